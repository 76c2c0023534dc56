#!/usr/bin/env python3
"""Benchmark of the FullyConnectedCompressed hot path on one MI355X.

One "step" is one decode pass (M = 1) over every FullyConnected of a Llama-3-8B-shaped model:
32 blocks x {q, k, v, o, gate, up, down}, int4 symmetric, group 128, f16 scales -- 224 launches over
3.6 GB of distinct weight buffers, so neither the per-XCD L2 nor the 256 MB Infinity Cache can serve
the weights.  All inputs are resident in HBM before the timed region.  The same run also times one
block's seven projections at M = 2048 (prefill) and reports TFLOP/s, and times the CPU oracle on the
host cores as a reported baseline.

Prints ONE JSON line on stdout; progress goes to stderr.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_F16_PEAK_TFLOPS = 2500.0

# HBM bytes per launch from the FETCH_SIZE / WRITE_SIZE counter runs recorded under profiles/ (counters cannot be
# read from inside this process): FETCH_SIZE x 2.000 (its reading for a copy kernel of known size) + WRITE_SIZE.
TRAFFIC_DECODE_M1 = {"qo": 8794112, "kv": 2283520, "gate_up": 30441472, "down": 30605312}
TRAFFIC_PREFILL_M2048 = {"qo": 85494784, "kv": 72139776, "gate_up": 264916992, "down": 255920128}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def algorithmic_bytes(K, N, M, bits=4, group=128, zp_bytes_per_group=0.0):
    ng = K // group
    return N * K * bits // 8 + N * ng * 2 + int(N * ng * zp_bytes_per_group) + M * K * 2 + M * N * 2


def results_table(dev, req, args) -> int:
    """All five benchmark configurations: kernel time with device-resident operands (HIP graph over a rotating set of
    weight copies larger than the caches), derived GB/s and TFLOP/s, and parity against the CPU oracle on a seeded
    sample of rows (every output channel)."""
    from openvino_amd import datagen, fc
    from oracle import oracle

    type_tag = {"u4": oracle.U4, "i4": oracle.I4, "u8": oracle.U8, "i8": oracle.I8, "none": oracle.NONE}
    rows = []

    def run(cfg, label, c, Ms, bits, zp_bytes_per_group, dtype):
        w = fc.CompressedWeights.from_case(dev, c)
        copies = [w]
        while sum(h.device_bytes for h in copies) < (600 << 20) and len(copies) < 48:
            copies.append(w.clone())
        x_dev = dev.malloc(c.x.nbytes)
        y_dev = dev.malloc(c.M * c.N * 2)
        for M in Ms:
            xs = np.ascontiguousarray(c.x[:M])
            y = req.infer(w, xs).astype(np.float32)
            info = req.last_kernel()
            pick = np.sort(np.random.default_rng(99).choice(M, size=min(16, M), replace=False))
            ref = oracle.fc_reference(xs[pick], c.w, type_tag[c.w_type], c.scale, c.zp, type_tag[c.zp_type], None,
                                      N=c.N, K=c.K, group_size=c.group_size)
            rl2, mab = oracle.rel_l2(y[pick], ref), oracle.max_abs(y[pick], ref)
            dev.upload(x_dev, xs)
            hs = copies if M <= 128 else copies[:1]
            reps = 20 if M <= 128 else 10
            best = min(req.bench_layers(hs, x_dev, y_dev, M, 3, reps, use_graph=True) for _ in range(2))
            us = best / reps / len(hs) * 1e3
            nbytes = algorithmic_bytes(c.K, c.N, M, bits, c.group_size, zp_bytes_per_group)
            gbs, tfs = nbytes / us / 1e3, 2.0 * M * c.N * c.K / us / 1e6
            rows.append(f"| {cfg} | {label} {c.K}->{c.N} | {M} | {dtype} | {info['name']} | {us:.1f} | "
                        f"{gbs:.0f} ({100 * gbs / HBM_PEAK_GBS:.1f} %) | {tfs:.1f} ({100 * tfs / 1000 / 2.5:.1f} %) | "
                        f"{rl2:.1e} | {mab:.1e} |")
            log(rows[-1])
        for h in copies:
            h.close()
        dev.free(x_dev)
        dev.free(y_dev)

    run(1, "q/o", datagen.config1(), [1], 4, 0.5, "u4 g128 asym")
    for shape in datagen.LLAMA3_8B_SHAPES:
        run(2, shape, datagen.config2(shape, 32), [1, 4, 16, 32], 4, 0.0, "i4 g128 sym")
    for shape in datagen.LLAMA3_8B_SHAPES:
        run(3, shape, datagen.config3(shape, 8192), [512, 2048, 8192], 4, 0.0, "i4 g128 sym")
    for shape in datagen.LLAMA3_70B_SHAPES:
        run(4, shape, datagen.config4(shape, 1024), [1, 32, 1024], 8, 1.0, "u8 per-channel asym")
    # Config 4's prefill row again with the node's activations allowed to be quantised per token to int8 (W8A8):
    # checked against the oracle of that arithmetic (exact integers) and, for reference, against the f16 oracle.
    for shape in datagen.LLAMA3_70B_SHAPES:
        c = datagen.config4(shape, 1024)
        w = fc.CompressedWeights.from_case(dev, c, dynamic_quantization=True)
        x_dev, y_dev = dev.malloc(c.x.nbytes), dev.malloc(c.M * c.N * 2)
        dev.upload(x_dev, c.x)
        y = req.infer(w, c.x).astype(np.float32)
        info = req.last_kernel()
        pick = np.sort(np.random.default_rng(99).choice(c.M, size=8, replace=False))
        zp = c.zp.astype(np.float32)
        ref_q = oracle.fc_dynquant_reference(c.x[pick], c.w, type_tag[c.w_type], c.scale, zp, None, N=c.N, K=c.K)
        ref_f = oracle.fc_reference(c.x[pick], c.w, type_tag[c.w_type], c.scale, c.zp, type_tag[c.zp_type], None,
                                    N=c.N, K=c.K, group_size=c.group_size)
        us = min(req.bench_layers([w], x_dev, y_dev, c.M, 3, 10, use_graph=True) for _ in range(2)) / 10 * 1e3
        nbytes = algorithmic_bytes(c.K, c.N, c.M, 8, c.group_size, 1.0)
        gbs, tfs = nbytes / us / 1e3, 2.0 * c.M * c.N * c.K / us / 1e6
        quantised = info["name"] == "fcc_prefill_i8_w8"
        rows.append(f"| 4 | {shape} {c.K}->{c.N}, int8 activations allowed | {c.M} | u8 per-channel asym"
                    f"{' x i8 per token' if quantised else ''} | {'fcc_dynquant + ' if quantised else ''}{info['name']} | "
                    f"{us:.1f} | {gbs:.0f} ({100 * gbs / HBM_PEAK_GBS:.1f} %) | {tfs:.1f} ({100 * tfs / 1000 / 2.5:.1f} % of f16 peak) | "
                    f"{oracle.rel_l2(y[pick], ref_q if quantised else ref_f):.1e} vs its own oracle, "
                    f"{oracle.rel_l2(y[pick], ref_f):.1e} vs f16 | {oracle.max_abs(y[pick], ref_q if quantised else ref_f):.1e} |")
        log(rows[-1])
        w.close()
        dev.free(x_dev)
        dev.free(y_dev)
    # Config 3's nodes at M = 2048 with int8 activations allowed (W4A8): per token, and per row and group of 128
    # inputs; checked against the oracle of that arithmetic and, for reference, against the f16 oracle.
    for mode, act_group in (("per_token", None), ("per_group", 128)):
        for shape in datagen.LLAMA3_8B_SHAPES:
            c = datagen.config3(shape, 2048)
            w = fc.CompressedWeights.from_case(dev, c, dynamic_quantization=mode)
            x_dev, y_dev = dev.malloc(c.x.nbytes), dev.malloc(c.M * c.N * 2)
            dev.upload(x_dev, c.x)
            y = req.infer(w, c.x).astype(np.float32)
            info = req.last_kernel()
            quantised = info["name"].startswith("fcc_prefill_i8_w4")
            pick = np.sort(np.random.default_rng(99).choice(c.M, size=8, replace=False))
            ref_f = oracle.fc_reference(c.x[pick], c.w, type_tag[c.w_type], c.scale, c.zp, type_tag[c.zp_type], None,
                                        N=c.N, K=c.K, group_size=c.group_size)
            ref_q = oracle.fc_dynquant_grouped_reference(c.x[pick], c.w, type_tag[c.w_type], c.scale, c.zp,
                                                         type_tag[c.zp_type], None, N=c.N, K=c.K,
                                                         group_size=c.group_size, act_group=act_group or c.K) \
                if quantised else ref_f
            us = min(req.bench_layers([w], x_dev, y_dev, c.M, 3, 10, use_graph=True) for _ in range(2)) / 10 * 1e3
            nbytes = algorithmic_bytes(c.K, c.N, c.M, 4, c.group_size, 0.0)
            gbs, tfs = nbytes / us / 1e3, 2.0 * c.M * c.N * c.K / us / 1e6
            rows.append(f"| 3 | {shape} {c.K}->{c.N}, int8 activations allowed ({mode.replace('_', ' ')}) | {c.M} | i4 g128 sym"
                        f"{' x i8 ' + mode.replace('_', ' ') if quantised else ''} | "
                        f"{'fcc_dynquant_w4 + ' if quantised else ''}{info['name']} | {us:.1f} | "
                        f"{gbs:.0f} ({100 * gbs / HBM_PEAK_GBS:.1f} %) | {tfs:.1f} ({100 * tfs / 1000 / 2.5:.1f} % of f16 peak) | "
                        f"{oracle.rel_l2(y[pick], ref_q):.1e} vs its own oracle, {oracle.rel_l2(y[pick], ref_f):.1e} vs f16 | "
                        f"{oracle.max_abs(y[pick], ref_q):.1e} |")
            log(rows[-1])
            w.close()
            dev.free(x_dev)
            dev.free(y_dev)


    routes = datagen.moe_routing()
    t_total, flops_total = 0.0, 0.0
    for e, tokens in enumerate(routes):
        for which in ("gate", "up", "down"):
            n0 = len(rows)
            run(5, f"expert {e} {which}", datagen.config5_expert(e, which, len(tokens)), [len(tokens)], 4, 0.5,
                "u4 g128 asym")
            us = float(rows[n0].split("|")[6])
            K, N = (4096, 14336) if which != "down" else (14336, 4096)
            t_total += us
            flops_total += 2.0 * len(tokens) * K * N
    log(f"config 5 as 24 separate launches: {t_total:.1f} us in total, {flops_total / t_total / 1e6:.1f} TFLOP/s")

    # The same 24 nodes as grouped runs: gate and up of all experts in one call (16 nodes of one shape), down in another.
    t_grouped = 0.0
    for label, names in (("experts gate+up, 16 nodes grouped", ("gate", "up")), ("experts down, 8 nodes grouped", ("down",))):
        cases = [datagen.config5_expert(e, which, len(routes[e])) for which in names for e in range(len(routes))]
        ws = [fc.CompressedWeights.from_case(dev, c) for c in cases]
        bufs = [(dev.malloc(c.x.nbytes), dev.malloc(c.M * c.N * 2)) for c in cases]
        for c, (xp, _) in zip(cases, bufs):
            dev.upload(xp, c.x)
        items = [(w, xp, yp, c.M) for w, c, (xp, yp) in zip(ws, cases, bufs)]
        req.infer_grouped_device(items)
        req.sync()
        info = req.last_kernel()
        rl2 = mab = 0.0
        for c, (_, yp) in zip(cases, bufs):
            y = dev.download(yp, (c.M, c.N), np.float16).astype(np.float32)
            pick = np.array([0, c.M // 2, c.M - 1])
            ref = oracle.fc_reference(c.x[pick], c.w, type_tag[c.w_type], c.scale, c.zp, type_tag[c.zp_type], None,
                                      N=c.N, K=c.K, group_size=c.group_size)
            rl2, mab = max(rl2, oracle.rel_l2(y[pick], ref)), max(mab, oracle.max_abs(y[pick], ref))
        us = min(req.bench_grouped(items, 3, 20) for _ in range(2)) / 20 * 1e3
        t_grouped += us
        nbytes = sum(algorithmic_bytes(c.K, c.N, c.M, 4, c.group_size, 0.5) for c in cases)
        gbs, tfs = nbytes / us / 1e3, sum(2.0 * c.M * c.N * c.K for c in cases) / us / 1e6
        rows.append(f"| 5 | {label} {cases[0].K}->{cases[0].N} | {'+'.join(str(len(t)) for t in routes)} | u4 g128 asym | "
                    f"{info['name']} | {us:.1f} | {gbs:.0f} ({100 * gbs / HBM_PEAK_GBS:.1f} %) | "
                    f"{tfs:.1f} ({100 * tfs / 1000 / 2.5:.1f} %) | {rl2:.1e} | {mab:.1e} |")
        log(rows[-1])
        for w in ws:
            w.close()
        for xp, yp in bufs:
            dev.free(xp)
            dev.free(yp)
    grouped_line = (f"config 5 as 2 grouped runs: {t_grouped:.1f} us in total, "
                    f"{flops_total / t_grouped / 1e6:.1f} TFLOP/s")
    log(grouped_line)

    # The same layer through the GatherMatmulCompressed entry point (routing indices in, gather and scatter on the
    # device): wall time per call over 20 back-to-back calls, host work included.
    import time
    tokens = 256
    indices = np.full((tokens, 2), -1, np.int32)
    for e, rows_e in enumerate(routes):
        for t in rows_e:
            indices[t, 0 if indices[t, 0] < 0 else 1] = e
    t_op = 0.0
    for label, which, batches in (("gate", "gate", 1), ("up", "up", 1), ("down", "down", 2)):
        cases = [datagen.config5_expert(e, which, 1) for e in range(len(routes))]
        ws = [fc.CompressedWeights.from_case(dev, c) for c in cases]
        K, N = cases[0].K, cases[0].N
        A = np.random.default_rng(5).standard_normal((batches, tokens, K)).astype(np.float16)
        a_ptr, y_ptr = dev.malloc(A.nbytes), dev.malloc(2 * tokens * N * 2)
        dev.upload(a_ptr, A)
        req.gather_matmul_device(ws, a_ptr, batches, indices, y_ptr)
        req.sync()
        y = dev.download(y_ptr, (2, tokens, N), np.float16).astype(np.float32)
        info = req.last_kernel()
        rl2 = mab = 0.0
        for t in (0, 101, 255):
            for i in range(2):
                c = cases[indices[t, i]]
                ref = oracle.fc_reference(A[i if batches > 1 else 0, t:t + 1], c.w, type_tag[c.w_type], c.scale, c.zp,
                                          type_tag[c.zp_type], None, N=N, K=K, group_size=c.group_size)
                rl2 = max(rl2, oracle.rel_l2(y[i, t:t + 1], ref))
                mab = max(mab, oracle.max_abs(y[i, t:t + 1], ref))
        best = 1e30
        for _ in range(3):
            t0 = time.perf_counter()
            for _ in range(20):
                req.gather_matmul_device(ws, a_ptr, batches, indices, y_ptr)
            req.sync()
            best = min(best, (time.perf_counter() - t0) / 20 * 1e6)
        t_op += best
        nbytes = sum(algorithmic_bytes(K, N, len(r_e), 4, 128, 0.5) for r_e in routes)
        gbs, tfs = nbytes / best / 1e3, 2.0 * 2 * tokens * N * K / best / 1e6
        rows.append(f"| 5 | gather-matmul op, {label} {K}->{N} (8 experts, top-2) | {tokens} tokens | u4 g128 asym | "
                    f"fcc_moe_route + {info['name']} (rows through the map) + scatter | {best:.1f} | {gbs:.0f} ({100 * gbs / HBM_PEAK_GBS:.1f} %) | "
                    f"{tfs:.1f} ({100 * tfs / 1000 / 2.5:.1f} %) | {rl2:.1e} | {mab:.1e} |")
        log(rows[-1])
        for w in ws:
            w.close()
        dev.free(a_ptr)
        dev.free(y_ptr)
    op_line = (f"config 5 as 3 gather-matmul calls (wall time, gather and scatter included): {t_op:.1f} us in total, "
               f"{flops_total / t_op / 1e6:.1f} TFLOP/s")
    log(op_line)
    # The whole layer as one call: MOECompressed (gate/up with a fused SwiGLU, down, routing-weighted sum).
    gu_cases, dn_cases, wg, wd = [], [], [], []
    for e in range(len(routes)):
        g, u = datagen.config5_expert(e, "gate", 1), datagen.config5_expert(e, "up", 1)
        gu_cases.append(datagen.FcCase(1, g.K, 2 * g.N, 128, "u4", "u4", np.concatenate([g.w, u.w]),
                                       np.concatenate([g.scale, u.scale]), np.concatenate([g.zp, u.zp]), g.x))
        dn_cases.append(datagen.config5_expert(e, "down", 1))
        wg.append(fc.CompressedWeights.from_case(dev, gu_cases[-1], glu="swish"))
        wd.append(fc.CompressedWeights.from_case(dev, dn_cases[-1]))
    rng5 = np.random.default_rng(55)
    xh = rng5.standard_normal((tokens, 4096)).astype(np.float16)
    rw = rng5.uniform(0.2, 0.8, size=(tokens, 1))
    routing = np.concatenate([rw, 1.0 - rw], axis=1).astype(np.float16)
    x_ptr, r_ptr, y_ptr = dev.malloc(xh.nbytes), dev.malloc(routing.nbytes), dev.malloc(tokens * 4096 * 2)
    dev.upload(x_ptr, xh)
    dev.upload(r_ptr, routing)
    req.moe_device(wg, wd, x_ptr, r_ptr, indices, y_ptr)
    req.sync()
    y = dev.download(y_ptr, (tokens, 4096), np.float16).astype(np.float32)
    pick = np.array([0, 101, 255])

    def eargs(c):
        return dict(w=c.w, w_type=type_tag[c.w_type], scale=c.scale, zp=c.zp, zp_type=type_tag[c.zp_type], bias=None,
                    N=c.N, K=c.K, group_size=c.group_size)
    ref = oracle.moe_reference(xh[pick], routing[pick], indices[pick], [eargs(c) for c in gu_cases],
                               [eargs(c) for c in dn_cases], 1)
    rl2, mab = oracle.rel_l2(y[pick], ref), oracle.max_abs(y[pick], ref)
    best = 1e30
    time.sleep(0.3)  # wall-clock timing: let the worker threads of the oracle's matrix products go idle first
    for _ in range(6):
        t0 = time.perf_counter()
        for _ in range(20):
            req.moe_device(wg, wd, x_ptr, r_ptr, indices, y_ptr)
        req.sync()
        best = min(best, (time.perf_counter() - t0) / 20 * 1e6)
    nbytes = 3 * sum(algorithmic_bytes(4096, 14336, len(r_e), 4, 128, 0.5) for r_e in routes)
    gbs, tfs = nbytes / best / 1e3, flops_total / best / 1e6
    rows.append(f"| 5 | mixture-of-experts block, 4096->14336->4096 (8 experts, top-2, SwiGLU fused) | {tokens} tokens | "
                f"u4 g128 asym | fcc_moe_route + 2 x fcc_prefill_async_grouped_w4 + weighted sum | {best:.1f} | "
                f"{gbs:.0f} ({100 * gbs / HBM_PEAK_GBS:.1f} %) | {tfs:.1f} ({100 * tfs / 1000 / 2.5:.1f} %) | "
                f"{rl2:.1e} | {mab:.1e} |")
    log(rows[-1])
    moe_line = (f"config 5 as one mixture-of-experts call (wall time; SwiGLU fused into gate/up, weighted sum over the "
                f"two experts of a token included): {best:.1f} us, {tfs:.1f} TFLOP/s")
    # the same call with the indices already in device memory (where a router's TopK leaves them)
    i_ptr = dev.malloc(indices.nbytes)
    dev.upload(i_ptr, np.ascontiguousarray(indices, dtype=np.int32))
    req.moe_routed_device(wg, wd, x_ptr, r_ptr, i_ptr, tokens, 2, y_ptr)
    req.sync()
    yd = dev.download(y_ptr, (tokens, 4096), np.float16).astype(np.float32)
    rl2d, mabd = oracle.rel_l2(yd[pick], ref), oracle.max_abs(yd[pick], ref)
    bestd = 1e30
    for _ in range(6):
        t0 = time.perf_counter()
        for _ in range(20):
            req.moe_routed_device(wg, wd, x_ptr, r_ptr, i_ptr, tokens, 2, y_ptr)
        req.sync()
        bestd = min(bestd, (time.perf_counter() - t0) / 20 * 1e6)
    gbsd, tfsd = nbytes / bestd / 1e3, flops_total / bestd / 1e6
    rows.append(f"| 5 | mixture-of-experts block, indices in device memory (routing kernel, no wait on the stream) | {tokens} tokens | "
                f"u4 g128 asym | fcc_moe_route + 2 x fcc_prefill_async_grouped_w4 + weighted sum | {bestd:.1f} | "
                f"{gbsd:.0f} ({100 * gbsd / HBM_PEAK_GBS:.1f} %) | {tfsd:.1f} ({100 * tfsd / 1000 / 2.5:.1f} %) | "
                f"{rl2d:.1e} | {mabd:.1e} |")
    log(rows[-1])
    dev.free(i_ptr)
    moe_line += f"; with the indices in device memory: {bestd:.1f} us"
    for w in wg + wd:
        w.close()
    for ptr in (x_ptr, r_ptr, y_ptr):
        dev.free(ptr)
    print("| Config | Shape (K->N) | M | dtype | GPU kernel | us | GB/s (% of 8 TB/s) | TFLOP/s (% of 2.5 PF) | "
          "rel-L2 vs fp32 | max-abs |")
    print("|---|---|---|---|---|---|---|---|---|---|")
    for r in rows:
        print(r)
    print(f"\nconfig 5 as 24 separate launches: {t_total:.1f} us in total, {flops_total / t_total / 1e6:.1f} TFLOP/s")
    print(grouped_line)
    print(op_line)
    print(moe_line)
    req.close()
    dev.close()
    return 0


def profile_moe(dev, req) -> int:
    """Short run for rocprofv3: the copy-kernel yardstick, then config 5's expert block (Mixtral-8x7B shapes, 8 experts,
    top-2, 256 tokens) a few times as one MOECompressed call with the routing indices in device memory."""
    from openvino_amd import datagen, fc

    dev.copy_bandwidth(256 << 20, 1)
    routes = datagen.moe_routing()
    tokens = 256
    indices = np.full((tokens, 2), -1, np.int32)
    for e, rows_e in enumerate(routes):
        for t in rows_e:
            indices[t, 0 if indices[t, 0] < 0 else 1] = e
    wg, wd = [], []
    for e in range(len(routes)):
        g, u = datagen.config5_expert(e, "gate", 1), datagen.config5_expert(e, "up", 1)
        gu = datagen.FcCase(1, g.K, 2 * g.N, 128, "u4", "u4", np.concatenate([g.w, u.w]),
                            np.concatenate([g.scale, u.scale]), np.concatenate([g.zp, u.zp]), g.x)
        wg.append(fc.CompressedWeights.from_case(dev, gu, glu="swish"))
        wd.append(fc.CompressedWeights.from_case(dev, datagen.config5_expert(e, "down", 1)))
    rng5 = np.random.default_rng(55)
    xh = rng5.standard_normal((tokens, 4096)).astype(np.float16)
    rw = rng5.uniform(0.2, 0.8, size=(tokens, 1))
    routing = np.concatenate([rw, 1.0 - rw], axis=1).astype(np.float16)
    x_ptr, r_ptr, y_ptr, i_ptr = (dev.malloc(xh.nbytes), dev.malloc(routing.nbytes), dev.malloc(tokens * 4096 * 2),
                                  dev.malloc(indices.nbytes))
    dev.upload(x_ptr, xh)
    dev.upload(r_ptr, routing)
    dev.upload(i_ptr, indices)
    for _ in range(5):
        req.moe_routed_device(wg, wd, x_ptr, r_ptr, i_ptr, tokens, 2, y_ptr)
    req.sync()
    log(f"rows per expert {[len(r) for r in routes]}; last launch {req.last_kernel()}")
    for w in wg + wd:
        w.close()
    for ptr in (x_ptr, r_ptr, y_ptr, i_ptr):
        dev.free(ptr)
    req.close()
    dev.close()
    return 0


def floors_table(dev, req, args) -> int:
    """Per Llama-3-8B shape at M = 1: the time of an empty graph node, of the best loads-only streaming kernel over the
    node's weight bytes (a sweep of workgroup shapes), and of the node itself -- all as nodes of replayed graphs over
    rotating buffers larger than the caches."""
    from openvino_amd import datagen, fc

    arena_bytes = 768 << 20
    arena = dev.malloc(arena_bytes)
    dev.copy_bandwidth(256 << 20, 1)
    empty = min(dev.floor_us(arena, arena_bytes, 0) for _ in range(3))
    x_dev, y_dev = dev.malloc(14336 * 2 * 4), dev.malloc(2 * 14336 * 2 * 4)
    print("| node | weight bytes | empty graph node us | loads-only streaming kernel us (GB/s) | fcc_gemv_w4 us (GB/s) | "
          "kernel / streaming |")
    print("|---|---|---|---|---|---|")
    total_probe = total_kernel = 0.0
    for name, (K, N) in datagen.LLAMA3_8B_SHAPES.items():
        wbytes = N * K // 2
        best = 1e30
        for waves in (4, 8, 16):
            for kpw in (8, 16, 32):
                if (wbytes >> 10) % (waves * kpw) or (wbytes >> 10) // (waves * kpw) < 64:
                    continue
                best = min(best, min(dev.floor_us(arena, arena_bytes, wbytes, 96, waves, kpw) for _ in range(2)))
        c = datagen.weights_only(2001, K, N, "i4", 128, "none")
        w = fc.CompressedWeights.from_case(dev, c)
        copies = [w]
        while sum(h.device_bytes for h in copies) < (600 << 20) and len(copies) < 48:
            copies.append(w.clone())
        t = min(req.bench_layers(copies, x_dev, y_dev, 1, 3, 20, use_graph=True) for _ in range(3)) / 20 / len(copies) * 1e3
        nbytes = algorithmic_bytes(K, N, 1)
        per_block = 2 if name in ("qo", "kv", "gate_up") else 1
        total_probe += per_block * best
        total_kernel += per_block * t
        print(f"| {name} {K}->{N} | {wbytes} | {empty:.2f} | {best:.2f} ({wbytes / best / 1e3:.0f}) | {t:.2f} "
              f"({nbytes / t / 1e3:.0f}) | {t / best:.2f} |")
        log(f"{name}: empty {empty:.2f} probe {best:.2f} kernel {t:.2f}")
        for h in copies:
            h.close()
    block_bytes = sum(algorithmic_bytes(*datagen.LLAMA3_8B_SHAPES[n], 1) for n in datagen.LLAMA3_8B_BLOCK)
    print(f"\none block (q, k, v, o, gate, up, down): streaming kernels {total_probe:.1f} us = "
          f"{block_bytes / total_probe / 1e3:.0f} GB/s ({100 * block_bytes / total_probe / 1e3 / HBM_PEAK_GBS:.1f} % of 8 TB/s); "
          f"fcc_gemv_w4 {total_kernel:.1f} us = {block_bytes / total_kernel / 1e3:.0f} GB/s "
          f"({100 * block_bytes / total_kernel / 1e3 / HBM_PEAK_GBS:.1f} %)")
    # what the matrix cores sustain with nothing else to do (the chip lowers its clock under this load)
    print("\n| matrix-core loop on registers, all compute units | TFLOP/s | of 2.5 PFLOP/s |")
    print("|---|---|---|")
    for shape, name in ((0, "v_mfma_f32_16x16x32_f16"), (1, "v_mfma_f32_32x32x16_f16")):
        for waves, valu in ((4, 0), (8, 0), (8, 2), (8, 3), (8, 4)):
            tf = max(dev.mfma_ceiling(waves, valu, shape=shape) for _ in range(2))
            print(f"| {name}, {waves // 4} wave(s) per SIMD, {valu} packed-f16 multiplications per 16 x 16 x 32 of "
                  f"matrix work | {tf:.0f} | {100 * tf / 2500:.1f} % |")
    # ... and how that depends on what the weight operand looks like (activation operand random halves)
    print("\n| v_mfma_f32_16x16x32_f16 on registers, two waves per SIMD, all compute units; one operand random halves, "
          "the other: | TFLOP/s | of 2.5 PFLOP/s |")
    print("|---|---|---|")
    for shape, name in ((0, "random halves too"), (4, "integers -8 .. 7 times a scale, rounded to half (what the prefill kernels feed)"),
                        (2, "integers -8 .. 7 as halves"), (3, "integers 0 .. 15 as subnormal halves (what the decode kernels feed)")):
        tf = max(dev.mfma_ceiling(8, 0, shape=shape) for _ in range(3))
        print(f"| {name} | {tf:.0f} | {100 * tf / 2500:.1f} % |")
    # how one SIMD overlaps matrix-core and vector instructions, in shader cycles: one compute unit alone, then all
    n_cus = 256
    print("\n| matrix-core loop with vector instructions after every MFMA (v_mfma_f32_16x16x32_f16, two waves per SIMD) | "
          "one compute unit: cycles, ns per MFMA and SIMD | all compute units: cycles, ns |")
    print("|---|---|---|")
    for mode, valu, what in ((0, 0, "no vector instruction"), (0, 2, "2 independent packed-f16 multiplications"),
                             (0, 3, "3 independent"), (0, 4, "4 independent"), (0, 6, "6 independent"),
                             (1, 3, "3 in one dependent chain"),
                             (2, 3, "3, the first writes a register of the B operand just read"),
                             (3, 3, "3 independent, MFMA destination is not its accumulator input")):
        one = dev.issue_probe(1, 8, mode, valu)
        all_ = dev.issue_probe(n_cus, 8, mode, valu)
        print(f"| {what} | {one[0]:.1f}, {one[1]:.2f} | {all_[0]:.1f}, {all_[1]:.2f} |")
    one = dev.issue_probe(1, 4, 0, 0)
    print(f"| no vector instruction, one wave per SIMD | {one[0]:.1f}, {one[1]:.2f} | |")
    for ptr in (arena, x_dev, y_dev):
        dev.free(ptr)
    req.close()
    dev.close()
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--layers", type=int, default=32, help="transformer blocks in the rotating weight set")
    ap.add_argument("--prefill-m", type=int, default=2048)
    ap.add_argument("--no-graph", action="store_true", help="launch eagerly instead of replaying a HIP graph")
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--cpu-seconds", type=float, default=10.0)
    ap.add_argument("--table", action="store_true",
                    help="time and parity-check every benchmark configuration (1-5) and print a markdown table on "
                         "stdout instead of the JSON line")
    ap.add_argument("--floors", action="store_true",
                    help="measure what bounds a decode node from below -- an empty graph node, a loads-only streaming "
                         "kernel over the node's weight bytes -- beside the node's own time, and print a markdown table")
    ap.add_argument("--profile", choices=["decode", "decode-graph", "batch", "prefill", "w8a8", "w4a8", "moe"], default=None,
                    help="short run for rocprofv3: one copy-kernel launch of known size (the counter yardstick), "
                         "then a few eager passes of the chosen kernel family; prints no JSON")
    ap.add_argument("--profile-rows", type=int, default=32,
                    help="row count of --profile batch (2..32; default: config 2's largest)")
    args = ap.parse_args()
    if args.gpus != 1:
        log("bench.py: this build measures one GPU only (the path has no collectives); run with --gpus 1")
        return 2

    from openvino_amd import _lib, datagen, fc

    if not os.path.exists(_lib.LIB_PATH):
        import __graft_entry__
        __graft_entry__.build()

    dev = fc.Device(0)
    req = fc.InferRequest(dev)
    if args.table:
        return results_table(dev, req, args)
    if args.floors:
        return floors_table(dev, req, args)
    if args.profile == "moe":
        return profile_moe(dev, req)

    # ---- weights: one host tensor set per shape, one device copy per use ----
    t0 = time.perf_counter()
    base = {}
    cases = {}
    for i, (name, (K, N)) in enumerate(datagen.LLAMA3_8B_SHAPES.items()):
        c = datagen.weights_only(2001 + i, K, N, "i4", 128, "none")
        cases[name] = c
        base[name] = fc.CompressedWeights.from_case(dev, c)
    layers = []
    for _ in range(args.layers):
        for name in datagen.LLAMA3_8B_BLOCK:
            layers.append((name, base[name].clone()))
    weight_bytes = sum(w.device_bytes for _, w in layers)
    log(f"rotating weight set: {len(layers)} nodes, {weight_bytes / 1e9:.2f} GB on device "
        f"({time.perf_counter() - t0:.1f} s to build)")

    max_k = max(K for K, _ in datagen.LLAMA3_8B_SHAPES.values())
    max_n = max(N for _, N in datagen.LLAMA3_8B_SHAPES.values())
    m_max = max(32, args.prefill_m)
    rng = np.random.default_rng(77)
    x_host = rng.standard_normal((m_max, max_k), dtype=np.float32).astype(np.float16)
    x_dev = dev.malloc(x_host.nbytes)
    y_dev = dev.malloc(m_max * 2 * max_n * 2)      # (the concatenated gate/up node has 2 max_n channels)
    dev.upload(x_dev, x_host)

    if args.profile:
        # yardstick: one 256 MiB device-to-device copy (reads 256 MiB, writes 256 MiB)
        dev.copy_bandwidth(256 << 20, 1)
        if args.profile == "w8a8":
            # Llama-3-70B u8 per-channel projections at M = 1024, int8 activations allowed (config 4 of the table)
            for shape in ("qo", "gate_up", "down"):
                c = datagen.config4(shape, 1024)
                w = fc.CompressedWeights.from_case(dev, c, dynamic_quantization=True)
                xq_dev, yq_dev = dev.malloc(c.x.nbytes), dev.malloc(c.M * c.N * 2)
                dev.upload(xq_dev, c.x)
                for _ in range(3):
                    req.infer_device(w, xq_dev, yq_dev, c.M)
                req.sync()
                w.close()
                dev.free(xq_dev)
                dev.free(yq_dev)
        elif args.profile == "w4a8":
            # Llama-3-8B i4 g128 projections at the prefill row count with int8 activations allowed: per token, then
            # per row and group of 128 inputs (config 3's nodes through the integer kernel)
            for mode in ("per_token", "per_group"):
                for shape in ("qo", "gate_up", "down"):
                    c = datagen.config3(shape, args.prefill_m)
                    w = fc.CompressedWeights.from_case(dev, c, dynamic_quantization=mode)
                    xq_dev, yq_dev = dev.malloc(c.x.nbytes), dev.malloc(c.M * c.N * 2)
                    dev.upload(xq_dev, c.x)
                    for _ in range(3):
                        req.infer_device(w, xq_dev, yq_dev, c.M)
                    req.sync()
                    w.close()
                    dev.free(xq_dev)
                    dev.free(yq_dev)
        elif args.profile == "decode-graph":
            # the headline pass as the benchmark runs it: all nodes captured into one HIP graph, replayed four times
            # (one capture and one instantiation in the whole process)
            req.bench_layers([w for _, w in layers], x_dev, y_dev, 1, 1, 3, use_graph=True)
        elif args.profile in ("decode", "batch"):
            rows = 1 if args.profile == "decode" else min(32, max(2, args.profile_rows))
            for _ in range(3):
                for _, w in layers:
                    req.infer_device(w, x_dev, y_dev, rows)
        else:
            for _ in range(3):
                for name in datagen.LLAMA3_8B_BLOCK:
                    req.infer_device(base[name], x_dev, y_dev, args.prefill_m)
        req.sync()
        log(f"profile run done ({args.profile})")
        return 0

    # ---- correctness of the timed path against the oracle, before timing ----
    from oracle import oracle
    parity = {}
    for name, M in (("kv", 1), ("qo", 1)):
        c = cases[name]
        xs = np.ascontiguousarray(x_host[:M, :c.K])
        y = req.infer(base[name], xs).astype(np.float32)
        ref = oracle.fc_reference(xs, c.w, oracle.I4, c.scale, None, oracle.NONE, None, N=c.N, K=c.K, group_size=128)
        parity[f"{name}_M{M}"] = {"rel_l2": oracle.rel_l2(y, ref), "max_abs": oracle.max_abs(y, ref)}
        assert parity[f"{name}_M{M}"]["rel_l2"] < 1e-3, parity

    # ---- decode: K timed passes over the rotating set ----
    M = 1
    handles = [w for _, w in layers]
    pass_bytes = sum(algorithmic_bytes(*datagen.LLAMA3_8B_SHAPES[name], M) for name, _ in layers)
    wall0 = time.perf_counter()
    ms = req.bench_layers(handles, x_dev, y_dev, M, args.warmup, args.steps, use_graph=not args.no_graph)
    wall = time.perf_counter() - wall0
    ms_per_step = ms / args.steps
    gbs = pass_bytes / (ms_per_step * 1e-3) / 1e9
    launches = len(layers)
    log(f"decode M=1: {ms_per_step:.4f} ms/pass, {launches} launches, {pass_bytes / 1e9:.3f} GB/pass -> {gbs:.1f} GB/s "
        f"({100 * gbs / HBM_PEAK_GBS:.1f} % of 8 TB/s); wall {wall:.2f} s incl. warm-up")

    # per-shape figures (each shape rotating over its own copies), for the results table
    per_shape = {}
    for name, (K, N) in datagen.LLAMA3_8B_SHAPES.items():
        hs = [w for n_, w in layers if n_ == name]
        for Mx in (1, 4, 8, 16, 32):
            t = req.bench_layers(hs, x_dev, y_dev, Mx, 2, max(5, args.steps // 5), use_graph=not args.no_graph)
            per = t / max(5, args.steps // 5) / len(hs)
            b = algorithmic_bytes(K, N, Mx)
            per_shape[f"{name}_M{Mx}"] = {"us": per * 1e3, "GBps": b / (per * 1e-3) / 1e9}
        log(f"  {name}: " + ", ".join(f"M={m}: {per_shape[f'{name}_M{m}']['us']:.2f} us "
                                      f"{per_shape[f'{name}_M{m}']['GBps']:.0f} GB/s" for m in (1, 4, 8, 16, 32)))
    # small batches: one block of seven nodes (q, k, v, o, gate, up, down) against its time at one row
    block_us = {m: sum(per_shape[f"{n_}_M{m}"]["us"] * reps for n_, reps in (("qo", 2), ("kv", 2), ("gate_up", 2), ("down", 1)))
                for m in (1, 4, 8, 16, 32)}
    small_batch = {f"M{m}": {"block_us": round(block_us[m], 2), "vs_M1": round(block_us[m] / block_us[1], 3)}
                   for m in (1, 4, 8, 16, 32)}
    log("  block of seven nodes: " + ", ".join(f"M={m}: {block_us[m]:.1f} us ({block_us[m] / block_us[1]:.2f} x)"
                                               for m in (1, 4, 8, 16, 32)))

    # horizontal fusion (q,k,v -> one node; gate,up -> one node): 4 launches per block instead of 7
    fused_base = {
        "qkv": fc.CompressedWeights.concat([base["qo"], base["kv"], base["kv"]]),
        "o": base["qo"],
        "gate_up2": fc.CompressedWeights.concat([base["gate_up"], base["gate_up"]]),
        "down": base["down"],
    }
    fused_layers = []
    for _ in range(args.layers):
        for name in ("qkv", "o", "gate_up2", "down"):
            fused_layers.append(fused_base[name].clone())
    fms = req.bench_layers(fused_layers, x_dev, y_dev, 1, args.warmup, args.steps, use_graph=not args.no_graph)
    fused_bytes = sum(w.N * w.K // 2 + w.N * (w.K // 128) * 2 + w.K * 2 + w.N * 2 for w in fused_layers)
    fused_gbs = fused_bytes / (fms / args.steps * 1e-3) / 1e9
    log(f"decode M=1 with q/k/v and gate/up fused: {fms / args.steps:.4f} ms/pass, {len(fused_layers)} launches -> "
        f"{fused_gbs:.1f} GB/s ({100 * fused_gbs / HBM_PEAK_GBS:.1f} % of 8 TB/s)")
    for w in fused_layers:
        w.close()

    # the same block with the gated MLP as one node (gate / up with SwiGLU, then down: the CPU plugin's LLMMLP): q/k/v, o,
    # mlp.  The node runs as two launches (4 per block); OVFCC_MLP_FUSED=1 selects its one-launch kernel (3 per block).
    mlp_base = {"qkv": fused_base["qkv"], "o": base["qo"]}
    glu_node = fc.CompressedWeights.glu(base["gate_up"], base["gate_up"], "swish")
    mlp_base["mlp"] = fc.CompressedWeights.mlp(glu_node, base["down"])
    glu_node.close()
    mlp_layers = [mlp_base[name].clone() for _ in range(args.layers) for name in ("qkv", "o", "mlp")]
    mlp_modes = {}
    saved = os.environ.get("OVFCC_MLP_FUSED")
    for mode, flag in (("two_launches", "0"), ("one_launch", "1")):
        os.environ["OVFCC_MLP_FUSED"] = flag
        _lib.sync_env()
        t = req.bench_layers(mlp_layers, x_dev, y_dev, 1, args.warmup, args.steps, use_graph=not args.no_graph)
        g = fused_bytes / (t / args.steps * 1e-3) / 1e9
        mlp_modes[mode] = {"ms_per_pass": round(t / args.steps, 5), "GBps": round(g, 1),
                           "pct_of_hbm_peak": round(100 * g / HBM_PEAK_GBS, 2), "kernel": req.last_kernel()["name"]}
        log(f"decode M=1 with q/k/v fused and the MLP as one node ({mode.replace('_', ' ')}): {t / args.steps:.4f} ms/pass -> "
            f"{g:.1f} GB/s ({100 * g / HBM_PEAK_GBS:.1f} % of 8 TB/s)")
    if saved is None:
        os.environ.pop("OVFCC_MLP_FUSED", None)
    else:
        os.environ["OVFCC_MLP_FUSED"] = saved
    _lib.sync_env()
    for w in mlp_layers:
        w.close()
    mlp_base["mlp"].close()

    copy_gbs = dev.copy_bandwidth(1 << 30, 10)
    log(f"plain copy kernel: {copy_gbs:.0f} GB/s (read + write)")

    out = {
        "metric": "int4 FC GB/s (% of 8TB/s) at M=1 + TFLOP/s at M=2048, Llama-3-8B shapes",
        "value": round(gbs, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16 activations x int4 weights, f32 accumulate",
        "data": "synthetic (seeded): i4 weights uniform -8..7, f16 scales U(0.002,0.02), f16 activations N(0,1)",
        "config": {
            "workload": f"Llama-3-8B decode pass, M=1: {args.layers} blocks x (q,k,v,o,gate,up,down) int4 g128 "
                        f"symmetric FullyConnectedCompressed, {launches} launches over {weight_bytes / 1e9:.2f} GB "
                        f"of distinct weight buffers",
            "launch": "eager" if args.no_graph else "hip graph replay",
            "pct_of_hbm_peak": round(100 * gbs / HBM_PEAK_GBS, 2),
        },
        "roofline": {
            "bound": "hbm", "kernel": "fcc_gemv_w4", "achieved": round(gbs, 2), "peak": HBM_PEAK_GBS,
            "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4),
            "traffic": (sum(TRAFFIC_DECODE_M1[name] for name, _ in layers) // launches
                        if set(n for n, _ in layers) <= set(TRAFFIC_DECODE_M1) else None),
            "traffic_source": "profiles/fcc_gemv_w4_llama3_8b_m1.md",
            "algorithmic_bytes_per_launch": pass_bytes // launches,
            "avg_launch_us": round(ms_per_step * 1e3 / launches, 3),
        },
        "copy_kernel_GBps": round(copy_gbs, 1),
        "decode_fused": {"note": "same pass with q/k/v and gate/up concatenated into one node each "
                                 "(ovfcc_weights_concat), 4 launches per block",
                         "launches": args.layers * 4, "ms_per_pass": round(fms / args.steps, 5),
                         "GBps": round(fused_gbs, 1), "pct_of_hbm_peak": round(100 * fused_gbs / HBM_PEAK_GBS, 2)},
        "decode_mlp_node": {"note": "same pass with q/k/v concatenated and gate/up (SwiGLU) + down as one MLP node "
                                    "(ovfcc_weights_mlp): as the two launches it runs by default, and as its one-launch "
                                    "kernel (OVFCC_MLP_FUSED=1); algorithmic bytes as in decode_fused", **mlp_modes},
        "decode_small_batch": small_batch,
        "decode_per_shape": {k: {"us": round(v["us"], 3), "GBps": round(v["GBps"], 1)} for k, v in per_shape.items()},
        "parity": {k: {a: float(f"{b:.3e}") for a, b in v.items()} for k, v in parity.items()},
    }

    # ---- prefill: one block's seven projections at M = 2048 ----
    if not args.no_prefill:
        Mp = args.prefill_m
        block = [w for _, w in layers[:len(datagen.LLAMA3_8B_BLOCK)]]
        flops = sum(2 * Mp * K * N for K, N in (datagen.LLAMA3_8B_SHAPES[n] for n in datagen.LLAMA3_8B_BLOCK))
        # parity of the timed kernel on a sample of rows
        c = cases["qo"]
        xs = np.ascontiguousarray(x_host[:Mp, :c.K])
        y = req.infer(base["qo"], xs).astype(np.float32)
        pick = np.sort(np.random.default_rng(5).choice(Mp, size=16, replace=False))
        ref = oracle.fc_reference(xs[pick], c.w, oracle.I4, c.scale, None, oracle.NONE, None, N=c.N, K=c.K,
                                  group_size=128)
        out["parity"][f"qo_M{Mp}"] = {"rel_l2": float(f"{oracle.rel_l2(y[pick], ref):.3e}"),
                                      "max_abs": float(f"{oracle.max_abs(y[pick], ref):.3e}")}
        assert out["parity"][f"qo_M{Mp}"]["rel_l2"] < 1e-3, out["parity"]
        psteps = max(10, args.steps // 2)
        pwarm = max(10, args.warmup)     # the clocks take some tens of milliseconds of MFMA load to settle
        pms = req.bench_layers(block, x_dev, y_dev, Mp, pwarm, psteps, use_graph=not args.no_graph)
        tflops = flops * psteps / (pms * 1e-3) / 1e12
        log(f"prefill M={Mp}: {pms / psteps:.3f} ms/block -> {tflops:.1f} TFLOP/s "
            f"({100 * tflops / MFMA_F16_PEAK_TFLOPS:.1f} % of 2.5 PFLOP/s)")
        pshape = {}
        for name, (K, N) in datagen.LLAMA3_8B_SHAPES.items():
            t = req.bench_layers([base[name]], x_dev, y_dev, Mp, pwarm, psteps, use_graph=not args.no_graph) / psteps
            pshape[name] = {"us": round(t * 1e3, 2), "TFLOPs": round(2 * Mp * K * N / (t * 1e-3) / 1e12, 1)}
        log("  " + ", ".join(f"{k}: {v['us']} us {v['TFLOPs']} TFLOP/s" for k, v in pshape.items()))
        # the same block with q/k/v and gate/up concatenated (4 launches, the same flops)
        fblock = [fused_base[n] for n in ("qkv", "o", "gate_up2", "down")]
        fpms = req.bench_layers(fblock, x_dev, y_dev, Mp, pwarm, psteps, use_graph=not args.no_graph)
        ftflops = flops * psteps / (fpms * 1e-3) / 1e12
        log(f"prefill M={Mp} with q/k/v and gate/up fused: {fpms / psteps:.3f} ms/block -> {ftflops:.1f} TFLOP/s "
            f"({100 * ftflops / MFMA_F16_PEAK_TFLOPS:.1f} % of 2.5 PFLOP/s)")
        out["prefill_fused"] = {"note": "same block with q/k/v and gate/up concatenated into one node each, 4 launches",
                                "M": Mp, "ms_per_block": round(fpms / psteps, 4), "TFLOPs": round(ftflops, 2),
                                "pct_of_mfma_peak": round(100 * ftflops / MFMA_F16_PEAK_TFLOPS, 2)}
        out["prefill"] = {
            "M": Mp, "TFLOPs": round(tflops, 2), "pct_of_mfma_peak": round(100 * tflops / MFMA_F16_PEAK_TFLOPS, 2),
            "ms_per_block": round(pms / psteps, 4), "steps": psteps, "per_shape": pshape,
            "roofline": {"bound": "mfma", "kernel": "fcc_prefill_big_w4 (gate, up) + fcc_prefill_async_w4", "achieved": round(tflops, 2),
                         "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                         "frac": round(tflops / MFMA_F16_PEAK_TFLOPS, 4),
                         "traffic": (sum(TRAFFIC_PREFILL_M2048[n] for n in datagen.LLAMA3_8B_BLOCK)
                                     // len(datagen.LLAMA3_8B_BLOCK) if Mp == 2048 else None),
                         "traffic_source": "profiles/fcc_prefill_w4_llama3_8b_m2048.md"},
        }

    # ---- CPU baseline: the blocked, vectorised port of the oracle's formula on the host cores, bounded samples ----
    if not args.no_cpu:
        c = cases["qo"]
        cores = oracle.lib().ovo_num_threads()

        def cpu_time(rows, budget):
            xs_ = np.ascontiguousarray(x_host[:rows, :c.K])
            n_, t_ = 0, time.perf_counter()
            while True:
                oracle.fc_reference(xs_, c.w, oracle.I4, c.scale, None, oracle.NONE, None, N=c.N, K=c.K, group_size=128,
                                    blocked=True)
                n_ += 1
                el_ = time.perf_counter() - t_
                if el_ >= budget or n_ >= 2000:
                    return n_, el_
        cpu_time(1, 0.2)   # page the weights in, start the worker threads
        n, el = cpu_time(1, args.cpu_seconds * 0.6)
        b = algorithmic_bytes(c.K, c.N, 1)
        out["cpu_baseline"] = {
            "value": round(b * n / el / 1e9, 3), "unit": "GB/s", "cores": int(cores), "kind": "port",
            "sample": f"{n} calls of the q/o projection (K=4096, N=4096, M=1, int4 g128) by the blocked C port of the "
                      f"oracle's formula (fp32 dequantise-then-dot, 16-lane partial sums, OpenMP) in {el:.1f} s",
        }
        log(f"cpu baseline: {out['cpu_baseline']['value']} GB/s on {cores} threads")
        if not args.no_prefill:
            Mp = args.prefill_m
            n, el = cpu_time(Mp, args.cpu_seconds * 0.4)
            tf = 2.0 * Mp * c.K * c.N * n / el / 1e12
            out["cpu_baseline"]["prefill"] = {
                "value": round(tf, 4), "unit": "TFLOP/s", "cores": int(cores), "kind": "port",
                "sample": f"{n} calls of the q/o projection at M={Mp} by the same port (panels of 32 dequantised channels, "
                          f"4 x 4 register-blocked micro-kernel) in {el:.1f} s",
            }
            log(f"cpu baseline, prefill: {tf:.3f} TFLOP/s on {cores} threads")

    print(json.dumps(out), flush=True)
    for _, w in layers:
        w.close()
    for k in ("qkv", "gate_up2"):
        fused_base[k].close()
    for w in base.values():
        w.close()
    dev.free(x_dev)
    dev.free(y_dev)
    req.close()
    dev.close()
    return 0


if __name__ == "__main__":
    sys.exit(main())
