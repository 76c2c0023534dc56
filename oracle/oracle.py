"""CPU oracle for FullyConnectedCompressed -- TEST INFRASTRUCTURE ONLY.

Loads ``oracle/liboracle.so`` (built from ``oracle/oracle.c`` by ``oracle/Makefile``) and
offers an independent numpy float64 restatement of the same formula for small cases.
Only tests, the smoke check and the benchmark's ``cpu_baseline`` leg may import this
module; the product package never does.

Formula (OpenVINO: fully_connected_gpu_bfyx_ref.cl:88-160, ov_ops/fully_connected.cpp:40-57)::

    y[m, n] = sum_k x[m, k] * ((q[n, k] - zp[n, k // G]) * s[n, k // G]) + bias[n]

with ``q`` stored row-major ``[N, K]``; u4/i4 buffers hold element ``i`` in byte ``i // 2``,
low nibble first (element_iterator.hpp:76,161-176), i4 sign-extended (:248-259).
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))

NONE, U4, I4, U8, I8, F16, F32 = range(7)
TYPE_NAMES = {"none": NONE, "u4": U4, "i4": I4, "u8": U8, "i8": I8, "f16": F16, "f32": F32}


class _FcArgs(ctypes.Structure):
    _fields_ = [
        ("M", ctypes.c_int64), ("N", ctypes.c_int64), ("K", ctypes.c_int64),
        ("group_size", ctypes.c_int64),
        ("w_type", ctypes.c_int32), ("scale_type", ctypes.c_int32),
        ("zp_type", ctypes.c_int32), ("zp_scalar", ctypes.c_int32),
        ("bias_type", ctypes.c_int32), ("x_type", ctypes.c_int32),
        ("acc_f64", ctypes.c_int32), ("reserved", ctypes.c_int32),
        ("w", ctypes.c_void_p), ("scale", ctypes.c_void_p), ("zp", ctypes.c_void_p),
        ("bias", ctypes.c_void_p), ("x", ctypes.c_void_p),
        ("n_index", ctypes.c_void_p), ("n_count", ctypes.c_int64),
    ]


_lib = None
_ref = None


def build(force: bool = False) -> None:
    """Compile liboracle.so (and oracle/_ref when the reference tree is present)."""
    args = ["make", "-C", HERE]
    if force:
        args.append("-B")
    subprocess.run(args, check=True, stdout=subprocess.DEVNULL)


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        path = os.path.join(HERE, "liboracle.so")
        if not os.path.exists(path):
            build()
        L = ctypes.CDLL(path)
        L.ovo_f32_to_f16.argtypes = [ctypes.c_float]
        L.ovo_f32_to_f16.restype = ctypes.c_uint16
        L.ovo_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.ovo_f16_to_f32.restype = ctypes.c_float
        for name in ("ovo_unpack_u4", "ovo_unpack_i4", "ovo_pack_u4", "ovo_pack_i4",
                     "ovo_f32_to_f16_n", "ovo_f16_to_f32_n"):
            getattr(L, name).argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]
            getattr(L, name).restype = None
        L.ovo_fc_reference.argtypes = [ctypes.POINTER(_FcArgs), ctypes.c_void_p]
        L.ovo_fc_reference.restype = ctypes.c_int
        L.ovo_fc_blocked.argtypes = [ctypes.POINTER(_FcArgs), ctypes.c_void_p]
        L.ovo_fc_blocked.restype = ctypes.c_int
        L.ovo_num_threads.restype = ctypes.c_int
        L.ovo_set_num_threads.argtypes = [ctypes.c_int]
        _lib = L
    return _lib


def ref_lib():
    """The reference's own element iterator / float16, or None where it was not built."""
    global _ref
    if _ref is None:
        path = os.path.join(HERE, "_ref", "libovref.so")
        if not os.path.exists(path):
            return None
        R = ctypes.CDLL(path)
        R.ref_f32_to_f16.argtypes = [ctypes.c_float]
        R.ref_f32_to_f16.restype = ctypes.c_uint16
        R.ref_f16_to_f32.argtypes = [ctypes.c_uint16]
        R.ref_f16_to_f32.restype = ctypes.c_float
        for name in ("ref_unpack_u4", "ref_unpack_i4", "ref_pack_u4", "ref_pack_i4"):
            getattr(R, name).argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]
            getattr(R, name).restype = None
        _ref = R
    return _ref


def _ptr(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


# ---------------------------------------------------------------- packing ----

def unpack_u4(packed: np.ndarray, n: int) -> np.ndarray:
    packed = np.ascontiguousarray(packed, dtype=np.uint8)
    assert packed.size >= (n + 1) // 2
    out = np.empty(n, dtype=np.uint8)
    lib().ovo_unpack_u4(_ptr(packed), n, _ptr(out))
    return out


def unpack_i4(packed: np.ndarray, n: int) -> np.ndarray:
    packed = np.ascontiguousarray(packed, dtype=np.uint8)
    assert packed.size >= (n + 1) // 2
    out = np.empty(n, dtype=np.int8)
    lib().ovo_unpack_i4(_ptr(packed), n, _ptr(out))
    return out


def pack_u4(values: np.ndarray) -> np.ndarray:
    values = np.ascontiguousarray(values, dtype=np.uint8).ravel()
    out = np.empty((values.size + 1) // 2, dtype=np.uint8)
    lib().ovo_pack_u4(_ptr(values), values.size, _ptr(out))
    return out


def pack_i4(values: np.ndarray) -> np.ndarray:
    values = np.ascontiguousarray(values, dtype=np.int8).ravel()
    out = np.empty((values.size + 1) // 2, dtype=np.uint8)
    lib().ovo_pack_i4(_ptr(values), values.size, _ptr(out))
    return out


def f32_to_f16_bits(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32).ravel()
    out = np.empty(x.size, dtype=np.uint16)
    lib().ovo_f32_to_f16_n(_ptr(x), x.size, _ptr(out))
    return out


def f16_bits_to_f32(h: np.ndarray) -> np.ndarray:
    h = np.ascontiguousarray(h, dtype=np.uint16).ravel()
    out = np.empty(h.size, dtype=np.float32)
    lib().ovo_f16_to_f32_n(_ptr(h), h.size, _ptr(out))
    return out


# ------------------------------------------------------------ FC reference ----

def _as_real(a, name):
    """float16 / float32 array -> (contiguous array, type tag)."""
    a = np.ascontiguousarray(a)
    if a.dtype == np.float16:
        return a, F16
    if a.dtype == np.float32:
        return a, F32
    raise TypeError(f"{name}: expected float16 or float32, got {a.dtype}")


def fc_reference(x, w, w_type, scale, zp=None, zp_type=NONE, bias=None, *, N, K, group_size,
                 zp_scalar=False, acc_f64=False, n_index=None, blocked=False) -> np.ndarray:
    """C oracle.  ``w`` and u4 ``zp`` are the raw packed bytes in OpenVINO order.  blocked: the blocked,
    vectorised port of the same formula (oracle_fast.c, the benchmark's CPU baseline) instead of the exact
    restatement; it agrees with it up to the order of the f32 sum.

    x: [M, K] float16/float32; scale: [N, K/G] float16/float32; zp: packed u4 bytes, u8 or
    float32 [N, K/G] (or one element with ``zp_scalar``); bias: [N].  Returns float32 [M, N]
    (or [M, len(n_index)]), not rounded to the output type.
    """
    x, x_type = _as_real(x, "x")
    x = x.reshape(-1, K)
    M = x.shape[0]
    w = np.ascontiguousarray(w, dtype=np.int8 if w_type == I8 else np.uint8)
    scale, scale_type = _as_real(scale, "scale")
    a = _FcArgs()
    a.M, a.N, a.K, a.group_size = M, N, K, group_size
    a.w_type, a.scale_type, a.x_type = w_type, scale_type, x_type
    a.zp_type, a.zp_scalar = zp_type, int(bool(zp_scalar))
    if zp_type != NONE:
        zp = np.ascontiguousarray(zp, dtype=np.float32 if zp_type == F32 else np.uint8)
    else:
        zp = None
    if bias is not None:
        bias, a.bias_type = _as_real(bias, "bias")
    else:
        a.bias_type = NONE
    a.acc_f64 = int(bool(acc_f64))
    a.w, a.scale, a.zp, a.bias, a.x = _ptr(w), _ptr(scale), _ptr(zp), _ptr(bias), _ptr(x)
    ncols = N
    idx = None
    if n_index is not None:
        idx = np.ascontiguousarray(n_index, dtype=np.int64)
        a.n_index, a.n_count = _ptr(idx), idx.size
        ncols = idx.size
    y = np.empty((M, ncols), dtype=np.float32)
    fn = lib().ovo_fc_blocked if blocked else lib().ovo_fc_reference
    rc = fn(ctypes.byref(a), _ptr(y))
    if rc != 0:
        raise ValueError(f"{'ovo_fc_blocked' if blocked else 'ovo_fc_reference'} rejected its arguments (code {rc})")
    return y


GLU_SWISH, GLU_GELU, GLU_GELU_TANH = 1, 2, 3


def glu(y, glu_type, gate_second=False) -> np.ndarray:
    """C oracle of the gated linear unit over the last axis of y [M, 2 L]: act(gate half) * up half, float32 [M, L]."""
    y = np.ascontiguousarray(y, dtype=np.float32)
    M, N = y.shape
    if N % 2:
        raise ValueError("the last axis must be even")
    out = np.empty((M, N // 2), dtype=np.float32)
    f = lib().ovo_glu
    f.restype = ctypes.c_int
    f.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p]
    if f(_ptr(y), M, N // 2, int(glu_type), int(bool(gate_second)), _ptr(out)) != 0:
        raise ValueError("ovo_glu rejected its arguments")
    return out


def moe_reference(x, routing, indices, gate_up, down, glu_type) -> np.ndarray:
    """Mixture-of-experts block with three projections per expert (ov::op::internal::MOE, GEMM3_SWIGLU), as the
    graph that MoE op fusion folds computes it (moe_op_fusion.cpp:55-105):

        y[m] = sum_j routing[m, j] * down_e(act(gate_e(x[m])) * up_e(x[m])),   e = indices[m, j]

    x float16 [M, H], routing [M, top_k], indices int [M, top_k].  gate_up[e] and down[e] are the keyword
    arguments of fc_reference for expert e's concatenated gate/up node ([2 I, H], gate rows first) and its down
    node ([H, I]).  Composed of fc_reference and glu; the activations between the two projections are rounded to
    float16 (they are a float16 tensor in the graph), the sum over a row's experts runs in float64.  float32 [M, H]."""
    x = np.ascontiguousarray(x, dtype=np.float16)
    routing = np.asarray(routing, dtype=np.float64)
    indices = np.asarray(indices)
    M, top_k = indices.shape
    H = down[0]["N"]
    y = np.zeros((M, H), np.float64)
    for e in range(len(gate_up)):
        for j in range(top_k):
            rows = np.nonzero(indices[:, j] == e)[0]
            if not rows.size:
                continue
            h = glu(fc_reference(x[rows], **gate_up[e]), glu_type).astype(np.float16)
            d = fc_reference(h, **down[e])
            y[rows] += routing[rows, j, None] * d.astype(np.float64)
    return y.astype(np.float32)


def grouped_matmul_reference(a, groups, offsets=None) -> np.ndarray:
    """GroupedMatMul over decompressed weights (ov::op::v17::GroupedMatMul; arithmetic of
    src/core/reference/include/openvino/reference/grouped_matmul.hpp:36-88 with B[g] = the decompressed weights of
    group g): groups[g] holds the keyword arguments of fc_reference for group g.

    offsets given (2-D x 3-D form, :61-88): a is [rows, K]; the output [rows, N] starts as zeros and group g fills
    rows [offsets[g-1], offsets[g]) -- offsets are cumulative row ends, a group may be empty, rows beyond the last
    offset stay zero.  offsets None (3-D x 3-D form, :36-58): a is [G, M, K], output [G, M, N].  float32."""
    a = np.asarray(a)
    N = groups[0]["N"]
    if offsets is None:
        return np.stack([fc_reference(a[g], **groups[g]) for g in range(len(groups))]).astype(np.float32)
    out = np.zeros((a.shape[0], N), np.float32)
    start = 0
    for g, end in enumerate(np.asarray(offsets).tolist()):
        if end > start:
            out[start:end] = fc_reference(a[start:end], **groups[g])
        start = end
    return out


def dynquant_rows(x):
    """C oracle: per-token symmetric int8 quantisation of x [M, K] float16 -> (q int8 [M, K], inv_scale float32 [M],
    qsum int32 [M])."""
    x = np.ascontiguousarray(x, dtype=np.float16)
    M, K = x.shape
    q, inv, qs = np.empty((M, K), np.int8), np.empty(M, np.float32), np.empty(M, np.int32)
    f = lib().ovo_dynquant_rows
    f.restype = ctypes.c_int
    f.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
    if f(_ptr(x), M, K, _ptr(q), _ptr(inv), _ptr(qs)) != 0:
        raise ValueError("ovo_dynquant_rows rejected its arguments")
    return q, inv, qs


def fc_dynquant_reference(x, w, w_type, scale, zp=None, bias=None, *, N, K) -> np.ndarray:
    """C oracle of the FullyConnected with per-token int8 activations: 8-bit weights [N, K], one float scale (and
    zero-point) per channel.  Returns float32 [M, N]."""
    if w_type not in (U8, I8):
        raise ValueError("8-bit weights only")
    q, inv, qs = dynquant_rows(np.asarray(x).reshape(-1, K))
    M = q.shape[0]
    w = np.ascontiguousarray(w).view(np.uint8).reshape(N, K)
    scale = np.ascontiguousarray(np.asarray(scale, dtype=np.float32).reshape(N))
    zp = None if zp is None else np.ascontiguousarray(np.asarray(zp, dtype=np.float32).reshape(N))
    bias = None if bias is None else np.ascontiguousarray(np.asarray(bias, dtype=np.float32).reshape(N))
    y = np.empty((M, N), np.float32)
    f = lib().ovo_fc_dynquant_reference
    f.restype = ctypes.c_int
    f.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64,
                  ctypes.c_void_p, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
    if f(_ptr(q), _ptr(inv), _ptr(qs), M, K, N, _ptr(w), int(w_type == I8), _ptr(scale), _ptr(zp), _ptr(bias), _ptr(y)) != 0:
        raise ValueError("ovo_fc_dynquant_reference rejected its arguments")
    return y


def dynquant_rows_asym(x):
    """C oracle: per-token asymmetric quantisation of x [M, K] float16 to unsigned bytes -> (q uint8 [M, K],
    inv_scale float32 [M], za int32 [M], qsum int32 [M])."""
    x = np.ascontiguousarray(x, dtype=np.float16)
    M, K = x.shape
    q, inv = np.empty((M, K), np.uint8), np.empty(M, np.float32)
    za, qs = np.empty(M, np.int32), np.empty(M, np.int32)
    f = lib().ovo_dynquant_rows_asym
    f.restype = ctypes.c_int
    f.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                  ctypes.c_void_p]
    if f(_ptr(x), M, K, _ptr(q), _ptr(inv), _ptr(za), _ptr(qs)) != 0:
        raise ValueError("ovo_dynquant_rows_asym rejected its arguments")
    return q, inv, za, qs


def fc_dynquant_asym_reference(x, w, w_type, scale, zp=None, bias=None, *, N, K) -> np.ndarray:
    """C oracle of the FullyConnected with per-token unsigned 8-bit activations and a zero-point per token: 8-bit
    weights [N, K], one float scale (and zero-point) per channel.  Returns float32 [M, N]."""
    if w_type not in (U8, I8):
        raise ValueError("8-bit weights only")
    q, inv, za, _ = dynquant_rows_asym(np.asarray(x).reshape(-1, K))
    M = q.shape[0]
    w = np.ascontiguousarray(w).view(np.uint8).reshape(N, K)
    scale = np.ascontiguousarray(np.asarray(scale, dtype=np.float32).reshape(N))
    zp = None if zp is None else np.ascontiguousarray(np.asarray(zp, dtype=np.float32).reshape(N))
    bias = None if bias is None else np.ascontiguousarray(np.asarray(bias, dtype=np.float32).reshape(N))
    y = np.empty((M, N), np.float32)
    f = lib().ovo_fc_dynquant_asym_reference
    f.restype = ctypes.c_int
    f.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64,
                  ctypes.c_void_p, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
    if f(_ptr(q), _ptr(inv), _ptr(za), M, K, N, _ptr(w), int(w_type == I8), _ptr(scale), _ptr(zp), _ptr(bias), _ptr(y)) != 0:
        raise ValueError("ovo_fc_dynquant_asym_reference rejected its arguments")
    return y


def dynquant_groups(x, G):
    """C oracle: symmetric int8 quantisation of x [M, K] float16 in groups of G inputs -> (q int8 [M, K],
    inv_scale float32 [M, K / G], qsum int32 [M, K / G])."""
    x = np.ascontiguousarray(x, dtype=np.float16)
    M, K = x.shape
    q, inv, qs = np.empty((M, K), np.int8), np.empty((M, K // G), np.float32), np.empty((M, K // G), np.int32)
    f = lib().ovo_dynquant_groups
    f.restype = ctypes.c_int
    f.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p,
                  ctypes.c_void_p]
    if f(_ptr(x), M, K, G, _ptr(q), _ptr(inv), _ptr(qs)) != 0:
        raise ValueError("ovo_dynquant_groups rejected its arguments")
    return q, inv, qs


def _codes(packed, type_, n):
    """One code per byte (two's complement for the signed types) from n packed 4- or 8-bit elements."""
    if type_ == U4:
        return unpack_u4(packed, n)
    if type_ == I4:
        return unpack_i4(packed, n).view(np.uint8)
    return np.ascontiguousarray(packed).view(np.uint8).ravel()[:n].copy()


def fc_dynquant_grouped_reference(x, w, w_type, scale, zp=None, zp_type=NONE, bias=None, *, N, K, group_size,
                                  act_group, zp_scalar=False) -> np.ndarray:
    """C oracle of the FullyConnected with int8 activations quantised in groups of act_group inputs (K: per token)
    over 4- or 8-bit weights with scales / zero-points per group of group_size inputs.  w, zp packed as for
    fc_reference.  Returns float32 [M, N]."""
    q, inv, _ = dynquant_groups(np.asarray(x).reshape(-1, K), act_group)
    M = q.shape[0]
    ng = K // group_size
    codes = _codes(w, w_type, N * K)
    scale = np.ascontiguousarray(np.asarray(scale, dtype=np.float32).reshape(N, ng))
    if zp is None or zp_type == NONE:
        zpf = None
    else:
        z = _codes(zp, zp_type, 1 if zp_scalar else N * ng).astype(np.float32)
        zpf = np.ascontiguousarray(np.broadcast_to(z, (N, ng)) if zp_scalar else z.reshape(N, ng), dtype=np.float32)
    bias = None if bias is None else np.ascontiguousarray(np.asarray(bias, dtype=np.float32).reshape(N))
    y = np.empty((M, N), np.float32)
    f = lib().ovo_fc_dynquant_grouped_reference
    f.restype = ctypes.c_int
    f.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64,
                  ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                  ctypes.c_void_p]
    signed = w_type in (I4, I8)
    if f(_ptr(q), _ptr(inv), M, K, act_group, N, _ptr(codes), int(signed), group_size, _ptr(scale), _ptr(zpf),
         _ptr(bias), _ptr(y)) != 0:
        raise ValueError("ovo_fc_dynquant_grouped_reference rejected its arguments")
    return y


# ---- independent numpy restatement (bit operations and float64 matmul) ----

def np_unpack_nibbles(packed: np.ndarray, n: int, signed: bool) -> np.ndarray:
    packed = np.asarray(packed, dtype=np.uint8).ravel()
    both = np.stack([packed & 0x0F, packed >> 4], axis=1).ravel()[:n].astype(np.int16)
    if signed:
        both = np.where(both >= 8, both - 16, both)
    return both


def np_dequantise(w, w_type, scale, zp=None, zp_type=NONE, *, N, K, group_size,
                  zp_scalar=False) -> np.ndarray:
    """Dequantised weights as float64 [N, K]: (q - zp) * s evaluated in float32 like the oracle."""
    ng = K // group_size
    if w_type in (U4, I4):
        q = np_unpack_nibbles(w, N * K, w_type == I4).reshape(N, K)
    else:
        q = np.asarray(w, dtype=np.int8 if w_type == I8 else np.uint8).reshape(N, K).astype(np.int16)
    s = np.asarray(scale).astype(np.float32).reshape(N, ng)
    if zp_type == NONE:
        z = np.zeros((N, ng), dtype=np.float32)
    else:
        if zp_type == U4:
            cnt = 1 if zp_scalar else N * ng
            zz = np_unpack_nibbles(zp, cnt, False).astype(np.float32)
        else:
            zz = np.asarray(zp).astype(np.float32).ravel()
        z = np.full((N, ng), zz[0], dtype=np.float32) if zp_scalar else zz.reshape(N, ng)
    qf = q.astype(np.float32).reshape(N, ng, group_size)
    deq = (qf - z[:, :, None]) * s[:, :, None]          # float32, as the reference kernel does
    return deq.reshape(N, K).astype(np.float64)


def fc_reference_numpy(x, w, w_type, scale, zp=None, zp_type=NONE, bias=None, *, N, K, group_size,
                       zp_scalar=False) -> np.ndarray:
    """float64 result [M, N] of the same formula, written with numpy only."""
    deq = np_dequantise(w, w_type, scale, zp, zp_type, N=N, K=K, group_size=group_size,
                        zp_scalar=zp_scalar)
    y = np.asarray(x).astype(np.float64).reshape(-1, K) @ deq.T
    if bias is not None:
        y = y + np.asarray(bias).astype(np.float64).reshape(1, N)
    return y


# ---- error measures used by every parity test ----

def rel_l2(y, y_ref) -> float:
    y = np.asarray(y, dtype=np.float64)
    y_ref = np.asarray(y_ref, dtype=np.float64)
    den = np.linalg.norm(y_ref.ravel())
    return float(np.linalg.norm((y - y_ref).ravel()) / (den if den > 0 else 1.0))


def max_abs(y, y_ref) -> float:
    return float(np.max(np.abs(np.asarray(y, dtype=np.float64) - np.asarray(y_ref, dtype=np.float64)))) \
        if np.size(y) else 0.0
