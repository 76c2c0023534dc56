"""Host-side mirror of the FullyConnectedCompressed node over the C ABI.

Argument names and meaning follow ov::op::internal::FullyConnectedCompressed
(src/common/transformations/include/ov_ops/fully_connected_compressed.hpp:15-37): inputs X, W,
bias, weight_scales, weight_zero_points; W is [N, K]; an absent input is ``None``.  Everything
executes in libovfcc.so on the GPU; there is no CPU path here.
"""
from __future__ import annotations

import ctypes
from typing import Optional, Sequence

import numpy as np

from . import _lib
from ._lib import FcDesc, KernelInfo, OvfccError, check


def _vp(a: Optional[np.ndarray]):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def make_desc(N: int, K: int, group_size: int, w_type: str, zp_type: str = "none", zp_scalar: bool = False,
              has_bias: bool = False, out_type: str = "f16", glu: Optional[str] = None,
              glu_gate_second: bool = False, dynamic_quantization: bool = False,
              input_major: bool = False) -> FcDesc:
    d = FcDesc()
    d.N, d.K, d.group_size = N, K, group_size
    d.w_type = _lib.TYPE[w_type]
    d.scale_type = _lib.F16
    d.zp_type = _lib.TYPE[zp_type]
    d.zp_scalar = int(zp_scalar)
    d.bias_type = _lib.F16 if has_bias else _lib.NONE
    d.act_type = _lib.F16
    d.out_type = _lib.TYPE[out_type]
    d.flags = (_lib.GLU[glu] | (_lib.GLU_GATE_SECOND if glu_gate_second else 0) |
               (_lib.DYNQUANT_I8 if dynamic_quantization else 0) |
               (_lib.DYNQUANT_PER_GROUP if dynamic_quantization == "per_group" else 0) |
               (_lib.DYNQUANT_ASYM if dynamic_quantization == "asymmetric" else 0) |
               (_lib.W_INPUT_MAJOR if input_major else 0))
    return d


class Device:
    """One MI355X and its library context (the plugin object's device half)."""

    def __init__(self, index: int = 0):
        self._lib = _lib.load()
        h = ctypes.c_void_p()
        check(self.lib.ovfcc_init(index, ctypes.byref(h)))
        self.handle = h

    @property
    def lib(self):
        """The loaded library, with environment overrides changed since the last call taken over first."""
        _lib.sync_env()
        return self._lib

    def close(self):
        if self.handle:
            self.lib.ovfcc_destroy(self.handle)
            self.handle = None

    def mem_info(self):
        """(free, total) bytes of device memory"""
        free, total = ctypes.c_size_t(), ctypes.c_size_t()
        check(self.lib.ovfcc_device_mem_info(self.handle, ctypes.byref(free), ctypes.byref(total)))
        return free.value, total.value

    # raw device buffers
    def malloc(self, nbytes: int) -> int:
        p = ctypes.c_void_p()
        check(self.lib.ovfcc_device_malloc(self.handle, nbytes, ctypes.byref(p)))
        return p.value

    def free(self, ptr: int) -> None:
        check(self.lib.ovfcc_device_free(self.handle, ctypes.c_void_p(ptr)))

    def upload(self, ptr: int, a: np.ndarray) -> None:
        a = np.ascontiguousarray(a)
        check(self.lib.ovfcc_memcpy_h2d(self.handle, ctypes.c_void_p(ptr), _vp(a), a.nbytes))

    def download(self, ptr: int, shape, dtype) -> np.ndarray:
        out = np.empty(shape, dtype=dtype)
        check(self.lib.ovfcc_memcpy_d2h(self.handle, _vp(out), ctypes.c_void_p(ptr), out.nbytes))
        return out

    def copy(self, dst_ptr: int, src_ptr: int, nbytes: int) -> None:
        """Device-to-device copy (blocking)."""
        check(self.lib.ovfcc_memcpy_d2d(self.handle, ctypes.c_void_p(dst_ptr), ctypes.c_void_p(src_ptr), nbytes))

    def floor_us(self, arena_ptr: int, arena_bytes: int, node_bytes: int, n_nodes: int = 96, waves: int = 8,
                 kib_per_wave: int = 8, iters: int = 20) -> float:
        """Microseconds per node of a replayed graph of probe launches: empty kernels (node_bytes = 0) or loads-only
        streaming kernels over node_bytes each (ovfcc_bench_floor)."""
        ms = ctypes.c_float()
        check(self.lib.ovfcc_bench_floor(self.handle, ctypes.c_void_p(arena_ptr), arena_bytes, node_bytes, n_nodes, waves,
                                         kib_per_wave, iters, ctypes.byref(ms)))
        return ms.value * 1e3 / iters / n_nodes

    def mfma_ceiling(self, waves: int = 8, valu: int = 0, rounds: int = 20000, shape: int = 0) -> float:
        """TFLOP/s of a loop of nothing but v_mfma_f32_16x16x32_f16 (shape 0) or v_mfma_f32_32x32x16_f16 (shape 1) on
        every compute unit, `waves` waves each (4 or 8), with `valu` packed-f16 vector multiplications after every
        16 x 16 x 32 MFMA's worth of work (ovfcc_bench_mfma)."""
        ms, flops = ctypes.c_float(), ctypes.c_double()
        check(self.lib.ovfcc_bench_mfma(self.handle, waves, valu, shape, rounds, ctypes.byref(ms), ctypes.byref(flops)))
        return flops.value / (ms.value * 1e-3) / 1e12

    def issue_probe(self, workgroups: int, waves: int, mode: int, valu: int, rounds: int = 20000):
        """(shader cycles, ns) per MFMA and SIMD of the matrix-core loop with `valu` vector instructions after every
        MFMA arranged by `mode` (ovfcc_bench_issue)."""
        cyc, ns = ctypes.c_double(), ctypes.c_double()
        check(self.lib.ovfcc_bench_issue(self.handle, workgroups, waves, mode, valu, rounds, ctypes.byref(cyc), ctypes.byref(ns)))
        return cyc.value, ns.value

    def copy_bandwidth(self, nbytes: int = 1 << 30, iters: int = 10) -> float:
        """GB/s (read + write) of the plain copy kernel."""
        src, dst = self.malloc(nbytes), self.malloc(nbytes)
        ms = ctypes.c_float()
        try:
            check(self.lib.ovfcc_bench_copy(self.handle, ctypes.c_void_p(dst), ctypes.c_void_p(src), nbytes, iters,
                                            ctypes.byref(ms)))
        finally:
            self.free(src)
            self.free(dst)
        return 2.0 * nbytes * iters / (ms.value * 1e-3) / 1e9


class _BlobHeader(ctypes.Structure):
    """Head of an exported node (ovfcc_weights_export): the device arrays follow, each padded to 16 bytes."""
    _fields_ = [("magic", ctypes.c_char * 8), ("version", ctypes.c_uint32), ("header_bytes", ctypes.c_uint32),
                ("desc", FcDesc), ("zp_const", ctypes.c_int32), ("tiled", ctypes.c_int32), ("sizes", ctypes.c_uint64 * 4)]


class CompressedWeights:
    """Repacked, device-resident constants of one FullyConnectedCompressed node."""

    def __init__(self, device: Device, W: np.ndarray, weight_scales: np.ndarray, weight_zero_points=None, bias=None, *,
                 N: int, K: int, group_size: int, w_type: str, zp_type: str = "none", zp_scalar: bool = False,
                 output_type: str = "f16", glu: Optional[str] = None, glu_gate_second: bool = False,
                 dynamic_quantization: bool = False, input_major: bool = False):
        """glu = "swish" | "gelu" | "gelu_tanh": W holds gate and up projection ([N, K], first and second half of
        the rows, or the other way round with glu_gate_second) and the node computes act(gate) * up, [M, N / 2].
        input_major: W is [K, N] and scales / zero-points [K / G, N] (a MatMul with transpose_b = false)."""
        self.device = device
        self.N, self.K, self.group_size = N, K, group_size
        self.desc = make_desc(N, K, group_size, w_type, zp_type if weight_zero_points is not None else "none",
                              zp_scalar, bias is not None, output_type, glu, glu_gate_second, dynamic_quantization,
                              input_major)
        W = np.ascontiguousarray(W).view(np.uint8)
        s = np.ascontiguousarray(weight_scales, dtype=np.float16)
        z = None if weight_zero_points is None else np.ascontiguousarray(weight_zero_points, dtype=np.uint8)
        b = None if bias is None else np.ascontiguousarray(bias, dtype=np.float16)
        h = ctypes.c_void_p()
        check(device.lib.ovfcc_weights_create(device.handle, ctypes.byref(self.desc), _vp(W), _vp(s), _vp(z), _vp(b),
                                              ctypes.byref(h)))
        self.handle = h

    @classmethod
    def from_case(cls, device: Device, c, output_type: str = "f16", glu: Optional[str] = None,
                  glu_gate_second: bool = False, dynamic_quantization: bool = False) -> "CompressedWeights":
        return cls(device, c.w, c.scale, c.zp, c.bias, N=c.N, K=c.K, group_size=c.group_size, w_type=c.w_type,
                   zp_type=c.zp_type, zp_scalar=c.zp_scalar, output_type=output_type, glu=glu,
                   glu_gate_second=glu_gate_second, dynamic_quantization=dynamic_quantization)

    @classmethod
    def adopt(cls, device: Device, handle, desc, extra_flags: int = 0) -> "CompressedWeights":
        """Wraps a node the library created by another route (graph.Graph.create_weights)."""
        other = object.__new__(CompressedWeights)
        other.device = device
        other.desc = FcDesc.from_buffer_copy(desc)
        other.desc.flags |= extra_flags
        other.N, other.K, other.group_size = other.desc.N, other.desc.K, other.desc.group_size
        other.handle = handle
        return other

    @property
    def N_out(self) -> int:
        """Row length of the node's output: N, or N / 2 with a gated-linear-unit epilogue; an MLP node's is its down
        projection's."""
        down = getattr(self, "down", None)
        if down is not None:
            return down.N_out
        return self.N // 2 if self.desc.flags & 3 else self.N

    @property
    def out_f32(self) -> bool:
        down = getattr(self, "down", None)
        return (down.desc if down is not None else self.desc).out_type == _lib.F32

    @classmethod
    def mlp(cls, gate_up: "CompressedWeights", down: "CompressedWeights") -> "CompressedWeights":
        """Gate / up node (with its gated linear unit) and down projection as one node: X [M, K] -> Y [M, N of down]
        (the CPU plugin's LLMMLP node).  The new node owns device copies of both."""
        h = ctypes.c_void_p()
        check(gate_up.device.lib.ovfcc_weights_mlp(gate_up.handle, down.handle, ctypes.byref(h)))
        other = object.__new__(CompressedWeights)
        other.device, other.N, other.K, other.group_size = gate_up.device, gate_up.N, gate_up.K, gate_up.group_size
        other.desc = FcDesc.from_buffer_copy(gate_up.desc)
        other.down = down          # shapes and types of the output side (the handle inside the node is its own copy)
        other.handle = h
        return other

    @classmethod
    def glu(cls, gate: "CompressedWeights", up: "CompressedWeights", kind: str = "swish") -> "CompressedWeights":
        """Gate and up projection fused into one node that computes act(gate(x)) * up(x)."""
        h = ctypes.c_void_p()
        check(gate.device.lib.ovfcc_weights_glu(gate.handle, up.handle, _lib.GLU[kind], ctypes.byref(h)))
        other = object.__new__(CompressedWeights)
        other.device, other.K, other.group_size = gate.device, gate.K, gate.group_size
        other.N = 2 * gate.N
        other.desc = FcDesc.from_buffer_copy(gate.desc)
        other.desc.N = other.N
        other.desc.flags = _lib.GLU[kind]
        other.handle = h
        return other

    def clone(self) -> "CompressedWeights":
        """Second device copy at distinct addresses (no host work)."""
        other = object.__new__(CompressedWeights)
        other.device, other.N, other.K, other.group_size, other.desc = (self.device, self.N, self.K,
                                                                        self.group_size, self.desc)
        if getattr(self, "down", None) is not None:
            other.down = self.down
        h = ctypes.c_void_p()
        check(self.device.lib.ovfcc_weights_clone(self.handle, ctypes.byref(h)))
        other.handle = h
        return other

    @classmethod
    def concat(cls, parts: Sequence["CompressedWeights"]) -> "CompressedWeights":
        """Horizontal fusion: one node whose output channels are the parts' channels in order."""
        first = parts[0]
        arr = (ctypes.c_void_p * len(parts))(*[p.handle for p in parts])
        h = ctypes.c_void_p()
        check(first.device.lib.ovfcc_weights_concat(arr, len(parts), ctypes.byref(h)))
        other = object.__new__(CompressedWeights)
        other.device, other.K, other.group_size = first.device, first.K, first.group_size
        other.N = sum(p.N for p in parts)
        other.desc = FcDesc.from_buffer_copy(first.desc)
        other.desc.N = other.N
        other.handle = h
        return other

    def export_blob(self) -> np.ndarray:
        """The node in its device form as one host blob (what a model cache stores instead of repacking again)."""
        n = ctypes.c_size_t()
        check(self.device.lib.ovfcc_weights_export_size(self.handle, ctypes.byref(n)))
        blob = np.empty(n.value, np.uint8)
        check(self.device.lib.ovfcc_weights_export(self.handle, _vp(blob), blob.nbytes))
        return blob

    @classmethod
    def import_blob(cls, device: Device, blob: np.ndarray) -> "CompressedWeights":
        blob = np.ascontiguousarray(blob, dtype=np.uint8)
        h = ctypes.c_void_p()
        check(device.lib.ovfcc_weights_import(device.handle, _vp(blob), blob.nbytes, ctypes.byref(h)))
        def described(at):
            """(stand-in carrying the descriptor of the node whose blob starts at byte `at`, where that blob ends,
            whether another node's blob follows)"""
            head = _BlobHeader.from_buffer_copy(blob[at:at + ctypes.sizeof(_BlobHeader)].tobytes())
            node = object.__new__(CompressedWeights)
            node.device, node.handle = device, None
            node.desc = FcDesc.from_buffer_copy(head.desc)
            node.N, node.K, node.group_size = node.desc.N, node.desc.K, node.desc.group_size
            pad = lambda n: (n + 15) & ~15
            end = at + pad(ctypes.sizeof(_BlobHeader)) + sum(pad(int(n)) for n in head.sizes)
            return node, end, bool(head.tiled & 2)

        other, end, has_down = described(0)
        if has_down:     # an MLP node: shapes and types of the output side come from the second blob
            other.down = described(end)[0]
        other.handle = h
        return other

    @property
    def tiled(self) -> bool:
        return bool(self.device.lib.ovfcc_weights_is_tiled(self.handle))

    @property
    def device_bytes(self) -> int:
        return int(self.device.lib.ovfcc_weights_device_bytes(self.handle))

    def close(self):
        if self.handle:
            self.device.lib.ovfcc_weights_destroy(self.handle)
            self.handle = None


class InferRequest:
    """One stream of execution (ov::ISyncInferRequest for this node)."""

    def __init__(self, device: Device):
        self.device = device
        h = ctypes.c_void_p()
        check(device.lib.ovfcc_request_create(device.handle, ctypes.byref(h)))
        self.handle = h

    def close(self):
        if self.handle:
            self.device.lib.ovfcc_request_destroy(self.handle)
            self.handle = None

    def force_kernel(self, kernel: int = _lib.KERNEL_AUTO, split_k: int = 0) -> None:
        check(self.device.lib.ovfcc_request_force_kernel(self.handle, kernel, split_k))

    def infer(self, weights: CompressedWeights, X: np.ndarray) -> np.ndarray:
        """X float16 [..., K] on the host -> Y [..., N] in the node's output_type (MatMul shape rules, transpose_b = true)."""
        X = np.ascontiguousarray(X, dtype=np.float16)
        if X.shape[-1] != weights.K:
            raise OvfccError(_lib.EINVAL, f"last dimension of X is {X.shape[-1]}, expected K = {weights.K}")
        M = int(np.prod(X.shape[:-1], dtype=np.int64))
        Y = np.empty(X.shape[:-1] + (weights.N_out,), dtype=np.float32 if weights.out_f32 else np.float16)
        check(self.device.lib.ovfcc_fc_run(self.handle, weights.handle, _vp(X), _vp(Y), M))
        return Y

    def infer_device(self, weights: CompressedWeights, x_ptr: int, y_ptr: int, M: int) -> None:
        check(self.device.lib.ovfcc_fc_run_device(self.handle, weights.handle, ctypes.c_void_p(x_ptr),
                                                  ctypes.c_void_p(y_ptr), M))

    def infer_device_static(self, weights: CompressedWeights, x_ptr: int, y_ptr: int, M: int) -> None:
        """infer_device through the entry point that allocates nothing (fixed scratch array instead of buffers of
        the request); calls that overlap on one GPU race."""
        check(self.device.lib.ovfcc_fc_run_device_static(self.handle, weights.handle, ctypes.c_void_p(x_ptr),
                                                         ctypes.c_void_p(y_ptr), M))

    def _group_items(self, items):
        arr = (_lib.GroupItem * len(items))()
        for a, (w, x_ptr, y_ptr, M) in zip(arr, items):
            a.weights, a.x_dev, a.y_dev, a.M = w.handle, x_ptr, y_ptr, M
        return arr

    def infer_grouped_device(self, items: Sequence[tuple]) -> None:
        """items: (weights, x_ptr, y_ptr, M) per independent node of one shape and format (e.g. the experts of a
        mixture-of-experts layer with their gathered rows); one launch where possible."""
        arr = self._group_items(items)
        check(self.device.lib.ovfcc_fc_run_grouped_device(self.handle, arr, len(items)))

    def infer_grouped(self, items: Sequence[tuple]) -> list:
        """items: (weights, X float16 [M_i, K] on the host) per node; returns the list of Y [M_i, N].  Stages the
        operands in device memory, runs infer_grouped_device, copies back."""
        dev, xs, ptrs = self.device, [], []
        try:
            for w, X in items:
                X = np.ascontiguousarray(X, dtype=np.float16)
                if X.ndim != 2 or X.shape[1] != w.K:
                    raise OvfccError(_lib.EINVAL, f"X has shape {X.shape}, expected [M, {w.K}]")
                xs.append(X)
                itemsize = 4 if w.desc.out_type == _lib.F32 else 2
                x_ptr, y_ptr = dev.malloc(max(X.nbytes, 16)), dev.malloc(max(X.shape[0] * w.N_out * itemsize, 16))
                ptrs.append((x_ptr, y_ptr))
                if X.size:
                    dev.upload(x_ptr, X)
            self.infer_grouped_device([(w, xp, yp, X.shape[0]) for (w, _), X, (xp, yp) in zip(items, xs, ptrs)])
            self.sync()
            return [dev.download(yp, (X.shape[0], w.N_out), np.float32 if w.desc.out_type == _lib.F32 else np.float16)
                    if X.shape[0] else np.empty((0, w.N_out), np.float32 if w.desc.out_type == _lib.F32 else np.float16)
                    for (w, _), X, (_, yp) in zip(items, xs, ptrs)]
        finally:
            for xp, yp in ptrs:
                dev.free(xp)
                dev.free(yp)

    def grouped_matmul_device(self, groups: Sequence[CompressedWeights], a_ptr: int, offsets: Optional[np.ndarray],
                              rows: int, y_ptr: int) -> None:
        """GroupedMatMulCompressed on device buffers.  offsets int32 [G] on the host (cumulative row ends): A
        [rows, K] at a_ptr, Y [rows, N_out] at y_ptr; offsets None: A [G, rows, K], Y [G, rows, N_out]."""
        arr = (ctypes.c_void_p * len(groups))(*[w.handle for w in groups])
        off = None
        if offsets is not None:
            off_arr = np.ascontiguousarray(offsets, dtype=np.int32)
            if off_arr.shape != (len(groups),):
                raise OvfccError(_lib.EINVAL, f"offsets have shape {off_arr.shape}, expected ({len(groups)},)")
            off = off_arr.ctypes.data_as(ctypes.POINTER(ctypes.c_int32))
        check(self.device.lib.ovfcc_grouped_matmul_device(self.handle, arr, len(groups), ctypes.c_void_p(a_ptr), off,
                                                          rows, ctypes.c_void_p(y_ptr)))

    def grouped_matmul_offsets_device(self, groups: Sequence[CompressedWeights], a_ptr: int, offsets_ptr: int,
                                      rows: int, y_ptr: int) -> None:
        """The 2-D x 3-D form with the offsets int32 [G] in device memory at offsets_ptr."""
        arr = (ctypes.c_void_p * len(groups))(*[w.handle for w in groups])
        check(self.device.lib.ovfcc_grouped_matmul_offsets_device(self.handle, arr, len(groups), ctypes.c_void_p(a_ptr),
                                                                  ctypes.c_void_p(offsets_ptr), rows, ctypes.c_void_p(y_ptr)))

    def grouped_matmul(self, groups: Sequence[CompressedWeights], A: np.ndarray,
                       offsets: Optional[np.ndarray] = None, y_fill: Optional[float] = None,
                       device_offsets: bool = False) -> np.ndarray:
        """Host convenience: with offsets A float16 [rows, K] -> Y [rows, N_out]; without, A [G, M, K] -> Y [G, M, N_out].
        y_fill: Y is preset to this value (the call must overwrite all of it); device_offsets: the offsets are uploaded
        and the entry point that reads them on the device is called."""
        A = np.ascontiguousarray(A, dtype=np.float16)
        w = groups[0]
        want = 2 if offsets is not None else 3
        if A.ndim != want or A.shape[-1] != w.K or (offsets is None and A.shape[0] != len(groups)):
            raise OvfccError(_lib.EINVAL, f"A has shape {A.shape}")
        rows = A.shape[0] if offsets is not None else A.shape[1]
        out_shape = (rows, w.N_out) if offsets is not None else (len(groups), rows, w.N_out)
        dt = np.float32 if w.desc.out_type == _lib.F32 else np.float16
        if rows == 0:
            self.grouped_matmul_device(groups, 0, offsets, 0, 0)
            return np.empty(out_shape, dt)
        dev = self.device
        a_ptr, y_ptr = dev.malloc(A.nbytes), dev.malloc(int(np.prod(out_shape)) * np.dtype(dt).itemsize)
        try:
            dev.upload(a_ptr, A)
            if y_fill is not None:
                dev.upload(y_ptr, np.full(out_shape, y_fill, dt))
            if device_offsets:
                off = np.ascontiguousarray(offsets, dtype=np.int32)
                o_ptr = dev.malloc(max(off.nbytes, 16))
                try:
                    dev.upload(o_ptr, off)
                    self.grouped_matmul_offsets_device(groups, a_ptr, o_ptr, rows, y_ptr)
                    self.sync()
                finally:
                    dev.free(o_ptr)
            else:
                self.grouped_matmul_device(groups, a_ptr, offsets, rows, y_ptr)
                self.sync()
            return dev.download(y_ptr, out_shape, dt)
        finally:
            dev.free(a_ptr)
            dev.free(y_ptr)

    def gather_matmul_device(self, experts: Sequence[CompressedWeights], a_ptr: int, a_batches: int,
                             indices: np.ndarray, y_ptr: int) -> None:
        """GatherMatmulCompressed on device buffers: A [a_batches, M, K] at a_ptr, indices int32 [M, top_k] on the
        host, Y [top_k, M, N_out] at y_ptr."""
        idx = np.ascontiguousarray(indices, dtype=np.int32)
        M, top_k = idx.shape
        arr = (ctypes.c_void_p * len(experts))(*[w.handle for w in experts])
        check(self.device.lib.ovfcc_gather_matmul_device(self.handle, arr, len(experts), ctypes.c_void_p(a_ptr), a_batches,
                                                         idx.ctypes.data_as(ctypes.POINTER(ctypes.c_int32)), M, top_k,
                                                         ctypes.c_void_p(y_ptr)))

    def gather_matmul_routed_device(self, experts: Sequence[CompressedWeights], a_ptr: int, a_batches: int,
                                    indices_ptr: int, M: int, top_k: int, y_ptr: int) -> None:
        """The same with the indices int32 [M, top_k] in device memory at indices_ptr: bucketed on the device."""
        arr = (ctypes.c_void_p * len(experts))(*[w.handle for w in experts])
        check(self.device.lib.ovfcc_gather_matmul_routed_device(self.handle, arr, len(experts), ctypes.c_void_p(a_ptr),
                                                                a_batches, ctypes.c_void_p(indices_ptr), M, top_k,
                                                                ctypes.c_void_p(y_ptr)))

    def gather_matmul(self, experts: Sequence[CompressedWeights], A: np.ndarray, indices: np.ndarray,
                      device_indices: bool = False, y_fill: Optional[float] = None) -> np.ndarray:
        """Host convenience: A float16 [a_batches, M, K] (a_batches 1 or top_k), indices [M, top_k] -> Y [top_k, M, N_out].
        device_indices: the indices are uploaded and the device-routed entry point is called; y_fill: Y is
        preset to this value (rows that no expert writes keep it)."""
        A = np.ascontiguousarray(A, dtype=np.float16)
        idx = np.ascontiguousarray(indices, dtype=np.int32)
        M, top_k = idx.shape
        w = experts[0]
        if A.ndim != 3 or A.shape[1] != M or A.shape[2] != w.K:
            raise OvfccError(_lib.EINVAL, f"A has shape {A.shape}, expected [1 or {top_k}, {M}, {w.K}]")
        dt = np.float32 if w.desc.out_type == _lib.F32 else np.float16
        if M == 0:
            return np.empty((top_k, 0, w.N_out), dt)
        dev = self.device
        a_ptr, y_ptr = dev.malloc(A.nbytes), dev.malloc(top_k * M * w.N_out * np.dtype(dt).itemsize)
        i_ptr = dev.malloc(max(idx.nbytes, 16)) if device_indices else None
        try:
            dev.upload(a_ptr, A)
            if y_fill is not None:
                dev.upload(y_ptr, np.full((top_k, M, w.N_out), y_fill, dt))
            if device_indices:
                dev.upload(i_ptr, idx)
                self.gather_matmul_routed_device(experts, a_ptr, A.shape[0], i_ptr, M, top_k, y_ptr)
            else:
                self.gather_matmul_device(experts, a_ptr, A.shape[0], idx, y_ptr)
            self.sync()
            return dev.download(y_ptr, (top_k, M, w.N_out), dt)
        finally:
            dev.free(a_ptr)
            dev.free(y_ptr)
            if i_ptr:
                dev.free(i_ptr)

    def moe_device(self, gate_up: Sequence[CompressedWeights], down: Sequence[CompressedWeights], x_ptr: int,
                   routing_ptr: int, indices: np.ndarray, y_ptr: int) -> None:
        """MOECompressed (three projections per expert, gated linear unit) on device buffers: hidden states
        [M, H] f16 at x_ptr, routing weights [M, top_k] f16 at routing_ptr, indices int32 [M, top_k] on the host,
        Y [M, H] at y_ptr."""
        idx = np.ascontiguousarray(indices, dtype=np.int32)
        M, top_k = idx.shape
        g = (ctypes.c_void_p * len(gate_up))(*[w.handle for w in gate_up])
        d = (ctypes.c_void_p * len(down))(*[w.handle for w in down])
        check(self.device.lib.ovfcc_moe_device(self.handle, g, d, len(gate_up), ctypes.c_void_p(x_ptr),
                                               ctypes.c_void_p(routing_ptr),
                                               idx.ctypes.data_as(ctypes.POINTER(ctypes.c_int32)), M, top_k,
                                               ctypes.c_void_p(y_ptr)))

    def moe_routed_device(self, gate_up: Sequence[CompressedWeights], down: Sequence[CompressedWeights], x_ptr: int,
                          routing_ptr: int, indices_ptr: int, M: int, top_k: int, y_ptr: int) -> None:
        """The same with the indices int32 [M, top_k] in device memory at indices_ptr: bucketed on the device."""
        g = (ctypes.c_void_p * len(gate_up))(*[w.handle for w in gate_up])
        d = (ctypes.c_void_p * len(down))(*[w.handle for w in down])
        check(self.device.lib.ovfcc_moe_routed_device(self.handle, g, d, len(gate_up), ctypes.c_void_p(x_ptr),
                                                      ctypes.c_void_p(routing_ptr), ctypes.c_void_p(indices_ptr), M,
                                                      top_k, ctypes.c_void_p(y_ptr)))

    def moe(self, gate_up: Sequence[CompressedWeights], down: Sequence[CompressedWeights], x: np.ndarray,
            routing: np.ndarray, indices: np.ndarray, device_indices: bool = False) -> np.ndarray:
        """Host convenience: x float16 [M, H], routing float16 [M, top_k], indices [M, top_k] -> Y [M, H].
        device_indices: the indices are uploaded and the device-routed entry point is called."""
        x = np.ascontiguousarray(x, dtype=np.float16)
        routing = np.ascontiguousarray(routing, dtype=np.float16)
        idx = np.ascontiguousarray(indices, dtype=np.int32)
        M, top_k = idx.shape
        H = down[0].N
        if x.shape != (M, gate_up[0].K) or routing.shape != (M, top_k) or len(gate_up) != len(down):
            raise OvfccError(_lib.EINVAL, f"x {x.shape}, routing {routing.shape}, indices {idx.shape} do not fit")
        dt = np.float32 if down[0].desc.out_type == _lib.F32 else np.float16
        if M == 0:
            return np.empty((0, H), dt)
        dev = self.device
        x_ptr, r_ptr, y_ptr = dev.malloc(x.nbytes), dev.malloc(max(routing.nbytes, 16)), dev.malloc(M * H * np.dtype(dt).itemsize)
        i_ptr = dev.malloc(max(idx.nbytes, 16)) if device_indices else None
        try:
            dev.upload(x_ptr, x)
            dev.upload(r_ptr, routing)
            if device_indices:
                dev.upload(i_ptr, idx)
                self.moe_routed_device(gate_up, down, x_ptr, r_ptr, i_ptr, M, top_k, y_ptr)
            else:
                self.moe_device(gate_up, down, x_ptr, r_ptr, idx, y_ptr)
            self.sync()
            return dev.download(y_ptr, (M, H), dt)
        finally:
            dev.free(x_ptr)
            dev.free(r_ptr)
            dev.free(y_ptr)
            if i_ptr:
                dev.free(i_ptr)

    def bench_grouped(self, items: Sequence[tuple], warmup: int, iters: int) -> float:
        """Milliseconds for `iters` grouped runs, HIP events on the launching stream."""
        arr = self._group_items(items)
        ms = ctypes.c_float()
        check(self.device.lib.ovfcc_bench_grouped(self.handle, arr, len(items), warmup, iters, ctypes.byref(ms)))
        return ms.value

    def sync(self) -> None:
        check(self.device.lib.ovfcc_request_sync(self.handle))

    def last_kernel(self) -> dict:
        info = KernelInfo()
        check(self.device.lib.ovfcc_last_kernel_info(self.handle, ctypes.byref(info)))
        return dict(kernel=info.kernel, name=info.name.decode(), grid=tuple(info.grid), block=info.block,
                    split_k=info.split_k, tile_m=info.tile_m, tile_n=info.tile_n)

    def bench_layers(self, layers: Sequence[CompressedWeights], x_ptr: int, y_ptr: int, M: int, warmup: int,
                     iters: int, use_graph: bool = True) -> float:
        """Milliseconds for `iters` passes over `layers`, HIP events on the launching stream."""
        arr = (ctypes.c_void_p * len(layers))(*[w.handle for w in layers])
        ms = ctypes.c_float()
        check(self.device.lib.ovfcc_bench_layers(self.handle, arr, len(layers), ctypes.c_void_p(x_ptr),
                                                 ctypes.c_void_p(y_ptr), M, warmup, iters, int(use_graph),
                                                 ctypes.byref(ms)))
        return ms.value


# ---- host-only helpers (no GPU needed) ----

def validate(desc: FcDesc) -> int:
    return _lib.load().ovfcc_desc_validate(ctypes.byref(desc))


def tiled_sizes(desc: FcDesc):
    L = _lib.load()
    a, b, c = ctypes.c_size_t(), ctypes.c_size_t(), ctypes.c_size_t()
    check(L.ovfcc_tiled_sizes(ctypes.byref(desc), ctypes.byref(a), ctypes.byref(b), ctypes.byref(c)))
    return a.value, b.value, c.value


def repack_host(desc: FcDesc, W, scales, zp=None):
    L = _lib.load()
    wb, sb, zb = tiled_sizes(desc)
    if wb == 0:
        raise OvfccError(_lib.EUNSUPPORTED, "descriptor keeps the OpenVINO layout")
    wt, st = np.empty(wb, np.uint8), np.empty(sb // 2, np.float16)
    zt = np.empty(zb, np.uint8) if zb else None
    W = np.ascontiguousarray(W)
    scales = np.ascontiguousarray(scales, dtype=np.float16)
    zp = None if zp is None else np.ascontiguousarray(zp, dtype=np.uint8)
    check(L.ovfcc_repack_host(ctypes.byref(desc), _vp(W), _vp(scales), _vp(zp), _vp(wt), _vp(st), _vp(zt)))
    return wt, st, zt


def unrepack_host(desc: FcDesc, wt, st, zt=None):
    L = _lib.load()
    four = desc.w_type in (_lib.U4, _lib.I4)
    ng = desc.K // desc.group_size
    W = np.empty(desc.N * desc.K // 2 if four else desc.N * desc.K, np.uint8)
    scales = np.empty((desc.N, ng), np.float16)
    zp = None
    if zt is not None:
        zp = np.empty((desc.N * ng + 1) // 2 if desc.zp_type == _lib.U4 else desc.N * ng, np.uint8)
    check(L.ovfcc_unrepack_host(ctypes.byref(desc), _vp(wt), _vp(st), _vp(zt), _vp(W), _vp(scales), _vp(zp)))
    return W, scales, zp
