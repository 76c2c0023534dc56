"""Plain-node description of a model fragment for the graph-side entry points (include/ovfcc_graph.h), and thin
wrappers over them: what the ov::IPlugin shim does with an ov::Model, in the vocabulary of OpenVINO's opset."""
from __future__ import annotations

import ctypes
from typing import Optional, Sequence

from . import _lib
from ._lib import OvfccError, check

_T = dict(_lib.TYPE, other=_lib.TYPE_OTHER, i32=_lib.TYPE_OTHER, i64=_lib.TYPE_OTHER, bf16=_lib.TYPE_OTHER)


class Graph:
    """Nodes are appended in topological order; every method returns the new node's index."""

    def __init__(self):
        self.nodes = []
        self.data = {}   # node index -> the Constant's bytes (numpy uint8, OpenVINO packing), where supplied

    def _add(self, op, type_, shape, inputs=(), transpose_a=False, transpose_b=False, attr=0, ints=None):
        n = _lib.GNode()
        n.op = _lib.OP[op]
        n.type = _T[type_]
        if shape is None:
            n.rank = -1
        else:
            n.rank = len(shape)
            for i, d in enumerate(shape):
                n.dims[i] = int(d)
        n.n_inputs = len(inputs)
        for i, v in enumerate(inputs):
            n.inputs[i] = -1 if v is None else int(v)
            if v is not None:
                self.nodes[v].consumers += 1
        n.transpose_a, n.transpose_b, n.attr = int(transpose_a), int(transpose_b), int(attr)
        if ints is None:
            n.n_ints = -1
        else:
            n.n_ints = len(ints)
            for i, v in enumerate(ints):
                n.ints[i] = int(v)
        self.nodes.append(n)
        return len(self.nodes) - 1

    def shape(self, i):
        n = self.nodes[i]
        return None if n.rank < 0 else [int(n.dims[k]) for k in range(n.rank)]

    def type(self, i):
        return {v: k for k, v in _T.items() if k in _lib.TYPE or k == "other"}[self.nodes[i].type]

    def parameter(self, type_, shape):
        return self._add("parameter", type_, shape)

    def constant(self, type_, shape, ints=None, data=None):
        """data: the Constant's bytes in OpenVINO's packing (any contiguous numpy array; 4-bit types two per byte,
        low nibble first), needed only by create_weights / create_expert_weights."""
        i = self._add("constant", type_, shape, ints=ints)
        if data is not None:
            self.set_data(i, data)
        return i

    def set_data(self, i, data):
        import numpy as np
        self.data[i] = np.ascontiguousarray(data).reshape(-1).view(np.uint8)

    def _data_table(self):
        table = (ctypes.c_void_p * len(self.nodes))()
        for i, a in self.data.items():
            table[i] = a.ctypes.data
        return table

    def convert(self, x, type_):
        return self._add("convert", type_, self.shape(x), [x])

    @staticmethod
    def _broadcast(a, b):
        r = max(len(a), len(b))
        a, b = [1] * (r - len(a)) + list(a), [1] * (r - len(b)) + list(b)
        return [max(p, q) for p, q in zip(a, b)]

    def subtract(self, a, b):
        return self._add("subtract", self.type(a), self._broadcast(self.shape(a), self.shape(b)), [a, b])

    def multiply(self, a, b):
        return self._add("multiply", self.type(a), self._broadcast(self.shape(a), self.shape(b)), [a, b])

    def add(self, a, b):
        return self._add("add", self.type(a), self._broadcast(self.shape(a), self.shape(b)), [a, b])

    def reshape(self, x, target):
        """target: the output shape (already resolved; -1 / 0 entries of the pattern are the caller's business)"""
        pattern = self.constant("i32", [len(target)], ints=target if len(target) <= _lib.MAX_RANK else None)
        return self._add("reshape", self.type(x), target, [x, pattern])

    def transpose(self, x, order):
        c = self.constant("i32", [len(order)], ints=order)
        s = self.shape(x)
        return self._add("transpose", self.type(x), [s[o] for o in order], [x, c])

    def matmul(self, a, b, transpose_a=False, transpose_b=False, type_=None):
        sa, sb = self.shape(a), self.shape(b)
        n = sb[-2] if transpose_b else sb[-1]
        return self._add("matmul", type_ or self.type(a), sa[:-1] + [n], [a, b], transpose_a, transpose_b)

    def fully_connected(self, a, w, bias=None, type_=None):
        """ov::op::internal::FullyConnected: W is [N, K]"""
        return self._add("fully_connected", type_ or self.type(a), self.shape(a)[:-1] + [self.shape(w)[-2]], [a, w, bias])

    def swish(self, x):
        return self._add("swish", self.type(x), self.shape(x), [x])

    def gelu(self, x, tanh=False):
        return self._add("gelu", self.type(x), self.shape(x), [x], attr=int(tanh))

    def unsqueeze(self, x, axis):
        s = self.shape(x)
        axis = axis if axis >= 0 else axis + len(s) + 1
        c = self.constant("i32", [1], ints=[axis])
        return self._add("unsqueeze", self.type(x), s[:axis] + [1] + s[axis:], [x, c])

    def slice(self, x, shape):
        """v8::Slice with constant begin / end / step / axes; shape: the resolved output shape"""
        cs = [self.constant("i32", [1]) for _ in range(4)]
        return self._add("slice", self.type(x), shape, [x] + cs)

    def reduce_sum(self, x, axis, keep_dims=False):
        s = self.shape(x)
        c = self.constant("i32", [1], ints=[axis])
        out = [d for i, d in enumerate(s) if i != axis] if not keep_dims else [1 if i == axis else d for i, d in enumerate(s)]
        return self._add("reduce_sum", self.type(x), out, [x, c], attr=int(keep_dims))

    def no_bias(self):
        """Constant(element::dynamic, Shape{0}): the reference's "no bias" input"""
        return self.constant("other", [0])

    def gather_matmul(self, a, b, indices, bias=None, type_=None):
        """ov::op::internal::GatherMatmul: A [1 or top_k, M, K], B [E, N, K], indices [M, top_k] -> [top_k, M, N]"""
        bias = self.no_bias() if bias is None else bias
        sa, sb, si = self.shape(a), self.shape(b), self.shape(indices)
        return self._add("gather_matmul", type_ or self.type(a), [si[1], sa[1], sb[1]], [a, b, indices, bias])

    def gather_matmul_compressed(self, a, b, indices, scale, zp=None, bias=None, type_=None):
        """ov::op::internal::GatherMatmulCompressed: B, scale, zp Constants of three dimensions"""
        bias = self.no_bias() if bias is None else bias
        zp = self.constant("other", [0]) if zp is None else zp
        sa, sb, si = self.shape(a), self.shape(b), self.shape(indices)
        return self._add("gather_matmul_compressed", type_ or self.type(a), [si[1], sa[1], sb[1]],
                         [a, b, indices, bias, scale, zp])

    def grouped_matmul(self, a, b, offsets=None, type_=None):
        """ov::op::v17::GroupedMatMul: A [rows, K] with offsets [G], or A [G, M, K]; B [G, N, K]"""
        sa, sb = self.shape(a), self.shape(b)
        return self._add("grouped_matmul", type_ or self.type(a), list(sa[:-1]) + [sb[1]],
                         [a, b] + ([offsets] if offsets is not None else []))

    def grouped_matmul_compressed(self, a, b, scale, zp=None, offsets=None, type_=None):
        """ov::op::internal::GroupedMatMulCompressed: (A, B, [offsets,] scale[, zp]), B, scale, zp Constants"""
        sa, sb = self.shape(a), self.shape(b)
        ins = [a, b] + ([offsets] if offsets is not None else []) + [scale] + ([zp] if zp is not None else [])
        return self._add("grouped_matmul_compressed", type_ or self.type(a), list(sa[:-1]) + [sb[1]], ins)

    def other(self, inputs, type_="f16", shape=None):
        return self._add("other", type_, shape, list(inputs))

    def result(self, x):
        return self._add("result", self.type(x), self.shape(x), [x])

    def _array(self):
        arr = (_lib.GNode * len(self.nodes))()
        for i, n in enumerate(self.nodes):
            arr[i] = n
        return arr

    # ---- the entry points ----
    def fold_match(self, root: int) -> _lib.Fold:
        out = _lib.Fold()
        check(_lib.load().ovfcc_fold_match(self._array(), len(self.nodes), root, ctypes.byref(out)))
        return out

    def fold_gather_matmul(self, root: int) -> _lib.GatherFold:
        out = _lib.GatherFold()
        check(_lib.load().ovfcc_fold_gather_matmul(self._array(), len(self.nodes), root, ctypes.byref(out)))
        return out

    def fold_grouped_matmul(self, root: int) -> _lib.GatherFold:
        out = _lib.GatherFold()
        check(_lib.load().ovfcc_fold_grouped_matmul(self._array(), len(self.nodes), root, ctypes.byref(out)))
        return out

    def fold_moe(self, root: int) -> _lib.MoeFold:
        out = _lib.MoeFold()
        check(_lib.load().ovfcc_fold_moe(self._array(), len(self.nodes), root, ctypes.byref(out)))
        return out

    def create_weights(self, device, fold: _lib.Fold, extra_flags: int = 0):
        """The node a fold describes, created from the data of its Constants (ovfcc_fold_weights_create)."""
        from .fc import CompressedWeights
        h = ctypes.c_void_p()
        check(device.lib.ovfcc_fold_weights_create(device.handle, self._array(), len(self.nodes), ctypes.byref(fold),
                                                   self._data_table(), extra_flags, ctypes.byref(h)))
        return CompressedWeights.adopt(device, h, fold.desc, extra_flags)

    def create_expert_weights(self, device, fold: _lib.GatherFold, expert: int, extra_flags: int = 0):
        """Expert (or group) `expert` of a gather / grouped fold as a node of its own."""
        from .fc import CompressedWeights
        h = ctypes.c_void_p()
        check(device.lib.ovfcc_fold_expert_weights_create(device.handle, self._array(), len(self.nodes), ctypes.byref(fold),
                                                          expert, self._data_table(), extra_flags, ctypes.byref(h)))
        return CompressedWeights.adopt(device, h, fold.desc, extra_flags)

    def fold_model(self, max_folds: int = 64):
        folds = (_lib.Fold * max_folds)()
        fused = (_lib.Fused * max_folds)()
        nf, nu = ctypes.c_int(0), ctypes.c_int(0)
        check(_lib.load().ovfcc_fold_model(self._array(), len(self.nodes), folds, max_folds, ctypes.byref(nf), fused,
                                           max_folds, ctypes.byref(nu)))
        return [folds[i] for i in range(nf.value)], [fused[i] for i in range(nu.value)]


def decompression_subgraph(g: Graph, w_type: str, w_shape: Sequence[int], scale_shape: Optional[Sequence[int]],
                           zp_shape: Optional[Sequence[int]] = None, zp_type: Optional[str] = None,
                           scale_type: str = "f32", compute_type: str = "f32", reshape_to: Optional[Sequence[int]] = None,
                           transpose: bool = False, convert_to: Optional[str] = None,
                           scale_const_shape: Optional[Sequence[int]] = None) -> int:
    """Constant -> Convert -> [Subtract] -> Multiply -> [Reshape] -> [Convert] -> [Transpose]: the chain that
    CompressedWeightsBlock matches, in the order the reference's builders emit it.  scale_const_shape: the scale
    (and zero-point) constant is stored in this squeezed shape and reshaped to scale_shape in the graph."""
    w = g.convert(g.constant(w_type, w_shape), compute_type)

    def param(type_, shape):
        stored = shape if scale_const_shape is None or len(shape) == 0 else scale_const_shape
        c = g.constant(type_, stored)
        if type_ != compute_type:
            c = g.convert(c, compute_type)
        if stored is not shape and list(stored) != list(shape):
            c = g.reshape(c, shape)
        return c
    body = w
    if zp_shape is not None:
        body = g.subtract(w, param(zp_type or w_type, list(zp_shape)))
    out = g.multiply(body, param(scale_type, list(scale_shape)))
    if reshape_to is not None:
        out = g.reshape(out, list(reshape_to))
    if convert_to is not None and convert_to != compute_type:
        out = g.convert(out, convert_to)
    if transpose:
        out = g.transpose(out, [1, 0])
    return out
