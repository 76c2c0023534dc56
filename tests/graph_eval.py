"""Evaluates a plain-node graph (openvino_amd.graph.Graph with constant data) node by node in float64 numpy, every
operation on its own as the opset defines it -- Convert, Subtract, Multiply, Reshape, Transpose, MatMul, Add, Swish,
Gelu, ReduceSum, GatherMatmul, GroupedMatMul -- with no knowledge of the fold: the value a plugin that fuses nothing
would produce (rounding of intermediate tensors aside).  Test infrastructure: a check on what the library makes of
the same graph, never part of the product path.

Semantics followed: MatMul src/core/reference/include/openvino/reference/matmul.hpp; Swish x * sigmoid(x)
(src/core/reference/include/openvino/reference/swish.hpp); Gelu erf / tanh forms
(src/core/reference/include/openvino/reference/gelu.hpp); GatherMatmul out[k, m] = A[k or 0, m] x B[indices[m, k]]^T
+ bias[indices[m, k]] (src/common/transformations/include/ov_ops/gather_matmul.hpp:17-41); GroupedMatMul rows
[offsets[g-1], offsets[g]) x B[g]^T (src/core/include/openvino/op/grouped_matmul.hpp:26-50)."""
import math

import numpy as np

from openvino_amd import _lib

_OP = {v: k for k, v in _lib.OP.items()}
_TYPE = {v: k for k, v in _lib.TYPE.items()}
_erf = np.vectorize(math.erf, otypes=[np.float64])


def decode_constant(type_name, shape, raw):
    """OpenVINO's packing -> float64 array of `shape`: 4-bit types two per byte, low nibble first."""
    count = int(np.prod(shape)) if len(shape) else 1
    raw = np.asarray(raw, np.uint8)
    if type_name in ("u4", "i4"):
        v = np.empty(2 * raw.size, np.int64)
        v[0::2], v[1::2] = raw & 15, raw >> 4
        v = v[:count]
        if type_name == "i4":
            v = np.where(v > 7, v - 16, v)
    elif type_name == "u8":
        v = raw[:count].astype(np.int64)
    elif type_name == "i8":
        v = raw[:count].view(np.int8).astype(np.int64)
    elif type_name == "f16":
        v = raw[:2 * count].view(np.float16)
    elif type_name == "f32":
        v = raw[:4 * count].view(np.float32)
    else:
        raise ValueError(type_name)
    return v.astype(np.float64).reshape(shape)


class Evaluator:
    def __init__(self, g, feeds):
        """feeds: node index of a Parameter -> array"""
        self.g, self.feeds, self.cache = g, feeds, {}

    def ints(self, i):
        n = self.g.nodes[i]
        assert n.n_ints >= 0, f"node {i} carries no integer values"
        return [int(n.ints[k]) for k in range(n.n_ints)]

    def decompress(self, w, scale, zp):
        """(W - zp) * scale for batched constants W [E, N, K] with scale / zero-point [E, N, K/G] (or one element)"""
        s = self.value(scale)
        E, N, K = w.shape
        ng = s.shape[2] if s.ndim == 3 else 1
        w = w.reshape(E, N, ng, K // ng)
        if zp >= 0 and int(np.prod(self.g.shape(zp))) > 0:
            z = self.value(zp)
            w = w - (z.reshape(E, N, ng, 1) if z.size > 1 else z.reshape(()))
        return (w * (s.reshape(E, N, ng, 1) if s.size > 1 else s.reshape(()))).reshape(E, N, K)

    def value(self, i):
        if i in self.cache:
            return self.cache[i]
        n = self.g.nodes[i]
        op = _OP[n.op]
        ins = [int(n.inputs[k]) for k in range(n.n_inputs)]
        if op == "parameter":
            v = np.asarray(self.feeds[i])
            v = v if v.dtype.kind in "iu" else v.astype(np.float64)
        elif op == "constant":
            v = decode_constant(_TYPE[n.type], self.g.shape(i), self.g.data[i])
        elif op in ("convert", "result"):
            v = self.value(ins[0])
        elif op == "subtract":
            v = self.value(ins[0]) - self.value(ins[1])
        elif op == "multiply":
            v = self.value(ins[0]) * self.value(ins[1])
        elif op == "add":
            v = self.value(ins[0]) + self.value(ins[1])
        elif op == "reshape":
            v = self.value(ins[0]).reshape([int(d) for d in self.g.shape(i)])
        elif op == "transpose":
            v = np.transpose(self.value(ins[0]), self.ints(ins[1]))
        elif op == "unsqueeze":
            v = np.expand_dims(self.value(ins[0]), self.ints(ins[1])[0])
        elif op == "reduce_sum":
            v = np.sum(self.value(ins[0]), axis=self.ints(ins[1])[0], keepdims=bool(n.attr))
        elif op == "matmul":
            a, b = self.value(ins[0]), self.value(ins[1])
            a = np.swapaxes(a, -1, -2) if n.transpose_a else a
            b = np.swapaxes(b, -1, -2) if n.transpose_b else b
            v = a @ b
        elif op == "fully_connected":
            v = self.value(ins[0]) @ self.value(ins[1]).T
            if len(ins) > 2 and ins[2] >= 0 and int(np.prod(self.g.shape(ins[2]))) > 0:
                v = v + self.value(ins[2]).reshape(-1)
        elif op == "swish":
            x = self.value(ins[0])
            v = x / (1.0 + np.exp(-x))
        elif op == "gelu":
            x = self.value(ins[0])
            if n.attr:
                v = 0.5 * x * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (x + 0.044715 * x ** 3)))
            else:
                v = 0.5 * x * (1.0 + _erf(x / math.sqrt(2.0)))
        elif op in ("gather_matmul", "gather_matmul_compressed"):
            a, b, idx = self.value(ins[0]), self.value(ins[1]), np.asarray(self.value(ins[2]), np.int64)
            if op == "gather_matmul_compressed":   # B, scale, zero-point [E, N, K/G]: decompress first
                b = self.decompress(b, ins[4], ins[5] if len(ins) > 5 else -1)
            bias = None
            if len(ins) > 3 and ins[3] >= 0 and int(np.prod(self.g.shape(ins[3]))) > 0:
                bias = self.value(ins[3])
            M, top_k = idx.shape
            v = np.zeros((top_k, M, b.shape[1]))
            for m in range(M):
                for k in range(top_k):
                    e = idx[m, k]
                    v[k, m] = b[e] @ a[k if a.shape[0] > 1 else 0, m]
                    if bias is not None:
                        v[k, m] += bias.reshape(-1, b.shape[1])[e if bias.size > b.shape[1] else 0]
        elif op in ("grouped_matmul", "grouped_matmul_compressed"):
            a, b = self.value(ins[0]), self.value(ins[1])
            offsets = ins[2] if len(ins) > 2 and self.g.nodes[ins[2]].op == _lib.OP["parameter"] else -1
            if op == "grouped_matmul_compressed":   # (A, B, [offsets,] scale[, zp])
                rest = ins[3:] if offsets >= 0 else ins[2:]
                b = self.decompress(b, rest[0], rest[1] if len(rest) > 1 else -1)
            if offsets >= 0:
                ends = np.asarray(self.value(offsets), np.int64)
                v = np.zeros((a.shape[0], b.shape[1]))
                first = 0
                for grp, end in enumerate(ends):
                    v[first:end] = a[first:end] @ b[grp].T
                    first = int(end)
            else:
                v = np.einsum("gmk,gnk->gmn", a, b)
        else:
            raise NotImplementedError(op)
        self.cache[i] = v
        return v
