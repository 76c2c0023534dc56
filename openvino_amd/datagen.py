"""Seeded synthetic inputs for the FullyConnectedCompressed workloads.

Every tensor comes out in the byte layout OpenVINO constants use: weights row-major [N, K],
4-bit types two per byte with the even element in the low nibble
(src/core/dev_api/openvino/core/type/element_iterator.hpp:76,161-176), scales float16
[N, K/G], zero-points u4 packed along the group axis or u8.  The distributions are the ones
the benchmark configurations name; one seed fixes every tensor of a case.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional

import numpy as np

# (K, N) of the four projection shapes of one transformer block
LLAMA3_8B_SHAPES = {"qo": (4096, 4096), "kv": (4096, 1024), "gate_up": (4096, 14336), "down": (14336, 4096)}
LLAMA3_70B_SHAPES = {"qo": (8192, 8192), "kv": (8192, 1024), "gate_up": (8192, 28672), "down": (28672, 8192)}
# FC launches of one Llama-3-8B block in execution order
LLAMA3_8B_BLOCK = ["qo", "kv", "kv", "qo", "gate_up", "gate_up", "down"]


def pack_nibbles(values: np.ndarray) -> np.ndarray:
    """Flattened 4-bit values (unsigned 0..15 or signed -8..7) -> bytes, low nibble first."""
    v = np.asarray(values).ravel().astype(np.uint8) & 0x0F
    if v.size % 2:
        v = np.concatenate([v, np.zeros(1, np.uint8)])
    return (v[0::2] | (v[1::2] << 4)).astype(np.uint8)


def unpack_nibbles(packed: np.ndarray, count: int) -> np.ndarray:
    """Bytes -> the first `count` 4-bit values (0..15), low nibble first."""
    b = np.asarray(packed, dtype=np.uint8).ravel()
    v = np.empty(b.size * 2, np.uint8)
    v[0::2] = b & 0x0F
    v[1::2] = b >> 4
    return v[:count]


def to_input_major(c: "FcCase"):
    """The constants of a case as a MatMul with transpose_b = false holds them: W [K, N], scales and zero-point
    table [K / G, N], each packed over its own flattened index.  Returns (w, scale, zp)."""
    N, K, ng = c.N, c.K, c.K // c.group_size
    if c.w_type in ("u4", "i4"):
        w = pack_nibbles(unpack_nibbles(c.w, N * K).reshape(N, K).T)
    else:
        w = np.ascontiguousarray(np.asarray(c.w, dtype=np.uint8).reshape(N, K).T).ravel()
    scale = np.ascontiguousarray(np.asarray(c.scale).reshape(N, ng).T)
    zp = c.zp
    if zp is not None and not c.zp_scalar:
        if c.zp_type == "u4":
            zp = pack_nibbles(unpack_nibbles(zp, N * ng).reshape(N, ng).T)
        else:
            zp = np.ascontiguousarray(np.asarray(zp, dtype=np.uint8).reshape(N, ng).T).ravel()
    return w, scale, zp


@dataclass
class FcCase:
    """One FullyConnectedCompressed problem in OpenVINO's constant layout."""
    M: int
    K: int
    N: int
    group_size: int
    w_type: str                 # "u4" | "i4" | "u8" | "i8"
    zp_type: str                # "none" | "u4" | "u8"
    w: np.ndarray               # raw bytes
    scale: np.ndarray           # float16 [N, K/G]
    zp: Optional[np.ndarray]    # raw bytes or None
    x: np.ndarray               # float16 [M, K]
    bias: Optional[np.ndarray] = None   # float16 [N] or None
    zp_scalar: bool = False
    meta: dict = field(default_factory=dict)

    @property
    def n_groups(self) -> int:
        return self.K // self.group_size

    def algorithmic_bytes(self) -> int:
        """W + S + ZP + X + Y, the traffic one call cannot avoid."""
        bits = 8 if self.w_type in ("u8", "i8") else 4
        ng = self.n_groups
        zp = {"none": 0, "u4": self.N * ng // 2, "u8": self.N * ng}[self.zp_type]
        if self.zp_scalar:
            zp = 1
        return self.N * self.K * bits // 8 + self.N * ng * 2 + zp + self.M * self.K * 2 + self.M * self.N * 2

    def flops(self) -> int:
        return 2 * self.M * self.N * self.K


def activations(rng: np.random.Generator, M: int, K: int, outlier_fraction: float = 0.0,
                outlier_scale: float = 20.0) -> np.ndarray:
    """float16 [M, K] ~ N(0,1); a fraction of the K channels (drawn once) is scaled up."""
    x = rng.standard_normal((M, K), dtype=np.float32)
    if outlier_fraction > 0:
        n_out = max(1, int(round(K * outlier_fraction)))
        cols = rng.choice(K, size=n_out, replace=False)
        x[:, cols] *= outlier_scale
    return x.astype(np.float16)


def weights_only(seed: int, K: int, N: int, w_type: str = "i4", group_size: int = 128,
                 zp_type: str = "none", scale_range=(0.002, 0.02), zp_range=None) -> FcCase:
    """Weights, scales and zero-points of one layer (x is left empty)."""
    return make_case(seed, 0, K, N, w_type, group_size, zp_type, scale_range, zp_range)


def make_case(seed: int, M: int, K: int, N: int, w_type: str = "u4", group_size: int = 128,
              zp_type: str = "u4", scale_range=(0.002, 0.02), zp_range=None,
              outlier_fraction: float = 0.0, with_bias: bool = False) -> FcCase:
    if group_size <= 0 or K % group_size:
        raise ValueError("group_size must divide K")
    rng = np.random.default_rng(seed)
    ng = K // group_size
    if w_type == "u4":
        w = pack_nibbles(rng.integers(0, 16, size=N * K, dtype=np.uint8))
    elif w_type == "i4":
        w = pack_nibbles(rng.integers(-8, 8, size=N * K, dtype=np.int8))
    elif w_type == "u8":
        w = rng.integers(0, 256, size=N * K, dtype=np.uint8)
    elif w_type == "i8":
        w = rng.integers(-128, 128, size=N * K, dtype=np.int8).view(np.uint8)
    else:
        raise ValueError(w_type)
    scale = rng.uniform(scale_range[0], scale_range[1], size=(N, ng)).astype(np.float16)
    if zp_type == "none":
        zp = None
    elif zp_type == "u4":
        lo, hi = zp_range or (0, 16)
        zp = pack_nibbles(rng.integers(lo, hi, size=N * ng, dtype=np.uint8))
    elif zp_type == "u8":
        lo, hi = zp_range or (0, 256)
        zp = rng.integers(lo, hi, size=N * ng, dtype=np.uint8)
    else:
        raise ValueError(zp_type)
    x = activations(rng, M, K, outlier_fraction)
    bias = rng.standard_normal(N).astype(np.float16) if with_bias else None
    return FcCase(M, K, N, group_size, w_type, zp_type, w, scale, zp, x, bias,
                  meta={"seed": seed})


# ---- the five benchmark configurations ----

def config1(seed: int = 1001) -> FcCase:
    """u4 asymmetric g128, [1,4096] x [4096,4096]."""
    return make_case(seed, 1, 4096, 4096, "u4", 128, "u4")


def config2(shape: str, M: int, seed: int = 2001) -> FcCase:
    """Llama-3-8B projection, i4 symmetric g128, decode M in {1,4,16,32}."""
    K, N = LLAMA3_8B_SHAPES[shape]
    return make_case(seed, M, K, N, "i4", 128, "none")


def config3(shape: str, M: int, seed: int = 3001) -> FcCase:
    """Same projections at prefill M in {512,2048,8192}, 0.1 % outlier channels x20."""
    K, N = LLAMA3_8B_SHAPES[shape]
    return make_case(seed, M, K, N, "i4", 128, "none", outlier_fraction=0.001)


def config4(shape: str, M: int, seed: int = 4001) -> FcCase:
    """Llama-3-70B projection, u8 asymmetric per output channel."""
    K, N = LLAMA3_70B_SHAPES[shape]
    return make_case(seed, M, K, N, "u8", K, "u8", scale_range=(1e-3, 1e-2), zp_range=(100, 157))


def moe_routing(seed: int = 5001, tokens: int = 256, experts: int = 8, top_k: int = 2):
    """Top-k routing from seeded softmax logits ~N(0,1): list of token-index arrays, one per expert."""
    rng = np.random.default_rng(seed)
    logits = rng.standard_normal((tokens, experts))
    p = np.exp(logits - logits.max(axis=1, keepdims=True))
    p /= p.sum(axis=1, keepdims=True)
    top = np.argsort(-p, axis=1, kind="stable")[:, :top_k]
    return [np.nonzero((top == e).any(axis=1))[0] for e in range(experts)]


def config5_expert(expert: int, which: str, M: int, seed: int = 5001) -> FcCase:
    """One Mixtral-8x7B expert matrix (gate/up 4096->14336, down 14336->4096), u4 asymmetric g128."""
    K, N = (4096, 14336) if which in ("gate", "up") else (14336, 4096)
    sub = {"gate": 0, "up": 1, "down": 2}[which]
    return make_case(seed + 10 * expert + sub + 1, M, K, N, "u4", 128, "u4")
