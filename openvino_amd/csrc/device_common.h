// Device-side types and the register unpack shared by the tiled kernels (gfx950, wave64).
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

#include "ovfcc_internal.h"

namespace ovfcc {

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));
typedef uint32_t uint2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void* lds_void_ptr;            // destination of a direct-to-LDS load
typedef __attribute__((address_space(3))) unsigned char* lds_byte_ptr;  // arithmetic stays in the LDS address space

__device__ __forceinline__ half2_t as_half2(uint32_t u) {
    return __builtin_bit_cast(half2_t, u);
}
__device__ __forceinline__ uint32_t as_u32(half2_t h) {
    return __builtin_bit_cast(uint32_t, h);
}

union Frag8 {
    half8_t v;
    uint32_t u[4];
    half2_t h2[4];
};

// One dword of the 4-bit tile layout -> 8 exact halves (q - zp), elements 0..7 in order.
// 0x6400 | q is the half 1024 + q; 0x5400 | (q << 4) is the half 64 + q.  Subtracting
// (1024 + zp) resp. (64 + zp) is exact in half precision.
__device__ __forceinline__ void unpack4(uint32_t w, half2_t off_lo, half2_t off_hi, Frag8& f) {
    const uint32_t w8 = w >> 8;
    f.h2[0] = as_half2((w & 0x000F000Fu) | 0x64006400u) - off_lo;
    f.h2[1] = as_half2((w & 0x00F000F0u) | 0x54005400u) - off_hi;
    f.h2[2] = as_half2((w8 & 0x000F000Fu) | 0x64006400u) - off_lo;
    f.h2[3] = as_half2((w8 & 0x00F000F0u) | 0x54005400u) - off_hi;
}

// Two dwords of the 8-bit tile layout (8 consecutive inputs) -> 8 exact halves (q - zp).
__device__ __forceinline__ void unpack8(uint32_t w0, uint32_t w1, half2_t off, Frag8& f) {
    // byte permute: result bytes {w.b0, 0x64, w.b1, 0x64} = halves (1024 + b0, 1024 + b1)
    f.h2[0] = as_half2(__builtin_amdgcn_perm(0x64646464u, w0, 0x04010400u)) - off;
    f.h2[1] = as_half2(__builtin_amdgcn_perm(0x64646464u, w0, 0x04030402u)) - off;
    f.h2[2] = as_half2(__builtin_amdgcn_perm(0x64646464u, w1, 0x04010400u)) - off;
    f.h2[3] = as_half2(__builtin_amdgcn_perm(0x64646464u, w1, 0x04030402u)) - off;
}

// The masks and magic numbers of the 4-bit unpack as values the compiler cannot fold: with register
// operands (w & mask) | magic selects the single instruction v_and_or_b32, with literals it becomes two.
// (Plain C on purpose: the compiler must see these VALU writes to keep its MFMA hazard spacing right.)
struct Unpack4Consts {
    uint32_t mask_lo, mask_hi, magic_lo, magic_hi;
};
__device__ __forceinline__ Unpack4Consts unpack4_consts() {
    Unpack4Consts c{0x000F000Fu, 0x00F000F0u, 0x64006400u, 0x54005400u};
    asm volatile("" : "+s"(c.mask_lo), "+s"(c.mask_hi));
    asm volatile("" : "+v"(c.magic_lo), "+v"(c.magic_hi));
    return c;
}

// Biased variants: the halves 1024 + q (elements 0,1,4,5) and 64 + q (elements 2,3,6,7) of a 4-bit dword,
// resp. 1024 + q for every element of two 8-bit dwords, without removing the bias.  A kernel that uses them
// cancels bias and zero-point with one extra MFMA whose weight operand is the constant fragment
// {-(1024 + zp), -(64 + zp), -(1024 + zp), -(64 + zp)} (resp. all -(1024 + zp)): the products are exact and
// the f32 accumulator sees sum x * (bias + q) - sum x * (bias + zp).
__device__ __forceinline__ void unpack4_biased(uint32_t w, const Unpack4Consts& c, Frag8& f) {
    const uint32_t w8 = w >> 8;
    f.u[0] = (w & c.mask_lo) | c.magic_lo;
    f.u[1] = (w & c.mask_hi) | c.magic_hi;
    f.u[2] = (w8 & c.mask_lo) | c.magic_lo;
    f.u[3] = (w8 & c.mask_hi) | c.magic_hi;
}

__device__ __forceinline__ void unpack8_biased(uint32_t w0, uint32_t w1, Frag8& f) {
    f.u[0] = __builtin_amdgcn_perm(0x64646464u, w0, 0x04010400u);
    f.u[1] = __builtin_amdgcn_perm(0x64646464u, w0, 0x04030402u);
    f.u[2] = __builtin_amdgcn_perm(0x64646464u, w1, 0x04010400u);
    f.u[3] = __builtin_amdgcn_perm(0x64646464u, w1, 0x04030402u);
}

// A pointer that is the same in every lane, told to the compiler (both halves through readfirstlane).
__device__ __forceinline__ const void* uniform_ptr(const void* p) {
    const uint64_t v = reinterpret_cast<uint64_t>(p);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return reinterpret_cast<const void*>(((uint64_t)hi << 32) | lo);
}

// Tile coordinates of this workgroup for a 2-D tile grid, arranged for the chip's eight XCDs.  The dispatcher
// hands consecutive workgroups to consecutive XCDs (workgroup L runs on XCD L % 8), every XCD has its own L2,
// and one XCD runs 32 workgroups of a one-per-CU kernel at a time.  Workgroups that run together on an XCD
// are therefore given one compact sm x sn block of tiles (sm sn <= 32), so that they share activation
// row-blocks and weight column-blocks through that L2; sm : sn is chosen to minimise the bytes the block
// fetches, row_cost and col_cost being the relative sizes of one tile's activation and weight strips.
// Blocks are dealt to the XCDs round-robin; when the number of blocks is no multiple of eight, the blocks
// of the last, partial round are cut into equal runs of tiles, one run per XCD.
// xcd_tile_at: the tile of position `linear` (< gx gy) in that order, for a gx x gy tile grid.
__device__ __forceinline__ void xcd_tile_at(unsigned linear, unsigned gx, unsigned gy, int& tile_x, int& tile_y,
                                            unsigned row_cost, unsigned col_cost) {
    const unsigned total = gx * gy;
    tile_x = (int)(linear % gx);
    tile_y = (int)(linear / gx);
    if (total & 7u)
        return;
    unsigned best_sn = 0, best_sm = 0;
    for (unsigned block = 32; block > 1 && best_sn == 0; block >>= 1) {
        unsigned best_cost = ~0u;
        for (unsigned sn = block; sn >= 1; sn >>= 1) {
            const unsigned sm = block / sn;
            const unsigned cost = row_cost * sm + col_cost * sn;
            if (gx % sn == 0 && gy % sm == 0 && cost < best_cost) {
                best_cost = cost;
                best_sn = sn;
                best_sm = sm;
            }
        }
    }
    if (best_sn == 0)
        return;
    const unsigned sn = best_sn, sm = best_sm, block = sn * sm;
    const unsigned xcd = linear & 7u, slot = linear >> 3;       // slot < total / 8
    const unsigned full_rounds = (total / block) >> 3;          // rounds in which every XCD owns a whole block
    unsigned super, within;
    if (slot < full_rounds * block) {
        super = (slot / block) * 8 + xcd;
        within = slot % block;
    } else {
        const unsigned share = (total >> 3) - full_rounds * block;    // tiles per XCD in the partial round
        const unsigned e = xcd * share + (slot - full_rounds * block);
        super = full_rounds * 8 + e / block;
        within = e % block;
    }
    const unsigned supers_x = gx / sn;
    tile_x = (int)((super % supers_x) * sn + within % sn);
    tile_y = (int)((super / supers_x) * sm + within / sn);
}

// The launch's own 2-D grid as the tile grid.
__device__ __forceinline__ void xcd_tile(int& tile_x, int& tile_y, unsigned row_cost, unsigned col_cost) {
    xcd_tile_at(blockIdx.y * gridDim.x + blockIdx.x, gridDim.x, gridDim.y, tile_x, tile_y, row_cost, col_cost);
}

// What one workgroup does: k-blocks [kb_lo, kb_hi) of the output tile at column block tile_x and rows m0.. of its
// node, as part z of split_k parts of that tile (split_k == 1: the whole tile), parked in workspace slot park_slot.
struct TileWork {
    int tile_x, tile_y, m0, z, split_k, kb_lo, kb_hi, park_slot;
};

// Work of workgroup blockIdx.x for a tiles_x x tiles_y tile grid (1-D launch) of the prefill kernels with
// 256-channel tiles; col_cost is the relative size of a tile's weight strip against 2 * tile_rows for its
// activation strip.  The first full_tiles workgroups take one whole tile each, in the XCD-aware order of
// xcd_tile_at; the remaining tiles are cut into tail_split
// parts along K, part by part (all first parts, then all second parts, ...), so that a launch whose tile count
// is a little more than a multiple of the compute units ends with a full round of shorter workgroups instead
// of a mostly idle round of whole tiles.  full_tiles = 0 splits every tile (few tiles, long K).
__device__ __forceinline__ TileWork tile_work(int tiles_x, int tiles_y, int full_tiles, int tail_split,
                                              int kb_per_split, int kb_total, int tile_rows, int col_cost) {
    TileWork wk;
    const int L = (int)blockIdx.x;
    int slot;
    if (L < full_tiles) {
        slot = L, wk.z = 0, wk.split_k = 1, wk.kb_lo = 0, wk.kb_hi = kb_total, wk.park_slot = 0;
    } else {
        const int tail = tiles_x * tiles_y - full_tiles, j = L - full_tiles;
        wk.z = j / tail, slot = full_tiles + j % tail, wk.split_k = tail_split;
        wk.kb_lo = wk.z * kb_per_split, wk.kb_hi = min(kb_total, wk.kb_lo + kb_per_split);
        wk.park_slot = j % tail;
    }
    xcd_tile_at((unsigned)slot, (unsigned)tiles_x, (unsigned)tiles_y, wk.tile_x, wk.tile_y, 2 * tile_rows, col_cost);
    wk.m0 = wk.tile_y * tile_rows;
    return wk;
}

// Gated-linear-unit epilogue on f32 values: act(gate) * up with act = Swish (1), Gelu (2), Gelu_Tanh (3), the
// formulas of the OpenVINO Intel-GPU plugin (cl_kernels/swiglu_gpu_ref.cl:74-85, swish beta = 1).  Exponential
// and reciprocal are the hardware's (about 1e-6 relative, far inside the f16 result): the epilogue of a prefill
// tile runs with the matrix cores idle, so its length is paid in full.  Both saturate correctly:
// exp -> inf gives 1 / inf = 0, exp -> 0 gives 1.  No multiply and add is contracted here: which ones the compiler
// fuses depends on the code around the call, and kernels that promise each other's bits must not differ in that.
__device__ __forceinline__ float glu_value(int type, float gate, float up) {
#pragma clang fp contract(off)
    // exp(t) as the hardware's 2^(t log2 e), one instruction: the library routine's range fix-ups are another place
    // where two kernels can come to differ
    constexpr float kLog2e = 1.44269504088896340736f;
    float a;
    if (type == 1) {
        a = gate * __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(-gate * kLog2e));
    } else if (type == 2) {
        a = 0.5f * gate * (1.f + erff(gate * 0.70710678118654752440f));
    } else {
        // tanh z = 1 - 2 / (1 + exp 2 z)
        const float z = 0.79788456080286535588f * gate * __builtin_fmaf(0.044715f * gate, gate, 1.f);
        a = gate * (1.f - __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(z * (2.f * kLog2e))));
    }
    return a * up;
}

// f32 -> f16, round to nearest even, of a value that exists in f32 first.  The empty asm statement keeps the compiler
// from folding the conversion into the multiply or fused multiply-add that produced the value (one rounding from the
// exact product instead of two): it does so in some kernels and not in others, and a result that sits on a rounding
// tie then differs by one f16 step between kernels that promise each other's bits.
__device__ __forceinline__ half_t to_half_rne(float v) {
    asm volatile("" : "+v"(v));
    return (half_t)v;
}

// Output cast: FullyConnected's output_type is f16 (default, the activation type) or f32.
__device__ __forceinline__ void store_out(void* y, size_t i, float v, int out_f32) {
    if (out_f32)
        static_cast<float*>(y)[i] = v;
    else
        static_cast<half_t*>(y)[i] = to_half_rne(v);
}

__device__ __forceinline__ half2_t splat(float v) {
    const half_t h = (half_t)v;
    return half2_t{h, h};
}

// s_waitcnt vmcnt(n) alone (export and LDS/scalar counters left at their maxima); n <= 63
constexpr int wait_vmcnt_imm(int n) {
    return (n & 15) | ((n >> 4) << 14) | 0x0F70;
}

}  // namespace ovfcc
