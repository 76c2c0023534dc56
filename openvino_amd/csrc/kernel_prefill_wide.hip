// Wide prefill kernel (M > 32): 128 x 256 output tile per workgroup, 8 waves, double-buffered LDS.
//
// grid = (N/256, ceil(M/128)), block = 512.  K advances 64 inputs per stage (K % 256 == 0).  Per stage the
// workgroup
//   - issues the global loads of the 128 x 64 activation tile (f16) and of the packed weight tiles that
//     will be needed four stages later (a register ring covers the memory latency),
//   - runs the MFMAs of the current stage out of LDS,
//   - dequantises the packed weights of the next stage to f16 and writes both next tiles to the other
//     LDS buffer, one barrier per stage.
// LDS tiles are row-major with 64 halves (128 bytes) per row, no padding; the eight 16-byte chunks of a
// row are stored at chunk ^ ((row >> 1) & 7).  LDS has 64 four-byte banks and serves a 128-bit access 16
// lanes at a time, so 16 consecutive rows (two per 256-byte bank wrap) must land on 16 distinct 16-byte
// slots: the row parity picks the half of the wrap, the swizzle the slot within it.
//
// Waves: two groups of four.  Both groups own the same 2 x 2 arrangement of 64 x 128 wave tiles; group 0
// contracts the first 32 inputs of every stage, group 1 the last 32, so every SIMD holds two waves that
// alternate on the matrix pipe while reading disjoint halves of the tiles.  After the last stage group 1
// passes its f32 accumulators to group 0 through LDS.
// v_mfma_f32_32x32x16_f16: operand lane = row (lane & 31), inputs 8 (lane >> 5) ..+8;
// result: column n = lane & 31, rows 8 (r >> 2) + 4 (lane >> 5) + (r & 3), r = 0..15.
//
// Weights: (q - zp) * s rounded once to f16 for grouped scales; with one group per channel the exact
// integers q - zp go to the matrix cores and the scale multiplies the f32 result.
#include "device_common.h"

namespace ovfcc {

constexpr int PW_BM = 128, PW_BN = 256, PW_BK = 64;
constexpr int PW_A_HALVES = PW_BM * PW_BK;  // per buffer
constexpr int PW_B_HALVES = PW_BN * PW_BK;
constexpr int PW_RING = 2;                             // LDS stages (double buffer)
constexpr unsigned PW_LDS_BYTES = 4u * 64 * 128 * 4;  // 128 KiB: the epilogue hand-over (the ring needs 96 KiB)

__device__ __forceinline__ int swz(int row, int chunk) {
    return row * PW_BK + ((chunk ^ ((row >> 1) & 7)) << 3);
}

template <int BITS, bool ZP_TABLE, bool PRESCALE>
__global__ __launch_bounds__(512) void fcc_prefill_wide_kernel(const uint4_t* __restrict__ wt,
                                                               const half_t* __restrict__ st,
                                                               const uint8_t* __restrict__ zt,
                                                               const half_t* __restrict__ x,
                                                               const half_t* __restrict__ bias,
                                                               void* __restrict__ y, int M, int N, int K,
                                                               int kb_total, int kb_per_group, int ng, int zp_const,
                                                               int out_f32, int glu) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    half_t* As = reinterpret_cast<half_t*>(lds_raw);  // [2][128 x 64]
    half_t* Bs = As + PW_RING * PW_A_HALVES;          // [2][256 x 64]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int kgrp = wave >> 2;            // which 32 inputs of a stage this wave contracts
    const int wm = (wave >> 1) & 1, wn = wave & 1;
    int tile_x, tile_y;
    xcd_tile(tile_x, tile_y, 2 * PW_BM * 2, PW_BN * BITS / 4);
    const int n0 = tile_x * PW_BN;
    const int m0 = tile_y * PW_BM;
    const int col = lane & 15, kq = lane >> 4;

    // Global loads run four stages ahead of the MFMAs (register ring), far enough to cover an L2 / HBM
    // round trip; every load goes through a range-checked descriptor (rows >= M and stages past the end of
    // K read zero), so the four-stage loop body below is straight-line and its waits count exactly.
    constexpr unsigned kOob = 0x80000000u;
    const __amdgpu_buffer_rsrc_t rx =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(x), 0, M * K * 2, 0x00020000);
    // thread covers chunks tid and tid + 512 of the 128 x 8 chunk grid: row = chunk / 8
    const int a_row0 = tid >> 3, a_chunk = tid & 7;
    unsigned a_off[2];
#pragma unroll
    for (int p = 0; p < 2; ++p) {
        const int m = m0 + a_row0 + 64 * p;
        a_off[p] = m < M ? (unsigned)(m * K + a_chunk * 8) * 2u : kOob;
    }
    // weights: wave covers channel tiles 2 wave, 2 wave + 1 of the 16 in this workgroup
    constexpr int TPB = BITS == 4 ? 1 : 2;
    const int nt0 = n0 / 16 + 2 * wave;
    const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint4_t*>(wt + (size_t)nt0 * kb_total * TPB * 64), 0, 2 * kb_total * TPB * kTileBytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<half_t*>(st + (size_t)nt0 * ng * 16), 0, 2 * ng * 32, 0x00020000);
    const __amdgpu_buffer_rsrc_t rz = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint8_t*>(ZP_TABLE ? zt + (size_t)nt0 * ng * 16 : zt), 0, ZP_TABLE ? 2 * ng * 16 : 0, 0x00020000);
    const unsigned g_mul = kb_per_group == 1 ? 0u : (unsigned)((0x100000000ull + kb_per_group - 1) / kb_per_group);

    const int stages = K / PW_BK;  // a multiple of 4 (K % 256 == 0)
    const Unpack4Consts uc = unpack4_consts();

    // register ring: activations of four stages; packed weights of two k-blocks (4-bit: a tile spans two
    // stages) or of four stages (8-bit: one 64-input tile per stage)
    constexpr int WSLOTS = BITS == 4 ? 2 : 4;
    uint4_t a_reg[4][2];
    uint4_t w_reg[WSLOTS][2];
    half_t w_scale[WSLOTS][2];
    uint8_t w_zp[WSLOTS][2];

    auto load_a = [&](int s, int slot) {
        const unsigned oob = (unsigned)((stages - 1 - s) >> 31) & kOob;
#pragma unroll
        for (int p = 0; p < 2; ++p)
            a_reg[slot][p] = __builtin_bit_cast(
                uint4_t, __builtin_amdgcn_raw_buffer_load_b128(rx, (a_off[p] + (unsigned)s * (PW_BK * 2)) | oob, 0, 0));
    };
    // unit = k-block (4-bit) or stage (8-bit)
    auto load_w = [&](int unit, int slot) {
        const int units = BITS == 4 ? kb_total : stages;
        const unsigned oob = (unsigned)((units - 1 - unit) >> 31) & kOob;
        const unsigned kb = BITS == 4 ? (unsigned)unit : (unsigned)unit >> 1;
        const unsigned g = kb_per_group == 1 ? kb : __umulhi(kb, g_mul);
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const unsigned tile = (unsigned)i * kb_total * TPB + (unsigned)unit;
            w_reg[slot][i] = __builtin_bit_cast(
                uint4_t, __builtin_amdgcn_raw_buffer_load_b128(rw, (tile * kTileBytes + lane * 16u) | oob, 0, 0));
            const unsigned sidx = (i * ng + g) * 16u + col;
            w_scale[slot][i] =
                __builtin_bit_cast(half_t, __builtin_amdgcn_raw_buffer_load_b16(rs, (sidx * 2u) | oob, 0, 0));
            if constexpr (ZP_TABLE)
                w_zp[slot][i] = __builtin_amdgcn_raw_buffer_load_b8(rz, sidx | oob, 0, 0);
        }
    };
    // writes one stage (activations from a_reg[aslot], weights from w_reg[wslot]) to LDS ring slot `buf`;
    // `second` selects the upper 64 inputs of a 4-bit tile
    auto store_stage = [&](int buf, int aslot, int wslot, bool second) {
        half_t* Ad = As + buf * PW_A_HALVES;
        half_t* Bd = Bs + buf * PW_B_HALVES;
#pragma unroll
        for (int p = 0; p < 2; ++p)
            *reinterpret_cast<uint4_t*>(&Ad[swz(a_row0 + 64 * p, a_chunk)]) = a_reg[aslot][p];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int row = 16 * (2 * wave + i) + col;
            const half_t sh = w_scale[wslot][i];
            const half2_t sc = half2_t{sh, sh};
            const float zpv = ZP_TABLE ? (float)w_zp[wslot][i] : (float)zp_const;
            const uint4_t wv = w_reg[wslot][i];
#pragma unroll
            for (int jj = 0; jj < 2; ++jj) {
                Frag8 b;
                if constexpr (BITS == 4) {
                    unpack4_biased(second ? (jj ? wv.w : wv.z) : (jj ? wv.y : wv.x), uc, b);
                    const half2_t off_lo = splat(1024.f + zpv);
                    const half2_t off_hi = splat(64.f + zpv);
                    b.h2[0] -= off_lo;
                    b.h2[1] -= off_hi;
                    b.h2[2] -= off_lo;
                    b.h2[3] -= off_hi;
                } else {
                    unpack8(jj ? wv.z : wv.x, jj ? wv.w : wv.y, splat(1024.f + zpv), b);
                }
                if constexpr (PRESCALE) {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        b.h2[e] = b.h2[e] * sc;
                }
                *reinterpret_cast<half8_t*>(&Bd[swz(row, 4 * jj + kq)]) = b.v;
            }
        }
    };

    float16_t acc[2][4];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                acc[i][j][r] = 0.f;

    const int frow = lane & 31, fhalf = lane >> 5;
    auto mfma_stage = [&](int buf) {
        const half_t* Ac = As + buf * PW_A_HALVES;
        const half_t* Bc = Bs + buf * PW_B_HALVES;
#pragma unroll
        for (int k2 = 0; k2 < 2; ++k2) {
            const int chunk = 2 * (2 * kgrp + k2) + fhalf;
            half8_t af[2], bf[4];
#pragma unroll
            for (int i = 0; i < 2; ++i)
                af[i] = *reinterpret_cast<const half8_t*>(&Ac[swz(64 * wm + 32 * i + frow, chunk)]);
#pragma unroll
            for (int j = 0; j < 4; ++j)
                bf[j] = *reinterpret_cast<const half8_t*>(&Bc[swz(128 * wn + 32 * j + frow, chunk)]);
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], bf[j], acc[i][j], 0, 0, 0);
        }
    };

    // prologue: four stages of activations and the matching weights in flight, stage 0 in LDS
#pragma unroll
    for (int u = 0; u < 4; ++u)
        load_a(u, u);
#pragma unroll
    for (int u = 0; u < WSLOTS; ++u)
        load_w(u, u);
    store_stage(0, 0, 0, false);
    __syncthreads();

    for (int s0 = 0; s0 < stages; s0 += 4) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int s = s0 + u;
            // stage s is in LDS buffer u & 1; a_reg[u] is free (stored last iteration): refill it four ahead
            load_a(s + 4, u);
            mfma_stage(u & 1);
            // stage s + 1 -> the other buffer
            if constexpr (BITS == 4) {
                store_stage((u + 1) & 1, (u + 1) & 3, ((u + 1) >> 1) & 1, (u + 1) & 1);
                // stage s + 1 odd: the second half of its k-block's tiles is now in LDS, so the slot is free
                // for the k-block two ahead
                if (!(u & 1))
                    load_w(s0 / 2 + 2 + (u >> 1), u >> 1);
            } else {
                store_stage((u + 1) & 1, (u + 1) & 3, (u + 1) & 3, false);
                load_w(s + 4, u);
            }
            __syncthreads();
        }
    }

    // ---- group 1 hands its accumulators to group 0 through LDS: [wave & 3][tile][r][lane] ----
    float* hand = reinterpret_cast<float*>(lds_raw) + (size_t)(wave & 3) * (8 * 16 * 64);
    if (kgrp == 1) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    hand[((i * 4 + j) * 16 + r) * 64 + lane] = acc[i][j][r];
    }
    __syncthreads();
    if (kgrp == 1)
        return;

#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int n = n0 + 128 * wn + 32 * j + (lane & 31);
        const float b = bias ? (float)bias[n] : 0.f;
        // one scale per output channel: applied here, to the f32 sum of exact integer products
        const float cs = PRESCALE ? 1.f : (float)st[(size_t)(n >> 4) * ng * 16 + (n & 15)];
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = m0 + 64 * wm + 32 * i + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                const float v = (acc[i][j][r] + hand[((i * 4 + j) * 16 + r) * 64 + lane]) * cs + b;
                if (glu) {
                    // gated linear unit: the 32 channels are a gate tile (lanes & 16 == 0) and its up tile
                    const float up = __shfl_xor(v, 16, 64);
                    if (m < M && !(lane & 16))
                        store_out(y, (size_t)m * (N / 2) + (n >> 5) * 16 + (lane & 15), glu_value(glu, v, up), out_f32);
                } else if (m < M) {
                    store_out(y, (size_t)m * N + n, v, out_f32);
                }
            }
    }
}

template <int BITS, bool ZPT, bool PRE>
static int launch_wide_impl(const FcDeviceArgs& a, const LaunchPlan& p, hipStream_t s) {
    const Layout& L = a.layout;
    auto kern = fcc_prefill_wide_kernel<BITS, ZPT, PRE>;
    static bool attr_set = false;  // per instantiation; the attribute is idempotent, a race only repeats it
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)PW_LDS_BYTES);
        if (e != hipSuccess)
            return (int)e;
        attr_set = true;
    }
    hipLaunchKernelGGL(kern, dim3(p.grid[0], p.grid[1], 1), dim3(512), PW_LDS_BYTES, s, (const uint4_t*)a.w,
                       (const half_t*)a.scale, (const uint8_t*)a.zp, (const half_t*)a.x, (const half_t*)a.bias, a.y,
                       (int)a.M, (int)a.N, (int)a.K, (int)L.k_blocks, (int)L.kblocks_per_group, (int)L.groups,
                       L.zp_const, a.out_f32, L.glu);
    return (int)hipGetLastError();
}

template <int BITS, bool ZPT>
static int launch_wide_bits(const FcDeviceArgs& a, const LaunchPlan& p, hipStream_t s) {
    return a.layout.groups == 1 ? launch_wide_impl<BITS, ZPT, false>(a, p, s)
                                : launch_wide_impl<BITS, ZPT, true>(a, p, s);
}

int launch_prefill_wide(const FcDeviceArgs& a, const LaunchPlan& p, void* stream) {
    hipStream_t s = static_cast<hipStream_t>(stream);
    const Layout& L = a.layout;
    if (L.groups_per_kblock != 1)
        return (int)hipErrorInvalidValue;  // groups below 128 inputs: the planner picks another kernel
    if (L.bits == 4)
        return L.zp_table ? launch_wide_bits<4, true>(a, p, s) : launch_wide_bits<4, false>(a, p, s);
    return L.zp_table ? launch_wide_bits<8, true>(a, p, s) : launch_wide_bits<8, false>(a, p, s);
}

}  // namespace ovfcc
