// Prefill kernel (M > 32) over the tiled layout: LDS-staged dequantisation feeding f16 MFMA.
#include "device_common.h"

namespace ovfcc {

// ------------------------------------------------------------------------------------------------
// Prefill kernel.  grid = (N/128, ceil(M/128)), block = 256 (4 waves as 2 x 2, 64 x 64 each).
// K advances 64 inputs per step; the 128-input weight tile of a 4-bit k-block is loaded once and
// dequantised half per step.  LDS rows are padded to 72 halves so that 128-bit operand reads by
// 32 consecutive rows spread over all banks.
// v_mfma_f32_32x32x16_f16: A operand lane = row (lane & 31), inputs 8 (lane >> 5) ..+8;
// result: column n = lane & 31, rows 8 (r >> 2) + 4 (lane >> 5) + (r & 3), r = 0..15.
// ------------------------------------------------------------------------------------------------
constexpr int PF_BM = kPrefillTileM, PF_BN = kPrefillTileN, PF_BK = 64, PF_LD = PF_BK + 8;

template <int BITS, bool ZP_TABLE, bool PRESCALE>
__global__ __launch_bounds__(256) void fcc_prefill_kernel(const uint4_t* __restrict__ wt,
                                                          const half_t* __restrict__ st,
                                                          const uint8_t* __restrict__ zt,
                                                          const half_t* __restrict__ x,
                                                          const half_t* __restrict__ bias, void* __restrict__ y,
                                                          int M, int N, int K, int kb_total, int kb_per_group, int ng,
                                                          int zp_const, int out_f32, int glu, int gpb) {
    constexpr int TPB = BITS == 4 ? 1 : 2;
    __shared__ __attribute__((aligned(16))) half_t As[PF_BM * PF_LD];
    __shared__ __attribute__((aligned(16))) half_t Bs[PF_BN * PF_LD];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    int tile_x, tile_y;
    xcd_tile(tile_x, tile_y, 2 * PF_BM * 2, PF_BN * BITS / 4);
    const int n0 = tile_x * PF_BN;
    const int m0 = tile_y * PF_BM;
    const int nt0 = n0 / 16;
    const int col = lane & 15, kq = lane >> 4;

    // activation staging: thread covers rows (tid >> 3) + 32 p, inputs 8 (tid & 7) ..+8
    const int a_row = tid >> 3, a_k = (tid & 7) * 8;
    uint4_t a_reg[4];
    // weight staging: wave covers channel tiles 2 wave, 2 wave + 1 of the 8 in this workgroup
    uint4_t w_reg[2];
    float w_scale[2][2], w_zp[2][2];  // [tile][32-input half of the step]

    float16_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                acc[i][j][r] = 0.f;

    const int steps = K / PF_BK;

    auto load_a = [&](int step) {
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const int m = m0 + a_row + 32 * p;
            if (m < M)
                a_reg[p] = *reinterpret_cast<const uint4_t*>(x + (size_t)m * K + step * PF_BK + a_k);
            else
                a_reg[p] = uint4_t{0, 0, 0, 0};
        }
    };
    auto load_w = [&](int step) {
        const int kb = step >> 1;
        if (gpb > 1) {
            // groups of 64 or 32 inputs (4-bit weights): the step's two 32-input halves are dwords 2 h, 2 h + 1
            // of the tile, groups (2 h + jj) gpb / 4 of the k-block
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const int nt = nt0 + 2 * wave + i;
#pragma unroll
                for (int jj = 0; jj < 2; ++jj) {
                    const int gi = (2 * (step & 1) + jj) * gpb / 4;
                    const size_t idx = (((size_t)nt * kb_total + kb) * 16 + col) * gpb + gi;
                    w_scale[i][jj] = (float)st[idx];
                    w_zp[i][jj] = ZP_TABLE ? (float)zt[idx] : (float)zp_const;
                }
            }
        }
        // 4-bit: a new 128-input tile every second step; 8-bit: a new 64-input tile every step
        if (BITS == 4 && (step & 1))
            return;
        const int g = kb / kb_per_group;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int nt = nt0 + 2 * wave + i;
            const size_t tile = BITS == 4 ? ((size_t)nt * kb_total + kb) : ((size_t)nt * kb_total * 2 + step);
            w_reg[i] = wt[tile * 64 + lane];
            if (gpb == 1) {
                w_scale[i][0] = w_scale[i][1] = (float)st[((size_t)nt * ng + g) * 16 + col];
                w_zp[i][0] = w_zp[i][1] = ZP_TABLE ? (float)zt[((size_t)nt * ng + g) * 16 + col] : (float)zp_const;
            }
        }
    };
    auto store_tiles = [&](int step) {
#pragma unroll
        for (int p = 0; p < 4; ++p)
            *reinterpret_cast<uint4_t*>(&As[(a_row + 32 * p) * PF_LD + a_k]) = a_reg[p];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int row = 16 * (2 * wave + i) + col;
            const uint32_t wd[4] = {w_reg[i].x, w_reg[i].y, w_reg[i].z, w_reg[i].w};
            if constexpr (BITS == 4) {
                const bool h = step & 1;
                const uint32_t half_w[2] = {h ? wd[2] : wd[0], h ? wd[3] : wd[1]};
#pragma unroll
                for (int jj = 0; jj < 2; ++jj) {
                    const half2_t sc = splat(w_scale[i][jj]);
                    const half2_t off_lo = splat(1024.f + w_zp[i][jj]);
                    const half2_t off_hi = splat(64.f + w_zp[i][jj]);
                    Frag8 b;
                    unpack4(half_w[jj], off_lo, off_hi, b);
                    if constexpr (PRESCALE) {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            b.h2[e] = b.h2[e] * sc;
                    }
                    *reinterpret_cast<half8_t*>(&Bs[row * PF_LD + 32 * jj + 8 * kq]) = b.v;
                }
            } else {
                const half2_t sc = splat(w_scale[i][0]);
                const half2_t off = splat(1024.f + w_zp[i][0]);
#pragma unroll
                for (int jj = 0; jj < 2; ++jj) {
                    Frag8 b;
                    unpack8(wd[2 * jj], wd[2 * jj + 1], off, b);
                    if constexpr (PRESCALE) {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            b.h2[e] = b.h2[e] * sc;
                    }
                    *reinterpret_cast<half8_t*>(&Bs[row * PF_LD + 32 * jj + 8 * kq]) = b.v;
                }
            }
        }
    };

    load_a(0);
    load_w(0);
    const int frow = lane & 31, fk = (lane >> 5) * 8;
    for (int step = 0; step < steps; ++step) {
        store_tiles(step);
        __syncthreads();
        if (step + 1 < steps) {
            load_a(step + 1);
            load_w(step + 1);
        }
#pragma unroll
        for (int kk = 0; kk < PF_BK / 16; ++kk) {
            half8_t af[2], bf[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                af[i] = *reinterpret_cast<const half8_t*>(&As[(64 * wm + 32 * i + frow) * PF_LD + 16 * kk + fk]);
                bf[i] = *reinterpret_cast<const half8_t*>(&Bs[(64 * wn + 32 * i + frow) * PF_LD + 16 * kk + fk]);
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], bf[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }

    // epilogue: bias, cast, store
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int n = n0 + 64 * wn + 32 * j + (lane & 31);
        const float b = bias ? (float)bias[n] : 0.f;
        // one scale per output channel: applied here, to the f32 sum of exact integer products
        const float cs = PRESCALE ? 1.f : (float)st[(size_t)(n >> 4) * ng * 16 + (n & 15)];
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = m0 + 64 * wm + 32 * i + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                const float v = acc[i][j][r] * cs + b;
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
static void launch_prefill_impl(const FcDeviceArgs& a, const LaunchPlan& p, hipStream_t s) {
    const Layout& L = a.layout;
    hipLaunchKernelGGL((fcc_prefill_kernel<BITS, ZPT, PRE>), dim3(p.grid[0], p.grid[1], 1), dim3(256), 0, s,
                       (const uint4_t*)a.w, (const half_t*)a.scale, (const uint8_t*)a.zp, (const half_t*)a.x,
                       (const half_t*)a.bias, a.y, (int)a.M, (int)a.N, (int)a.K, (int)L.k_blocks,
                       (int)L.kblocks_per_group, (int)L.groups, L.zp_const, a.out_f32, L.glu, L.groups_per_kblock);
}

// Grouped scales are folded into the f16 weights in LDS; a single group per channel (G == K) keeps the
// weights as exact integers and scales the f32 result once.
template <int BITS, bool ZPT>
static void launch_prefill(const FcDeviceArgs& a, const LaunchPlan& p, hipStream_t s) {
    if (a.layout.groups == 1)
        launch_prefill_impl<BITS, ZPT, false>(a, p, s);
    else
        launch_prefill_impl<BITS, ZPT, true>(a, p, s);
}

int launch_prefill(const FcDeviceArgs& a, const LaunchPlan& p, void* stream) {
    hipStream_t s = static_cast<hipStream_t>(stream);
    const Layout& L = a.layout;
    if (L.groups_per_kblock != 1 && (L.bits != 4 || L.groups == 1))
        return (int)hipErrorInvalidValue;
    if (L.bits == 4)
        L.zp_table ? launch_prefill<4, true>(a, p, s) : launch_prefill<4, false>(a, p, s);
    else
        L.zp_table ? launch_prefill<8, true>(a, p, s) : launch_prefill<8, false>(a, p, s);
    return (int)hipGetLastError();
}

}  // namespace ovfcc
