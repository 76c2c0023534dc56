// HIP kernels for FullyConnectedCompressed on gfx950 (CDNA4, wave64).
//
//   Y[m,n] = sum_k X[m,k] * ((W[n,k] - ZP[n,k/G]) * S[n,k/G]) (+ bias[n])
//
// Semantics follow the scalar reference kernel of the OpenVINO Intel-GPU plugin
// (src/plugins/intel_gpu/src/kernel_selector/cl_kernels/fully_connected_gpu_bfyx_ref.cl:88-160);
// none of the code below derives from that plugin's OpenCL kernels.
//
// Three kernel families:
//   fcc_plain_kernel    any shape, OpenVINO constant layout, one wave per (n, m)
//   fcc_decode_kernel   M <= 32, tiled layout: every wave streams 1 KiB weight tiles with one
//                       128-bit load per lane, unpacks nibbles in registers to exact (q - zp)
//                       halves and contracts them on the matrix cores against the activation
//                       rows; the group scale multiplies the f32 group partial sum.  K is split
//                       over the four waves of a workgroup (LDS reduction) and over workgroups
//                       (partials + arrival counter; the last workgroup sums in fixed order).
//   fcc_prefill_kernel  M > 32, tiled layout: 128x128 output tile per workgroup; weight tiles
//                       are dequantised to f16 into LDS ((q - zp) * s for grouped scales, exact
//                       q - zp with the scale applied to the f32 result for per-channel scales),
//                       activations staged in LDS, v_mfma_f32_32x32x16_f16 with f32 accumulators.
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

// Output cast: FullyConnected's output_type is f16 (default, the activation type) or f32.
__device__ __forceinline__ void store_out(void* y, size_t i, float v, int out_f32) {
    if (out_f32)
        static_cast<float*>(y)[i] = v;
    else
        static_cast<half_t*>(y)[i] = (half_t)v;
}

__device__ __forceinline__ half2_t splat(float v) {
    const half_t h = (half_t)v;
    return half2_t{h, h};
}

// ------------------------------------------------------------------------------------------------
// Plain kernel: OpenVINO layout, any N/K/G.  One wave per (n, m); lanes stride over k.
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(64) void fcc_plain_kernel(const uint8_t* __restrict__ w, const half_t* __restrict__ s,
                                                       const uint8_t* __restrict__ zp,
                                                       const half_t* __restrict__ bias,
                                                       const half_t* __restrict__ x, void* __restrict__ y, int M,
                                                       int N, int K, int G, int w_type, int zp_type, int zp_scalar,
                                                       int out_f32) {
    const int n = blockIdx.x;
    const int m = blockIdx.y;
    const int lane = threadIdx.x;
    const int ng = K / G;
    float acc = 0.f;
    for (int k = lane; k < K; k += 64) {
        const size_t wi = (size_t)n * K + k;
        float q;
        if (w_type == OVFCC_U4 || w_type == OVFCC_I4) {
            const unsigned b = w[wi >> 1];
            int v = (wi & 1) ? (b >> 4) : (b & 0xF);
            if (w_type == OVFCC_I4 && v >= 8)
                v -= 16;
            q = (float)v;
        } else if (w_type == OVFCC_U8) {
            q = (float)w[wi];
        } else {
            q = (float)(int8_t)w[wi];
        }
        const int g = k / G;
        float z = 0.f;
        if (zp_type != OVFCC_NONE) {
            const size_t zi = zp_scalar ? 0 : (size_t)n * ng + g;
            if (zp_type == OVFCC_U4) {
                const unsigned b = zp[zi >> 1];
                z = (float)((zi & 1) ? (b >> 4) : (b & 0xF));
            } else {
                z = (float)zp[zi];
            }
        }
        const float sc = (float)s[(size_t)n * ng + g];
        acc += (float)x[(size_t)m * K + k] * ((q - z) * sc);
    }
    for (int off = 32; off > 0; off >>= 1)
        acc += __shfl_down(acc, off, 64);
    if (lane == 0) {
        if (bias)
            acc += (float)bias[n];
        store_out(y, (size_t)m * N + n, acc, out_f32);
    }
}

// ------------------------------------------------------------------------------------------------
// Decode kernel (M <= 16*MT).  grid = (N/16, split_k), block = 256 (4 waves).
// Workgroup (nt, ks) owns output channels [16 nt, 16 nt + 16) and k-blocks
// [ks * kb_per_split, min(KB, (ks+1) * kb_per_split)); wave w takes every fourth k-block.
// MFMA roles: A = activations (rows m), B = weights (columns n); a lane's B operand for k-step j
// is dword j of its 128-bit load, a lane's A operand is X[m][128 kb + 32 j + 8 (lane >> 4) ..+8].
// Result layout of v_mfma_f32_16x16x32_f16: lane holds column n = lane & 15, rows 4 (lane >> 4) + r.
// ------------------------------------------------------------------------------------------------
template <int BITS, int MT, bool ZP_TABLE>
__global__ __launch_bounds__(256) void fcc_decode_kernel(const uint4_t* __restrict__ wt,
                                                         const half_t* __restrict__ st,
                                                         const uint8_t* __restrict__ zt,
                                                         const half_t* __restrict__ x,
                                                         const half_t* __restrict__ bias, void* __restrict__ y,
                                                         float* __restrict__ ws, unsigned* __restrict__ counters,
                                                         int M, int N, int K, int kb_total, int kb_per_group,
                                                         int ng, int zp_const, int kb_per_split, int split_k,
                                                         int out_f32) {
    constexpr int TPB = BITS == 4 ? 1 : 2;  // tiles per k-block
    const int nt = blockIdx.x;
    const int ks = blockIdx.y;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int col = lane & 15;
    const int kq = lane >> 4;

    const int kb_begin = ks * kb_per_split;
    const int kb_end = min(kb_total, kb_begin + kb_per_split);

    float4_t acc[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t)
        acc[t] = float4_t{0.f, 0.f, 0.f, 0.f};

    const uint4_t* wrow = wt + (size_t)nt * kb_total * TPB * 64 + lane;
    const half_t* srow = st + (size_t)nt * ng * 16 + col;
    const uint8_t* zrow = ZP_TABLE ? zt + (size_t)nt * ng * 16 + col : nullptr;
    // activation row pointers of this lane (row m = col, and col + 16 for the second M tile)
    const half_t* xrow[MT];
    bool xvalid[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        const int m = col + 16 * t;
        xvalid[t] = m < M;
        xrow[t] = x + (size_t)(xvalid[t] ? m : 0) * K + 8 * kq;
    }

    for (int kb = kb_begin + wave; kb < kb_end; kb += 4) {
        uint4_t wv[TPB];
#pragma unroll
        for (int i = 0; i < TPB; ++i)
            wv[i] = __builtin_nontemporal_load(wrow + (size_t)(kb * TPB + i) * 64);
        const int g = kb / kb_per_group;
        const float scale = (float)srow[g * 16];
        const float zpv = ZP_TABLE ? (float)zrow[g * 16] : (float)zp_const;

        Frag8 a[MT][4];
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (xvalid[t])
                    a[t][j].v = *reinterpret_cast<const half8_t*>(xrow[t] + (size_t)kb * 128 + 32 * j);
                else
                    a[t][j].v = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
            }

        float4_t part[MT];
#pragma unroll
        for (int t = 0; t < MT; ++t)
            part[t] = float4_t{0.f, 0.f, 0.f, 0.f};

        if constexpr (BITS == 4) {
            const half2_t off_lo = splat(1024.f + zpv);
            const half2_t off_hi = splat(64.f + zpv);
            const uint32_t wd[4] = {wv[0].x, wv[0].y, wv[0].z, wv[0].w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                Frag8 b;
                unpack4(wd[j], off_lo, off_hi, b);
#pragma unroll
                for (int t = 0; t < MT; ++t)
                    part[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[t][j].v, b.v, part[t], 0, 0, 0);
            }
        } else {
            const half2_t off = splat(1024.f + zpv);
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const uint32_t wd[4] = {wv[i].x, wv[i].y, wv[i].z, wv[i].w};
#pragma unroll
                for (int jj = 0; jj < 2; ++jj) {
                    Frag8 b;
                    unpack8(wd[2 * jj], wd[2 * jj + 1], off, b);
#pragma unroll
                    for (int t = 0; t < MT; ++t)
                        part[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[t][2 * i + jj].v, b.v, part[t], 0, 0, 0);
                }
            }
        }
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            acc[t].x += scale * part[t].x;
            acc[t].y += scale * part[t].y;
            acc[t].z += scale * part[t].z;
            acc[t].w += scale * part[t].w;
        }
    }

    // ---- reduce the four waves through LDS (fixed order) ----
    __shared__ float red[4][MT][64][4];
    __shared__ unsigned ticket_s;
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        red[wave][t][lane][0] = acc[t].x;
        red[wave][t][lane][1] = acc[t].y;
        red[wave][t][lane][2] = acc[t].z;
        red[wave][t][lane][3] = acc[t].w;
    }
    __syncthreads();
    if (wave != 0 && split_k == 1)
        return;

    float sum[MT][4];
    if (wave == 0) {
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r)
                sum[t][r] = ((red[0][t][lane][r] + red[1][t][lane][r]) + red[2][t][lane][r]) + red[3][t][lane][r];
    }

    if (split_k > 1) {
        // partial layout: [nt][ks][MT][4 r][64 lanes] floats
        float* mine = ws + ((size_t)nt * split_k + ks) * (MT * 256);
        if (wave == 0) {
#pragma unroll
            for (int t = 0; t < MT; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if (4 * kq + r + 16 * t < M)
                        __hip_atomic_store(mine + (t * 4 + r) * 64 + lane, sum[t][r], __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_AGENT);
            __threadfence();
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            const unsigned prev = __hip_atomic_fetch_add(counters + nt, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
            ticket_s = prev;
        }
        __syncthreads();
        if (ticket_s != (unsigned)(split_k - 1) || wave != 0)
            return;
        __threadfence();
        // last arrival: sum all partials in split order, independent of arrival order
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r)
                sum[t][r] = 0.f;
        for (int s = 0; s < split_k; ++s) {
            const float* p = ws + ((size_t)nt * split_k + s) * (MT * 256);
#pragma unroll
            for (int t = 0; t < MT; ++t)
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if (4 * kq + r + 16 * t < M)
                        sum[t][r] += __hip_atomic_load(p + (t * 4 + r) * 64 + lane, __ATOMIC_RELAXED,
                                                       __HIP_MEMORY_SCOPE_AGENT);
        }
        if (lane == 0)
            __hip_atomic_store(counters + nt, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }

    const int n = nt * 16 + col;
    const float b = bias ? (float)bias[n] : 0.f;
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int m = 4 * kq + r + 16 * t;
            if (m < M)
                store_out(y, (size_t)m * N + n, sum[t][r] + b, out_f32);
        }
}

// ------------------------------------------------------------------------------------------------
// Prefill kernel.  grid = (N/128, ceil(M/128)), block = 256 (4 waves as 2 x 2, 64 x 64 each).
// K advances 64 inputs per step; the 128-input weight tile of a 4-bit k-block is loaded once and
// dequantised half per step.  LDS rows are padded to 72 halves so that 128-bit operand reads by
// 32 consecutive rows spread over all banks.
// v_mfma_f32_32x32x16_f16: A operand lane = row (lane & 31), inputs 8 (lane >> 5) ..+8;
// result: column n = lane & 31, rows 8 (r >> 2) + 4 (lane >> 5) + (r & 3), r = 0..15.
// ------------------------------------------------------------------------------------------------
constexpr int PF_BM = 128, PF_BN = 128, PF_BK = 64, PF_LD = PF_BK + 8;

template <int BITS, bool ZP_TABLE, bool PRESCALE>
__global__ __launch_bounds__(256) void fcc_prefill_kernel(const uint4_t* __restrict__ wt,
                                                          const half_t* __restrict__ st,
                                                          const uint8_t* __restrict__ zt,
                                                          const half_t* __restrict__ x,
                                                          const half_t* __restrict__ bias, void* __restrict__ y,
                                                          int M, int N, int K, int kb_total, int kb_per_group, int ng,
                                                          int zp_const, int out_f32) {
    constexpr int TPB = BITS == 4 ? 1 : 2;
    __shared__ __attribute__((aligned(16))) half_t As[PF_BM * PF_LD];
    __shared__ __attribute__((aligned(16))) half_t Bs[PF_BN * PF_LD];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int n0 = blockIdx.x * PF_BN;
    const int m0 = blockIdx.y * PF_BM;
    const int nt0 = n0 / 16;
    const int col = lane & 15, kq = lane >> 4;

    // activation staging: thread covers rows (tid >> 3) + 32 p, inputs 8 (tid & 7) ..+8
    const int a_row = tid >> 3, a_k = (tid & 7) * 8;
    uint4_t a_reg[4];
    // weight staging: wave covers channel tiles 2 wave, 2 wave + 1 of the 8 in this workgroup
    uint4_t w_reg[2];
    float w_scale[2], w_zp[2];

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
        // 4-bit: a new 128-input tile every second step; 8-bit: a new 64-input tile every step
        if (BITS == 4 && (step & 1))
            return;
        const int kb = step >> 1;
        const int g = kb / kb_per_group;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int nt = nt0 + 2 * wave + i;
            const size_t tile = BITS == 4 ? ((size_t)nt * kb_total + kb) : ((size_t)nt * kb_total * 2 + step);
            w_reg[i] = wt[tile * 64 + lane];
            w_scale[i] = (float)st[((size_t)nt * ng + g) * 16 + col];
            w_zp[i] = ZP_TABLE ? (float)zt[((size_t)nt * ng + g) * 16 + col] : (float)zp_const;
        }
    };
    auto store_tiles = [&](int step) {
#pragma unroll
        for (int p = 0; p < 4; ++p)
            *reinterpret_cast<uint4_t*>(&As[(a_row + 32 * p) * PF_LD + a_k]) = a_reg[p];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int row = 16 * (2 * wave + i) + col;
            const half2_t sc = splat(w_scale[i]);
            const uint32_t wd[4] = {w_reg[i].x, w_reg[i].y, w_reg[i].z, w_reg[i].w};
            if constexpr (BITS == 4) {
                const half2_t off_lo = splat(1024.f + w_zp[i]);
                const half2_t off_hi = splat(64.f + w_zp[i]);
                const bool h = step & 1;
                const uint32_t half_w[2] = {h ? wd[2] : wd[0], h ? wd[3] : wd[1]};
#pragma unroll
                for (int jj = 0; jj < 2; ++jj) {
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
                const half2_t off = splat(1024.f + w_zp[i]);
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
                if (m < M)
                    store_out(y, (size_t)m * N + n, acc[i][j][r] * cs + b, out_f32);
            }
    }
}

// ------------------------------------------------------------------------------------------------
// Plain 128-bit copy, the yardstick for bandwidth figures and counter scaling.
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void fcc_copy_kernel(uint4_t* __restrict__ dst, const uint4_t* __restrict__ src,
                                                       size_t n16) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n16; i += stride)
        dst[i] = __builtin_nontemporal_load(src + i);
}

// ------------------------------------------------------------------------------------------------
// Host side: planning and launching
// ------------------------------------------------------------------------------------------------
int plan_launch(const FcDeviceArgs& a, int force_kernel, int force_split, int n_cus, LaunchPlan* plan) {
    LaunchPlan p;
    const Layout& L = a.layout;
    int kernel = force_kernel;
    if (kernel == OVFCC_KERNEL_AUTO)
        kernel = !L.tiled ? OVFCC_KERNEL_PLAIN : (a.M <= 32 ? OVFCC_KERNEL_DECODE : OVFCC_KERNEL_PREFILL);
    if (kernel != OVFCC_KERNEL_PLAIN && !L.tiled)
        return fail(OVFCC_EUNSUPPORTED, "this node keeps the OpenVINO layout; only the plain kernel can run it");
    if (kernel == OVFCC_KERNEL_PLAIN && L.tiled)
        return fail(OVFCC_EUNSUPPORTED, "this node was repacked into tiles; the plain kernel needs the OpenVINO layout");
    if (kernel == OVFCC_KERNEL_DECODE && a.M > 32)
        return fail(OVFCC_EUNSUPPORTED, "the decode kernel handles at most 32 rows");
    if (kernel == OVFCC_KERNEL_PREFILL && (a.N % PF_BN) != 0)
        kernel = OVFCC_KERNEL_AUTO;  // resolved below
    p.kernel = kernel;
    if (kernel == OVFCC_KERNEL_PLAIN) {
        if (a.M > 65535)
            return fail(OVFCC_EUNSUPPORTED, "the plain kernel handles at most 65535 rows");
        p.grid[0] = (unsigned)a.N;
        p.grid[1] = (unsigned)a.M;
        p.block = 64;
        p.name = "fcc_plain";
    } else if (kernel == OVFCC_KERNEL_DECODE) {
        const int kb = (int)L.k_blocks;
        int split = force_split;
        if (split <= 0) {
            // aim for about four workgroups per compute unit, at least one k-block per wave
            const int64_t want = (int64_t)4 * n_cus;
            split = (int)((want + L.n_tiles - 1) / L.n_tiles);
            const int max_split = kb >= 4 ? kb / 4 : 1;
            if (split > max_split)
                split = max_split;
            if (split < 1)
                split = 1;
        }
        if (split > kb)
            split = kb;
        int per = (kb + split - 1) / split;
        split = (kb + per - 1) / per;  // no empty splits
        p.split_k = split;
        p.kblocks_per_split = per;
        p.grid[0] = (unsigned)L.n_tiles;
        p.grid[1] = (unsigned)split;
        p.block = 256;
        p.tile_m = a.M <= 16 ? 16 : 32;
        p.tile_n = 16;
        const int mt = a.M <= 16 ? 1 : 2;
        p.workspace_bytes = split > 1 ? (size_t)L.n_tiles * split * mt * 256 * sizeof(float) : 0;
        p.counter_count = split > 1 ? (size_t)L.n_tiles : 0;
        p.name = L.bits == 4 ? "fcc_decode_w4" : "fcc_decode_w8";
    } else if (kernel == OVFCC_KERNEL_PREFILL) {
        p.grid[0] = (unsigned)(a.N / PF_BN);
        p.grid[1] = (unsigned)((a.M + PF_BM - 1) / PF_BM);
        p.block = 256;
        p.tile_m = PF_BM;
        p.tile_n = PF_BN;
        p.name = L.bits == 4 ? "fcc_prefill_w4" : "fcc_prefill_w8";
    } else {
        return fail(OVFCC_EUNSUPPORTED, "no tiled kernel covers this shape (prefill needs N % 128 == 0)");
    }
    *plan = p;
    return OVFCC_OK;
}

template <int BITS, int MT, bool ZPT>
static void launch_decode(const FcDeviceArgs& a, const LaunchPlan& p, hipStream_t s) {
    const Layout& L = a.layout;
    hipLaunchKernelGGL((fcc_decode_kernel<BITS, MT, ZPT>), dim3(p.grid[0], p.grid[1], 1), dim3(256), 0, s,
                       (const uint4_t*)a.w, (const half_t*)a.scale, (const uint8_t*)a.zp, (const half_t*)a.x,
                       (const half_t*)a.bias, a.y, a.workspace, a.counters, (int)a.M, (int)a.N, (int)a.K,
                       (int)L.k_blocks, (int)L.kblocks_per_group, (int)L.groups, L.zp_const, p.kblocks_per_split,
                       p.split_k, a.out_f32);
}

template <int BITS, bool ZPT, bool PRE>
static void launch_prefill_impl(const FcDeviceArgs& a, const LaunchPlan& p, hipStream_t s) {
    const Layout& L = a.layout;
    hipLaunchKernelGGL((fcc_prefill_kernel<BITS, ZPT, PRE>), dim3(p.grid[0], p.grid[1], 1), dim3(256), 0, s,
                       (const uint4_t*)a.w, (const half_t*)a.scale, (const uint8_t*)a.zp, (const half_t*)a.x,
                       (const half_t*)a.bias, a.y, (int)a.M, (int)a.N, (int)a.K, (int)L.k_blocks,
                       (int)L.kblocks_per_group, (int)L.groups, L.zp_const, a.out_f32);
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

int launch_fc(const FcDeviceArgs& a, const LaunchPlan& p, void* stream) {
    hipStream_t s = static_cast<hipStream_t>(stream);
    const Layout& L = a.layout;
    if (a.M == 0)
        return 0;
    if (p.kernel == OVFCC_KERNEL_PLAIN) {
        hipLaunchKernelGGL(fcc_plain_kernel, dim3(p.grid[0], p.grid[1], 1), dim3(64), 0, s, (const uint8_t*)a.w,
                           (const half_t*)a.scale, (const uint8_t*)a.zp, (const half_t*)a.bias, (const half_t*)a.x,
                           a.y, (int)a.M, (int)a.N, (int)a.K, (int)a.group_size, a.w_type, a.zp_type,
                           a.zp_scalar, a.out_f32);
    } else if (p.kernel == OVFCC_KERNEL_DECODE) {
        const bool two = a.M > 16;
        if (L.bits == 4) {
            if (L.zp_table)
                two ? launch_decode<4, 2, true>(a, p, s) : launch_decode<4, 1, true>(a, p, s);
            else
                two ? launch_decode<4, 2, false>(a, p, s) : launch_decode<4, 1, false>(a, p, s);
        } else {
            if (L.zp_table)
                two ? launch_decode<8, 2, true>(a, p, s) : launch_decode<8, 1, true>(a, p, s);
            else
                two ? launch_decode<8, 2, false>(a, p, s) : launch_decode<8, 1, false>(a, p, s);
        }
    } else {
        if (L.bits == 4)
            L.zp_table ? launch_prefill<4, true>(a, p, s) : launch_prefill<4, false>(a, p, s);
        else
            L.zp_table ? launch_prefill<8, true>(a, p, s) : launch_prefill<8, false>(a, p, s);
    }
    return (int)hipGetLastError();
}

int launch_copy(void* dst, const void* src, size_t bytes, void* stream) {
    const size_t n16 = bytes / 16;
    hipLaunchKernelGGL(fcc_copy_kernel, dim3(256 * 8), dim3(256), 0, static_cast<hipStream_t>(stream), (uint4_t*)dst,
                       (const uint4_t*)src, n16);
    return (int)hipGetLastError();
}

}  // namespace ovfcc
