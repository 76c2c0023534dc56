// Prefill kernel for 8-bit per-channel weights over dynamically quantised activations (W8A8), and the kernel that
// quantises the activations.  What the OpenVINO Intel-GPU plugin does for large batches with its DynamicQuantize
// primitive (src/plugins/intel_gpu/src/kernel_selector/cl_kernels/dynamic_quantize_gpu_ref.cl:100-250) and the
// integer path of its FullyConnected (cl_kernels/fully_connected_gpu_bf_tiled.cl:1257-1291): activations become
// int8 with one scale per row, the contraction runs on the integer matrix cores (v_mfma_i32_16x16x64_i8, twice
// the f16 rate and no weight unpack at all), and the result is
//     y[m, n] = (sum_k q[m, k] w[n, k] - zp[n] sum_k q[m, k]) * (s[n] * inv_scale[m]) + bias[n].
//
// Quantisation (fcc_dynquant_kernel, one workgroup per row): max |x| clamped below at 0.003, scale = 127 / max
// rounded to half, q = rte(half(x * scale)), inv_scale = half(1 / scale), qsum = sum q.  q is written with the 64
// inputs of every weight tile permuted into the order the tile's lanes hold them (byte p of lane group kq is input
// 32 (p >> 3) + 8 kq + (p & 7)), so that activations and weights enter the MFMA as 16 verbatim bytes per lane.
//
// The asymmetric form (fcc_dynquant_asym_kernel; the reference's QuantizationType::Asymmetric with unsigned 8-bit
// output, same file, ASYMMETRIC_QUANTIZATION and UNSIGNED_OUTPUT): d = max - min in half (0.003 if equal), scale =
// half(255 / d), zp = half(-min (255 / d)), q = sat_u8(rte(half(x scale) + zp)), za = sat_u8(rte(zp)).  The main
// kernel's operands are signed bytes, so q - 128 is stored and za - 128 kept per row; with cw[n] = sum_k (w[n, k] -
// zp[n]) per channel (fcc_i8_colsum_kernel, once per node)
//     y[m, n] = (sum_k q' w' - zp' sum_k q' - za' cw[n]) * (s[n] * inv_scale[m]) + bias[n]
// is sum_k (q - za)(w - zp) exactly (primes: minus 128).
//
// Main kernel: 128 x 256 output tile, 8 waves, grid = (N / 256, ceil(M / 128)) in XCD-aware order.  wn = wave & 3
// owns 64 channels, kg = wave >> 2 the first or second 64-input tile of every 128-input k-block.  The int8
// activation tile (128 rows x 128 bytes) travels to LDS by direct-to-LDS loads two k-blocks ahead (three 16 KiB
// stages; the 16-byte chunks of row r sit at chunk ^ ((r >> 1) & 7), conflict-free for 128-bit reads of 16 rows);
// the wave's four weight tiles come straight from memory into a two-slot register ring and are only XORed with
// 0x80 (stored unsigned -> signed operand; the zero-point is shifted to match).  k-group 1 hands its i32
// accumulators over through LDS; all integer arithmetic is exact.
#include "device_common.h"

namespace ovfcc {

typedef int int4_t __attribute__((ext_vector_type(4)));

constexpr int PI_BM = 128, PI_BN = 256, PI_BK = 128;
constexpr int PI_STAGES = 3;
constexpr int PI_XQ = 3;                      // activation operands in registers
constexpr int PI_A_BYTES = PI_BM * PI_BK;     // 16 KiB per stage
constexpr unsigned PI_LDS_BYTES = 64 * 1024;  // three stages need 48 KiB, the hand-over at the end 64 KiB

// ------------------------------------------------------------------------------------------------
// Per-row quantisation.  grid = M, block = 256; K % 128 == 0.
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void fcc_dynquant_kernel(const half_t* __restrict__ x, int8_t* __restrict__ xq,
                                                           float* __restrict__ inv_scale, int* __restrict__ qsum,
                                                           int K) {
    __shared__ float red_f[4];
    __shared__ int red_i[4];
    const int row = blockIdx.x;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const half_t* xr = x + (size_t)row * K;
    // pass 1: largest magnitude (exact in half)
    float mx = 0.f;
    for (int c = tid; c < K / 8; c += 256) {
        const half8_t v = *reinterpret_cast<const half8_t*>(xr + c * 8);
#pragma unroll
        for (int j = 0; j < 8; ++j)
            mx = fmaxf(mx, fabsf((float)v[j]));
    }
    for (int off = 32; off > 0; off >>= 1)
        mx = fmaxf(mx, __shfl_xor(mx, off, 64));
    if (lane == 0)
        red_f[wave] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(red_f[0], red_f[1]), fmaxf(red_f[2], red_f[3]));
    mx = fmaxf(mx, (float)(half_t)0.003f);
    const half_t scale = (half_t)(127.f / mx);  // one f32 division rounded to half = the half division
    // pass 2: 16 bytes (one lane group's share of a 64-input tile) per thread and step
    int sum = 0;
    for (int ch = tid; ch < K / 16; ch += 256) {
        const int tile = ch >> 2, kq = ch & 3;  // 64-input tile, lane group
        uint32_t packed[4];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const half8_t v = *reinterpret_cast<const half8_t*>(xr + tile * 64 + 32 * h + 8 * kq);
#pragma unroll
            for (int d = 0; d < 2; ++d) {
                uint32_t wrd = 0;
#pragma unroll
                for (int b = 0; b < 4; ++b) {
                    const half_t p = v[4 * d + b] * scale;  // half product, as the reference rounds it
                    int q = (int)__builtin_rintf((float)p);
                    q = q > 127 ? 127 : (q < -128 ? -128 : q);
                    sum += q;
                    wrd |= (uint32_t)(q & 0xFF) << (8 * b);
                }
                packed[2 * h + d] = wrd;
            }
        }
        *reinterpret_cast<uint4_t*>(xq + (size_t)row * K + (size_t)ch * 16) =
            uint4_t{packed[0], packed[1], packed[2], packed[3]};
    }
    for (int off = 32; off > 0; off >>= 1)
        sum += __shfl_xor(sum, off, 64);
    if (lane == 0)
        red_i[wave] = sum;
    __syncthreads();
    if (tid == 0) {
        inv_scale[row] = (float)(half_t)(1.f / (float)scale);
        qsum[row] = red_i[0] + red_i[1] + red_i[2] + red_i[3];
    }
}

// ------------------------------------------------------------------------------------------------
// Per-row asymmetric quantisation.  grid = M, block = 256; K % 128 == 0.  xq holds q - 128 (the signed operand
// of the integer kernel), qsum their sum, za the row's zero-point minus 128.
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void fcc_dynquant_asym_kernel(const half_t* __restrict__ x, int8_t* __restrict__ xq,
                                                                float* __restrict__ inv_scale, int* __restrict__ qsum,
                                                                int* __restrict__ za, int K) {
    __shared__ float red_mx[4], red_mn[4];
    __shared__ int red_i[4];
    const int row = blockIdx.x;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const half_t* xr = x + (size_t)row * K;
    // pass 1: largest and smallest value (exact in half)
    float mx = -65504.f, mn = 65504.f;  // the reference starts from the type's lowest and largest finite values
    for (int c = tid; c < K / 8; c += 256) {
        const half8_t v = *reinterpret_cast<const half8_t*>(xr + c * 8);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            mx = fmaxf(mx, (float)v[j]);
            mn = fminf(mn, (float)v[j]);
        }
    }
    for (int off = 32; off > 0; off >>= 1) {
        mx = fmaxf(mx, __shfl_xor(mx, off, 64));
        mn = fminf(mn, __shfl_xor(mn, off, 64));
    }
    if (lane == 0)
        red_mx[wave] = mx, red_mn[wave] = mn;
    __syncthreads();
    mx = fmaxf(fmaxf(red_mx[0], red_mx[1]), fmaxf(red_mx[2], red_mx[3]));
    mn = fminf(fminf(red_mn[0], red_mn[1]), fminf(red_mn[2], red_mn[3]));
    const half_t mxh = (half_t)mx, mnh = (half_t)mn;
    const half_t range = mxh - mnh;  // half subtraction, as the reference's
    const float diff = mxh == mnh ? (float)(half_t)0.003f : (float)range;
    const float scale_f = 255.f / diff;
    const half_t scale = (half_t)scale_f;
    const half_t zp = (half_t)(-(float)mnh * scale_f);
    auto to_u8 = [](half_t v) {  // round to nearest even, saturate; NaN -> 0
        return (int)fminf(fmaxf(__builtin_rintf((float)v), 0.f), 255.f);
    };
    // pass 2: 16 bytes (one lane group's share of a 64-input tile) per thread and step
    int sum = 0;
    for (int ch = tid; ch < K / 16; ch += 256) {
        const int tile = ch >> 2, kq = ch & 3;
        uint32_t packed[4];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const half8_t v = *reinterpret_cast<const half8_t*>(xr + tile * 64 + 32 * h + 8 * kq);
#pragma unroll
            for (int d = 0; d < 2; ++d) {
                uint32_t wrd = 0;
#pragma unroll
                for (int b = 0; b < 4; ++b) {
                    half_t p = v[4 * d + b] * scale;  // half product, then half sum, as the reference rounds them
                    asm volatile("" : "+v"(p));       // (two roundings: keep the compiler from fusing them)
                    p = p + zp;
                    const int q = to_u8(p) - 128;
                    sum += q;
                    wrd |= (uint32_t)(q & 0xFF) << (8 * b);
                }
                packed[2 * h + d] = wrd;
            }
        }
        *reinterpret_cast<uint4_t*>(xq + (size_t)row * K + (size_t)ch * 16) =
            uint4_t{packed[0], packed[1], packed[2], packed[3]};
    }
    for (int off = 32; off > 0; off >>= 1)
        sum += __shfl_xor(sum, off, 64);
    if (lane == 0)
        red_i[wave] = sum;
    __syncthreads();
    if (tid == 0) {
        inv_scale[row] = (float)(half_t)(1.f / (float)scale);
        qsum[row] = red_i[0] + red_i[1] + red_i[2] + red_i[3];
        za[row] = to_u8(zp) - 128;
    }
}

// ------------------------------------------------------------------------------------------------
// cw[n] = sum_k (w[n, k] - zp[n]) over tiled 8-bit weights (stored unsigned, zero-point raised to match), channels
// in tiled order.  grid = N / 16, block = 256: wave w sums the 64-input tiles w, w + 4, ... of the channel tile.
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void fcc_i8_colsum_kernel(const uint4_t* __restrict__ wt,
                                                            const uint8_t* __restrict__ zt, int zp_const,
                                                            int* __restrict__ cw, int kb_total) {
    __shared__ unsigned red[4][16];
    const int nt = blockIdx.x;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint4_t* base = wt + (size_t)nt * kb_total * 2 * 64;
    unsigned sum = 0;
    for (int j = wave; j < kb_total * 2; j += 4) {
        const uint4_t v = base[(size_t)j * 64 + lane];
        sum = __builtin_amdgcn_sad_u8(v.x, 0u, sum);
        sum = __builtin_amdgcn_sad_u8(v.y, 0u, sum);
        sum = __builtin_amdgcn_sad_u8(v.z, 0u, sum);
        sum = __builtin_amdgcn_sad_u8(v.w, 0u, sum);
    }
    sum += __shfl_xor(sum, 16, 64);  // the four lane groups hold the four quarters of a tile's inputs
    sum += __shfl_xor(sum, 32, 64);
    if (lane < 16)
        red[wave][lane] = sum;
    __syncthreads();
    if (tid < 16) {
        const unsigned total = red[0][tid] + red[1][tid] + red[2][tid] + red[3][tid];
        const int zp = zt ? (int)zt[nt * 16 + tid] : zp_const;
        cw[nt * 16 + tid] = (int)total - kb_total * 128 * zp;
    }
}

// ------------------------------------------------------------------------------------------------
// Integer FullyConnected.
// ------------------------------------------------------------------------------------------------
template <bool ZP_TABLE>
__global__ __launch_bounds__(512) void fcc_prefill_i8_kernel(const uint4_t* __restrict__ wt, const half_t* __restrict__ st,
                                                             const uint8_t* __restrict__ zt,
                                                             const int8_t* __restrict__ xq,
                                                             const float* __restrict__ inv_scale,
                                                             const int* __restrict__ qsum,
                                                             const int* __restrict__ za, const int* __restrict__ cw,
                                                             const half_t* __restrict__ bias, void* __restrict__ y,
                                                             int M, int N, int K, int kb_total, int zp_const,
                                                             int out_f32, int glu) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    const lds_byte_ptr lds3 = (lds_byte_ptr)lds_raw;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wn = wave & 3, kg = wave >> 2;
    int tile_x, tile_y;
    xcd_tile(tile_x, tile_y, PI_BM, PI_BN);
    const int n0 = tile_x * PI_BN;
    const int m0 = tile_y * PI_BM;
    const int col = lane & 15, kq = lane >> 4;

    constexpr unsigned kOob = 0x80000000u;
    constexpr int kRsrcFlags = 0x00020000;
    // Every offset goes through the vector operand: the scalar offset of a buffer load is not range-checked.
    const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(xq), 0, M * K, kRsrcFlags);
    const int nt0 = n0 / 16 + 4 * wn;  // the wave's four channel tiles
    const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint4_t*>(wt + (size_t)nt0 * kb_total * 2 * 64), 0, 4 * kb_total * 2 * kTileBytes, kRsrcFlags);

    // ---- activations: direct-to-LDS load i (0, 1) of the wave covers rows 64 i + 8 wave .. + 7; lane -> row
    // lane >> 3 of those, LDS chunk slot lane & 7, which holds global chunk (lane & 7) ^ ((row >> 1) & 7) with
    // (row >> 1) & 7 = 4 (wave & 1) + (lane >> 4).  Rows >= M lie beyond the descriptor's range: zeros. ----
    const unsigned a_row0 = (unsigned)((m0 + 8 * wave + (lane >> 3)) * K);
    const unsigned a_chunk = (unsigned)(((lane & 7) ^ (4 * (wave & 1) + (lane >> 4))) << 4);
    auto dma_a = [&](int kb, int i) {
        const unsigned oob = (unsigned)((kb_total - 1 - kb) >> 31) & kOob;
        const int stage = kb % PI_STAGES;
        const unsigned sterm = __builtin_amdgcn_readfirstlane((unsigned)(64 * i * K + kb * PI_BK));
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, (lds_void_ptr)(lds3 + stage * PI_A_BYTES + i * 8192 + wave * 1024), 16,
                                                 (a_row0 + sterm + a_chunk) | oob, 0, 0, 0);
    };
    // ---- weights: two-slot register ring, 16 bytes per lane and channel tile (the wave's 64-input tile kg) ----
    uint4_t raw[2][4];
    auto load_w = [&](int kb, int slot, int r) {
        const unsigned oob = (unsigned)((kb_total - 1 - kb) >> 31) & kOob;
        const unsigned sofs = __builtin_amdgcn_readfirstlane((unsigned)((r * kb_total + kb) * 2 + kg) * kTileBytes);
        raw[slot][r] = __builtin_bit_cast(uint4_t, __builtin_amdgcn_raw_buffer_load_b128(rw, (lane * 16u + sofs) | oob, 0, 0));
    };

    int4_t acc[4][8];  // [channel tile][row tile]
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int t = 0; t < 8; ++t)
            acc[r][t] = int4_t{0, 0, 0, 0};

    // One k-block: 32 MFMAs of the wave's four signed weight operands against the eight row tiles of its 64-input
    // tile in `stage`, the memory instructions of mem(i) in between.
    typedef __attribute__((address_space(3))) const int4_t* lds_i4_ptr;
    auto block = [&](int stage, int slot, auto&& mem) {
        int4_t w[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const uint4_t u = raw[slot][r];
            w[r] = int4_t{(int)(u.x ^ 0x80808080u), (int)(u.y ^ 0x80808080u), (int)(u.z ^ 0x80808080u),
                          (int)(u.w ^ 0x80808080u)};
        }
        // operand of row tile t: row 16 t + col, chunk (4 kg + kq) ^ ((col >> 1) & 7)
        const lds_byte_ptr xa = lds3 + stage * PI_A_BYTES + col * 128 + (((4 * kg + kq) ^ ((col >> 1) & 7)) << 4);
        int4_t xo[PI_XQ];
#pragma unroll
        for (int t = 0; t < PI_XQ - 1; ++t)
            xo[t] = *(lds_i4_ptr)(xa + t * 2048);
#pragma unroll
        for (int i = 0; i < 32; ++i) {
            const int t = i >> 2, r = i & 3;
            if (r == 0 && t + PI_XQ - 1 < 8)
                xo[(t + PI_XQ - 1) % PI_XQ] = *(lds_i4_ptr)(xa + (t + PI_XQ - 1) * 2048);
            acc[r][t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(w[r], xo[t % PI_XQ], acc[r][t], 0, 0, 0);
            mem(i);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // ---- prologue: issue order as in the loop (activations of a k-block, then its weights) ----
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        dma_a(j, 0);
        dma_a(j, 1);
#pragma unroll
        for (int r = 0; r < 4; ++r)
            load_w(j, j, r);
    }
    // ---- main loop: two k-blocks per trip so that ring slots are static; k-blocks past the end load zeros ----
    for (int kb0 = 0; kb0 < kb_total; kb0 += 2) {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int kb = kb0 + u;
            // own loads of k-block kb have landed once only the six issued after them (k-block kb + 1) are out
            __builtin_amdgcn_s_waitcnt(wait_vmcnt_imm(6));
            asm volatile("" ::: "memory");
            __builtin_amdgcn_s_barrier();  // everyone's have; everyone is done with the stage of k-block kb - 1
            asm volatile("" ::: "memory");
            block(kb % PI_STAGES, u, [&](int i) {
                if (i == 2 || i == 10)
                    dma_a(kb + 2, i >> 3);
                if ((i & 7) == 6 && i >= 14)
                    load_w(kb + 2, u, (i - 14) >> 3);
                if (i == 31)
                    load_w(kb + 2, u, 3);
            });
        }
    }

    // ---- epilogue: k-group 1 -> k-group 0 through LDS (i32, exact), two channel tiles at a time ----
    __builtin_amdgcn_s_waitcnt(wait_vmcnt_imm(0));  // the out-of-range loads of the last trips still target LDS
    __syncthreads();
    int* ex = reinterpret_cast<int*>(lds_raw);  // [wn][2 x 8 x 4][64 lanes]
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) {
        if (kg == 1) {
#pragma unroll
            for (int r2 = 0; r2 < 2; ++r2)
#pragma unroll
                for (int t = 0; t < 8; ++t) {
                    const int4_t v = acc[2 * hh + r2][t];
                    int* p = ex + ((wn * 64 + (r2 * 8 + t) * 4) * 64) + lane;
                    p[0] = v.x, p[64] = v.y, p[128] = v.z, p[192] = v.w;
                }
        }
        __syncthreads();
        if (kg == 0 && glu) {
            // gated linear unit: channel tiles 2 hh and 2 hh + 1 of the wave are gate and up of output channels
            // (n0 + 64 wn) / 2 + 16 hh .. of the [M, N / 2] result
            const int ng_ch = n0 + 64 * wn + 32 * hh + 4 * kq;  // gate channels; up channels are 16 further
            int zadj[2][4], cwv[2][4];
            float sc[2][4], bs[2][4];
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    cwv[h][q] = za ? cw[ng_ch + 16 * h + q] : 0;  // asymmetric activations: sum_k (w - zp) of the channel
                    zadj[h][q] = (ZP_TABLE ? (int)zt[ng_ch + 16 * h + q] : zp_const) - 128;
                    sc[h][q] = (float)st[ng_ch + 16 * h + q];
                    bs[h][q] = bias ? (float)bias[ng_ch + 16 * h + q] : 0.f;
                }
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                const int m = m0 + 16 * t + col;
                if (m < M) {
                    const int rs = qsum[m];
                    const int zr = za ? za[m] : 0;
                    const float inv = inv_scale[m];
                    float o[4];
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const int g = acc[2 * hh][t][q] + ex[((wn * 64 + t * 4 + q) * 64) + lane];
                        const int u = acc[2 * hh + 1][t][q] + ex[((wn * 64 + (8 + t) * 4 + q) * 64) + lane];
                        o[q] = glu_value(glu,
                                         (float)(g - zadj[0][q] * rs - zr * cwv[0][q]) * (sc[0][q] * inv) + bs[0][q],
                                         (float)(u - zadj[1][q] * rs - zr * cwv[1][q]) * (sc[1][q] * inv) + bs[1][q]);
                    }
                    const size_t at = (size_t)m * (N / 2) + (n0 + 64 * wn) / 2 + 16 * hh + 4 * kq;
                    if (out_f32)
                        *reinterpret_cast<float4_t*>(static_cast<float*>(y) + at) = float4_t{o[0], o[1], o[2], o[3]};
                    else
                        *reinterpret_cast<half4_t*>(static_cast<half_t*>(y) + at) =
                            half4_t{(half_t)o[0], (half_t)o[1], (half_t)o[2], (half_t)o[3]};
                }
            }
        } else if (kg == 0) {
#pragma unroll
            for (int r2 = 0; r2 < 2; ++r2) {
                const int r = 2 * hh + r2;
                const int n = n0 + 64 * wn + 16 * r + 4 * kq;  // four consecutive channels
                int zadj[4], cwv[4];
                float sc[4], bs[4];
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    cwv[q] = za ? cw[n + q] : 0;
                    zadj[q] = (ZP_TABLE ? (int)zt[n + q] : zp_const) - 128;  // weights entered as w - 128
                    sc[q] = (float)st[n + q];
                    bs[q] = bias ? (float)bias[n + q] : 0.f;
                }
#pragma unroll
                for (int t = 0; t < 8; ++t) {
                    const int* p = ex + ((wn * 64 + (r2 * 8 + t) * 4) * 64) + lane;
                    const int4_t a = acc[r][t];
                    const int v[4] = {a.x + p[0], a.y + p[64], a.z + p[128], a.w + p[192]};
                    const int m = m0 + 16 * t + col;
                    if (m < M) {
                        const int rs = qsum[m];
                        const int zr = za ? za[m] : 0;
                        const float inv = inv_scale[m];
                        float o[4];
#pragma unroll
                        for (int q = 0; q < 4; ++q)
                            o[q] = (float)(v[q] - zadj[q] * rs - zr * cwv[q]) * (sc[q] * inv) + bs[q];
                        if (out_f32)
                            *reinterpret_cast<float4_t*>(static_cast<float*>(y) + (size_t)m * N + n) =
                                float4_t{o[0], o[1], o[2], o[3]};
                        else
                            *reinterpret_cast<half4_t*>(static_cast<half_t*>(y) + (size_t)m * N + n) =
                                half4_t{(half_t)o[0], (half_t)o[1], (half_t)o[2], (half_t)o[3]};
                    }
                }
            }
        }
        __syncthreads();
    }
}

int launch_dynquant(const void* x, void* xq, float* inv_scale, int* qsum, int64_t M, int64_t K, void* stream) {
    if (M <= 0 || K <= 0 || (K % PI_BK) != 0 || M > 0x7fffffff)
        return (int)hipErrorInvalidValue;
    hipLaunchKernelGGL(fcc_dynquant_kernel, dim3((unsigned)M), dim3(256), 0, static_cast<hipStream_t>(stream),
                       (const half_t*)x, (int8_t*)xq, inv_scale, qsum, (int)K);
    return (int)hipGetLastError();
}

int launch_dynquant_asym(const void* x, void* xq, float* inv_scale, int* qsum, int* za, int64_t M, int64_t K,
                         void* stream) {
    if (M <= 0 || K <= 0 || (K % PI_BK) != 0 || M > 0x7fffffff || !za)
        return (int)hipErrorInvalidValue;
    hipLaunchKernelGGL(fcc_dynquant_asym_kernel, dim3((unsigned)M), dim3(256), 0, static_cast<hipStream_t>(stream),
                       (const half_t*)x, (int8_t*)xq, inv_scale, qsum, za, (int)K);
    return (int)hipGetLastError();
}

int launch_i8_colsum(const void* w_tiled, const void* zp_tiled, int zp_const, int* cw, int64_t n_tiles, int64_t k_blocks,
                     void* stream) {
    if (!w_tiled || !cw || n_tiles <= 0 || n_tiles > 0x7fffffff || k_blocks <= 0 || k_blocks * 128 > kI8AsymMaxK)
        return (int)hipErrorInvalidValue;
    hipLaunchKernelGGL(fcc_i8_colsum_kernel, dim3((unsigned)n_tiles), dim3(256), 0, static_cast<hipStream_t>(stream),
                       (const uint4_t*)w_tiled, (const uint8_t*)zp_tiled, zp_const, cw, (int)k_blocks);
    return (int)hipGetLastError();
}

template <bool ZPT>
static int launch_i8_impl(const FcDeviceArgs& a, const void* xq, const float* inv_scale, const int* qsum, const int* za,
                          const int* cw, hipStream_t s) {
    const Layout& L = a.layout;
    auto kern = fcc_prefill_i8_kernel<ZPT>;
    static bool attr_set = false;  // per instantiation; the attribute is idempotent, a race only repeats it
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)PI_LDS_BYTES);
        if (e != hipSuccess)
            return (int)e;
        attr_set = true;
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)(a.N / PI_BN), (unsigned)((a.M + PI_BM - 1) / PI_BM), 1), dim3(512),
                       PI_LDS_BYTES, s, (const uint4_t*)a.w, (const half_t*)a.scale, (const uint8_t*)a.zp,
                       (const int8_t*)xq, inv_scale, qsum, za, cw, (const half_t*)a.bias, a.y, (int)a.M, (int)a.N, (int)a.K,
                       (int)L.k_blocks, L.zp_const, a.out_f32, L.glu);
    return (int)hipGetLastError();
}

// a describes the node and y; xq / inv_scale / qsum are the outputs of launch_dynquant for the same M and K, or, with
// za (the rows' zero-points) and cw (the node's column sums, launch_i8_colsum), of launch_dynquant_asym.
int launch_prefill_i8(const FcDeviceArgs& a, const void* xq, const float* inv_scale, const int* qsum, const int* za,
                      const int* cw, void* stream) {
    const Layout& L = a.layout;
    // what the kernel's indexing assumes: tiled 8-bit weights, one group per channel, whole 256-channel tiles,
    // 32-bit byte offsets into the quantised activations and into one wave's weight strip
    if (!L.tiled || L.bits != 8 || L.groups != 1 || (a.N % PI_BN) != 0 || a.M < 1 ||
        a.M * a.K >= ((int64_t)1 << 31) || (int64_t)4 * L.k_blocks * 2 * kTileBytes >= ((int64_t)1 << 31) ||
        (a.M + PI_BM - 1) / PI_BM > 65535 || !xq || !inv_scale || !qsum || (za != nullptr) != (cw != nullptr) ||
        (za && a.K > kI8AsymMaxK))
        return (int)hipErrorInvalidValue;
    hipStream_t s = static_cast<hipStream_t>(stream);
    return L.zp_table ? launch_i8_impl<true>(a, xq, inv_scale, qsum, za, cw, s)
                      : launch_i8_impl<false>(a, xq, inv_scale, qsum, za, cw, s);
}

}  // namespace ovfcc
