// Prefill kernel for 4-bit weights with one scale (and zero-point) per 128 inputs over dynamically quantised
// activations (W4A8), and the kernel that quantises the activations for it.  The reference's plugins run their
// weight-compressed FullyConnected this way for large batches: the CPU plugin quantises the source in groups of
// ov::hint::dynamic_quantization_group_size inputs where the weights are u8 / u4
// (src/plugins/intel_cpu/src/nodes/executors/dnnl/dnnl_fullyconnected_primitive.cpp:161-241,284-298), the GPU
// plugin inserts a DynamicQuantize node in front of FullyConnectedCompressed -- per token on matrix-engine
// hardware, else per group (src/plugins/intel_gpu/src/plugin/transformations/dynamic_quantize_fully_connected.cpp:
// 24-140, src/plugins/intel_gpu/src/runtime/execution_config.cpp:348-354) -- and its kernel scales every group's
// integer sum into a float accumulator (cl_kernels/fully_connected_gpu_bf_tiled.cl:1257-1291).
//
//     y[m, n] = sum_g ( sum_{k in g} q[m, k] (w[n, k] - zp[n, g]) ) * s[n, g] * inv[m, g or -]   (+ bias[n])
//
// with g the weight groups of 128 inputs = the k-blocks of the tile layout, q the int8 activations and inv their
// scales, one per row (per token) or one per row and k-block (GROUPED).  The integer sums run on
// v_mfma_i32_16x16x64_i8 and are exact; every k-block's sums are converted and scaled into f32 accumulators.
//
// Weights: a lane's 16 bytes of a 4-bit tile are the nibbles of inputs 32 j + 8 kq + e (dword j, element e at
// nibble (e >> 1) + 4 (e & 1)).  (d & 0x0F0F0F0F) and ((d >> 4) & 0x0F0F0F0F) are four codes each, as bytes,
// of elements {0, 4, 1, 5} and {2, 6, 3, 7}; the zero-point leaves byte-wise, ((c | 0x80) - zp) ^ 0x80 = c - zp
// as a signed byte, no borrow between bytes for c, zp <= 15.  MFMA step s (of two per k-block) takes dwords 2 s
// and 2 s + 1; the quantisation kernel writes q in the same byte order, so that both operands are verbatim
// registers.
//
// Main kernel: 128 x 256 output tile, 8 waves, one workgroup per tile in XCD-aware order.  Wave w owns channel
// tiles 2 w and 2 w + 1 (with a gated linear unit: a gate tile and its up tile) against all eight row tiles and
// the whole k-block: 32 MFMAs and 16 rescaled accumulator tiles per wave and k-block.  Activations travel to LDS
// by direct-to-LDS loads two k-blocks ahead (three 16 KiB stages, chunks XOR-swizzled as in the 8-bit kernel);
// weights, scales, zero-points and activation scales come from memory into two-slot register rings.
#include "device_common.h"

namespace ovfcc {

typedef int int4_t __attribute__((ext_vector_type(4)));

constexpr int PW_BM = 128, PW_BN = 256, PW_BK = 128;
constexpr int PW_STAGES = 3;
constexpr int PW_A_BYTES = PW_BM * PW_BK;  // 16 KiB per stage
constexpr unsigned PW_LDS_BYTES = PW_STAGES * PW_A_BYTES;

// ------------------------------------------------------------------------------------------------
// Quantisation.  grid = M, block = 256; K % 128 == 0.  Thread and step: one 16-byte chunk of q, the 16 inputs
// 32 (2 s + jj) + 8 kq + e (jj < 2, e < 8) of k-block kb, chunk index 8 kb + 4 s + kq.
// Arithmetic of the reference kernel (cl_kernels/dynamic_quantize_gpu_ref.cl:100-250): max |x| clamped below at
// 0.003, scale = 127 / max rounded to half, q = rte(half(x * scale)), stored scale half(1 / scale).
// inv: [M] (per token), or GROUPED one per row and k-block at [kb][m / 128][m % 16][(m % 128) / 16], the order in
// which the main kernel's lanes read them.
// ------------------------------------------------------------------------------------------------
template <bool GROUPED>
__global__ __launch_bounds__(256) void fcc_dynquant_w4_kernel(const half_t* __restrict__ x, int8_t* __restrict__ xq,
                                                              float* __restrict__ inv, int K, int tiles_m) {
    __shared__ float red_f[4];
    const int row = blockIdx.x;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const half_t* xr = x + (size_t)row * K;
    const float floor_max = (float)(half_t)0.003f;
    half_t scale = (half_t)0.f;
    if constexpr (!GROUPED) {
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
        mx = fmaxf(mx, floor_max);
        scale = (half_t)(127.f / mx);  // one f32 division rounded to half = the half division
        if (tid == 0)
            inv[row] = (float)(half_t)(1.f / (float)scale);
    }
    for (int ch = tid; ch < K / 16; ch += 256) {
        const int kb = ch >> 3, s = (ch >> 2) & 1, kq = ch & 3;
        half8_t v[2];
#pragma unroll
        for (int jj = 0; jj < 2; ++jj)
            v[jj] = *reinterpret_cast<const half8_t*>(xr + kb * PW_BK + 32 * (2 * s + jj) + 8 * kq);
        if constexpr (GROUPED) {
            // the eight chunks of a k-block sit in eight consecutive lanes
            float mx = 0.f;
#pragma unroll
            for (int jj = 0; jj < 2; ++jj)
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    mx = fmaxf(mx, fabsf((float)v[jj][e]));
            mx = fmaxf(mx, __shfl_xor(mx, 1, 64));
            mx = fmaxf(mx, __shfl_xor(mx, 2, 64));
            mx = fmaxf(mx, __shfl_xor(mx, 4, 64));
            mx = fmaxf(mx, floor_max);
            scale = (half_t)(127.f / mx);
            if ((ch & 7) == 0)
                inv[(((size_t)kb * tiles_m + (row >> 7)) * 16 + (row & 15)) * 8 + ((row & 127) >> 4)] =
                    (float)(half_t)(1.f / (float)scale);
        }
        uint32_t packed[4];
#pragma unroll
        for (int jj = 0; jj < 2; ++jj)
#pragma unroll
            for (int hi = 0; hi < 2; ++hi) {
                uint32_t wrd = 0;
#pragma unroll
                for (int b = 0; b < 4; ++b) {
                    const int e = 2 * hi + 4 * (b & 1) + (b >> 1);  // bytes: elements {0, 4, 1, 5} / {2, 6, 3, 7}
                    const half_t p = v[jj][e] * scale;              // half product, as the reference rounds it
                    int q = (int)__builtin_rintf((float)p);
                    q = q > 127 ? 127 : (q < -128 ? -128 : q);
                    wrd |= (uint32_t)(q & 0xFF) << (8 * b);
                }
                packed[2 * jj + hi] = wrd;
            }
        *reinterpret_cast<uint4_t*>(xq + (size_t)row * K + (size_t)ch * 16) =
            uint4_t{packed[0], packed[1], packed[2], packed[3]};
    }
}

// ------------------------------------------------------------------------------------------------
// Integer FullyConnected over 4-bit weights.
// ------------------------------------------------------------------------------------------------
template <bool ZP_TABLE, bool GROUPED>
__global__ __launch_bounds__(512) void fcc_prefill_i8w4_kernel(const uint4_t* __restrict__ wt, const half_t* __restrict__ st,
                                                               const uint8_t* __restrict__ zt,
                                                               const int8_t* __restrict__ xq,
                                                               const float* __restrict__ inv,
                                                               const half_t* __restrict__ bias, void* __restrict__ y,
                                                               int M, int N, int K, int kb_total, int zp_const,
                                                               int out_f32, int glu, int tiles_m) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    const lds_byte_ptr lds3 = (lds_byte_ptr)lds_raw;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    int tile_x, tile_y;
    xcd_tile(tile_x, tile_y, PW_BM, PW_BN / 2);
    const int n0 = tile_x * PW_BN;
    const int m0 = tile_y * PW_BM;
    const int col = lane & 15, kq = lane >> 4;

    constexpr unsigned kOob = 0x80000000u;
    constexpr int kRsrcFlags = 0x00020000;
    // Every offset goes through the vector operand: the scalar offset of a buffer load is not range-checked.
    const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(xq), 0, M * K, kRsrcFlags);
    const int nt0 = n0 / 16 + 2 * wave;  // the wave's two channel tiles
    const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint4_t*>(wt + (size_t)nt0 * kb_total * 64), 0, 2 * kb_total * kTileBytes, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<half_t*>(st + (size_t)nt0 * kb_total * 16), 0, 2 * kb_total * 32, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t rz = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint8_t*>(ZP_TABLE ? zt + (size_t)nt0 * kb_total * 16 : nullptr), 0, ZP_TABLE ? 2 * kb_total * 16 : 0,
        kRsrcFlags);
    const __amdgpu_buffer_rsrc_t ri = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float*>(inv), 0, GROUPED ? kb_total * tiles_m * 128 * 4 : M * 4, kRsrcFlags);

    // ---- activations: as in the 8-bit kernel -- load i (0, 1) of the wave covers rows 64 i + 8 wave .. + 7 ----
    const unsigned a_row0 = (unsigned)((m0 + 8 * wave + (lane >> 3)) * K);
    const unsigned a_chunk = (unsigned)(((lane & 7) ^ (4 * (wave & 1) + (lane >> 4))) << 4);
    auto dma_a = [&](int kb, int i) {
        const unsigned oob = (unsigned)((kb_total - 1 - kb) >> 31) & kOob;
        const int stage = kb % PW_STAGES;
        const unsigned sterm = __builtin_amdgcn_readfirstlane((unsigned)(64 * i * K + kb * PW_BK));
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, (lds_void_ptr)(lds3 + stage * PW_A_BYTES + i * 8192 + wave * 1024), 16,
                                                 (a_row0 + sterm + a_chunk) | oob, 0, 0, 0);
    };
    // ---- per-k-block operands from memory: two-slot rings ----
    uint4_t raw[2][2];   // weights: 16 bytes per lane and channel tile
    uint2_t scr[2][2];   // scales of channels 4 kq .. + 3 of the tile (four halves)
    uint32_t zpr[2][2];  // zero-point of channel col of the tile
    float4_t sxr[2][2];  // GROUPED: activation scales of rows 16 t + col, t = 0..7
    auto load_w = [&](int kb, int slot, int r) {
        const unsigned oob = (unsigned)((kb_total - 1 - kb) >> 31) & kOob;
        const unsigned base = __builtin_amdgcn_readfirstlane((unsigned)(r * kb_total + kb));
        raw[slot][r] = __builtin_bit_cast(uint4_t, __builtin_amdgcn_raw_buffer_load_b128(rw, (lane * 16u + base * kTileBytes) | oob, 0, 0));
        scr[slot][r] = __builtin_bit_cast(uint2_t, __builtin_amdgcn_raw_buffer_load_b64(rs, (kq * 8u + base * 32u) | oob, 0, 0));
        if constexpr (ZP_TABLE)
            zpr[slot][r] = __builtin_amdgcn_raw_buffer_load_b8(rz, ((unsigned)col + base * 16u) | oob, 0, 0);
    };
    auto load_sx = [&](int kb, int slot) {
        if constexpr (GROUPED) {
            const unsigned oob = (unsigned)((kb_total - 1 - kb) >> 31) & kOob;
            const unsigned base = __builtin_amdgcn_readfirstlane((unsigned)((kb * tiles_m + tile_y) * 16) * 32u);
            sxr[slot][0] = __builtin_bit_cast(float4_t, __builtin_amdgcn_raw_buffer_load_b128(ri, (col * 32u + base) | oob, 0, 0));
            sxr[slot][1] = __builtin_bit_cast(float4_t, __builtin_amdgcn_raw_buffer_load_b128(ri, (col * 32u + 16u + base) | oob, 0, 0));
        }
    };
    // loads per wave and k-block, for the wait counts
    constexpr int kLoads = 2 + 2 * (2 + (ZP_TABLE ? 1 : 0)) + (GROUPED ? 2 : 0);

    float4_t acc[2][8];  // [channel tile][row tile]
#pragma unroll
    for (int r = 0; r < 2; ++r)
#pragma unroll
        for (int t = 0; t < 8; ++t)
            acc[r][t] = float4_t{0.f, 0.f, 0.f, 0.f};

    typedef __attribute__((address_space(3))) const int4_t* lds_i4_ptr;
    const uint32_t zconst4 = (uint32_t)zp_const * 0x01010101u;
    // One k-block: unpack the two weight tiles, 32 MFMAs, 16 accumulator tiles rescaled; mem() issues the loads of
    // the k-block after next.
    auto block = [&](int stage, int slot, auto&& mem) {
        int4_t w[2][2];
        float sw[2][4];
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            const uint32_t z4 = ZP_TABLE ? (zpr[slot][r] & 0xFFu) * 0x01010101u : zconst4;
            const uint4_t u = raw[slot][r];
            auto codes = [&](uint32_t d) { return (int)((((d & 0x0F0F0F0Fu) | 0x80808080u) - z4) ^ 0x80808080u); };
            w[r][0] = int4_t{codes(u.x), codes(u.x >> 4), codes(u.y), codes(u.y >> 4)};
            w[r][1] = int4_t{codes(u.z), codes(u.z >> 4), codes(u.w), codes(u.w >> 4)};
            const half2_t s01 = as_half2(scr[slot][r].x), s23 = as_half2(scr[slot][r].y);
            sw[r][0] = (float)s01[0], sw[r][1] = (float)s01[1], sw[r][2] = (float)s23[0], sw[r][3] = (float)s23[1];
        }
        float sx[8];
        if constexpr (GROUPED) {
#pragma unroll
            for (int t = 0; t < 8; ++t)
                sx[t] = sxr[slot][t >> 2][t & 3];
        }
        mem();
        // operand of row tile t, step s: row 16 t + col, chunk (4 s + kq) ^ ((col >> 1) & 7)
        const lds_byte_ptr xa = lds3 + stage * PW_A_BYTES + col * 128;
        const unsigned c0 = (unsigned)((kq ^ ((col >> 1) & 7)) << 4), c1 = (unsigned)(((4 + kq) ^ ((col >> 1) & 7)) << 4);
        // Software pipeline over the row tiles: the four MFMAs of row tile t are issued, then the sums of row tile
        // t - 1 (long finished) are converted and scaled while the matrix pipe works, then the operands of row tile
        // t + 2 are fetched.  The scheduling barriers keep that order.
        int4_t xo[3][2];
        xo[0][0] = *(lds_i4_ptr)(xa + c0), xo[0][1] = *(lds_i4_ptr)(xa + c1);
        xo[1][0] = *(lds_i4_ptr)(xa + 2048 + c0), xo[1][1] = *(lds_i4_ptr)(xa + 2048 + c1);
        int4_t d[2][2];  // [parity of t][channel tile]
        auto rescale = [&](int t) {
#pragma unroll
            for (int r = 0; r < 2; ++r)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const float p = GROUPED ? sw[r][q] * sx[t] : sw[r][q];
                    acc[r][t][q] += (float)d[t & 1][r][q] * p;
                }
        };
#pragma unroll
        for (int t = 0; t < 8; ++t) {
#pragma unroll
            for (int r = 0; r < 2; ++r) {
                d[t & 1][r] = __builtin_amdgcn_mfma_i32_16x16x64_i8(w[r][0], xo[t % 3][0], int4_t{0, 0, 0, 0}, 0, 0, 0);
                d[t & 1][r] = __builtin_amdgcn_mfma_i32_16x16x64_i8(w[r][1], xo[t % 3][1], d[t & 1][r], 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
            if (t > 0)
                rescale(t - 1);
            if (t + 2 < 8) {
                xo[(t + 2) % 3][0] = *(lds_i4_ptr)(xa + (t + 2) * 2048 + c0);
                xo[(t + 2) % 3][1] = *(lds_i4_ptr)(xa + (t + 2) * 2048 + c1);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        rescale(7);
    };

    // ---- prologue: k-blocks 0 and 1 ----
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        dma_a(j, 0);
        dma_a(j, 1);
        load_w(j, j, 0);
        load_w(j, j, 1);
        load_sx(j, j);
    }
    // ---- main loop: two k-blocks per trip so that ring slots are static; k-blocks past the end load zeros ----
    for (int kb0 = 0; kb0 < kb_total; kb0 += 2) {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int kb = kb0 + u;
            // own loads of k-block kb have landed once only those of k-block kb + 1, issued after them, are out
            __builtin_amdgcn_s_waitcnt(wait_vmcnt_imm(kLoads));
            asm volatile("" ::: "memory");
            __builtin_amdgcn_s_barrier();  // everyone's have; everyone is done with the stage of k-block kb - 1
            asm volatile("" ::: "memory");
            block(kb % PW_STAGES, u, [&]() {
                dma_a(kb + 2, 0);
                dma_a(kb + 2, 1);
                load_w(kb + 2, u, 0);
                load_w(kb + 2, u, 1);
                load_sx(kb + 2, u);
                __builtin_amdgcn_sched_barrier(0);  // the wait counts assume this issue order
            });
        }
    }
    __builtin_amdgcn_s_waitcnt(wait_vmcnt_imm(0));  // the out-of-range loads of the last trips still target LDS

    // ---- epilogue: per-token scale, bias, gated linear unit, store; lane holds channels 4 kq .. + 3 of each of its
    // two tiles for rows 16 t + col ----
    const int nch = n0 + 32 * wave + 4 * kq;  // first of the lane's channels of tile 0 in the tiled channel order
    float bs[2][4];
#pragma unroll
    for (int r = 0; r < 2; ++r)
#pragma unroll
        for (int q = 0; q < 4; ++q)
            bs[r][q] = bias ? (float)bias[nch + 16 * r + q] : 0.f;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
        const int m = m0 + 16 * t + col;
        if (m >= M)
            continue;
        const float im = GROUPED ? 1.f : inv[m];
        if (glu) {
            float o[4];
#pragma unroll
            for (int q = 0; q < 4; ++q)
                o[q] = glu_value(glu, acc[0][t][q] * im + bs[0][q], acc[1][t][q] * im + bs[1][q]);
            const size_t at = (size_t)m * (N / 2) + n0 / 2 + 16 * wave + 4 * kq;
            if (out_f32)
                *reinterpret_cast<float4_t*>(static_cast<float*>(y) + at) = float4_t{o[0], o[1], o[2], o[3]};
            else
                *reinterpret_cast<half4_t*>(static_cast<half_t*>(y) + at) =
                    half4_t{(half_t)o[0], (half_t)o[1], (half_t)o[2], (half_t)o[3]};
        } else {
#pragma unroll
            for (int r = 0; r < 2; ++r) {
                float o[4];
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    o[q] = acc[r][t][q] * im + bs[r][q];
                const size_t at = (size_t)m * N + nch + 16 * r;
                if (out_f32)
                    *reinterpret_cast<float4_t*>(static_cast<float*>(y) + at) = float4_t{o[0], o[1], o[2], o[3]};
                else
                    *reinterpret_cast<half4_t*>(static_cast<half_t*>(y) + at) =
                        half4_t{(half_t)o[0], (half_t)o[1], (half_t)o[2], (half_t)o[3]};
            }
        }
    }
}

size_t dynquant_w4_scale_floats(int64_t M, int64_t K, bool grouped) {
    return grouped ? (size_t)(K / PW_BK) * (size_t)((M + PW_BM - 1) / PW_BM) * PW_BM : (size_t)M;
}

int launch_dynquant_w4(const void* x, void* xq, float* inv, int64_t M, int64_t K, bool grouped, void* stream) {
    if (M <= 0 || K <= 0 || (K % PW_BK) != 0 || M > 0x7fffffff || !x || !xq || !inv)
        return (int)hipErrorInvalidValue;
    const int tiles_m = (int)((M + PW_BM - 1) / PW_BM);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (grouped)
        hipLaunchKernelGGL(fcc_dynquant_w4_kernel<true>, dim3((unsigned)M), dim3(256), 0, s, (const half_t*)x, (int8_t*)xq,
                           inv, (int)K, tiles_m);
    else
        hipLaunchKernelGGL(fcc_dynquant_w4_kernel<false>, dim3((unsigned)M), dim3(256), 0, s, (const half_t*)x, (int8_t*)xq,
                           inv, (int)K, tiles_m);
    return (int)hipGetLastError();
}

template <bool ZPT, bool GROUPED>
static int launch_i8w4_impl(const FcDeviceArgs& a, const void* xq, const float* inv, hipStream_t s) {
    const Layout& L = a.layout;
    auto kern = fcc_prefill_i8w4_kernel<ZPT, GROUPED>;
    hipLaunchKernelGGL(kern, dim3((unsigned)(a.N / PW_BN), (unsigned)((a.M + PW_BM - 1) / PW_BM), 1), dim3(512),
                       PW_LDS_BYTES, s, (const uint4_t*)a.w, (const half_t*)a.scale, (const uint8_t*)a.zp,
                       (const int8_t*)xq, inv, (const half_t*)a.bias, a.y, (int)a.M, (int)a.N, (int)a.K,
                       (int)L.k_blocks, L.zp_const, a.out_f32, L.glu, (int)((a.M + PW_BM - 1) / PW_BM));
    return (int)hipGetLastError();
}

// Whether the kernel can run the node: tiled 4-bit weights, one group per k-block, whole 256-channel tiles,
// zero-points that fit a nibble (a table of the 4-bit type, or a scalar of at most 15 including the offset of
// signed weights).
bool prefill_i8w4_applies(const Layout& L, int64_t N, int zp_type) {
    return L.tiled && L.bits == 4 && L.groups_per_kblock == 1 && L.kblocks_per_group == 1 && (N % PW_BN) == 0 &&
           (L.zp_table ? zp_type == OVFCC_U4 : (L.zp_const >= 0 && L.zp_const <= 15));
}

// a describes the node and y; xq / inv are the outputs of launch_dynquant_w4 for the same M, K and grouping.
int launch_prefill_i8w4(const FcDeviceArgs& a, const void* xq, const float* inv, bool grouped, void* stream) {
    const Layout& L = a.layout;
    // what the kernel's indexing assumes, and 32-bit byte offsets into the quantised activations, the scale table
    // and one wave's weight strip
    if (!prefill_i8w4_applies(L, a.N, a.zp_type) || a.M < 1 || a.M * a.K >= ((int64_t)1 << 31) ||
        (int64_t)2 * L.k_blocks * kTileBytes >= ((int64_t)1 << 31) || (a.M + PW_BM - 1) / PW_BM > 65535 ||
        (grouped && (int64_t)dynquant_w4_scale_floats(a.M, a.K, true) * 4 >= ((int64_t)1 << 31)) || !xq || !inv)
        return (int)hipErrorInvalidValue;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (grouped)
        return L.zp_table ? launch_i8w4_impl<true, true>(a, xq, inv, s) : launch_i8w4_impl<false, true>(a, xq, inv, s);
    return L.zp_table ? launch_i8w4_impl<true, false>(a, xq, inv, s) : launch_i8w4_impl<false, false>(a, xq, inv, s);
}

}  // namespace ovfcc
