// Prefill kernel with register-fed weights (M > 128): 128 x 256 output tile per workgroup, 8 waves.
//
// grid = (N/256, ceil(M/128)), block = 512.  K advances one k-block (128 inputs) per step.
//
// Weights never pass through LDS as f16.  A packed weight tile already has the matrix cores' operand layout
// (lane = channel (lane & 15), eight consecutive inputs per dword at 8 (lane >> 4)), so every wave loads the
// tiles of its own 64 output channels straight into a two-slot register ring (two k-blocks ahead), unpacks
// one dword into one f16 operand and feeds it to v_mfma_f32_16x16x32_f16.  The activation tile (128 rows x
// 128 inputs, f16, 32 KiB) travels HBM/L2 -> LDS with buffer loads that write LDS directly, two k-blocks
// ahead, into one of three stages; rows are 256 bytes without padding and the sixteen 16-byte chunks of row r
// sit at chunk ^ (r & 15), so the 16 rows of one 128-bit read phase hit 16 different bank groups (the
// swizzle is applied on the global side: a lane fetches the chunk that belongs in its linear LDS slot).
// A wave waits for its own loads (the vector-memory counter is in order); one bare barrier per k-block
// publishes the stage and frees the oldest one (a fence would also wait for the loads meant to stay in
// flight).
//
// Waves: wn = wave & 3 picks 64 of the 256 channels, kg = wave >> 2 picks which two of the four 32-input
// steps of every k-block the wave contracts (for 8-bit weights: which of the k-block's two 64-input tiles).
// A wave unpacks every weight it uses exactly once and multiplies it with all 128 rows (eight 16-row operands
// read from LDS): 32 MFMAs per step and 4 unpacked dwords.  After the last k-block k-group 1 hands its f32
// accumulators to k-group 0 through LDS, which adds, applies per-channel scale and bias and stores.
//
// The inner loop is software-pipelined by hand and pinned with scheduling barriers: between every two MFMAs
// of a step sit one or two vector-ALU operations of the *next* step's unpack, and every few MFMAs one memory
// instruction (an LDS read of an activation operand two ahead, a direct-to-LDS load, a weight load).  Left
// to itself the compiler emits these in bursts; the two waves of a SIMD run in lockstep between barriers, so
// a burst in one is a burst in both and the matrix pipe idles.
//
// MFMA roles: A = weights (rows = channels), B = activations (columns = rows m of X); result lane holds
// column m = lane & 15, channels 4 (lane >> 4) + r, so a lane stores four consecutive outputs of one row.
//
// Weights: (q - zp) * s rounded once to f16 for grouped scales; with one group per channel the exact
// integers q - zp go to the matrix cores and the scale multiplies the f32 result.
#include "device_common.h"

namespace ovfcc {

constexpr int PD_BM = 128, PD_BN = 256, PD_BK = 128;
constexpr int PD_STAGES = 3;
constexpr int PD_XQ = 2;  // activation operands in registers: the one in use and PD_XQ - 1 on their way from LDS
constexpr int PD_A_BYTES = PD_BM * PD_BK * 2;                        // 32 KiB per stage
constexpr unsigned PD_LDS_BYTES = (unsigned)(PD_STAGES * PD_A_BYTES);  // 96 KiB (the epilogue needs 64)


template <int BITS, bool ZP_TABLE, bool PRESCALE>
__global__ __launch_bounds__(512) void fcc_prefill_direct_kernel(const uint4_t* __restrict__ wt,
                                                                 const half_t* __restrict__ st,
                                                                 const uint8_t* __restrict__ zt,
                                                                 const half_t* __restrict__ x,
                                                                 const half_t* __restrict__ bias,
                                                                 void* __restrict__ y, int M, int N, int K,
                                                                 int kb_total, int kb_per_group, int ng, int zp_const,
                                                                 int out_f32, int glu) {
    constexpr int TPB = BITS == 4 ? 1 : 2;   // tiles per k-block and channel tile
    constexpr int WD = BITS == 4 ? 2 : 4;    // packed dwords per lane, channel tile and k-block for this k-group
    constexpr int NOPS = (BITS == 4 ? 5 : 4) + 4 + (PRESCALE ? 4 : 0);  // unpack micro-operations per dword (pair)
    // memory instructions a wave issues per k-block, in this order: 4 direct-to-LDS, then weights and parameters
    constexpr int RING_LOADS = 4 + (PRESCALE ? 4 : 0) + (ZP_TABLE ? 4 : 0);
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    const lds_byte_ptr lds3 = (lds_byte_ptr)lds_raw;  // arithmetic stays in the LDS address space (no null checks)

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wn = wave & 3, kg = wave >> 2;
    int tile_x, tile_y;
    xcd_tile(tile_x, tile_y, 2 * PD_BM, PD_BN * BITS / 8);
    const int n0 = tile_x * PD_BN;
    const int m0 = tile_y * PD_BM;
    const int col = lane & 15, kq = lane >> 4;

    constexpr unsigned kOob = 0x80000000u;
    constexpr int kRsrcFlags = 0x00020000;
    // Every offset goes through the vector operand: the scalar offset of a buffer load is not range-checked.
    const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(x), 0, M * K * 2, kRsrcFlags);
    const int nt0 = n0 / 16 + 4 * wn;  // the wave's four channel tiles
    const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint4_t*>(wt + (size_t)nt0 * kb_total * TPB * 64), 0, 4 * kb_total * TPB * kTileBytes, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t rs =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(st + (size_t)nt0 * ng * 16), 0, 4 * ng * 32, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t rz = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint8_t*>(ZP_TABLE ? zt + (size_t)nt0 * ng * 16 : zt), 0, ZP_TABLE ? 4 * ng * 16 : 0, kRsrcFlags);
    const unsigned g_mul = kb_per_group == 1 ? 0u : (unsigned)((0x100000000ull + kb_per_group - 1) / kb_per_group);

    // ---- activations: direct-to-LDS load i of the wave covers rows 16 wave + 4 i .. +3 of the tile; lane ->
    // row 4 i + (lane >> 4) of those, LDS slot lane & 15 of that row, which holds global chunk
    // (lane & 15) ^ (row & 15).  Rows >= M lie beyond the descriptor's range and arrive as zeros. ----
    // (row & 15 = 4 i + (lane >> 4) = 4 i ^ (lane >> 4), so the chunk of load i is c0 ^ 4 i.)
    const unsigned a_row0 = (unsigned)((m0 + 16 * wave + (lane >> 4)) * K) * 2u;
    const unsigned a_c0 = (unsigned)((lane & 15) ^ (lane >> 4));
    auto dma_a = [&](int kb, int i) {
        const unsigned oob = (unsigned)((kb_total - 1 - kb) >> 31) & kOob;
        const int stage = kb % PD_STAGES;
        const unsigned sterm = __builtin_amdgcn_readfirstlane((unsigned)(4 * i * K + kb * PD_BK) * 2u);
        const unsigned voff = a_row0 + sterm + ((a_c0 ^ (unsigned)(4 * i)) << 4);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, (lds_void_ptr)(lds3 + stage * PD_A_BYTES + (4 * wave + i) * 1024),
                                                 16, voff | oob, 0, 0, 0);
    };

    // ---- weights and their parameters: two-slot register ring ----
    uint32_t raw[2][4][WD];
    uint32_t rscale[2][4];  // two adjacent channels' f16 scales
    uint32_t rzp[2][4];
    const unsigned w_voff = BITS == 4 ? lane * 16u + kg * 8u : lane * 16u;
    auto load_w = [&](int kb, int slot, int r) {
        const unsigned oob = (unsigned)((kb_total - 1 - kb) >> 31) & kOob;
        if constexpr (BITS == 4) {
            const unsigned sofs = __builtin_amdgcn_readfirstlane((unsigned)(r * kb_total + kb) * kTileBytes);
            const uint2_t v =
                __builtin_bit_cast(uint2_t, __builtin_amdgcn_raw_buffer_load_b64(rw, (w_voff + sofs) | oob, 0, 0));
            raw[slot][r][0] = v.x, raw[slot][r][1] = v.y;
        } else {
            const unsigned sofs = __builtin_amdgcn_readfirstlane((unsigned)((r * kb_total + kb) * 2 + kg) * kTileBytes);
            const uint4_t v =
                __builtin_bit_cast(uint4_t, __builtin_amdgcn_raw_buffer_load_b128(rw, (w_voff + sofs) | oob, 0, 0));
            raw[slot][r][0] = v.x, raw[slot][r][1] = v.y, raw[slot][r][2] = v.z, raw[slot][r][3] = v.w;
        }
    };
    // a lane loads the dword that holds its channel's f16 scale and the neighbour's; scale_sel picks its half
    // into both halves of a register when the scale is used
    const uint32_t scale_sel = (col & 1) ? 0x03020302u : 0x01000100u;
    auto load_s = [&](int kb, int slot, int r) {
        const unsigned oob = (unsigned)((kb_total - 1 - kb) >> 31) & kOob;
        const unsigned g = kb_per_group == 1 ? (unsigned)kb : __umulhi((unsigned)kb, g_mul);
        rscale[slot][r] =
            __builtin_amdgcn_raw_buffer_load_b32(
                rs, (__builtin_amdgcn_readfirstlane((r * ng + g) * 32u) + (unsigned)(col & ~1) * 2u) | oob, 0, 0);
    };
    auto load_z = [&](int kb, int slot, int r) {
        const unsigned oob = (unsigned)((kb_total - 1 - kb) >> 31) & kOob;
        const unsigned g = kb_per_group == 1 ? (unsigned)kb : __umulhi((unsigned)kb, g_mul);
        rzp[slot][r] = (uint8_t)__builtin_amdgcn_raw_buffer_load_b8(
            rz, (__builtin_amdgcn_readfirstlane((r * ng + g) * 16u) + (unsigned)col) | oob, 0, 0);
    };

    // ---- unpack, one micro-operation at a time: dword (pair) `js` of tile r in ring slot `slot` -> f ----
    const Unpack4Consts uc = unpack4_consts();
    // uniform values the vector ALU can take as its one scalar operand are kept in scalar registers
    const half2_t off_lo_c = as_half2(__builtin_amdgcn_readfirstlane(as_u32(splat(1024.f + (float)zp_const))));
    const half2_t off_hi_c = as_half2(__builtin_amdgcn_readfirstlane(as_u32(splat(64.f + (float)zp_const))));
    auto unpack_op = [&](int slot, int r, int js, int op, Frag8& f) {
        if constexpr (BITS == 4) {
            const uint32_t w = raw[slot][r][js];
            if (op == 0)
                f.u[3] = w >> 8;
            else if (op == 1)
                f.u[0] = (w & uc.mask_lo) | uc.magic_lo;
            else if (op == 2)
                f.u[1] = (w & uc.mask_hi) | uc.magic_hi;
            else if (op == 3)
                f.u[2] = (f.u[3] & uc.mask_lo) | uc.magic_lo;
            else if (op == 4)
                f.u[3] = (f.u[3] & uc.mask_hi) | uc.magic_hi;
        } else {
            const uint32_t w = raw[slot][r][2 * js + (op >> 1 & 1)];
            if (op < 4)
                f.u[op] = __builtin_amdgcn_perm(0x64646464u, w, (op & 1) ? 0x04030402u : 0x04010400u);
        }
        constexpr int SUB0 = BITS == 4 ? 5 : 4;
        if (op >= SUB0 && op < SUB0 + 4) {
            const int k = op - SUB0;
            half2_t off;
            if constexpr (ZP_TABLE) {
                const float zpv = (float)rzp[slot][r];
                off = (BITS == 4 && (k & 1)) ? splat(64.f + zpv) : splat(1024.f + zpv);
            } else {
                off = (BITS == 4 && (k & 1)) ? off_hi_c : off_lo_c;
            }
            f.h2[k] = f.h2[k] - off;
        }
        if constexpr (PRESCALE) {
            if (op >= SUB0 + 4) {
                f.h2[op - SUB0 - 4] *= as_half2(__builtin_amdgcn_perm(rscale[slot][r], rscale[slot][r], scale_sel));
            }
        }
    };

    float4_t acc[4][8];  // [channel tile][row tile]
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int t = 0; t < 8; ++t)
            acc[r][t] = float4_t{0.f, 0.f, 0.f, 0.f};

    // One step: 32 MFMAs of operand `cur` against the eight row tiles of k-step `js` in `stage`, with the
    // unpack of (slot_n, js_n) into `nxt` and the memory instructions of `mem(i)` interleaved.
    auto step = [&](int stage, int js, const Frag8 (&cur)[4], int slot_n, int js_n, Frag8 (&nxt)[4], auto&& mem) {
        // activation operand of row tile t: row 16 t + col, chunk (4 (2 kg + js) + kq) ^ col
        typedef __attribute__((address_space(3))) const half8_t* lds_frag_ptr;
        const lds_byte_ptr xa = lds3 + stage * PD_A_BYTES + col * 256 + (((4 * (2 * kg + js) + kq) ^ col) << 4);
        half8_t xq[PD_XQ];
#pragma unroll
        for (int t = 0; t < PD_XQ - 1; ++t)
            xq[t] = *(lds_frag_ptr)(xa + t * 16 * 256);
#pragma unroll
        for (int i = 0; i < 32; ++i) {
            const int t = i >> 2, r = i & 3;
            if (r == 0 && t + PD_XQ - 1 < 8)
                xq[(t + PD_XQ - 1) % PD_XQ] = *(lds_frag_ptr)(xa + (t + PD_XQ - 1) * 16 * 256);
            acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(cur[r].v, xq[t % PD_XQ], acc[r][t], 0, 0, 0);
            // micro-operations [i * 4 NOPS / 32, (i + 1) * 4 NOPS / 32) of the next operand's unpack
#pragma unroll
            for (int g = i * 4 * NOPS / 32; g < (i + 1) * 4 * NOPS / 32; ++g)
                unpack_op(slot_n, g / NOPS, js_n, g % NOPS, nxt[g / NOPS]);
            mem(i);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // ---- prologue.  Memory instructions are issued in the same order as in the main loop (direct-to-LDS
    // loads of a k-block, then its ring loads), which the wait below counts on. ----
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int i = 0; i < 4; ++i)
            dma_a(kb, i);
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
        for (int r = 0; r < 4; ++r)
            load_w(kb, kb, r);
        if constexpr (PRESCALE)
#pragma unroll
            for (int r = 0; r < 4; ++r)
                load_s(kb, kb, r);
        if constexpr (ZP_TABLE)
#pragma unroll
            for (int r = 0; r < 4; ++r)
                load_z(kb, kb, r);
    }
    Frag8 wf0[4], wf1[4];
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int op = 0; op < NOPS; ++op)
            unpack_op(0, r, 0, op, wf0[r]);

    // ---- main loop: two k-blocks per trip so that ring slots are static.  k-blocks past the end are loaded
    // out of range (zeros) and add nothing. ----
    for (int kb0 = 0; kb0 < kb_total; kb0 += 2) {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int kb = kb0 + u;
            const int stage = kb % PD_STAGES;
            // This wave's direct-to-LDS loads of k-block kb have landed once at most the memory instructions
            // issued after them are outstanding: the ring loads of that k-block, and all of the next one's.
            __builtin_amdgcn_s_waitcnt(wait_vmcnt_imm(4 + 2 * RING_LOADS));
            asm volatile("" ::: "memory");
            __builtin_amdgcn_s_barrier();  // everyone's have; everyone is done with the stage k-block kb - 1 used
            asm volatile("" ::: "memory");
            // first step: unpack this k-block's second dword; request the activations of k-block kb + 2
            step(stage, 0, wf0, u, 1, wf1, [&](int i) {
                if ((i & 7) == 2)
                    dma_a(kb + 2, i >> 3);
            });
            // second step: refill this ring slot for k-block kb + 2 (its dwords are unpacked); unpack the
            // first dword of k-block kb + 1 from the other slot
            step(stage, 1, wf1, u ^ 1, 0, wf0, [&](int i) {
                if ((i & 3) == 1 && i < 16)
                    load_w(kb + 2, u, i >> 2);
                if constexpr (PRESCALE)
                    if ((i & 3) == 1 && i >= 16)
                        load_s(kb + 2, u, (i - 16) >> 2);
                if constexpr (ZP_TABLE)
                    if ((i & 3) == 3 && i >= 16)
                        load_z(kb + 2, u, (i - 16) >> 2);
            });
        }
    }

    // ---- epilogue: k-group 1 -> k-group 0 through LDS, two channel tiles at a time ----
    __builtin_amdgcn_s_waitcnt(wait_vmcnt_imm(0));  // the out-of-range loads of the last trips still target LDS
    __syncthreads();
    float* ex = reinterpret_cast<float*>(lds_raw);  // [wn][2 x 8 x 4][64 lanes]
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) {
        if (kg == 1) {
#pragma unroll
            for (int r2 = 0; r2 < 2; ++r2)
#pragma unroll
                for (int t = 0; t < 8; ++t) {
                    const float4_t v = acc[2 * hh + r2][t];
                    float* p = ex + ((wn * 64 + (r2 * 8 + t) * 4) * 64) + lane;
                    p[0] = v.x, p[64] = v.y, p[128] = v.z, p[192] = v.w;
                }
        }
        __syncthreads();
        if (kg == 0 && glu) {
            // gated linear unit: channel tiles 2 hh and 2 hh + 1 of the wave are gate and up of output channels
            // (n0 + 64 wn) / 2 + 16 hh .. of the [M, N / 2] result
            const int ng_ch = n0 + 64 * wn + 32 * hh + 4 * kq;  // gate channels; up channels are 16 further
            float sc[2][4], bs[2][4];
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    sc[h][q] = PRESCALE ? 1.f : (float)st[ng_ch + 16 * h + q];
                    bs[h][q] = bias ? (float)bias[ng_ch + 16 * h + q] : 0.f;
                }
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                float o[4];
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const float g = acc[2 * hh][t][q] + ex[((wn * 64 + t * 4 + q) * 64) + lane];
                    const float u = acc[2 * hh + 1][t][q] + ex[((wn * 64 + (8 + t) * 4 + q) * 64) + lane];
                    o[q] = glu_value(glu, g * sc[0][q] + bs[0][q], u * sc[1][q] + bs[1][q]);
                }
                const int m = m0 + 16 * t + col;
                const size_t at = (size_t)m * (N / 2) + (n0 + 64 * wn) / 2 + 16 * hh + 4 * kq;
                if (m < M) {
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
                float sc[4] = {1.f, 1.f, 1.f, 1.f}, bs[4] = {0.f, 0.f, 0.f, 0.f};
                if constexpr (!PRESCALE) {  // one group per channel: scales are st[n]
                    const half4_t s4 = *reinterpret_cast<const half4_t*>(st + n);
#pragma unroll
                    for (int q = 0; q < 4; ++q)
                        sc[q] = (float)s4[q];
                }
                if (bias) {
                    const half4_t b4 = *reinterpret_cast<const half4_t*>(bias + n);
#pragma unroll
                    for (int q = 0; q < 4; ++q)
                        bs[q] = (float)b4[q];
                }
#pragma unroll
                for (int t = 0; t < 8; ++t) {
                    const float* p = ex + ((wn * 64 + (r2 * 8 + t) * 4) * 64) + lane;
                    const float4_t a = acc[r][t];
                    const float v[4] = {(a.x + p[0]) * sc[0] + bs[0], (a.y + p[64]) * sc[1] + bs[1],
                                        (a.z + p[128]) * sc[2] + bs[2], (a.w + p[192]) * sc[3] + bs[3]};
                    const int m = m0 + 16 * t + col;
                    if (m < M) {
                        if (out_f32) {
                            *reinterpret_cast<float4_t*>(static_cast<float*>(y) + (size_t)m * N + n) =
                                float4_t{v[0], v[1], v[2], v[3]};
                        } else {
                            *reinterpret_cast<half4_t*>(static_cast<half_t*>(y) + (size_t)m * N + n) =
                                half4_t{(half_t)v[0], (half_t)v[1], (half_t)v[2], (half_t)v[3]};
                        }
                    }
                }
            }
        }
        __syncthreads();
    }
}

template <int BITS, bool ZPT, bool PRE>
static int launch_direct_impl(const FcDeviceArgs& a, const LaunchPlan& p, hipStream_t s) {
    const Layout& L = a.layout;
    auto kern = fcc_prefill_direct_kernel<BITS, ZPT, PRE>;
    static bool attr_set = false;  // per instantiation; the attribute is idempotent, a race only repeats it
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)PD_LDS_BYTES);
        if (e != hipSuccess)
            return (int)e;
        attr_set = true;
    }
    hipLaunchKernelGGL(kern, dim3(p.grid[0], p.grid[1], 1), dim3(512), PD_LDS_BYTES, s, (const uint4_t*)a.w,
                       (const half_t*)a.scale, (const uint8_t*)a.zp, (const half_t*)a.x, (const half_t*)a.bias, a.y,
                       (int)a.M, (int)a.N, (int)a.K, (int)L.k_blocks, (int)L.kblocks_per_group, (int)L.groups,
                       L.zp_const, a.out_f32, L.glu);
    return (int)hipGetLastError();
}

template <int BITS, bool ZPT>
static int launch_direct_bits(const FcDeviceArgs& a, const LaunchPlan& p, hipStream_t s) {
    return a.layout.groups == 1 ? launch_direct_impl<BITS, ZPT, false>(a, p, s)
                                : launch_direct_impl<BITS, ZPT, true>(a, p, s);
}

int launch_prefill_direct(const FcDeviceArgs& a, const LaunchPlan& p, void* stream) {
    hipStream_t s = static_cast<hipStream_t>(stream);
    const Layout& L = a.layout;
    if (L.bits == 4)
        return L.zp_table ? launch_direct_bits<4, true>(a, p, s) : launch_direct_bits<4, false>(a, p, s);
    return L.zp_table ? launch_direct_bits<8, true>(a, p, s) : launch_direct_bits<8, false>(a, p, s);
}

}  // namespace ovfcc
