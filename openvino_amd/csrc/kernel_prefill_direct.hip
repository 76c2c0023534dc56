// Prefill kernel with register-fed weights: 128 x 256 output tile per workgroup, 8 waves.  Runs the 8-bit
// nodes (three stages of an 8-bit k-block of tiles do not fit in LDS beside the activations, so the 4-bit
// kernel's all-asynchronous form does not carry over) and, on request, 4-bit ones.
//
// 1-D grid, block = 512: workgroup -> (tile, part of K) by tile_work (device_common.h), deterministic split-K
// and the rest of the epilogue in prefill_epilogue.h.  K advances one k-block (128 inputs) per step.
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
// accumulators to k-group 0 through LDS, which adds, applies per-channel scale, bias and the gated linear unit
// and stores.
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
#include "prefill_epilogue.h"

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
                                                                 void* __restrict__ y, float* __restrict__ ws,
                                                                 unsigned* __restrict__ counters, int M, int N, int K,
                                                                 int kb_total, int kb_per_group, int ng, int zp_const,
                                                                 int out_f32, int glu, int tiles_x, int tiles_y,
                                                                 int full_tiles, int tail_split, int kb_per_split) {
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
    // split-K: this workgroup contracts k-blocks [kb_lo, kb_hi); loads of k-blocks past kb_hi are sent out of range
    const TileWork wk = tile_work(tiles_x, tiles_y, full_tiles, tail_split, kb_per_split, kb_total, PD_BM, PD_BN * BITS / 8);
    const int n0 = wk.tile_x * PD_BN;
    const int m0 = wk.m0;
    const int kb_lo = wk.kb_lo, kb_hi = wk.kb_hi;
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
        const unsigned oob = (unsigned)((kb_hi - 1 - kb) >> 31) & kOob;
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
        const unsigned oob = (unsigned)((kb_hi - 1 - kb) >> 31) & kOob;
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
        const unsigned oob = (unsigned)((kb_hi - 1 - kb) >> 31) & kOob;
        const unsigned g = kb_per_group == 1 ? (unsigned)kb : __umulhi((unsigned)kb, g_mul);
        rscale[slot][r] =
            __builtin_amdgcn_raw_buffer_load_b32(
                rs, (__builtin_amdgcn_readfirstlane((r * ng + g) * 32u) + (unsigned)(col & ~1) * 2u) | oob, 0, 0);
    };
    auto load_z = [&](int kb, int slot, int r) {
        const unsigned oob = (unsigned)((kb_hi - 1 - kb) >> 31) & kOob;
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
    for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i)
            dma_a(kb_lo + j, i);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
#pragma unroll
        for (int r = 0; r < 4; ++r)
            load_w(kb_lo + j, j, r);
        if constexpr (PRESCALE)
#pragma unroll
            for (int r = 0; r < 4; ++r)
                load_s(kb_lo + j, j, r);
        if constexpr (ZP_TABLE)
#pragma unroll
            for (int r = 0; r < 4; ++r)
                load_z(kb_lo + j, j, r);
    }
    Frag8 wf0[4], wf1[4];
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int op = 0; op < NOPS; ++op)
            unpack_op(0, r, 0, op, wf0[r]);

    // ---- main loop: two k-blocks per trip so that ring slots are static.  k-blocks past the end are loaded
    // out of range (zeros) and add nothing. ----
    for (int kb0 = kb_lo; kb0 < kb_hi; kb0 += 2) {
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

    // ---- epilogue (prefill_epilogue.h): k-group hand-over, scale / bias / gated linear unit, split-K fix-up ----
    __builtin_amdgcn_s_waitcnt(wait_vmcnt_imm(0));  // the out-of-range loads of the last trips still target LDS
    tile_epilogue<PRESCALE, 8>(acc, lds_raw, st, bias, y, ws, counters, M, N, n0, m0, wk.split_k, wk.z, wk.park_slot,
                               out_f32, glu);
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
    hipLaunchKernelGGL(kern, dim3(p.grid[0], p.grid[1], p.grid[2]), dim3(512), PD_LDS_BYTES, s, (const uint4_t*)a.w,
                       (const half_t*)a.scale, (const uint8_t*)a.zp, (const half_t*)a.x, (const half_t*)a.bias, a.y,
                       a.workspace, a.counters, (int)a.M, (int)a.N, (int)a.K, (int)L.k_blocks,
                       (int)L.kblocks_per_group, (int)L.groups, L.zp_const, a.out_f32, L.glu, p.tiles_x, p.tiles_y,
                       p.full_tiles, p.split_k, p.kblocks_per_split);
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
    // the launch must be what tile_work assumes: a 1-D grid of full_tiles whole tiles plus split_k parts of each
    // remaining tile, parts that cover K and rows that cover M
    const int64_t tiles = (int64_t)p.tiles_x * p.tiles_y;
    if (L.groups_per_kblock != 1)
        return (int)hipErrorInvalidValue;  // groups below 128 inputs: the planner picks another kernel
    if (p.tile_m != PD_BM || p.tiles_x != a.N / PD_BN || (int64_t)p.tiles_y * PD_BM < a.M || p.full_tiles < 0 ||
        p.full_tiles > tiles || p.split_k < 1 || (int64_t)p.kblocks_per_split * p.split_k < L.k_blocks ||
        p.grid[0] != (unsigned)(p.full_tiles + (tiles - p.full_tiles) * p.split_k) || p.grid[1] != 1 || p.grid[2] != 1 ||
        (p.split_k > 1 && !(a.workspace && a.counters)))
        return (int)hipErrorInvalidValue;
    if (L.bits == 4)
        return L.zp_table ? launch_direct_bits<4, true>(a, p, s) : launch_direct_bits<4, false>(a, p, s);
    return L.zp_table ? launch_direct_bits<8, true>(a, p, s) : launch_direct_bits<8, false>(a, p, s);
}

}  // namespace ovfcc
