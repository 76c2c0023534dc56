// Prefill kernel for 4-bit weights with register-fed matrix-core operands and fully asynchronous data
// movement: 128 x 256 output tile per workgroup (NT = 8 row tiles of 16), 8 waves; also built with 64 x 256
// tiles (NT = 4) for grids that 128-row tiles would underfill and, for grouped runs whose slices have between 64
// and 128 rows (the experts of a mixture-of-experts layer), with 80 and 96 rows (NT = 5, 6; four stages of
// weights).  The text below describes NT = 8.
//
// 1-D grid, block = 512: workgroup -> (tile, part of K) by tile_work (device_common.h); the first full_tiles
// workgroups own whole tiles in XCD-aware order, the others one of split_k parts of a tile (deterministic
// split-K, prefill_epilogue.h).  K advances one k-block (128 inputs) per step.  The grouped kernel at the end of
// the file runs the same body over a table of nodes, one tile row per node.
//
// Every operand of a k-block travels HBM/L2 -> LDS with buffer loads that write LDS directly (no registers,
// no LDS store instructions), 16 bytes per lane:
//   - the activation tile, 128 rows x 128 inputs f16 = 32 KiB, two k-blocks ahead, three stages; rows are
//     256 bytes without padding and the sixteen 16-byte chunks of row r sit at chunk ^ (r & 15), so the 16
//     rows of one 128-bit read phase hit 16 different bank groups (the swizzle is applied on the global
//     side: a lane fetches the chunk that belongs in its linear LDS slot);
//   - the 16 packed weight tiles of the workgroup's 256 channels (16 KiB), copied verbatim three k-blocks
//     ahead, three stages.  A tile already has the matrix cores' operand layout (lane = channel (lane & 15),
//     eight consecutive inputs per dword at 8 (lane >> 4)): a wave reads its 8 bytes per tile back with one
//     LDS read and unpacks them in registers -- dequantised weights never exist in memory;
//   - the group scales (and zero-points) of the k-block, 512 (+256) bytes, with the weights.
// LDS holds the parameter stages first, then the weight stages, then the activation stages.
// That is 6 to 7 vector-memory instructions per wave and k-block; each one costs the compute unit some
// 15 cycles that nothing overlaps, which is why weights do not come as four 8-byte register loads per wave.
// None of them needs vector address arithmetic in the loop: a lane's part of the offset is fixed, the part that
// advances with the k-block goes in the instruction's scalar offset, and a load past the end of K is switched off
// by a descriptor of length zero.
// A wave waits for its own loads (the vector-memory counter is in order); one bare barrier per k-block
// publishes the activations of this k-block and the weights of the next, and frees the oldest stages (a fence
// would also wait for the loads meant to stay in flight).
//
// Waves: wn = wave & 3 picks 64 of the 256 channels, kg = wave >> 2 picks which two of the four 32-input
// steps of every k-block the wave contracts.  A wave unpacks every weight it uses exactly once and multiplies
// it with all 128 rows (eight 16-row operands read from LDS): 32 v_mfma_f32_16x16x32_f16 per step and 4
// unpacked dwords.  After the last k-block the k-groups exchange halves of their f32 accumulators through LDS
// (each finishes half of the row tiles), add, apply per-channel scale, bias and the gated linear unit and store
// whole 128-byte lines (prefill_epilogue.h).
//
// The inner loop is software-pipelined by hand and pinned with scheduling barriers: between every two MFMAs
// of a step sit one or two vector-ALU operations of the *next* step's unpack, and every few MFMAs one memory
// instruction.  Left to itself the compiler emits these in bursts; the two waves of a SIMD run in lockstep
// between barriers, so a burst in one is a burst in both and the matrix pipe idles.
//
// MFMA roles: A = weights (rows = channels), B = activations (columns = rows m of X); result lane holds
// column m = lane & 15, channels 4 (lane >> 4) + r, so a lane stores four consecutive outputs of one row.
//
// Weights: (q - zp) * s rounded once to f16 for grouped scales; with one group per channel the exact
// integers q - zp go to the matrix cores and the scale multiplies the f32 result.
#include "device_common.h"
#include "prefill_epilogue.h"

namespace ovfcc {

constexpr int PA_BM = 128, PA_BN = 256, PA_BK = 128;  // PA_BM: rows of the full tile (NT = 8 row tiles of 16)
constexpr int PA_STAGES = 3;
constexpr int PA_XQ = 3;  // activation operands in registers: the one in use and PA_XQ - 1 on their way from LDS
constexpr int PA_W_BYTES = 16 * kTileBytes;    // 16 KiB per stage
constexpr int PA_P_BYTES = 1024;               // per group of a k-block: scales (512) + zero-points (256)
// Tiles of 80 and 96 rows stage 96 rows of activations (24 KiB instead of 32) and spend the room on more stages of
// weights and parameters: their weights come from memory rather than from L2 (every slice of a grouped run has its
// own) and need the longer lead.
constexpr int pa_a_bytes(int nt) { return nt == 5 || nt == 6 ? 96 * PA_BK * 2 : PA_BM * PA_BK * 2; }
constexpr int pa_w_stages(int nt) { return nt == 5 || nt == 6 ? 4 : PA_STAGES; }
// 128- and 64-row tiles: 147 KiB with one group per k-block, 150 and 156 KiB with two and four
constexpr unsigned pa_lds_bytes(int nt, int gpb) {
    return (unsigned)(PA_STAGES * pa_a_bytes(nt) + pa_w_stages(nt) * (PA_W_BYTES + PA_P_BYTES * gpb));
}

// The whole kernel for one workgroup's share of one node.  The two kernels below differ only in where the node's
// operands come from.
// GPB: groups per k-block.  With groups of 64 or 32 inputs (GPB = 2 or 4) a staged k-block carries GPB scales and
// zero-points per channel, stored [tile][channel][group]; a wave's k-group kg and step js contract inputs
// 32 (2 kg + js) ..+32 of the k-block, that is group kg (GPB = 2) or 2 kg + js (GPB = 4).
template <bool ZP_TABLE, bool PRESCALE, int NT, int GPB>
__device__ __forceinline__ void prefill_async_body(const uint4_t* __restrict__ wt, const half_t* __restrict__ st,
                                                   const uint8_t* __restrict__ zt, const half_t* __restrict__ x,
                                                   const half_t* __restrict__ bias, void* __restrict__ y,
                                                   float* __restrict__ ws, unsigned* __restrict__ counters, int M, int N,
                                                   int K, int kb_total, int kb_per_group, int ng, int zp_const,
                                                   int out_f32, int glu, const TileWork wk,
                                                   const int* __restrict__ row_map = nullptr, int x_rows = 0) {
    static_assert(NT == 8 || NT == 6 || NT == 5 || NT == 4, "tiles of 128, 96, 80 or 64 rows");
    static_assert(GPB == 1 || ((GPB == 2 || GPB == 4) && PRESCALE), "several groups per k-block: scales go into the weights");
    constexpr int PB = PA_P_BYTES * GPB;  // parameter bytes per stage
    constexpr int WS = pa_w_stages(NT);   // stages of weights and parameters
    // LDS: parameters first, then weights, then activations -- the small, scattered reads of scales and zero-points
    // keep their offsets within the 16 bits of an LDS instruction's immediate
    constexpr int PA_A_BYTES = pa_a_bytes(NT), PA_W_OFF = WS * PB, PA_A_OFF = PA_W_OFF + WS * PA_W_BYTES;
    constexpr int ZOFF = 512 * GPB;       // zero-points follow the scales
    constexpr int NOPS = 5 + 4 + (PRESCALE ? 4 : 0);  // unpack micro-operations per dword
    constexpr int AL = (NT + 1) / 2;                    // activation loads per wave and k-block (32 AL rows staged)
    constexpr int S = 4 * NT;                           // MFMA slots per step (a wave's two steps make a k-block)
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    const lds_byte_ptr lds3 = (lds_byte_ptr)lds_raw;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wn = wave & 3, kg = wave >> 2;
    const int n0 = wk.tile_x * PA_BN, m0 = wk.m0, tile_id = wk.park_slot, split_k = wk.split_k;
    const int col = lane & 15, kq = lane >> 4;
    // split-K: this workgroup contracts k-blocks [kb_lo, kb_hi); loads of k-blocks past kb_hi are sent out of range
    const int kb_lo = wk.kb_lo, kb_hi = wk.kb_hi;

    constexpr unsigned kOob = 0x80000000u;
    constexpr int kRsrcFlags = 0x00020000;
    // Buffer loads: the per-lane part of an offset (row, chunk, lane) is computed once and travels in the vector
    // operand, which the hardware checks against the descriptor's range (rows >= M read zeros); the part that
    // advances with the k-block is uniform and travels in the scalar operand, which is not checked -- a load for a
    // k-block past kb_hi uses a descriptor of length zero instead.  That keeps the loop free of vector address
    // arithmetic.
    const int nt0 = n0 / 16;  // the workgroup's 16 channel tiles
    auto live = [&](int kb, int bytes) { return kb < kb_hi ? bytes : 0; };
#define PA_DESC_X(kb) \
    __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(x), 0, live(kb, (row_map ? x_rows : M) * K * 2), kRsrcFlags)
#define PA_DESC_W(kb)                                                                                  \
    __builtin_amdgcn_make_buffer_rsrc(const_cast<uint4_t*>(wt + (size_t)nt0 * kb_total * 64), 0,        \
                                      live(kb, 16 * kb_total * kTileBytes), kRsrcFlags)
#define PA_DESC_S(kb) \
    __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(st + (size_t)nt0 * ng * 16), 0, live(kb, 16 * ng * 32), kRsrcFlags)
#define PA_DESC_Z(kb)                                                                                       \
    __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(ZP_TABLE ? zt + (size_t)nt0 * ng * 16 : zt), 0, \
                                      ZP_TABLE ? live(kb, 16 * ng * 16) : 0, kRsrcFlags)
    const unsigned g_mul = kb_per_group == 1 ? 0u : (unsigned)((0x100000000ull + kb_per_group - 1) / kb_per_group);

    // ---- activations: direct-to-LDS load i of the wave covers rows 4 AL wave + 4 i .. +3 of the tile (AL loads per
    // wave; 16 wave + 4 i with 128-row tiles); lane -> row (lane >> 4) of those, LDS slot lane & 15 of that row,
    // which holds global chunk (lane & 15) ^ (row & 15).  4 AL wave + 4 i is a multiple of four, so
    // row & 15 = ((4 AL wave + 4 i) & 15) ^ (lane >> 4).  80-row tiles stage 96 rows; the loads of rows past the
    // tile go out of range. ----
    unsigned a_voff[4];  // AL entries in use (a bound that depends on NT does not pass the host pass)
#pragma unroll
    for (int i = 0; i < AL; ++i) {
        const int r0 = 4 * AL * wave + 4 * i;  // first of the load's four rows, uniform
        int row = m0 + r0 + (lane >> 4);
        unsigned dead = r0 >= 16 * NT ? kOob : 0u;
        if (row_map) {
            // the slice gathers its rows itself: row_map[.] names the row of x; rows past the slice and entries that
            // name no row are switched off here (the descriptor spans the whole of x)
            const int src = row < M ? row_map[row] : -1;
            dead |= src < 0 ? kOob : 0u;
            row = src < 0 ? 0 : src;
        }
        a_voff[i] = ((unsigned)(row * K) * 2u + ((unsigned)((lane & 15) ^ (lane >> 4) ^ (r0 & 15)) << 4)) | dead;
    }
    auto dma_a = [&](int kb, int stage, int i) {
        { const __amdgpu_buffer_rsrc_t d_ = PA_DESC_X(kb); __builtin_amdgcn_raw_ptr_buffer_load_lds(d_,
                                                 (lds_void_ptr)(lds3 + PA_A_OFF + stage * PA_A_BYTES + (AL * wave + i) * 1024),
                                                 16, a_voff[i], kb * (PA_BK * 2), 0, 0); }
    };
    // ---- weights: the wave copies tiles 2 wave, 2 wave + 1 of the workgroup's 16 ----
    const unsigned w_voff = lane * 16u;
    auto dma_w = [&](int kb, int stage, int i) {
        const int t = 2 * wave + i;
        { const __amdgpu_buffer_rsrc_t d_ = PA_DESC_W(kb); __builtin_amdgcn_raw_ptr_buffer_load_lds(d_, (lds_void_ptr)(lds3 + PA_W_OFF + stage * PA_W_BYTES + t * kTileBytes),
                                                 16, w_voff, (t * kb_total + kb) * kTileBytes, 0, 0); }
    };
    // ---- parameters: waves 0 and 1 fetch the scales of eight channel tiles each (32 bytes per tile, 4 per
    // lane), wave 2 the zero-points of all sixteen (16 bytes per tile, 4 per lane); other waves fetch nothing ----
    // With two groups per k-block (64 and 32 bytes per tile): wave 0 the scales, 16 bytes per lane; waves 2 and 3
    // the zero-points of eight tiles each.  With four (128 and 64 bytes per tile): waves 0 and 1 the scales of
    // eight tiles each and wave 2 the zero-points, 16 bytes per lane.  No wave issues more than one such load.
    const bool has_p = GPB == 1   ? (PRESCALE && wave < 2) || (ZP_TABLE && wave == 2)
                       : GPB == 2 ? wave == 0 || (ZP_TABLE && (wave == 2 || wave == 3))
                                  : wave < 2 || (ZP_TABLE && wave == 2);
    // the lane's part of its parameter load's offset (the tile's row of the table and the lane's bytes in it)
    unsigned p_voff = 0;
    if constexpr (GPB == 1) {
        if (PRESCALE && wave < 2)
            p_voff = (8u * wave + (lane >> 3)) * ng * 32u + (lane & 7) * 4u;
        else if (ZP_TABLE && wave == 2)
            p_voff = (lane >> 2) * ng * 16u + (lane & 3) * 4u;
    } else if constexpr (GPB == 2) {
        if (wave == 0)
            p_voff = (lane >> 2) * kb_total * 64u + (lane & 3) * 16u;
        else if (ZP_TABLE && (wave == 2 || wave == 3))
            p_voff = (8u * (wave - 2) + (lane >> 3)) * kb_total * 32u + (lane & 7) * 4u;
    } else {
        if (wave < 2)
            p_voff = (8u * wave + (lane >> 3)) * kb_total * 128u + (lane & 7) * 16u;
        else if (ZP_TABLE && wave == 2)
            p_voff = (lane >> 2) * kb_total * 64u + (lane & 3) * 16u;
    }
    auto dma_p = [&](int kb, int stage) {
        const lds_byte_ptr pbase = lds3 + stage * PB;
        if constexpr (GPB == 1) {
            const int g = kb_per_group == 1 ? kb : (int)__umulhi((unsigned)kb, g_mul);
            if (PRESCALE && wave < 2)
                { const __amdgpu_buffer_rsrc_t d_ = PA_DESC_S(kb); __builtin_amdgcn_raw_ptr_buffer_load_lds(d_, (lds_void_ptr)(pbase + 256 * wave), 4, p_voff, g * 32, 0, 0); }
            else if (ZP_TABLE && wave == 2)
                { const __amdgpu_buffer_rsrc_t d_ = PA_DESC_Z(kb); __builtin_amdgcn_raw_ptr_buffer_load_lds(d_, (lds_void_ptr)(pbase + ZOFF), 4, p_voff, g * 16, 0, 0); }
        } else if constexpr (GPB == 2) {
            if (wave == 0)
                { const __amdgpu_buffer_rsrc_t d_ = PA_DESC_S(kb); __builtin_amdgcn_raw_ptr_buffer_load_lds(d_, (lds_void_ptr)pbase, 16, p_voff, kb * 64, 0, 0); }
            else if (ZP_TABLE && (wave == 2 || wave == 3))
                { const __amdgpu_buffer_rsrc_t d_ = PA_DESC_Z(kb); __builtin_amdgcn_raw_ptr_buffer_load_lds(d_, (lds_void_ptr)(pbase + ZOFF + 256 * (wave - 2)), 4,
                                                         p_voff, kb * 32, 0, 0); }
        } else {
            if (wave < 2)
                { const __amdgpu_buffer_rsrc_t d_ = PA_DESC_S(kb); __builtin_amdgcn_raw_ptr_buffer_load_lds(d_, (lds_void_ptr)(pbase + 1024 * wave), 16, p_voff, kb * 128, 0, 0); }
            else if (ZP_TABLE && wave == 2)
                { const __amdgpu_buffer_rsrc_t d_ = PA_DESC_Z(kb); __builtin_amdgcn_raw_ptr_buffer_load_lds(d_, (lds_void_ptr)(pbase + ZOFF), 16, p_voff, kb * 64, 0, 0); }
        }
    };
    // Per k-block a wave issues, in this order: AL activation loads (for k-block + 2), then 2 weight
    // loads and at most one parameter load (for k-block + WS).  The wait at the top of a k-block needs the
    // activations of this k-block and the weights and parameters of the next; the instructions issued after those
    // are one k-block's worth, at least AL + 2; with more than three stages the weights of the next k-block were
    // requested before the activations of this one, and the two weight loads that followed those may be in flight too.
    constexpr int kWaitTop = WS == 3 ? AL + 2 : AL + 4;

    // ---- the wave's share of a staged k-block of weights: 8 bytes per tile, plus scale and zero-point ----
    typedef __attribute__((address_space(3))) const uint2_t* lds_u2_ptr;
    typedef __attribute__((address_space(3))) const half_t* lds_half_ptr;
    uint32_t wraw[2][4][2];
    typedef __attribute__((address_space(3))) const uint32_t* lds_u32_ptr;
    typedef __attribute__((address_space(3))) const uint16_t* lds_u16_ptr;
    uint32_t wscale[2][4];  // f16 scale in both halves; GPB == 4: the scales of step 0 and step 1
    uint32_t wzp[2][4];     // zero-point; GPB == 4: those of step 0 and step 1 in bytes 0 and 1
    auto read_w = [&](int par, int stage, int r) {
        const uint2_t v = *(lds_u2_ptr)(lds3 + PA_W_OFF + stage * PA_W_BYTES + (4 * wn + r) * kTileBytes + lane * 16 + kg * 8);
        wraw[par][r][0] = v.x, wraw[par][r][1] = v.y;
    };
    auto read_p = [&](int par, int stage, int r) {
        const lds_byte_ptr pbase = lds3 + stage * PB;
        if constexpr (GPB == 4) {
            // groups 2 kg (step 0) and 2 kg + 1 (step 1) of the lane's channel
            const uint32_t v = *(lds_u32_ptr)(pbase + (4 * wn + r) * 128 + col * 8 + kg * 4);
            wscale[par][r] = v;
            if constexpr (ZP_TABLE)
                wzp[par][r] = *(lds_u16_ptr)(pbase + ZOFF + (4 * wn + r) * 64 + col * 4 + kg * 2);
        } else {
            // GPB == 2: group kg of the lane's channel
            if constexpr (PRESCALE) {
                const half_t h = *(lds_half_ptr)(pbase + (4 * wn + r) * 32 * GPB + col * 2 * GPB + (GPB == 2 ? kg * 2 : 0));
                wscale[par][r] = as_u32(half2_t{h, h});
            }
            if constexpr (ZP_TABLE)
                wzp[par][r] = pbase[ZOFF + (4 * wn + r) * 16 * GPB + col * GPB + (GPB == 2 ? kg : 0)];
        }
    };

    // ---- unpack, one micro-operation at a time: dword js of tile r of parity par -> f ----
    const Unpack4Consts uc = unpack4_consts();
    // uniform values the vector ALU can take as its one scalar operand are kept in scalar registers
    const half2_t off_lo_c = as_half2(__builtin_amdgcn_readfirstlane(as_u32(splat(1024.f + (float)zp_const))));
    const half2_t off_hi_c = as_half2(__builtin_amdgcn_readfirstlane(as_u32(splat(64.f + (float)zp_const))));
    auto unpack_op = [&](int par, int r, int js, int op, Frag8& f) {
        const uint32_t w = wraw[par][r][js];
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
        else if (op < 9) {
            const int k = op - 5;
            half2_t off;
            if constexpr (ZP_TABLE) {
                // 1024 + zp in both halves with one integer operation (f16 1024 .. 2047 are 0x6400 + n), and
                // 64 + zp = (1024 + zp) - 960 with one packed subtraction; both exact for zp <= 255
                const uint32_t zpv = GPB == 4 ? (wzp[par][r] >> (8 * js)) & 0xFFu : wzp[par][r];
                const half2_t lo = as_half2(zpv * 0x00010001u + 0x64006400u);
                off = (k & 1) ? lo - half2_t{(half_t)960.f, (half_t)960.f} : lo;
            } else {
                off = (k & 1) ? off_hi_c : off_lo_c;
            }
            f.h2[k] = f.h2[k] - off;
        } else if constexpr (PRESCALE) {
            const half2_t sv = as_half2(wscale[par][r]);
            f.h2[op - 9] *= GPB == 4 ? half2_t{sv[js], sv[js]} : sv;
        }
    };

    float4_t acc[4][NT];  // [channel tile][row tile]
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int t = 0; t < NT; ++t)
            acc[r][t] = float4_t{0.f, 0.f, 0.f, 0.f};

    // One k-block: 64 MFMAs -- step 0 with operand wf0 while the unpack of (par_a, dword 1) fills wf1, then
    // step 1 with wf1 while the unpack of (par_b, dword 0) refills wf0 -- against the eight row tiles of this
    // wave's two k-steps in activation stage `stage`; mem(i) adds the memory instructions of slot i.  The
    // activation operands run PA_XQ - 1 row tiles ahead of the MFMAs, across the boundary between the steps.
    auto block = [&](int stage, Frag8 (&wf0)[4], Frag8 (&wf1)[4], int par_a, int par_b, auto&& mem) {
        typedef __attribute__((address_space(3))) const half8_t* lds_frag_ptr;
        // operand of row tile t and step js: row 16 t + col, chunk (4 (2 kg + js) + kq) ^ col
        const lds_byte_ptr xa0 = lds3 + PA_A_OFF + stage * PA_A_BYTES + col * 256 + (((8 * kg + kq) ^ col) << 4);
        const lds_byte_ptr xa1 = lds3 + PA_A_OFF + stage * PA_A_BYTES + col * 256 + (((8 * kg + 4 + kq) ^ col) << 4);
        auto x_at = [&](int tt) { return *(lds_frag_ptr)((tt < NT ? xa0 : xa1) + (tt % NT) * 16 * 256); };
        half8_t xq[PA_XQ];
#pragma unroll
        for (int tt = 0; tt < PA_XQ - 1; ++tt)
            xq[tt] = x_at(tt);
        auto slot = [&](int i) {
            const int tt = i >> 2, r = i & 3;  // tt = NT js + t
            if (r == 0 && tt + PA_XQ - 1 < 2 * NT)
                xq[(tt + PA_XQ - 1) % PA_XQ] = x_at(tt + PA_XQ - 1);
            const int t = tt % NT;
            if (i < S) {
                acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wf0[r].v, xq[tt % PA_XQ], acc[r][t], 0, 0, 0);
#pragma unroll
                for (int g = i * 4 * NOPS / S; g < (i + 1) * 4 * NOPS / S; ++g)
                    unpack_op(par_a, g / NOPS, 1, g % NOPS, wf1[g / NOPS]);
            } else {
                acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wf1[r].v, xq[tt % PA_XQ], acc[r][t], 0, 0, 0);
#pragma unroll
                for (int g = (i - S) * 4 * NOPS / S; g < (i - S + 1) * 4 * NOPS / S; ++g)
                    unpack_op(par_b, g / NOPS, 0, g % NOPS, wf0[g / NOPS]);
            }
            mem(i);
            __builtin_amdgcn_sched_barrier(0);
        };
#pragma unroll
        for (int i = 0; i < S; ++i)
            slot(i);
#pragma unroll
        for (int i = S; i < 2 * S; ++i)
            slot(i);
    };

    // ---- prologue: activations of k-blocks 0, 1; weights and parameters of k-blocks 0, 1, 2; everything
    // landed and published; first operand unpacked ----
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int i = 0; i < AL; ++i)
            dma_a(kb_lo + j, j, i);
#pragma unroll
    for (int j = 0; j < WS; ++j) {
        dma_w(kb_lo + j, j, 0);
        dma_w(kb_lo + j, j, 1);
        if (has_p)
            dma_p(kb_lo + j, j);
    }
    __builtin_amdgcn_s_waitcnt(wait_vmcnt_imm(0));
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    Frag8 wf0[4], wf1[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        read_w(0, 0, r);
        read_p(0, 0, r);
    }
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int op = 0; op < NOPS; ++op)
            unpack_op(0, r, 0, op, wf0[r]);

    // ---- main loop: two k-blocks per trip so that the parity of the weight registers is static.  k-blocks
    // past the end are loaded out of range (zeros) and add nothing. ----
    int s0 = 0;  // stage of k-block kb's activations: kb % 3
    int w0 = 0;  // stage of its weights and parameters: kb % WS
    for (int kb0 = kb_lo; kb0 < kb_hi; kb0 += 2) {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int kb = kb0 + u;
            const int s1 = s0 == 2 ? 0 : s0 + 1;  // stage of k-block kb + 1 and kb - 2
            const int s2 = s1 == 2 ? 0 : s1 + 1;  // stage of k-block kb + 2 and kb - 1
            const int w1 = w0 == WS - 1 ? 0 : w0 + 1;
            // own loads landed: activations of kb, weights and parameters of kb + 1
            __builtin_amdgcn_s_waitcnt(wait_vmcnt_imm(kWaitTop));
            asm volatile("" ::: "memory");
            __builtin_amdgcn_s_barrier();  // everyone's have; everyone is done with k-block kb - 1
            asm volatile("" ::: "memory");
            // Slots 0-31 (first step): request the activations of k-block kb + 2 into the stage k-block kb - 1
            // used; towards the end fetch the next k-block's weight bits and parameters from LDS.  Slots 32-63:
            // request the weights and parameters of k-block kb + 3 into the stage those of k-block kb used
            // (every wave read them before the barrier above).
            block(s0, wf0, wf1, u, u ^ 1, [&](int i) {
                if (i < S && (i & 7) == 2)
                    dma_a(kb + 2, s2, i >> 3);
                if (i >= S - 8 && i < S - 4)
                    read_p(u ^ 1, w1, i - (S - 8));
                if (i >= S - 4 && i < S)
                    read_w(u ^ 1, w1, i - (S - 4));
                if (i == S + 4)
                    dma_w(kb + WS, w0, 0);
                if (i == S + 4 + S / 2)
                    dma_w(kb + WS, w0, 1);
                if (i == S + 4 + S / 4 && has_p)
                    dma_p(kb + WS, w0);
            });
            s0 = s1;
            w0 = w1;
        }
    }

    // ---- epilogue (prefill_epilogue.h): the k-groups exchange halves, scale / bias / gated linear unit, split-K fix-up ----
    __builtin_amdgcn_s_waitcnt(wait_vmcnt_imm(0));  // the out-of-range loads of the last trips still target LDS
    static_assert(pa_lds_bytes(NT, GPB) >= 8u * 4u * ((NT + 1) / 2) * 1024u, "the epilogue's exchange buffer");
    tile_epilogue_shared<PRESCALE, NT>(acc, lds_raw, st, bias, y, ws, counters, M, N, n0, m0, split_k, wk.z, tile_id,
                                       out_f32, glu);
}
#undef PA_DESC_X
#undef PA_DESC_W
#undef PA_DESC_S
#undef PA_DESC_Z

template <bool ZP_TABLE, bool PRESCALE, int NT, int GPB>
__global__ __launch_bounds__(512) void fcc_prefill_async_kernel(const uint4_t* __restrict__ wt,
                                                                const half_t* __restrict__ st,
                                                                const uint8_t* __restrict__ zt,
                                                                const half_t* __restrict__ x,
                                                                const half_t* __restrict__ bias,
                                                                void* __restrict__ y, float* __restrict__ ws,
                                                                unsigned* __restrict__ counters, int M, int N, int K,
                                                                int kb_total, int kb_per_group, int ng, int zp_const,
                                                                int out_f32, int glu, int tiles_x, int tiles_y,
                                                                int full_tiles, int tail_split, int kb_per_split) {
    const TileWork wk = tile_work(tiles_x, tiles_y, full_tiles, tail_split, kb_per_split, kb_total, 16 * NT, PA_BN / 2);
    prefill_async_body<ZP_TABLE, PRESCALE, NT, GPB>(wt, st, zt, x, bias, y, ws, counters, M, N, K, kb_total,
                                                    kb_per_group, ng, zp_const, out_f32, glu, wk);
}

// Grouped launch: tile row tile_y is item tile_y of the table, a node of the common shape and format with at most
// 128 rows of its own (the experts of a mixture-of-experts layer over their gathered rows).  Workgroups of one
// item sit together in a super-tile and share its activations in L2.
template <bool ZP_TABLE, bool PRESCALE, int NT, int GPB>
__global__ __launch_bounds__(512) void fcc_prefill_async_grouped_kernel(const BatchGroupTable tab,
                                                                        const BatchGroupItem* __restrict__ dev_tab,
                                                                        const RoutedHeader* __restrict__ dev_hdr,
                                                                        float* __restrict__ ws,
                                                                        unsigned* __restrict__ counters, int N, int K,
                                                                        int kb_total, int kb_per_group, int ng,
                                                                        int zp_const, int out_f32, int glu,
                                                                        int tiles_x, int tiles_y, int full_tiles,
                                                                        int tail_split, int kb_per_split,
                                                                        const int* __restrict__ row_map, int x_rows) {
    // the table travels in the kernel arguments, or -- when the rows were bucketed on the device -- lies in memory,
    // with the slice count and the cut along K that the routing kernel chose for it
    if (dev_tab) {
        const RoutedHeader h = *dev_hdr;
        if ((int)blockIdx.x >= h.grid)
            return;
        tiles_y = h.tiles_y, tail_split = h.split_k, kb_per_split = h.kb_per_split, full_tiles = h.full_tiles;
    }
    TileWork wk = tile_work(tiles_x, tiles_y, full_tiles, tail_split, kb_per_split, kb_total, 16 * NT, PA_BN / 2);
    BatchGroupItem it = dev_tab ? dev_tab[wk.tile_y] : tab.item[wk.tile_y];
    // The item is the same for every lane, but the compiler cannot tell: without this, every buffer load of the body
    // sits in a loop that looks for lanes with equal descriptors (six vector instructions and a branch per load).
    it.w = uniform_ptr(it.w), it.scale = uniform_ptr(it.scale), it.zp = uniform_ptr(it.zp);
    it.bias = uniform_ptr(it.bias), it.x = uniform_ptr(it.x), it.y = const_cast<void*>(uniform_ptr(it.y));
    it.M = __builtin_amdgcn_readfirstlane(it.M);
    if (it.M <= 0)
        return;
    wk.m0 = 0;
    prefill_async_body<ZP_TABLE, PRESCALE, NT, GPB>((const uint4_t*)it.w, (const half_t*)it.scale,
                                                    (const uint8_t*)it.zp, (const half_t*)it.x, (const half_t*)it.bias,
                                                    it.y, ws, counters, it.M, N, K, kb_total, kb_per_group, ng, zp_const,
                                                    out_f32, glu, wk,
                                                    row_map ? row_map + __builtin_amdgcn_readfirstlane(it.reserved) : nullptr,
                                                    x_rows);
}

template <typename Kern>
static int allow_lds(Kern kern, bool* done, unsigned bytes) {
    if (*done)
        return 0;  // the attribute is idempotent, a race only repeats it
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)bytes);
    if (e == hipSuccess)
        *done = true;
    return (int)e;
}

// The launch must be what async_work assumes: a 1-D grid of full_tiles whole tiles plus split_k parts of each
// remaining tile, parts that cover K.
static bool async_plan_ok(const FcDeviceArgs& a, const LaunchPlan& p) {
    const int64_t tiles = (int64_t)p.tiles_x * p.tiles_y;
    return (p.tile_m == 128 || p.tile_m == 96 || p.tile_m == 80 || p.tile_m == 64) && p.tiles_x == a.N / PA_BN && p.tiles_y >= 1 && p.full_tiles >= 0 && p.full_tiles <= tiles && p.split_k >= 1 &&
           (int64_t)p.kblocks_per_split * p.split_k >= a.layout.k_blocks && (p.full_tiles == tiles || p.kblocks_per_split >= 1) &&
           p.grid[0] == (unsigned)(p.full_tiles + (tiles - p.full_tiles) * p.split_k) && p.grid[1] == 1 && p.grid[2] == 1 &&
           (p.split_k == 1 || (a.workspace && a.counters));
}

template <bool ZPT, bool PRE, int NT, int GPB>
static int launch_async_gpb(const FcDeviceArgs& a, const LaunchPlan& p, hipStream_t s) {
    const Layout& L = a.layout;
    auto kern = fcc_prefill_async_kernel<ZPT, PRE, NT, GPB>;
    static bool attr_set = false;  // per instantiation
    if (int e = allow_lds(kern, &attr_set, pa_lds_bytes(NT, GPB)))
        return e;
    hipLaunchKernelGGL(kern, dim3(p.grid[0], p.grid[1], p.grid[2]), dim3(512), pa_lds_bytes(NT, GPB), s, (const uint4_t*)a.w,
                       (const half_t*)a.scale, (const uint8_t*)a.zp, (const half_t*)a.x, (const half_t*)a.bias, a.y,
                       a.workspace, a.counters, (int)a.M, (int)a.N, (int)a.K, (int)L.k_blocks,
                       (int)L.kblocks_per_group, (int)L.groups, L.zp_const, a.out_f32, L.glu, p.tiles_x,
                       p.tiles_y, p.full_tiles, p.split_k, p.kblocks_per_split);
    return (int)hipGetLastError();
}

template <bool ZPT, bool PRE, int NT>
static int launch_async_impl(const FcDeviceArgs& a, const LaunchPlan& p, hipStream_t s) {
    if constexpr (PRE) {
        if (a.layout.groups_per_kblock == 2)
            return launch_async_gpb<ZPT, PRE, NT, 2>(a, p, s);
        if (a.layout.groups_per_kblock == 4)
            return launch_async_gpb<ZPT, PRE, NT, 4>(a, p, s);
    }
    return launch_async_gpb<ZPT, PRE, NT, 1>(a, p, s);
}

template <bool ZPT, bool PRE, int NT, int GPB>
static int launch_async_grouped_gpb(const BatchGroupTable& tab, const BatchGroupItem* dev_tab,
                                    const RoutedHeader* dev_hdr, const FcDeviceArgs& a, const LaunchPlan& p,
                                    hipStream_t s) {
    const Layout& L = a.layout;
    auto kern = fcc_prefill_async_grouped_kernel<ZPT, PRE, NT, GPB>;
    static bool attr_set = false;  // per instantiation
    if (int e = allow_lds(kern, &attr_set, pa_lds_bytes(NT, GPB)))
        return e;
    hipLaunchKernelGGL(kern, dim3(p.grid[0], p.grid[1], p.grid[2]), dim3(512), pa_lds_bytes(NT, GPB), s, tab, dev_tab,
                       dev_hdr, a.workspace, a.counters, (int)a.N, (int)a.K, (int)L.k_blocks, (int)L.kblocks_per_group, (int)L.groups,
                       L.zp_const, a.out_f32, L.glu, p.tiles_x, p.tiles_y, p.full_tiles, p.split_k,
                       p.kblocks_per_split, a.row_map, (int)a.x_rows);
    return (int)hipGetLastError();
}

template <bool ZPT, bool PRE, int NT>
static int launch_async_grouped_impl(const BatchGroupTable& tab, const BatchGroupItem* dev_tab,
                                     const RoutedHeader* dev_hdr, const FcDeviceArgs& a, const LaunchPlan& p,
                                     hipStream_t s) {
    if constexpr (PRE) {
        if (a.layout.groups_per_kblock == 2)
            return launch_async_grouped_gpb<ZPT, PRE, NT, 2>(tab, dev_tab, dev_hdr, a, p, s);
        if (a.layout.groups_per_kblock == 4)
            return launch_async_grouped_gpb<ZPT, PRE, NT, 4>(tab, dev_tab, dev_hdr, a, p, s);
    }
    return launch_async_grouped_gpb<ZPT, PRE, NT, 1>(tab, dev_tab, dev_hdr, a, p, s);
}

// dispatch on zero-point table, per-group scales and tile height
#define OVFCC_ASYNC_DISPATCH(FN, ...)                                                                    \
    (L.groups == 1 ? (L.zp_table ? (nt8 ? FN<true, false, 8>(__VA_ARGS__) : FN<true, false, 4>(__VA_ARGS__))    \
                                 : (nt8 ? FN<false, false, 8>(__VA_ARGS__) : FN<false, false, 4>(__VA_ARGS__)))  \
                   : (L.zp_table ? (nt8 ? FN<true, true, 8>(__VA_ARGS__) : FN<true, true, 4>(__VA_ARGS__))      \
                                 : (nt8 ? FN<false, true, 8>(__VA_ARGS__) : FN<false, true, 4>(__VA_ARGS__))))

int launch_prefill_async(const FcDeviceArgs& a, const LaunchPlan& p, void* stream) {
    hipStream_t s = static_cast<hipStream_t>(stream);
    const Layout& L = a.layout;
    // (the planner sends 8-bit nodes to the register-ring kernel)
    if (L.bits != 4 || !async_plan_ok(a, p) || (int64_t)p.tiles_y * p.tile_m < a.M || (p.tile_m != PA_BM && p.tile_m != PA_BM / 2))
        return (int)hipErrorInvalidValue;
    const bool nt8 = p.tile_m == PA_BM;
    return OVFCC_ASYNC_DISPATCH(launch_async_impl, a, p, s);
}

// p plans one node of n_items * tile_m rows: its tile rows are the items of the table.  dev_tab and dev_hdr
// (optional, both or none): table and header in device memory, written by the routing kernel earlier on the same
// stream -- at most n_items entries of at most tile_m rows each; how many are in use and how K is cut for them is
// the header's word, and p only sizes the launch: a 1-D grid, workspace and counters that hold
// routed_header(tiles_x, t, k_blocks, .).grid workgroups for every t <= n_items.  `tab` is then ignored and n_items
// is not limited to kMaxGroupItems.
int launch_prefill_async_grouped(const BatchGroupTable& tab, int n_items, const FcDeviceArgs& a, const LaunchPlan& p,
                                 void* stream, const BatchGroupItem* dev_tab, const RoutedHeader* dev_hdr) {
    hipStream_t s = static_cast<hipStream_t>(stream);
    const Layout& L = a.layout;
    if (L.bits != 4 || n_items < 1 || p.tiles_y != n_items || !dev_tab != !dev_hdr ||
        (a.row_map && (!dev_tab || a.x_rows < 1 || a.x_rows * a.K * 2 >= ((int64_t)1 << 31))))
        return (int)hipErrorInvalidValue;
    if (!dev_tab) {
        if (!async_plan_ok(a, p) || n_items > kMaxGroupItems)
            return (int)hipErrorInvalidValue;
        for (int i = 0; i < n_items; ++i)
            if (tab.item[i].M < 1 || tab.item[i].M > p.tile_m)
                return (int)hipErrorInvalidValue;
    } else {
        if ((p.tile_m != 128 && p.tile_m != 96 && p.tile_m != 80 && p.tile_m != 64) || p.tiles_x != a.N / PA_BN || p.grid[1] != 1 || p.grid[2] != 1)
            return (int)hipErrorInvalidValue;
        for (int t = 1; t <= n_items; ++t) {
            const RoutedHeader h = routed_header(p.tiles_x, t, (int)L.k_blocks, p.n_cus);
            if ((unsigned)h.grid > p.grid[0] ||
                (h.split_k > 1 && (!a.workspace || !a.counters ||
                                   (size_t)routed_parked_tiles(h, p.tiles_x) * p.tile_m * PA_BN * sizeof(float) > p.workspace_bytes ||
                                   (size_t)p.tiles_x * t > p.counter_count)))
                return (int)hipErrorInvalidValue;
        }
    }
    if (p.tile_m == 80 || p.tile_m == 96) {
        // slices of 80 and 96 rows: one group per k-block only
        if (L.groups_per_kblock != 1)
            return (int)hipErrorInvalidValue;
        const bool nt5 = p.tile_m == 80;
#define OVFCC_ASYNC_MID(ZPT, PRE)                                                                          \
    (nt5 ? launch_async_grouped_gpb<ZPT, PRE, 5, 1>(tab, dev_tab, dev_hdr, a, p, s)                         \
         : launch_async_grouped_gpb<ZPT, PRE, 6, 1>(tab, dev_tab, dev_hdr, a, p, s))
        return L.groups == 1 ? (L.zp_table ? OVFCC_ASYNC_MID(true, false) : OVFCC_ASYNC_MID(false, false))
                             : (L.zp_table ? OVFCC_ASYNC_MID(true, true) : OVFCC_ASYNC_MID(false, true));
#undef OVFCC_ASYNC_MID
    }
    const bool nt8 = p.tile_m == PA_BM;
    return OVFCC_ASYNC_DISPATCH(launch_async_grouped_impl, tab, dev_tab, dev_hdr, a, p, s);
}
#undef OVFCC_ASYNC_DISPATCH

}  // namespace ovfcc
