// Prefill kernel for 4-bit weights with 256 x 256 output tiles: four waves per workgroup, one per SIMD, each with
// the 512 registers a wave owns when it has a SIMD to itself -- the 256 accumulation registers hold the wave's
// 64 channels x 256 rows of f32 results, the 256 ordinary ones everything else.  Against the 128 x 256 kernel
// (kernel_prefill_async.hip) every unpacked weight meets twice as many rows, so the vector-ALU work per MFMA and the
// weight traffic per flop halve, and no two waves contract the same outputs: there is no hand-over at the end.
//
// 1-D grid, block = 256: workgroup -> tile in XCD-aware order (tile_work, device_common.h); whole tiles only, no
// split along K.  Wave w owns channel tiles 4 w .. 4 w + 3 of the workgroup's 16 and all sixteen 16-row tiles.
//
// Data movement per k-block (128 inputs):
//   - weights: the wave's four packed tiles come HBM/L2 -> registers, one 128-bit load per lane and tile, one
//     k-block ahead.  A tile has the matrix cores' operand layout (lane = channel (lane & 15), dword j = inputs
//     32 j + 8 (lane >> 4) ..+8), and no other wave needs them: they never touch LDS.  Scales and zero-points of the
//     lane's channel travel with them.
//   - activations: 256 rows x 64 inputs (32 KiB, half a k-block) per stage, four stages, HBM/L2 -> LDS by
//     direct-to-LDS loads (16 bytes per lane, eight rows of 128 bytes per instruction), three halves ahead.  The
//     eight 16-byte chunks of row r sit at chunk ^ ((r >> 1) & 7), applied on the global side, so that the sixteen
//     rows of a 128-bit operand read fall into sixteen different bank groups.
// One barrier per half k-block (128 MFMAs per wave) publishes the stage of this half and frees the oldest one.
//
// MFMA roles as in the 128 x 256 kernel: A = weights (rows = channels), B = activations (columns = rows m of X);
// a lane holds column m = lane & 15, channels 4 (lane >> 4) + q of a 16 x 16 result and stores four consecutive
// channels of one row.  Grouped scales: (q - zp) * s rounded once to f16; one group per channel: exact integers,
// scale in the epilogue.
#include "device_common.h"

namespace ovfcc {

constexpr int PB_BM = 256, PB_BN = 256;
constexpr int PB_HALF_K = 64;
constexpr int PB_STAGE_BYTES = PB_BM * PB_HALF_K * 2;  // 32 KiB
constexpr int PB_STAGES = 4;
constexpr unsigned PB_LDS_BYTES = PB_STAGES * PB_STAGE_BYTES;  // 128 KiB
constexpr int PB_AL = 8;  // activation loads per wave and half k-block

// acc += a x b on the matrix cores with the accumulator updated in place in its accumulation registers.  The 64
// accumulator tiles of a wave fill all 256 of them; the compiler's own MFMA wants a destination that does not
// overlap its source and, finding none free, moves accumulators through ordinary registers around every MFMA
// (two register moves and a pipeline drain per MFMA).  As an asm statement the instruction is opaque to the
// compiler's hazard tables, so the kernel keeps the distances itself: an operand written by the vector ALU is read
// a whole k-step (64 MFMAs) later, an accumulator is touched again 64 MFMAs later, and the epilogue waits out the
// last MFMAs before it reads the accumulators.
__device__ __forceinline__ void mfma_in_place(float4_t& acc, half8_t a, half8_t b) {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
}

template <bool ZP_TABLE, bool PRESCALE>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void fcc_prefill_big_kernel(
    const uint4_t* __restrict__ wt, const half_t* __restrict__ st, const uint8_t* __restrict__ zt,
    const half_t* __restrict__ x, const half_t* __restrict__ bias, void* __restrict__ y, int M, int N, int K,
    int kb_total, int kb_per_group, int ng, int zp_const, int out_f32, int glu, int tiles_x, int tiles_y) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    const lds_byte_ptr lds3 = (lds_byte_ptr)lds_raw;
    typedef __attribute__((address_space(3))) const half8_t* lds_frag_ptr;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int col = lane & 15, kq = lane >> 4;
    const TileWork wk = tile_work(tiles_x, tiles_y, tiles_x * tiles_y, 1, kb_total, kb_total, PB_BM, PB_BN / 2);
    const int n0 = wk.tile_x * PB_BN, m0 = wk.m0;
    const int halves = 2 * kb_total;

    constexpr unsigned kOob = 0x80000000u;
    constexpr int kRsrcFlags = 0x00020000;
    // Every offset goes through the vector operand: the scalar offset of a buffer load is not range-checked.
    const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(x), 0, M * K * 2, kRsrcFlags);
    const int nt0 = n0 / 16 + 4 * wave;  // the wave's four channel tiles
    const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint4_t*>(wt + (size_t)nt0 * kb_total * 64), 0, 4 * kb_total * kTileBytes, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t rs =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(st + (size_t)nt0 * ng * 16), 0, 4 * ng * 32, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t rz = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint8_t*>(ZP_TABLE ? zt + (size_t)nt0 * ng * 16 : zt), 0, ZP_TABLE ? 4 * ng * 16 : 0, kRsrcFlags);
    const unsigned g_mul = kb_per_group == 1 ? 0u : (unsigned)((0x100000000ull + kb_per_group - 1) / kb_per_group);

    // ---- activations: load i of the wave fills rows 64 wave + 8 i .. +7 of a stage; lane -> row 8 i + (lane >> 3)
    // of those, 16-byte slot lane & 7 of that row, which holds chunk (lane & 7) ^ ((row >> 1) & 7) of the half
    // k-block.  ((row >> 1) & 7 = (4 i + (lane >> 4)) & 7 = (4 i & 7) ^ (lane >> 4).)  Rows >= M lie beyond the
    // descriptor's range and arrive as zeros. ----
    const unsigned a_row0 = (unsigned)((m0 + 64 * wave + (lane >> 3)) * K) * 2u;
    const unsigned a_c0 = (unsigned)((lane & 7) ^ (lane >> 4));
    auto dma_a = [&](int hh, int stage, int i) {
        const unsigned oob = (unsigned)((halves - 1 - hh) >> 31) & kOob;
        const unsigned sterm = __builtin_amdgcn_readfirstlane((unsigned)(8 * i * K + hh * PB_HALF_K) * 2u);
        const unsigned voff = a_row0 + sterm + ((a_c0 ^ (unsigned)((4 * i) & 7)) << 4);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            rx, (lds_void_ptr)(lds3 + stage * PB_STAGE_BYTES + (64 * wave + 8 * i) * 128), 16, voff | oob, 0, 0, 0);
    };

    // ---- weights of one k-block in registers: raw tile dwords, scale and zero-point of the lane's channel ----
    struct WSlot {
        uint4_t w[4];
        uint32_t scale[4];
        uint32_t zp[4];
        uint32_t off_lo[4], off_hi[4];  // the halves 1024 + zp and 64 + zp, twice each (prepare; zero-point tables)
    };
    auto load_w = [&](int kb, WSlot& s) {
        const unsigned oob = (unsigned)((kb_total - 1 - kb) >> 31) & kOob;
        const unsigned g = kb_per_group == 1 ? (unsigned)kb : __umulhi((unsigned)kb, g_mul);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const unsigned wofs = ((unsigned)(r * kb_total + kb) * (unsigned)kTileBytes + lane * 16u) | oob;
            s.w[r] = __builtin_bit_cast(uint4_t, __builtin_amdgcn_raw_buffer_load_b128(rw, wofs, 0, 0));
            const unsigned sidx = ((unsigned)r * ng + g) * 16u + col;
            if constexpr (PRESCALE)
                s.scale[r] = __builtin_amdgcn_raw_buffer_load_b16(rs, (sidx * 2u) | oob, 0, 0);
            if constexpr (ZP_TABLE)
                s.zp[r] = __builtin_amdgcn_raw_buffer_load_b8(rz, sidx | oob, 0, 0);
        }
    };
    constexpr int kWLoads = 4 + (PRESCALE ? 4 : 0) + (ZP_TABLE ? 4 : 0);  // vector-memory loads of load_w

    // ---- unpack, one micro-operation at a time: dword j of tile r of slot s -> f (the 128 x 256 kernel's scheme) ----
    constexpr int NOPS = 5 + 4 + (PRESCALE ? 4 : 0);  // per dword
    const Unpack4Consts uc = unpack4_consts();
    const half2_t off_lo_c = as_half2(__builtin_amdgcn_readfirstlane(as_u32(splat(1024.f + (float)zp_const))));
    const half2_t off_hi_c = as_half2(__builtin_amdgcn_readfirstlane(as_u32(splat(64.f + (float)zp_const))));
    // Once per k-block and tile, before the first dword of a slot is unpacked: the two offsets its subtractions use.
    auto prepare = [&](WSlot& s) {
        if constexpr (ZP_TABLE) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float zpv = (float)s.zp[r];
                s.off_lo[r] = as_u32(splat(1024.f + zpv));
                s.off_hi[r] = as_u32(splat(64.f + zpv));
            }
        }
    };
    auto unpack_op = [&](const WSlot& s, int r, int j, int op, Frag8& f) {
        const uint32_t w = j == 0 ? s.w[r].x : j == 1 ? s.w[r].y : j == 2 ? s.w[r].z : s.w[r].w;
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
                off = as_half2((k & 1) ? s.off_hi[r] : s.off_lo[r]);
            } else {
                off = (k & 1) ? off_hi_c : off_lo_c;
            }
            f.h2[k] = f.h2[k] - off;
        } else if constexpr (PRESCALE) {
            const half_t h = __builtin_bit_cast(half_t, (uint16_t)s.scale[r]);
            f.h2[op - 9] *= half2_t{h, h};
        }
    };

    float4_t acc[4][16];  // [channel tile][row tile]
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int t = 0; t < 16; ++t)
            acc[r][t] = float4_t{0.f, 0.f, 0.f, 0.f};

    // One half k-block = two k-steps of 64 MFMAs.  Step js multiplies the unpacked weights wa (js == 0) / wb (js == 1)
    // with the sixteen row tiles of inputs 32 js ..+32 of the stage while the vector ALU unpacks the *next* step's
    // weights into the other set, a few micro-operations after every MFMA: dword ja of `sa` during step 0 (into wb),
    // dword jb of `sb` during step 1 (into wa).  The activation operands run PB_XQ - 1 row tiles ahead of the
    // MFMAs, across the boundary between the steps; mem(i) adds the memory instructions of slot i (0 .. 127).
    // Ring of activation operands, eight deep (a divisor of the 32 operands of a half, so ring positions repeat from
    // half to half): operand n of a half is row tile n & 15 of step n >> 4.  The ring runs seven operands ahead of
    // the MFMAs and carries on into the next half's stage, so no half starts with an empty ring.
    constexpr int PB_XQ = 8;
    constexpr int PB_SYNC_SLOT = 100;  // the first slot whose ring read belongs to the next half
    half8_t xq[PB_XQ];
    const int x_sw = (col >> 1) & 7;
    // operand n of the half in `stage`: row 16 (n & 15) + col, chunk (4 (n >> 4) + kq) ^ ((col >> 1) & 7)
    auto x_at = [&](int stage, int n) {
        return *(lds_frag_ptr)(lds3 + stage * PB_STAGE_BYTES + ((n & 15) * 16 + col) * 128 + ((((n >> 4) * 4 + kq) ^ x_sw) << 4));
    };
    auto half = [&](int stage, Frag8 (&wa)[4], Frag8 (&wb)[4], const WSlot& sa, int ja, WSlot& sb, int jb,
                    auto&& sync_next, auto&& mem) {
        auto slot = [&](int i) {
            const int tt = i >> 2, r = i & 3;  // tt = 16 js + t
            if (i == PB_SYNC_SLOT)
                sync_next();  // the next half's activations are in LDS for every wave
            if (r == 0) {
                constexpr int ahead = PB_XQ - 1;
                xq[(tt + ahead) % PB_XQ] = tt + ahead < 32 ? x_at(stage, tt + ahead) : x_at((stage + 1) & 3, tt + ahead - 32);
            }
            const int t = tt & 15;
            if (i < 64) {
                mfma_in_place(acc[r][t], wa[r].v, xq[tt % PB_XQ]);
#pragma unroll
                for (int g = i * 4 * NOPS / 64; g < (i + 1) * 4 * NOPS / 64; ++g)
                    unpack_op(sa, g / NOPS, ja, g % NOPS, wb[g / NOPS]);
            } else {
                if (i == 64 && jb == 0)
                    prepare(sb);  // step 1 starts on a fresh slot
                mfma_in_place(acc[r][t], wb[r].v, xq[tt % PB_XQ]);
#pragma unroll
                for (int g = (i - 64) * 4 * NOPS / 64; g < (i - 63) * 4 * NOPS / 64; ++g)
                    unpack_op(sb, g / NOPS, jb, g % NOPS, wa[g / NOPS]);
            }
            mem(i);
            __builtin_amdgcn_sched_barrier(0);
        };
        // (eight loops: the unroller gives up on longer ones)
#pragma unroll
        for (int i = 0; i < 16; ++i)
            slot(i);
#pragma unroll
        for (int i = 16; i < 32; ++i)
            slot(i);
#pragma unroll
        for (int i = 32; i < 48; ++i)
            slot(i);
#pragma unroll
        for (int i = 48; i < 64; ++i)
            slot(i);
#pragma unroll
        for (int i = 64; i < 80; ++i)
            slot(i);
#pragma unroll
        for (int i = 80; i < 96; ++i)
            slot(i);
#pragma unroll
        for (int i = 96; i < 112; ++i)
            slot(i);
#pragma unroll
        for (int i = 112; i < 128; ++i)
            slot(i);
    };

    // ---- prologue: weights of k-blocks 0 and 1, activations of halves 0, 1, 2; first operand unpacked ----
    WSlot ws0, ws1;
    load_w(0, ws0);
    load_w(1, ws1);
#pragma unroll
    for (int hh = 0; hh < 3; ++hh)
#pragma unroll
        for (int i = 0; i < PB_AL; ++i)
            dma_a(hh, hh, i);
    Frag8 wf0[4], wf1[4];
    prepare(ws0);
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int op = 0; op < NOPS; ++op)
            unpack_op(ws0, r, 0, op, wf0[r]);
    __builtin_amdgcn_s_waitcnt(wait_vmcnt_imm(2 * PB_AL));  // half 0 has landed
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
#pragma unroll
    for (int n = 0; n < PB_XQ - 1; ++n)
        xq[n] = x_at(0, n);

    // ---- main loop: two k-blocks (four halves, the four stages) per trip so that stages and weight slots are
    // static.  Halves and k-blocks past the end are loaded out of range (zeros) and add nothing. ----
    for (int kb0 = 0; kb0 < kb_total; kb0 += 2) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int hh = 2 * kb0 + u;
            // The one barrier of a half sits where the operand ring first reaches into the next half: by then the
            // wave needs that half's activations.  Issued after them by this wave: the rest of the activation loads
            // of the half before this one and seven of this half's (fifteen in all) and, in one of the two halves, a
            // k-block's weight loads (none yet in the very first half).  Past the barrier no wave reads this half's
            // stage any more (its last operand was fetched four slots earlier, and the wave's own LDS reads are
            // waited for here), so the loads of half hh + 4, which start in the next half, may overwrite it.
            auto sync_next = [&]() {
                constexpr int lds_reads_done = ~0x0F00;
                if (u == 0)  // (later trips: this also waits for loads issued more than a half ago, long since in)
                    __builtin_amdgcn_s_waitcnt(wait_vmcnt_imm(2 * PB_AL - 1) & lds_reads_done);
                else
                    __builtin_amdgcn_s_waitcnt(wait_vmcnt_imm(2 * PB_AL - 1 + kWLoads) & lds_reads_done);
                asm volatile("" ::: "memory");
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
            };
            // Memory instructions between the MFMAs: the stage that half hh - 1 used takes half hh + 3 (slots 1, 17,
            // ..).  A k-block's weight slot is free once the last step that unpacks from it has run -- step 0 of its
            // second half -- so the loads of the k-block after next go out at the start of step 1 of that half.
            auto mem = [&](int i) {
                if ((i & 15) == 1)
                    dma_a(hh + 3, (u + 3) & 3, i >> 4);
                if (i == 64 && u == 1)
                    load_w(kb0 + 2, ws0);
                if (i == 64 && u == 3)
                    load_w(kb0 + 3, ws1);
            };
            // steps of this half: dwords 2 (u & 1), 2 (u & 1) + 1 of the k-block's slot; unpacked meanwhile: the
            // next step's dword -- of the same slot, or dword 0 of the other slot at the end of a k-block
            if (u == 0)
                half(0, wf0, wf1, ws0, 1, ws0, 2, sync_next, mem);
            else if (u == 1)
                half(1, wf0, wf1, ws0, 3, ws1, 0, sync_next, mem);
            else if (u == 2)
                half(2, wf0, wf1, ws1, 1, ws1, 2, sync_next, mem);
            else
                half(3, wf0, wf1, ws1, 3, ws0, 0, sync_next, mem);
        }
    }
    __builtin_amdgcn_s_waitcnt(wait_vmcnt_imm(0));  // the out-of-range loads of the last trips still target LDS
    // the last MFMAs retire (a 16 x 16 x 32 MFMA writes its result up to 18 cycles after issue; the compiler does not
    // know the asm statements are MFMAs and would read the accumulators at once)
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");

    // ---- epilogue: per-channel scale, bias, gated linear unit, stores ----
    auto channel_params = [&](int r, float (&sc)[4], float (&bs)[4]) {
        const int n = n0 + 64 * wave + 16 * r + 4 * kq;
#pragma unroll
        for (int q = 0; q < 4; ++q)
            sc[q] = 1.f, bs[q] = 0.f;
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
    };
    auto put = [&](size_t idx, const float (&o)[4]) {
        if (out_f32)
            *reinterpret_cast<float4_t*>(static_cast<float*>(y) + idx) = float4_t{o[0], o[1], o[2], o[3]};
        else
            *reinterpret_cast<half4_t*>(static_cast<half_t*>(y) + idx) =
                half4_t{to_half_rne(o[0]), to_half_rne(o[1]), to_half_rne(o[2]), to_half_rne(o[3])};
    };
    if (glu) {
        // channel tiles 2 j and 2 j + 1 of the wave are gate and up of output channels (n0 + 64 wave) / 2 + 16 j ..
        float scg[2][4], bsg[2][4], scu[2][4], bsu[2][4];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            channel_params(2 * j, scg[j], bsg[j]);
            channel_params(2 * j + 1, scu[j], bsu[j]);
        }
#pragma unroll
        for (int t = 0; t < 16; ++t) {
            const int m = m0 + 16 * t + col;
#pragma unroll
            for (int j = 0; j < 2; ++j) {  // the two pairs' results are neighbours in the output row
                const int n = (n0 + 64 * wave) / 2 + 16 * j + 4 * kq;
                const float4_t g = acc[2 * j][t], u = acc[2 * j + 1][t];
                const float o[4] = {glu_value(glu, g.x * scg[j][0] + bsg[j][0], u.x * scu[j][0] + bsu[j][0]),
                                    glu_value(glu, g.y * scg[j][1] + bsg[j][1], u.y * scu[j][1] + bsu[j][1]),
                                    glu_value(glu, g.z * scg[j][2] + bsg[j][2], u.z * scu[j][2] + bsu[j][2]),
                                    glu_value(glu, g.w * scg[j][3] + bsg[j][3], u.w * scu[j][3] + bsu[j][3])};
                if (m < M)
                    put((size_t)m * (N / 2) + n, o);
            }
        }
        return;
    }
    if (!out_f32 && (reinterpret_cast<uintptr_t>(y) & 15) == 0) {
        // f16 output: the four lanes of a row (lane bits 4 and 5 = kq) hold four channels of each of the wave's four
        // channel tiles.  A 4 x 4 exchange between them -- halves of the wave swapped, then neighbouring rows of 16
        // lanes -- leaves lane kq with all 16 channels of tile kq: 32 contiguous bytes per lane, and the four lanes
        // of a row write its whole 128-byte line with two store instructions.
        float sc[4][4], bs[4][4];
#pragma unroll
        for (int r = 0; r < 4; ++r)
            channel_params(r, sc[r], bs[r]);
        half_t* yh = static_cast<half_t*>(y);
#pragma unroll
        for (int t = 0; t < 16; ++t) {
            uint32_t p[4][2];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float4_t v = acc[r][t];
                const half4_t h = half4_t{to_half_rne(v.x * sc[r][0] + bs[r][0]), to_half_rne(v.y * sc[r][1] + bs[r][1]),
                                          to_half_rne(v.z * sc[r][2] + bs[r][2]), to_half_rne(v.w * sc[r][3] + bs[r][3])};
                const uint2_t u = __builtin_bit_cast(uint2_t, h);
                p[r][0] = u.x, p[r][1] = u.y;
            }
            uint32_t q[8];  // channels 4 k' .. 4 k' + 3 of tile kq, from lane k' of the row: dwords 2 k', 2 k' + 1
#pragma unroll
            for (int d = 0; d < 2; ++d) {
                // lanes 0-31 keep tiles 0 and 1, lanes 32-63 tiles 2 and 3; .x comes from the lane with kq bit 1
                // clear, .y from the one with it set
                const uint2_t s02 = __builtin_amdgcn_permlane32_swap(p[0][d], p[2][d], false, false);
                const uint2_t s13 = __builtin_amdgcn_permlane32_swap(p[1][d], p[3][d], false, false);
                // even rows of 16 lanes keep the even tile, odd rows the odd one; .x from kq bit 0 clear, .y set
                const uint2_t lo = __builtin_amdgcn_permlane16_swap(s02.x, s13.x, false, false);
                const uint2_t hi = __builtin_amdgcn_permlane16_swap(s02.y, s13.y, false, false);
                q[d] = lo.x, q[2 + d] = lo.y, q[4 + d] = hi.x, q[6 + d] = hi.y;
            }
            const int m = m0 + 16 * t + col;
            if (m < M) {
                uint4_t* dst = reinterpret_cast<uint4_t*>(yh + (size_t)m * N + n0 + 64 * wave + 16 * kq);
                dst[0] = uint4_t{q[0], q[1], q[2], q[3]};
                dst[1] = uint4_t{q[4], q[5], q[6], q[7]};
            }
        }
        return;
    }
    // Row tile by row tile, the four channel tiles one after the other: a wave's 64 channels are one 128-byte line
    // of an f16 output row, written as four 32-byte pieces by consecutive store instructions.
    float sc[4][4], bs[4][4];
#pragma unroll
    for (int r = 0; r < 4; ++r)
        channel_params(r, sc[r], bs[r]);
#pragma unroll
    for (int t = 0; t < 16; ++t) {
        const int m = m0 + 16 * t + col;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int n = n0 + 64 * wave + 16 * r + 4 * kq;  // four consecutive channels
            const float4_t v = acc[r][t];
            const float o[4] = {v.x * sc[r][0] + bs[r][0], v.y * sc[r][1] + bs[r][1], v.z * sc[r][2] + bs[r][2],
                                v.w * sc[r][3] + bs[r][3]};
            if (m < M)
                put((size_t)m * N + n, o);
        }
    }
}

// The launch must be what the kernel assumes: a 1-D grid of whole 256 x 256 tiles.
static bool big_plan_ok(const FcDeviceArgs& a, const LaunchPlan& p) {
    const Layout& L = a.layout;
    return L.tiled && L.bits == 4 && L.groups_per_kblock == 1 && a.N % PB_BN == 0 && p.tile_m == PB_BM &&
           p.tile_n == PB_BN && p.tiles_x == a.N / PB_BN && p.tiles_y >= 1 && (int64_t)p.tiles_y * PB_BM >= a.M &&
           p.split_k == 1 && p.full_tiles == p.tiles_x * p.tiles_y && p.grid[0] == (unsigned)(p.tiles_x * p.tiles_y) &&
           p.grid[1] == 1 && p.grid[2] == 1 && p.block == 256 && a.M * a.K * 2 < ((int64_t)1 << 31) &&
           (int64_t)4 * L.k_blocks * kTileBytes < ((int64_t)1 << 31);
}

template <bool ZPT, bool PRE>
static int launch_big_impl(const FcDeviceArgs& a, const LaunchPlan& p, hipStream_t s) {
    const Layout& L = a.layout;
    auto kern = fcc_prefill_big_kernel<ZPT, PRE>;
    static bool attr_set = false;  // per instantiation; the attribute is idempotent, a race only repeats it
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)PB_LDS_BYTES);
        if (e != hipSuccess)
            return (int)e;
        attr_set = true;
    }
    hipLaunchKernelGGL(kern, dim3(p.grid[0], 1, 1), dim3(256), PB_LDS_BYTES, s, (const uint4_t*)a.w,
                       (const half_t*)a.scale, (const uint8_t*)a.zp, (const half_t*)a.x, (const half_t*)a.bias, a.y,
                       (int)a.M, (int)a.N, (int)a.K, (int)L.k_blocks, (int)L.kblocks_per_group, (int)L.groups, L.zp_const,
                       a.out_f32, L.glu, p.tiles_x, p.tiles_y);
    return (int)hipGetLastError();
}

int launch_prefill_big(const FcDeviceArgs& a, const LaunchPlan& p, void* stream) {
    hipStream_t s = static_cast<hipStream_t>(stream);
    const Layout& L = a.layout;
    if (!big_plan_ok(a, p))
        return (int)hipErrorInvalidValue;
    if (L.groups == 1)
        return L.zp_table ? launch_big_impl<true, false>(a, p, s) : launch_big_impl<false, false>(a, p, s);
    return L.zp_table ? launch_big_impl<true, true>(a, p, s) : launch_big_impl<false, true>(a, p, s);
}

}  // namespace ovfcc
