// The gated MLP of a decoder block as one launch for one to four rows: gate / up projection with the gated linear
// unit, then the down projection, both 4-bit with groups of 128 inputs (the node the OpenVINO CPU plugin calls
// LLMMLP: src/plugins/intel_cpu/src/nodes/llm_mlp.cpp:495-526, fused by
// src/plugins/intel_cpu/src/transformations/cpu_opset/x64/pass/mlp_fusion.cpp:48-120).  A launch of the down
// projection on its own costs its start and its wind-down a second time; here its weights are already on their way
// while the last gate / up tiles are reduced.
//
// Both phases are the matrix-vector kernel's arithmetic (kernel_gemv.hip) with eight k-blocks per wave, instruction
// for instruction, so that the result has the bits of the two launches it replaces.
//
// grid = one workgroup of sixteen waves per compute unit, all resident at once (the host checks).
// Phase 1: a gate / up tile pair takes 2 x nwt1 waves (nwt1 = K1 / 1024), so a workgroup works on PS = 8 / nwt1
// pairs at a time: pair blockIdx.x + G (PS it + ps) in round `it`, pair slot ps.  The activations are staged once
// per workgroup (one copy per share of K); the weights of round it + 1 are requested before round it is computed.
// The waves of a pair leave their partial sums in LDS, the last to arrive (a ticket per pair) adds them, applies
// bias and the unit and stores sixteen f16 values of the intermediate row with device-scope stores.  When a
// workgroup's last pair is stored and acknowledged it adds one to an arrival counter in memory.
// Phase 2: every wave requests its eight weight tiles of down tile blockIdx.x (+ G j) *first*, then wave 0 waits for
// the workgroup's go flag, which the workgroup that brings the arrival counter to G raises -- a bounded wait: past the limit it raises a flag in host-visible memory and goes
// on, so the grid always drains -- and the workgroup passes a barrier.  The intermediate row is then read with
// device-scope loads (other XCDs wrote it; this L2 may hold an older launch's lines), staged per wave, and the
// down projection proceeds as in the matrix-vector kernel.  The counter and the flags return to zero on the way (the
// workgroup that completes the count clears it, every workgroup clears its own flag).
#include "device_common.h"

namespace ovfcc {

namespace {

constexpr int kMlpC = 8;                          // k-blocks per wave in both phases
constexpr int kMlpRowBytes = kMlpC * 256 + 64;    // one staged row; the pad keeps rows on different banks
constexpr int kMlpWaves = 16;
constexpr int kMlpMaxRounds = 8;                  // rounds of pairs / of down tiles one workgroup may take
constexpr unsigned kMlpOob = 0x80000000u;
constexpr int kMlpRsrcFlags = 0x00020000;
constexpr int kMlpAuxDeviceScope = 16;            // sc1: the load bypasses this XCD's L2
// The go flag of workgroup g, in 32-bit words from the start of the sync buffer: 4 352 bytes apart, so that the
// workgroups poll addresses spread over the memory channels.  (Polling one word from every waiting workgroup kept
// that word's channel half busy, and since every wave's tiles are spread over all channels the whole weight stream
// ran at half speed: the workgroups still in phase 1 arrived at 29 instead of 17 us.)
constexpr size_t kMlpFlagStride = 1088, kMlpFlagBase = 1024;
__host__ __device__ constexpr size_t mlp_flag_at(size_t g) {
    return kMlpFlagBase + kMlpFlagStride * g;
}

// sum over the 16 lanes of a DPP row; lane 15 of every row ends with the row's total
__device__ __forceinline__ float mlp_row_sum16(float v) {
    int t;
    t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x111, 0xF, 0xF, true);  // row_shr:1
    v += __builtin_bit_cast(float, t);
    t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x112, 0xF, 0xF, true);  // row_shr:2
    v += __builtin_bit_cast(float, t);
    t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x114, 0xF, 0xF, true);  // row_shr:4
    v += __builtin_bit_cast(float, t);
    t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x118, 0xF, 0xF, true);  // row_shr:8
    v += __builtin_bit_cast(float, t);
    return v;
}

// keeps a loaded value from being moved down to a later, conditional use
__device__ __forceinline__ void mlp_needed_here(uint32_t& v) {
    asm volatile("" : "+v"(v));
}
__device__ __forceinline__ void mlp_needed_here(uint4_t& v) {
    uint32_t a = v.x, b = v.y, c = v.z, d = v.w;
    asm volatile("" : "+v"(a), "+v"(b), "+v"(c), "+v"(d));
    v = uint4_t{a, b, c, d};
}

// weights and group parameters of one wave for one tile: eight packed tiles, the eight scales (and zero-points) of
// the lane's channel in lanes 0-15
struct MlpTile {
    uint4_t wv[kMlpC];
    uint4_t sv;
    uint32_t zv[2];
};

// Requests them: tile `tile` of a node with kb k-blocks per channel tile cut over nwt waves, share `part`; live =
// false requests nothing (every offset out of range, zeros arrive).
template <bool ZP_TABLE>
__device__ __forceinline__ void mlp_load_tile(MlpTile& t, const uint4_t* wt, const half_t* scale_cm, const uint8_t* zp_cm,
                                              int tile, int kb, int nwt, int part, bool live, int lane) {
    const int col = lane & 15, kq = lane >> 4;
    const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint4_t*>(wt + ((size_t)tile * kb + part) * 64), 0, live ? ((kMlpC - 1) * nwt + 1) * kTileBytes : 0,
        kMlpRsrcFlags);
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<half_t*>(scale_cm + (size_t)tile * 16 * kb), 0, live ? 16 * kb * 2 : 0, kMlpRsrcFlags);
    const unsigned pofs = kq == 0 ? (unsigned)(col * kb + part * kMlpC) : kMlpOob;
    t.sv = __builtin_bit_cast(uint4_t, __builtin_amdgcn_raw_buffer_load_b128(rs, kq == 0 ? pofs * 2u : kMlpOob, 0, 0));
    t.zv[0] = t.zv[1] = 0u;
    if constexpr (ZP_TABLE) {
        const __amdgpu_buffer_rsrc_t rz = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<uint8_t*>(zp_cm + (size_t)tile * 16 * kb), 0, live ? 16 * kb : 0, kMlpRsrcFlags);
        const uint2_t v = __builtin_bit_cast(uint2_t, __builtin_amdgcn_raw_buffer_load_b64(rz, pofs, 0, 0));
        t.zv[0] = v.x, t.zv[1] = v.y;
    }
#pragma unroll
    for (int i = 0; i < kMlpC; ++i)
        t.wv[i] = __builtin_bit_cast(
            uint4_t, __builtin_amdgcn_raw_buffer_load_b128(rw, (unsigned)(i * nwt * kTileBytes + lane * 16), 0, 2));
}

// Rows 0 .. MR-1 of a [M, K] f16 matrix, the wave's k-blocks part + nwt s (s = 0 .. 7): two loads per row, lane ->
// k-block 4 i + (lane >> 4), 16-byte chunk lane & 15.
template <int MR>
__device__ __forceinline__ void mlp_load_rows(uint4_t (&xr)[MR][2], const __amdgpu_buffer_rsrc_t rx, int M, int K, int part,
                                              int nwt, int aux_device_scope, int lane) {
    const int col = lane & 15, kq = lane >> 4;
#pragma unroll
    for (int m = 0; m < MR; ++m)
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const unsigned ofs = m < M ? (unsigned)(m * K + (part + nwt * (4 * i + kq)) * 128 + col * 8) * 2u : kMlpOob;
            xr[m][i] = aux_device_scope
                           ? __builtin_bit_cast(uint4_t, __builtin_amdgcn_raw_buffer_load_b128(rx, ofs, 0, kMlpAuxDeviceScope))
                           : __builtin_bit_cast(uint4_t, __builtin_amdgcn_raw_buffer_load_b128(rx, ofs, 0, 0));
        }
}

// Group sums of the loaded rows (times cmul) into scalars, and the rows themselves into `xs` in operand order
// (elements that meet nibbles four bits up in their halves times 2^-4), where `write` says so.
template <int MR>
__device__ __forceinline__ void mlp_stage_rows(const uint4_t (&xr)[MR][2], float cmul, unsigned char* xs, bool write,
                                               float (&csum)[MR][kMlpC], int lane) {
    const half2_t ones = half2_t{(half_t)1.f, (half_t)1.f};
    const half2_t sixteenth = half2_t{(half_t)0.0625f, (half_t)0.0625f};
#pragma unroll
    for (int m = 0; m < MR; ++m)
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const uint4_t v = xr[m][i];
            float s = __builtin_amdgcn_fdot2(as_half2(v.x), ones, 0.f, false);
            s = __builtin_amdgcn_fdot2(as_half2(v.y), ones, s, false);
            s = __builtin_amdgcn_fdot2(as_half2(v.z), ones, s, false);
            s = __builtin_amdgcn_fdot2(as_half2(v.w), ones, s, false);
            s = mlp_row_sum16(s) * cmul;
#pragma unroll
            for (int r = 0; r < 4; ++r)
                csum[m][4 * i + r] =
                    __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, s), 16 * r + 15));
            uint4_t p = v;
            p.y = as_u32(as_half2(v.y) * sixteenth);
            p.w = as_u32(as_half2(v.w) * sixteenth);
            if (write)
                *reinterpret_cast<uint4_t*>(xs + m * kMlpRowBytes + (i * 64 + lane) * 16) = p;
        }
}

// The wave's partial sums over its eight k-blocks: acc[r] for the lane's channel (lanes 0-15 hold rows 0-3).
template <int MR, bool ZP_TABLE>
__device__ __forceinline__ void mlp_partial(const MlpTile& t, const unsigned char* xs_lane, const float (&csum)[MR][kMlpC],
                                            float (&acc)[MR]) {
    const uint32_t mask_lo = 0x000F000Fu, mask_hi = 0x00F000F0u;
#pragma unroll
    for (int r = 0; r < MR; ++r)
        acc[r] = 0.f;
#pragma unroll
    for (int i = 0; i < kMlpC; ++i) {
        const uint32_t wd[4] = {t.wv[i].x, t.wv[i].y, t.wv[i].z, t.wv[i].w};
        float4_t p = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const half8_t a = *reinterpret_cast<const half8_t*>(xs_lane + (i * 16 + 4 * j) * 16);
            const uint32_t w8 = wd[j] >> 8;
            Frag8 b;
            b.u[0] = wd[j] & mask_lo;
            b.u[1] = wd[j] & mask_hi;
            b.u[2] = w8 & mask_lo;
            b.u[3] = w8 & mask_hi;
            p = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b.v, p, 0, 0, 0);
        }
        const uint32_t sbits = (i < 2 ? t.sv.x : i < 4 ? t.sv.y : i < 6 ? t.sv.z : t.sv.w) >> (16 * (i & 1));
        const float scale = (float)__builtin_bit_cast(half_t, (uint16_t)sbits);
        const float pr[4] = {p.x, p.y, p.z, p.w};
        if constexpr (ZP_TABLE) {
            const float zpf = (float)((t.zv[i >> 2] >> (8 * (i & 3))) & 0xFFu);
#pragma unroll
            for (int r = 0; r < MR; ++r)
                acc[r] = __builtin_fmaf(scale, __builtin_fmaf(-zpf, csum[r][i], pr[r]), acc[r]);
        } else {
#pragma unroll
            for (int r = 0; r < MR; ++r)
                acc[r] = __builtin_fmaf(scale, pr[r] + csum[r][i], acc[r]);
        }
    }
}

// Sum over the rows of sixteen lanes of a wave, every lane ends with the total: (g0 + g2) + (g1 + g3).  (The second
// result of an exchange passes through an empty asm statement: converted straight to a float, this compiler reads
// the first result in its place.)
__device__ __forceinline__ float mlp_across_rows(float v) {
    const uint32_t a = __builtin_bit_cast(uint32_t, v);
    const uint2_t h = __builtin_amdgcn_permlane32_swap(a, a, false, false);
    uint32_t hy = h.y;
    asm volatile("" : "+v"(hy));
    const float t = __builtin_bit_cast(float, h.x) + __builtin_bit_cast(float, hy);
    const uint32_t b = __builtin_bit_cast(uint32_t, t);
    const uint2_t q = __builtin_amdgcn_permlane16_swap(b, b, false, false);
    uint32_t qy = q.y;
    asm volatile("" : "+v"(qy));
    return __builtin_bit_cast(float, q.x) + __builtin_bit_cast(float, qy);
}

// Sum of the partial sums red[first .. first + count) [MR][16] of row r, channel lane & 15 (count <= 16).
template <int MR>
__device__ __forceinline__ float mlp_tile_sum(const float* red, int first, int count, int r, int lane) {
    const int col = lane & 15, kq = lane >> 4;
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int w = kq + 4 * j;
        const float v = red[((first + (w < count ? w : 0)) * MR + r) * 16 + col];
        s += w < count ? v : 0.f;
    }
    return mlp_across_rows(s);
}

}  // namespace

struct MlpKernelArgs {
    const uint4_t* w1;
    const half_t* s1;
    const uint8_t* z1;
    const half_t* b1;
    const uint4_t* w2;
    const half_t* s2;
    const uint8_t* z2;
    const half_t* b2;
    const half_t* x;
    half_t* h;         // [M, K2] f16, the request's intermediate buffer
    void* y;
    unsigned* sync;    // [0] workgroups whose intermediate values are in memory; one go flag per workgroup (mlp_flag_at)
    unsigned* error;   // host-visible: set when a wait ran out
    int M, K1, K2, N2;
    int kb1, nwt1, kb2, nwt2;
    int pairs1, tiles2, rounds1, rounds2;
    int zp_const1, zp_const2, glu, out_f32;
    unsigned spin_limit;
};

// MR: rows the kernel carries (M <= MR); ZP1 / ZP2: zero-point tables of the gate / up and the down node
template <int MR, bool ZP1, bool ZP2>
__global__ __launch_bounds__(1024) void fcc_mlp_gemv_kernel(const MlpKernelArgs a) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    __shared__ unsigned arrived[2 * 8 * kMlpMaxRounds];  // tickets: pair (round, slot) of phase 1, then tile rounds of phase 2
    __shared__ unsigned pairs_done;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int col = lane & 15, kq = lane >> 4;
    const int G = gridDim.x;
    const int nwt1 = a.nwt1, nwt2 = a.nwt2;
    const int PS = 8 / nwt1;                       // pair slots of a workgroup: 16 waves / (2 nwt1)
    const int ps = wave / (2 * nwt1), sub = (wave / nwt1) & 1, part1 = wave % nwt1;
    const int wp = sub * nwt1 + part1;             // the wave within its pair: gate waves, then up waves
    if (threadIdx.x < 2 * 8 * kMlpMaxRounds)
        arrived[threadIdx.x] = 0;
    if (threadIdx.x == 0)
        pairs_done = 0;
    // pairs of this workgroup: blockIdx.x + G j < pairs1
    const int my_pairs = (int)blockIdx.x < a.pairs1 ? (a.pairs1 - 1 - (int)blockIdx.x) / G + 1 : 0;
    // One wave per workgroup reports that the workgroup's share of the intermediate row is in memory (`mine`: this
    // wave is the one).  The workgroup that completes the count returns the counter to zero -- nobody reads it any
    // more -- and raises every workgroup's go flag.
    auto arrive = [&](bool mine) {
        unsigned last = 0;
        if (mine && lane == 0)
            last = __hip_atomic_fetch_add(a.sync, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == (unsigned)G - 1 ? 1u : 0u;
        if (__builtin_amdgcn_readfirstlane(last)) {
            if (lane == 0)
                __hip_atomic_store(a.sync, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            for (int g = lane; g < G; g += 64)
                __hip_atomic_store(a.sync + mlp_flag_at(g), 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    };
    if (my_pairs == 0 && wave == 0)
        arrive(true);

    // ---- phase 1: activations, then the first round's weights; staged copies: one per share of K ----
    const __amdgpu_buffer_rsrc_t rx =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(a.x), 0, a.M * a.K1 * 2, kMlpRsrcFlags);
    uint4_t xr[MR][2];
    mlp_load_rows<MR>(xr, rx, a.M, a.K1, part1, nwt1, 0, lane);
    auto pair_of = [&](int round) { return (int)blockIdx.x + G * (round * PS + ps); };
    MlpTile ta, tb;
    __builtin_amdgcn_sched_barrier(0);
    mlp_load_tile<ZP1>(ta, a.w1, a.s1, a.z1, 2 * pair_of(0) + sub, a.kb1, nwt1, part1, pair_of(0) < a.pairs1, lane);
    __builtin_amdgcn_sched_barrier(0);
    float csum[MR][kMlpC];
    unsigned char* stage1 = lds;                                     // [nwt1][MR] rows
    float* red1 = reinterpret_cast<float*>(lds + nwt1 * MR * kMlpRowBytes);  // [round][slot][2 nwt1][MR][16]
    mlp_stage_rows<MR>(xr, ZP1 ? 0x1p-24f : -(float)a.zp_const1 * 0x1p-24f, stage1 + part1 * MR * kMlpRowBytes,
                       ps == 0 && sub == 0, csum, lane);
    __syncthreads();  // staged rows and zeroed tickets are visible
    const unsigned char* xs_lane = stage1 + part1 * MR * kMlpRowBytes + (col < MR ? col : 0) * kMlpRowBytes + kq * 16;

    auto round1 = [&](MlpTile& t, int round) {
        const int pair = pair_of(round);
        const bool live = pair < a.pairs1;
        mlp_needed_here(t.sv);
        if constexpr (ZP1) {
            mlp_needed_here(t.zv[0]);
            mlp_needed_here(t.zv[1]);
        }
        float acc[MR];
        mlp_partial<MR, ZP1>(t, xs_lane, csum, acc);
        float* red = red1 + (size_t)(round * PS + ps) * 2 * nwt1 * MR * 16;
        if (kq == 0) {
#pragma unroll
            for (int r = 0; r < MR; ++r)
                red[(wp * MR + r) * 16 + col] = acc[r];
        }
        unsigned ticket = 0;
        if (lane == 0)
            ticket = __hip_atomic_fetch_add(&arrived[round * PS + ps], 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_WORKGROUP);
        ticket = __builtin_amdgcn_readfirstlane(ticket);
        if (ticket != (unsigned)(2 * nwt1 - 1) || !live)
            return;
        // last wave of the pair: gate and up sums, bias, the unit, sixteen values of the intermediate row
        const int n = pair * 32 + col;  // position of the gate channel in the tiled bias order
        const float bg = a.b1 ? (float)a.b1[n] : 0.f, bu = a.b1 ? (float)a.b1[n + 16] : 0.f;
#pragma unroll
        for (int r = 0; r < MR; ++r) {
            const float g = mlp_tile_sum<MR>(red, 0, nwt1, r, lane), u = mlp_tile_sum<MR>(red, nwt1, nwt1, r, lane);
            const half_t hv = to_half_rne(glu_value(a.glu, __builtin_fmaf(g, 0x1p24f, bg), __builtin_fmaf(u, 0x1p24f, bu)));
            if (r < a.M && kq == 0)
                __hip_atomic_store(reinterpret_cast<unsigned short*>(a.h) + (size_t)r * a.K2 + pair * 16 + col,
                                   __builtin_bit_cast(unsigned short, hv), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        // device-scope stores write through; once they are acknowledged the pair counts, and the workgroup's last
        // pair makes the workgroup count
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        unsigned done = 0;
        if (lane == 0)
            done = __hip_atomic_fetch_add(&pairs_done, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_WORKGROUP);
        arrive((int)__builtin_amdgcn_readfirstlane(done) + 1 == my_pairs);
    };
    // One round ahead and no more: with two rounds requested up front the memory system's queues held 64 MB, and
    // everything asked for later -- the activations of workgroups that start late, the intermediate row, the flags
    // -- waited its turn behind them (activations staged 9 us into the kernel instead of 3).
    for (int round = 0; round < a.rounds1; round += 2) {
        {
            const int p = pair_of(round + 1);
            mlp_load_tile<ZP1>(tb, a.w1, a.s1, a.z1, 2 * p + sub, a.kb1, nwt1, part1, round + 1 < a.rounds1 && p < a.pairs1, lane);
        }
        __builtin_amdgcn_sched_barrier(0);
        round1(ta, round);
        if (round + 1 >= a.rounds1)
            break;
        {
            const int p = pair_of(round + 2);
            mlp_load_tile<ZP1>(ta, a.w1, a.s1, a.z1, 2 * p + sub, a.kb1, nwt1, part1, round + 2 < a.rounds1 && p < a.pairs1, lane);
        }
        __builtin_amdgcn_sched_barrier(0);
        round1(tb, round + 1);
    }

    // ---- phase 2: the first down tile's weights leave before anything waits ----
    const bool works2 = wave < nwt2;
    auto tile_of = [&](int round) { return (int)blockIdx.x + G * round; };
    mlp_load_tile<ZP2>(ta, a.w2, a.s2, a.z2, tile_of(0), a.kb2, nwt2, works2 ? wave : 0, works2 && tile_of(0) < a.tiles2, lane);
    __builtin_amdgcn_sched_barrier(0);
    if (wave == 0 && lane == 0) {
        unsigned* go = a.sync + mlp_flag_at(blockIdx.x);
        unsigned spins = 0;
        bool ok = true;
        while (__hip_atomic_load(go, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0u) {
            if (++spins > a.spin_limit) {
                ok = false;
                break;
            }
            __builtin_amdgcn_s_sleep(4);
        }
        if (!ok)
            __hip_atomic_store(a.error, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        else
            __hip_atomic_store(go, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // for the next launch
    }
    __syncthreads();  // every wave of this workgroup is done with phase 1's LDS, and the intermediate row is complete
    if (!works2)
        return;

    const __amdgpu_buffer_rsrc_t rh =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(a.h), 0, a.M * a.K2 * 2, kMlpRsrcFlags);
    mlp_load_rows<MR>(xr, rh, a.M, a.K2, wave, nwt2, 1, lane);
    unsigned char* stage2 = lds + wave * MR * kMlpRowBytes;                    // [nwt2][MR] rows, one set per wave
    float* red2 = reinterpret_cast<float*>(lds + nwt2 * MR * kMlpRowBytes);    // [round][nwt2][MR][16]
    mlp_stage_rows<MR>(xr, ZP2 ? 0x1p-24f : -(float)a.zp_const2 * 0x1p-24f, stage2, true, csum, lane);
    const unsigned char* hs_lane = stage2 + (col < MR ? col : 0) * kMlpRowBytes + kq * 16;
    unsigned* arrived2 = arrived + 8 * kMlpMaxRounds;

    auto round2 = [&](MlpTile& t, int round) {
        const int tile = tile_of(round);
        const bool live = tile < a.tiles2;
        mlp_needed_here(t.sv);
        if constexpr (ZP2) {
            mlp_needed_here(t.zv[0]);
            mlp_needed_here(t.zv[1]);
        }
        float acc[MR];
        mlp_partial<MR, ZP2>(t, hs_lane, csum, acc);
        float* red = red2 + (size_t)round * nwt2 * MR * 16;
        if (kq == 0) {
#pragma unroll
            for (int r = 0; r < MR; ++r)
                red[(wave * MR + r) * 16 + col] = acc[r];
        }
        unsigned ticket = 0;
        if (lane == 0)
            ticket = __hip_atomic_fetch_add(&arrived2[round], 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_WORKGROUP);
        ticket = __builtin_amdgcn_readfirstlane(ticket);
        if (ticket != (unsigned)(nwt2 - 1) || !live)
            return;
        const int n = tile * 16 + col;
        const float b = a.b2 ? (float)a.b2[n] : 0.f;
#pragma unroll
        for (int r = 0; r < MR; ++r) {
            const float s = mlp_tile_sum<MR>(red, 0, nwt2, r, lane);
            if (r < a.M && kq == 0)
                store_out(a.y, (size_t)r * a.N2 + n, __builtin_fmaf(s, 0x1p24f, b), a.out_f32);
        }
    };
    for (int round = 0; round < a.rounds2; round += 2) {
        mlp_load_tile<ZP2>(tb, a.w2, a.s2, a.z2, tile_of(round + 1), a.kb2, nwt2, wave,
                           round + 1 < a.rounds2 && tile_of(round + 1) < a.tiles2, lane);
        __builtin_amdgcn_sched_barrier(0);
        round2(ta, round);
        if (round + 1 >= a.rounds2)
            break;
        mlp_load_tile<ZP2>(ta, a.w2, a.s2, a.z2, tile_of(round + 2), a.kb2, nwt2, wave,
                           round + 2 < a.rounds2 && tile_of(round + 2) < a.tiles2, lane);
        __builtin_amdgcn_sched_barrier(0);
        round2(tb, round + 1);
    }
}

// Dynamic LDS of a launch: the larger of the two phases' staged rows and partial sums.
size_t mlp_lds_bytes(int mr, int nwt1, int rounds1, int nwt2, int rounds2) {
    const size_t p1 = (size_t)nwt1 * mr * kMlpRowBytes + (size_t)rounds1 * 16 * mr * 16 * sizeof(float);
    const size_t p2 = (size_t)nwt2 * mr * kMlpRowBytes + (size_t)rounds2 * nwt2 * mr * 16 * sizeof(float);
    return p1 > p2 ? p1 : p2;
}

size_t mlp_sync_bytes(int grid) {
    return (mlp_flag_at((size_t)grid) + 64) * sizeof(unsigned);
}

// Whether the one-launch kernel can run this pair of nodes at M rows on `grid` workgroups.
bool mlp_fused_applies(const Layout& g, const Layout& d, int64_t M, int grid) {
    auto node_ok = [](const Layout& L) {
        return L.tiled && L.bits == 4 && L.groups_per_kblock == 1 && L.kblocks_per_group == 1 && L.gemv_c == kMlpC &&
               L.k_blocks % kMlpC == 0;
    };
    if (M < 1 || M > 4 || grid < 1 || !node_ok(g) || !node_ok(d) || !g.glu || d.glu || (g.n_tiles & 1))
        return false;
    const int64_t nwt1 = g.k_blocks / kMlpC, nwt2 = d.k_blocks / kMlpC;
    if ((nwt1 != 1 && nwt1 != 2 && nwt1 != 4 && nwt1 != 8) || nwt2 < 1 || nwt2 > kMlpWaves)
        return false;
    const int64_t ps = 8 / nwt1, pairs = g.n_tiles / 2;
    const int64_t rounds1 = (pairs + (int64_t)grid * ps - 1) / (grid * ps), rounds2 = (d.n_tiles + grid - 1) / grid;
    return rounds1 <= kMlpMaxRounds && rounds2 <= kMlpMaxRounds && d.k_blocks * 128 == pairs * 16;
}

template <int MR, bool ZP1, bool ZP2>
static int launch_mlp_impl(const MlpKernelArgs& k, int grid, int n_cus, size_t lds_bytes, hipStream_t s) {
    auto kern = fcc_mlp_gemv_kernel<MR, ZP1, ZP2>;
    static bool attr_set = false;  // per instantiation; the attribute is idempotent, a race only repeats it
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024 - 1024);
        if (e != hipSuccess)
            return (int)e;
        attr_set = true;
    }
    // every workgroup must be resident at once: the wait in the middle of the kernel is for all of them
    // (asked once per instantiation and LDS size; a race only repeats the question)
    static size_t asked_lds = ~(size_t)0;
    static int per_cu = 0;
    if (asked_lds != lds_bytes) {
        int n = 0;
        hipError_t e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kern, 64 * kMlpWaves, lds_bytes);
        if (e != hipSuccess)
            return (int)e;
        per_cu = n, asked_lds = lds_bytes;
    }
    if (per_cu < 1 || (int64_t)grid > (int64_t)per_cu * n_cus)
        return (int)hipErrorLaunchOutOfResources;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(64 * kMlpWaves), lds_bytes, s, k);
    return (int)hipGetLastError();
}

// gate / up node `g` (with its gated linear unit), down node `d`: x [M, K1] -> mid [M, K2] (scratch) -> y [M, N2].
// sync: the arrival counter and the go flags (mlp_sync_bytes(grid) bytes), zero between launches; error: host-visible
// flag.
int launch_mlp(const FcDeviceArgs& g, const FcDeviceArgs& d, void* mid, unsigned* sync, unsigned* error, int grid,
               int n_cus, unsigned spin_limit, void* stream) {
    const Layout &L1 = g.layout, &L2 = d.layout;
    if (!mlp_fused_applies(L1, L2, g.M, grid) || n_cus < 1 || g.M != d.M || !g.scale_cm || !d.scale_cm || (L1.zp_table && !g.zp_cm) ||
        (L2.zp_table && !d.zp_cm) || !mid || !sync || !error || g.K * 2 * g.M >= ((int64_t)1 << 31) ||
        d.K * 2 * d.M >= ((int64_t)1 << 31) || (int64_t)16 * L1.k_blocks * 2 >= ((int64_t)1 << 31) ||
        (int64_t)16 * L2.k_blocks * 2 >= ((int64_t)1 << 31))
        return (int)hipErrorInvalidValue;
    MlpKernelArgs k;
    k.w1 = (const uint4_t*)g.w, k.s1 = (const half_t*)g.scale_cm, k.z1 = (const uint8_t*)g.zp_cm, k.b1 = (const half_t*)g.bias;
    k.w2 = (const uint4_t*)d.w, k.s2 = (const half_t*)d.scale_cm, k.z2 = (const uint8_t*)d.zp_cm, k.b2 = (const half_t*)d.bias;
    k.x = (const half_t*)g.x, k.h = (half_t*)mid, k.y = d.y, k.sync = sync, k.error = error;
    k.M = (int)g.M, k.K1 = (int)g.K, k.K2 = (int)d.K, k.N2 = (int)d.N;
    k.kb1 = (int)L1.k_blocks, k.nwt1 = k.kb1 / kMlpC, k.kb2 = (int)L2.k_blocks, k.nwt2 = k.kb2 / kMlpC;
    k.pairs1 = (int)(L1.n_tiles / 2), k.tiles2 = (int)L2.n_tiles;
    const int ps = 8 / k.nwt1;
    k.rounds1 = (k.pairs1 + grid * ps - 1) / (grid * ps), k.rounds2 = (k.tiles2 + grid - 1) / grid;
    k.zp_const1 = L1.zp_const, k.zp_const2 = L2.zp_const, k.glu = L1.glu, k.out_f32 = d.out_f32;
    k.spin_limit = spin_limit;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int mr = g.M == 1 ? 1 : g.M == 2 ? 2 : 4;
    const size_t lds_bytes = mlp_lds_bytes(mr, k.nwt1, k.rounds1, k.nwt2, k.rounds2);
    if (lds_bytes > 160 * 1024 - 1024)
        return (int)hipErrorInvalidValue;
#define OVFCC_MLP_CASE(MR)                                                                                   \
    (L1.zp_table ? (L2.zp_table ? launch_mlp_impl<MR, true, true>(k, grid, n_cus, lds_bytes, s)                     \
                                : launch_mlp_impl<MR, true, false>(k, grid, n_cus, lds_bytes, s))                   \
                 : (L2.zp_table ? launch_mlp_impl<MR, false, true>(k, grid, n_cus, lds_bytes, s)                    \
                                : launch_mlp_impl<MR, false, false>(k, grid, n_cus, lds_bytes, s)))
    const int rc = mr == 1 ? OVFCC_MLP_CASE(1) : mr == 2 ? OVFCC_MLP_CASE(2) : OVFCC_MLP_CASE(4);
#undef OVFCC_MLP_CASE
    return rc;
}

}  // namespace ovfcc
