// Epilogue shared by the prefill kernels with 256-channel tiles and 8 waves (wn = wave & 3 owns 64 channels as four
// 16-channel tiles, kg = wave >> 2 owns half of every k-block): acc[r][t] is the wave's f32 result for channel tile r
// and row tile t in the 16x16 MFMA layout (lane: column m = lane & 15, channels 4 (lane >> 4) + q).
#pragma once

#include <type_traits>

#include "device_common.h"

namespace ovfcc {

// Split-K, after a workgroup has parked its f32 tile (layout [split][wn][channel tile r][row tile t][lane] float4
// behind rp) with device-scope stores: wait for them, draw a ticket from the tile's arrival counter; the last
// arrival adds the parked tiles in split order with device-scope loads (the result does not depend on arrival
// order), finishes the outputs and returns the counter to zero.
template <bool PRESCALE, int NT>
__device__ __forceinline__ void split_k_last_arrival(const __amdgpu_buffer_rsrc_t rp, const half_t* __restrict__ st,
                                                     const half_t* __restrict__ bias, void* __restrict__ y,
                                                     unsigned* __restrict__ counters, int M, int N, int n0, int m0,
                                                     int split_k, int tile_id, int out_f32, int glu) {
    constexpr int kAuxDeviceScope = 16;
    constexpr unsigned kParkBytes = 4 * (4 * NT) * 64 * 16;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wn = wave & 3, kg = wave >> 2;
    const int col = lane & 15, kq = lane >> 4;
    __shared__ unsigned ticket_s;
    auto finish = [&](int r, int t, float4_t v, const float (&sc)[4], const float (&bs)[4]) {
        const int n = n0 + 64 * wn + 16 * r + 4 * kq;  // four consecutive channels
        const int m = m0 + 16 * t + col;
        const float o[4] = {v.x * sc[0] + bs[0], v.y * sc[1] + bs[1], v.z * sc[2] + bs[2], v.w * sc[3] + bs[3]};
        if (m < M) {
            if (out_f32) {
                *reinterpret_cast<float4_t*>(static_cast<float*>(y) + (size_t)m * N + n) = float4_t{o[0], o[1], o[2], o[3]};
            } else {
                *reinterpret_cast<half4_t*>(static_cast<half_t*>(y) + (size_t)m * N + n) =
                    half4_t{to_half_rne(o[0]), to_half_rne(o[1]), to_half_rne(o[2]), to_half_rne(o[3])};
            }
        }
    };
    auto finish_glu = [&](int j, int t, float4_t g, float4_t u, const float (&scg)[4], const float (&bsg)[4],
                          const float (&scu)[4], const float (&bsu)[4]) {
        const int n = (n0 + 64 * wn) / 2 + 16 * j + 4 * kq;
        const int m = m0 + 16 * t + col;
        const float o[4] = {glu_value(glu, g.x * scg[0] + bsg[0], u.x * scu[0] + bsu[0]),
                            glu_value(glu, g.y * scg[1] + bsg[1], u.y * scu[1] + bsu[1]),
                            glu_value(glu, g.z * scg[2] + bsg[2], u.z * scu[2] + bsu[2]),
                            glu_value(glu, g.w * scg[3] + bsg[3], u.w * scu[3] + bsu[3])};
        if (m < M) {
            if (out_f32) {
                *reinterpret_cast<float4_t*>(static_cast<float*>(y) + (size_t)m * (N / 2) + n) =
                    float4_t{o[0], o[1], o[2], o[3]};
            } else {
                *reinterpret_cast<half4_t*>(static_cast<half_t*>(y) + (size_t)m * (N / 2) + n) =
                    half4_t{to_half_rne(o[0]), to_half_rne(o[1]), to_half_rne(o[2]), to_half_rne(o[3])};
            }
        }
    };
    auto channel_params = [&](int r, float (&sc)[4], float (&bs)[4]) {
        const int n = n0 + 64 * wn + 16 * r + 4 * kq;
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
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the parked tile has reached memory before the ticket is drawn
    __syncthreads();
    if (tid == 0)
        ticket_s = __hip_atomic_fetch_add(counters + tile_id, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (ticket_s != (unsigned)(split_k - 1))
        return;
    // Last arrival: every wave adds up two of its k-group pair's four channel tiles (k-group kg takes tiles 2 kg and
    // 2 kg + 1 -- a gate tile and its up tile), all row tiles, parts in ascending order.  The loads of two parts,
    // 2 x 2 NT of them, are in flight together (a part index past split_k falls outside the descriptor's range
    // and reads zero); issued one at a time behind their additions they cost 9 us per part.
    float4_t sum[2][NT];
#pragma unroll
    for (int r2 = 0; r2 < 2; ++r2)
#pragma unroll
        for (int t = 0; t < NT; ++t)
            sum[r2][t] = float4_t{0.f, 0.f, 0.f, 0.f};
    for (int z0 = 0; z0 < split_k; z0 += 2) {
        float4_t part[2][2][NT];
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int r2 = 0; r2 < 2; ++r2)
#pragma unroll
                for (int t = 0; t < NT; ++t)
                    part[u][r2][t] = __builtin_bit_cast(
                        float4_t, __builtin_amdgcn_raw_buffer_load_b128(
                                      rp, (unsigned)(z0 + u) * kParkBytes +
                                              (unsigned)(((wn * 4 + 2 * kg + r2) * NT + t) * 64 + lane) * 16u,
                                      0, kAuxDeviceScope));
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int r2 = 0; r2 < 2; ++r2)
#pragma unroll
                for (int t = 0; t < NT; ++t) {
                    sum[r2][t].x += part[u][r2][t].x, sum[r2][t].y += part[u][r2][t].y;
                    sum[r2][t].z += part[u][r2][t].z, sum[r2][t].w += part[u][r2][t].w;
                }
    }
    if (glu) {
        float scg[4], bsg[4], scu[4], bsu[4];
        channel_params(2 * kg, scg, bsg);
        channel_params(2 * kg + 1, scu, bsu);
#pragma unroll
        for (int t = 0; t < NT; ++t)
            finish_glu(kg, t, sum[0][t], sum[1][t], scg, bsg, scu, bsu);
    } else {
        float sc[2][4], bs[2][4];
        channel_params(2 * kg, sc[0], bs[0]);
        channel_params(2 * kg + 1, sc[1], bs[1]);
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int r2 = 0; r2 < 2; ++r2)
                finish(2 * kg + r2, t, sum[r2][t], sc[r2], bs[r2]);
    }
    if (tid == 0)
        __hip_atomic_store(counters + tile_id, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// k-group 1 -> k-group 0 through LDS, two channel tiles at a time.  Without split-K k-group 0
// finishes the outputs; with split-K it parks the f32 tile in the workspace with device-scope stores and
// waits for them, the workgroup draws a ticket from the tile's arrival counter, and the last arrival adds
// the parked tiles in split order with device-scope loads (the result does not depend on arrival order),
// finishes the outputs and returns the counter to zero.  No fences: a device-scope fence writes back and
// invalidates whole caches, which costs more than the kernel.
// The caller has waited for its own outstanding loads into LDS; lds_raw is the workgroup's dynamic LDS (at least
// NT * 8 KiB), n0 / m0 the tile's first channel and row, z_part this workgroup's part of split_k, park_slot the
// tile's slot in workspace and counters.
template <bool PRESCALE, int NT>
__device__ __forceinline__ void tile_epilogue(float4_t (&acc)[4][NT], unsigned char* lds_raw,
                                              const half_t* __restrict__ st, const half_t* __restrict__ bias,
                                              void* __restrict__ y, float* __restrict__ ws,
                                              unsigned* __restrict__ counters, int M, int N, int n0, int m0, int split_k,
                                              int z_part, int park_slot, int out_f32, int glu) {
    constexpr int kRsrcFlags = 0x00020000;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wn = wave & 3, kg = wave >> 2;
    const int col = lane & 15, kq = lane >> 4;
    const int tile_id = park_slot;
    __syncthreads();
    float* ex = reinterpret_cast<float*>(lds_raw);  // [wn][2 x 8 x 4][64 lanes]
    // parked tile layout: [tile][split][wn][channel tile r][row tile t][lane] float4
    constexpr int kAuxDeviceScope = 16;              // sc1: write through to / read from memory shared by all XCDs
    constexpr unsigned kParkBytes = 4 * (4 * NT) * 64 * 16;  // one workgroup's f32 tile
    const __amdgpu_buffer_rsrc_t rp = __builtin_amdgcn_make_buffer_rsrc(
        reinterpret_cast<char*>(ws) + (size_t)tile_id * split_k * kParkBytes, 0, split_k * (int)kParkBytes, kRsrcFlags);
    auto finish = [&](int r, int t, float4_t v, const float (&sc)[4], const float (&bs)[4]) {
        const int n = n0 + 64 * wn + 16 * r + 4 * kq;  // four consecutive channels
        const int m = m0 + 16 * t + col;
        const float o[4] = {v.x * sc[0] + bs[0], v.y * sc[1] + bs[1], v.z * sc[2] + bs[2], v.w * sc[3] + bs[3]};
        if (m < M) {
            if (out_f32) {
                *reinterpret_cast<float4_t*>(static_cast<float*>(y) + (size_t)m * N + n) = float4_t{o[0], o[1], o[2], o[3]};
            } else {
                *reinterpret_cast<half4_t*>(static_cast<half_t*>(y) + (size_t)m * N + n) =
                    half4_t{to_half_rne(o[0]), to_half_rne(o[1]), to_half_rne(o[2]), to_half_rne(o[3])};
            }
        }
    };
    // gated linear unit: channel tiles 2 j and 2 j + 1 of the wave are gate and up of output channels
    // (n0 + 64 wn) / 2 + 16 j .. of the [M, N / 2] result
    auto finish_glu = [&](int j, int t, float4_t g, float4_t u, const float (&scg)[4], const float (&bsg)[4],
                          const float (&scu)[4], const float (&bsu)[4]) {
        const int n = (n0 + 64 * wn) / 2 + 16 * j + 4 * kq;
        const int m = m0 + 16 * t + col;
        const float o[4] = {glu_value(glu, g.x * scg[0] + bsg[0], u.x * scu[0] + bsu[0]),
                            glu_value(glu, g.y * scg[1] + bsg[1], u.y * scu[1] + bsu[1]),
                            glu_value(glu, g.z * scg[2] + bsg[2], u.z * scu[2] + bsu[2]),
                            glu_value(glu, g.w * scg[3] + bsg[3], u.w * scu[3] + bsu[3])};
        if (m < M) {
            if (out_f32) {
                *reinterpret_cast<float4_t*>(static_cast<float*>(y) + (size_t)m * (N / 2) + n) =
                    float4_t{o[0], o[1], o[2], o[3]};
            } else {
                *reinterpret_cast<half4_t*>(static_cast<half_t*>(y) + (size_t)m * (N / 2) + n) =
                    half4_t{to_half_rne(o[0]), to_half_rne(o[1]), to_half_rne(o[2]), to_half_rne(o[3])};
            }
        }
    };
    auto channel_params = [&](int r, float (&sc)[4], float (&bs)[4]) {
        const int n = n0 + 64 * wn + 16 * r + 4 * kq;
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
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) {
        if (kg == 1) {
#pragma unroll
            for (int r2 = 0; r2 < 2; ++r2)
#pragma unroll
                for (int t = 0; t < NT; ++t) {
                    const float4_t v = acc[2 * hh + r2][t];
                    float* p = ex + ((wn * 8 * NT + (r2 * NT + t) * 4) * 64) + lane;
                    p[0] = v.x, p[64] = v.y, p[128] = v.z, p[192] = v.w;
                }
        }
        __syncthreads();
        if (kg == 0 && glu && split_k == 1) {
            float scg[4], bsg[4], scu[4], bsu[4];
            channel_params(2 * hh, scg, bsg);
            channel_params(2 * hh + 1, scu, bsu);
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                const float* pg = ex + ((wn * 8 * NT + t * 4) * 64) + lane;
                const float* pu = ex + ((wn * 8 * NT + (NT + t) * 4) * 64) + lane;
                const float4_t a = acc[2 * hh][t], b = acc[2 * hh + 1][t];
                finish_glu(hh, t, float4_t{a.x + pg[0], a.y + pg[64], a.z + pg[128], a.w + pg[192]},
                           float4_t{b.x + pu[0], b.y + pu[64], b.z + pu[128], b.w + pu[192]}, scg, bsg, scu, bsu);
            }
        } else if (kg == 0) {
            // row tile by row tile, the two channel tiles back to back: their pieces of an output row are
            // neighbours in one 128-byte line, and stores to a line that follow each other closely merge
            float sc[2][4], bs[2][4];
            channel_params(2 * hh, sc[0], bs[0]);
            channel_params(2 * hh + 1, sc[1], bs[1]);
#pragma unroll
            for (int t = 0; t < NT; ++t) {
#pragma unroll
                for (int r2 = 0; r2 < 2; ++r2) {
                    const int r = 2 * hh + r2;
                    const float* p = ex + ((wn * 8 * NT + (r2 * NT + t) * 4) * 64) + lane;
                    const float4_t a = acc[r][t];
                    const float4_t v = float4_t{a.x + p[0], a.y + p[64], a.z + p[128], a.w + p[192]};
                    if (split_k == 1)
                        finish(r, t, v, sc[r2], bs[r2]);
                    else
                        __builtin_amdgcn_raw_buffer_store_b128(
                            __builtin_bit_cast(uint4_t, v), rp,
                            z_part * kParkBytes + (unsigned)(((wn * 4 + r) * NT + t) * 64 + lane) * 16u, 0,
                            kAuxDeviceScope);
                }
            }
        }
        __syncthreads();
    }
    if (split_k == 1)
        return;
    split_k_last_arrival<PRESCALE, NT>(rp, st, bias, y, counters, M, N, n0, m0, split_k, tile_id, out_f32, glu);
}


// The same epilogue for kernels whose LDS holds NT x 16 KiB: the k-groups share the output instead of one handing
// everything to the other.  k-group 0 finishes row tiles [0, T0), k-group 1 row tiles [T0, NT) (T0 = NT / 2 rounded
// up): each wave sends its partner (wave ^ 4) the partial sums of the partner's row tiles through LDS -- 16 bytes per
// lane and accumulator, one barrier -- adds what it receives and then holds all four channel tiles of its own row
// tiles, so all eight waves convert and store.  An f16 result without a gated linear unit leaves in whole 128-byte
// lines: the four lanes of a row (lane bits 4 and 5) hold four channels of each of the wave's four channel tiles, a
// 4 x 4 exchange between them (halves of the wave swapped, then neighbouring rows of 16 lanes) leaves lane kq with
// all 16 channels of tile kq, 32 contiguous bytes, and the four lanes write the row's line with two store
// instructions.  The sums are the same as the other form's (a + b with the k-groups' roles swapped for half of the
// tiles), split-K parks the same tile layout and is finished by the same last arrival.
template <bool PRESCALE, int NT>
__device__ __forceinline__ void tile_epilogue_shared(float4_t (&acc)[4][NT], unsigned char* lds_raw,
                                                     const half_t* __restrict__ st, const half_t* __restrict__ bias,
                                                     void* __restrict__ y, float* __restrict__ ws,
                                                     unsigned* __restrict__ counters, int M, int N, int n0, int m0,
                                                     int split_k, int z_part, int park_slot, int out_f32, int glu) {
    constexpr int kRsrcFlags = 0x00020000;
    constexpr int T0 = (NT + 1) / 2;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wn = wave & 3, kg = wave >> 2;
    const int col = lane & 15, kq = lane >> 4;
    const int tile_id = park_slot;
    constexpr int kAuxDeviceScope = 16;
    constexpr unsigned kParkBytes = 4 * (4 * NT) * 64 * 16;
    const __amdgpu_buffer_rsrc_t rp = __builtin_amdgcn_make_buffer_rsrc(
        reinterpret_cast<char*>(ws) + (size_t)tile_id * split_k * kParkBytes, 0, split_k * (int)kParkBytes, kRsrcFlags);
    float4_t* ex = reinterpret_cast<float4_t*>(lds_raw);  // [wave][4 x T0][64 lanes]
    __syncthreads();                                      // everyone has left the main loop's LDS
    auto channel_params = [&](int r, float (&sc)[4], float (&bs)[4]) {
        const int n = n0 + 64 * wn + 16 * r + 4 * kq;
#pragma unroll
        for (int q = 0; q < 4; ++q)
            sc[q] = 1.f, bs[q] = 0.f;
        if constexpr (!PRESCALE) {
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
    // KG: this wave's k-group; it owns row tiles [LO, LO + CNT) and sends [SLO, SLO + SCNT)
    auto send = [&](auto kg_const) {
        constexpr int KG = decltype(kg_const)::value;
        constexpr int SLO = KG == 0 ? T0 : 0, SCNT = KG == 0 ? NT - T0 : T0;
        float4_t* mine = ex + (size_t)(wave * 4 * T0) * 64 + lane;
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int i = 0; i < SCNT; ++i)
                mine[(r * T0 + i) * 64] = acc[r][SLO + i];
    };
    auto run = [&](auto kg_const) {
        constexpr int KG = decltype(kg_const)::value;
        constexpr int LO = KG == 0 ? 0 : T0, CNT = KG == 0 ? T0 : NT - T0;
        const float4_t* theirs = ex + (size_t)((wave ^ 4) * 4 * T0) * 64 + lane;
        float4_t v[4][CNT > 0 ? CNT : 1];
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int i = 0; i < CNT; ++i) {
                const float4_t a = acc[r][LO + i], b = theirs[(r * T0 + i) * 64];
                v[r][i] = float4_t{a.x + b.x, a.y + b.y, a.z + b.z, a.w + b.w};
            }
        if (split_k != 1) {
#pragma unroll
            for (int r = 0; r < 4; ++r)
#pragma unroll
                for (int i = 0; i < CNT; ++i)
                    __builtin_amdgcn_raw_buffer_store_b128(
                        __builtin_bit_cast(uint4_t, v[r][i]), rp,
                        z_part * kParkBytes + (unsigned)(((wn * 4 + r) * NT + LO + i) * 64 + lane) * 16u, 0,
                        kAuxDeviceScope);
            return;
        }
        if (glu) {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                float scg[4], bsg[4], scu[4], bsu[4];
                channel_params(2 * j, scg, bsg);
                channel_params(2 * j + 1, scu, bsu);
                const int n = (n0 + 64 * wn) / 2 + 16 * j + 4 * kq;
#pragma unroll
                for (int i = 0; i < CNT; ++i) {
                    const int m = m0 + 16 * (LO + i) + col;
                    const float4_t g = v[2 * j][i], u = v[2 * j + 1][i];
                    const float o[4] = {glu_value(glu, g.x * scg[0] + bsg[0], u.x * scu[0] + bsu[0]),
                                        glu_value(glu, g.y * scg[1] + bsg[1], u.y * scu[1] + bsu[1]),
                                        glu_value(glu, g.z * scg[2] + bsg[2], u.z * scu[2] + bsu[2]),
                                        glu_value(glu, g.w * scg[3] + bsg[3], u.w * scu[3] + bsu[3])};
                    if (m < M) {
                        if (out_f32)
                            *reinterpret_cast<float4_t*>(static_cast<float*>(y) + (size_t)m * (N / 2) + n) =
                                float4_t{o[0], o[1], o[2], o[3]};
                        else
                            *reinterpret_cast<half4_t*>(static_cast<half_t*>(y) + (size_t)m * (N / 2) + n) =
                                half4_t{to_half_rne(o[0]), to_half_rne(o[1]), to_half_rne(o[2]), to_half_rne(o[3])};
                    }
                }
            }
            return;
        }
        float sc[4][4], bs[4][4];
#pragma unroll
        for (int r = 0; r < 4; ++r)
            channel_params(r, sc[r], bs[r]);
        if (!out_f32 && (reinterpret_cast<uintptr_t>(y) & 15) == 0 && (N & 7) == 0) {
            half_t* yh = static_cast<half_t*>(y);
#pragma unroll
            for (int i = 0; i < CNT; ++i) {
                uint32_t p[4][2];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float4_t a = v[r][i];
                    const half4_t h = half4_t{to_half_rne(a.x * sc[r][0] + bs[r][0]), to_half_rne(a.y * sc[r][1] + bs[r][1]),
                                              to_half_rne(a.z * sc[r][2] + bs[r][2]), to_half_rne(a.w * sc[r][3] + bs[r][3])};
                    const uint2_t u = __builtin_bit_cast(uint2_t, h);
                    p[r][0] = u.x, p[r][1] = u.y;
                }
                uint32_t q[8];  // channels 4 k' .. 4 k' + 3 of tile kq, from lane k' of the row: dwords 2 k', 2 k' + 1
#pragma unroll
                for (int d = 0; d < 2; ++d) {
                    // lanes 0-31 keep tiles 0 and 1, lanes 32-63 tiles 2 and 3; .x comes from the lane with kq bit
                    // 1 clear, .y from the one with it set
                    const uint2_t s02 = __builtin_amdgcn_permlane32_swap(p[0][d], p[2][d], false, false);
                    const uint2_t s13 = __builtin_amdgcn_permlane32_swap(p[1][d], p[3][d], false, false);
                    // even rows of 16 lanes keep the even tile, odd rows the odd one; .x from kq bit 0 clear, .y set
                    const uint2_t lo = __builtin_amdgcn_permlane16_swap(s02.x, s13.x, false, false);
                    const uint2_t hi = __builtin_amdgcn_permlane16_swap(s02.y, s13.y, false, false);
                    q[d] = lo.x, q[2 + d] = lo.y, q[4 + d] = hi.x, q[6 + d] = hi.y;
                }
                const int m = m0 + 16 * (LO + i) + col;
                if (m < M) {
                    uint4_t* dst = reinterpret_cast<uint4_t*>(yh + (size_t)m * N + n0 + 64 * wn + 16 * kq);
                    // whole lines that nobody reads again in this launch: the non-temporal hint is worth 0.7 % on a
                    // launch of one tile per compute unit (14336 -> 4096 at 2048 rows: 187.5 -> 186.2 us)
                    __builtin_nontemporal_store(uint4_t{q[0], q[1], q[2], q[3]}, dst);
                    __builtin_nontemporal_store(uint4_t{q[4], q[5], q[6], q[7]}, dst + 1);
                }
            }
            return;
        }
#pragma unroll
        for (int i = 0; i < CNT; ++i) {
            const int m = m0 + 16 * (LO + i) + col;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int n = n0 + 64 * wn + 16 * r + 4 * kq;
                const float4_t a = v[r][i];
                const float o[4] = {a.x * sc[r][0] + bs[r][0], a.y * sc[r][1] + bs[r][1], a.z * sc[r][2] + bs[r][2],
                                    a.w * sc[r][3] + bs[r][3]};
                if (m < M) {
                    if (out_f32)
                        *reinterpret_cast<float4_t*>(static_cast<float*>(y) + (size_t)m * N + n) =
                            float4_t{o[0], o[1], o[2], o[3]};
                    else
                        *reinterpret_cast<half4_t*>(static_cast<half_t*>(y) + (size_t)m * N + n) =
                            half4_t{to_half_rne(o[0]), to_half_rne(o[1]), to_half_rne(o[2]), to_half_rne(o[3])};
                }
            }
        }
    };
    if (kg == 0)
        send(std::integral_constant<int, 0>{});
    else
        send(std::integral_constant<int, 1>{});
    __syncthreads();
    if (kg == 0)
        run(std::integral_constant<int, 0>{});
    else
        run(std::integral_constant<int, 1>{});
    if (split_k == 1)
        return;
    split_k_last_arrival<PRESCALE, NT>(rp, st, bias, y, counters, M, N, n0, m0, split_k, tile_id, out_f32, glu);
}

}  // namespace ovfcc
