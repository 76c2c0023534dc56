// Small-batch decode kernel (M <= 48) over the tiled layout.
//
// With more than a few activation rows the streaming decode kernel re-reads X once per 16 output channels,
// which costs more than the weights.  Here a workgroup owns NW * RT channel tiles and one slice of K instead:
//
//   grid = (ceil(N / 16 / (NW RT)), split_k), block = 64 NW.  Workgroup (g, ks) stages X[0:M, its k-range]
//   in LDS once (rows >= M are zero) and wave w streams the k-range of its own RT channel tiles
//   (g NW + w) RT .. +RT, one 1 KiB tile per 128-bit load per lane, DEPTH k-blocks in flight, straight
//   from HBM into the MFMA weight operand.  The activation operand is read from LDS (lanes 0-15 of a
//   128-bit read hit 16 different rows; the row pitch of 16 bytes more than a multiple of 256 spreads
//   them over all banks).
//
// Arithmetic as in the streaming kernel: exact halves q - zp, v_mfma_f32_16x16x32_f16 with A = activations,
// f32 partial per k-block multiplied by the group scale.  Bias and zero-point are removed on the vector
// ALU here (one packed subtract per two weights): with two or more row tiles per weight tile the matrix
// cores are the scarcer unit.
//
// No reduction inside the workgroup.  With split_k > 1 each workgroup publishes its partial tiles with
// device-scope stores, waits for them, and draws a ticket from the group's arrival counter; the last
// arrival adds the partials in split order (independent of arrival order) and zeroes the counter.
#include "device_common.h"

namespace ovfcc {

template <int TPB, int RT, int GPB>
struct BatchSlot {
    uint4_t w[RT][TPB];
    uint32_t scale[RT][GPB == 4 ? 2 : 1];  // GPB f16 scales, packed
    uint32_t zp[RT];                       // GPB zero-points, one per byte
};

// GPB: groups per k-block (2 or 4 for groups of 64 or 32 inputs, 4-bit weights only); MFMA j of a k-block
// covers inputs 32 j ..+32 and adds into the partial sum of group j GPB / 4.
template <int BITS, int MT, bool ZP_TABLE, int RT, int GPB>
__device__ __forceinline__ void batch_body(const uint4_t* __restrict__ wt, const half_t* __restrict__ st,
                                           const uint8_t* __restrict__ zt, const half_t* __restrict__ x,
                                           const half_t* __restrict__ bias, void* __restrict__ y,
                                           float* __restrict__ ws, unsigned* __restrict__ counters, int M, int N, int K,
                                           int kb_total, int kb_per_group, int ng, int zp_const, int kb_per_split,
                                           int split_k, int n_tiles, int out_f32, int glu) {
    static_assert(GPB == 1 || ((GPB == 2 || GPB == 4) && BITS == 4), "groups below 128 inputs: 4-bit weights only");
    constexpr int TPB = BITS == 4 ? 1 : 2;                    // tiles per k-block
    constexpr int DEPTH = (RT * TPB >= 4) ? 2 : 4 / TPB;      // k-blocks in flight per wave
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    __shared__ unsigned ticket_s;
    half_t* xs = reinterpret_cast<half_t*>(lds);              // [16 MT][x_stride]

    const int grp = blockIdx.x;
    const int ks = blockIdx.y;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nw = blockDim.x >> 6;
    const int col = lane & 15;
    const int kq = lane >> 4;

    const int kb_begin = ks * kb_per_split;
    const int kb_end = min(kb_total, kb_begin + kb_per_split);
    const int cnt = kb_end - kb_begin;
    const int x_stride = cnt * 128 + 8;  // halves

    const int tile0 = (grp * nw + wave) * RT;
    const int tiles_here = max(0, min(RT, n_tiles - tile0));  // 0: this wave has no channels (ragged last group)

    constexpr unsigned kOob = 0x80000000u;
    constexpr int kRsrcFlags = 0x00020000;
    const size_t tile_base = tiles_here ? (size_t)tile0 : 0;
    const __amdgpu_buffer_rsrc_t rw =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<uint4_t*>(wt + tile_base * kb_total * TPB * 64), 0,
                                          tiles_here * kb_total * TPB * kTileBytes, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(st + tile_base * ng * 16),
                                                                        0, tiles_here * ng * 32, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t rz = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint8_t*>(ZP_TABLE ? zt + tile_base * ng * 16 : zt), 0, ZP_TABLE ? tiles_here * ng * 16 : 0,
        kRsrcFlags);
    const __amdgpu_buffer_rsrc_t rx =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(x), 0, M * K * 2, kRsrcFlags);

    const unsigned g_mul = kb_per_group == 1 ? 0u : (unsigned)((0x100000000ull + kb_per_group - 1) / kb_per_group);
    using Slot = BatchSlot<TPB, RT, GPB>;
    auto issue = [&](int i, Slot& s) {
        // bit 31 of every offset of a slot past the end of the k-range is set: out of range, reads zero
        const unsigned oob = (unsigned)((cnt - 1 - i) >> 31) & kOob;
        const unsigned kb = (unsigned)(kb_begin + i);
        const unsigned g = kb_per_group == 1 ? kb : __umulhi(kb, g_mul);
#pragma unroll
        for (int r = 0; r < RT; ++r) {
            const unsigned wofs = ((r * kb_total + kb) * (unsigned)(TPB * kTileBytes) + lane * 16u) | oob;
#pragma unroll
            for (int t = 0; t < TPB; ++t)
                s.w[r][t] =
                    __builtin_bit_cast(uint4_t, __builtin_amdgcn_raw_buffer_load_b128(rw, wofs + t * kTileBytes, 0, 2));
            if constexpr (GPB == 1) {
                const unsigned sidx = (r * ng + g) * 16u + col;
                s.scale[r][0] = __builtin_amdgcn_raw_buffer_load_b16(rs, (sidx * 2u) | oob, 0, 0);
                if constexpr (ZP_TABLE)
                    s.zp[r] = __builtin_amdgcn_raw_buffer_load_b8(rz, sidx | oob, 0, 0);
            } else {
                const unsigned sidx = ((r * kb_total + kb) * 16u + col) * GPB;
                if constexpr (GPB == 2) {
                    s.scale[r][0] = __builtin_amdgcn_raw_buffer_load_b32(rs, (sidx * 2u) | oob, 0, 0);
                    if constexpr (ZP_TABLE)
                        s.zp[r] = __builtin_amdgcn_raw_buffer_load_b16(rz, sidx | oob, 0, 0);
                } else {
                    const uint2_t v = __builtin_bit_cast(uint2_t, __builtin_amdgcn_raw_buffer_load_b64(rs, (sidx * 2u) | oob, 0, 0));
                    s.scale[r][0] = v.x, s.scale[r][1] = v.y;
                    if constexpr (ZP_TABLE)
                        s.zp[r] = __builtin_amdgcn_raw_buffer_load_b32(rz, sidx | oob, 0, 0);
                }
            }
        }
    };

    // Stage X[0 : 16 MT, k-range] in LDS; 16-byte chunks, coalesced along k; rows >= M read zeros.  The loads go
    // out BEFORE the first weight loads: the memory counter retires in order, so a wave that asked for its weights
    // first could not write the staged activations until all of those weights had landed, and the workgroup would
    // start computing only after the first DEPTH k-blocks of every wave were in.  (Twelve chunks per thread cover
    // the 96 KiB budget with eight waves; a workgroup of four waves stages the rest afterwards.)
    constexpr int kXChunks = 12;
    uint4_t xr[kXChunks];
    const int x_cpr = cnt * 16;  // chunks per row
    const int x_total = 16 * MT * x_cpr;
    const int x_iters = (x_total + (int)blockDim.x - 1) / (int)blockDim.x;
    const unsigned x_rcp = (unsigned)((0x100000000ull + x_cpr - 1) / x_cpr);  // idx / x_cpr for idx < 2^16
    auto x_chunk = [&](int it, int& m, int& c) {
        const int idx = (int)threadIdx.x + it * (int)blockDim.x;
        m = (int)__umulhi((unsigned)idx, x_rcp);
        c = idx - m * x_cpr;
        return idx < x_total;
    };
#pragma unroll
    for (int it = 0; it < kXChunks; ++it)
        if (it < x_iters) {
            int m, c;
            const bool ok = x_chunk(it, m, c);
            const unsigned ofs = ok ? (unsigned)(m * K + kb_begin * 128 + c * 8) * 2u : kOob;
            xr[it] = __builtin_bit_cast(uint4_t, __builtin_amdgcn_raw_buffer_load_b128(rx, ofs, 0, 0));
        }

    Slot slot[DEPTH];
#pragma unroll
    for (int u = 0; u < DEPTH; ++u)
        issue(u, slot[u]);

#pragma unroll
    for (int it = 0; it < kXChunks; ++it)
        if (it < x_iters) {
            int m, c;
            if (x_chunk(it, m, c))
                *reinterpret_cast<uint4_t*>(&xs[m * x_stride + c * 8]) = xr[it];
        }
    for (int it = kXChunks; it < x_iters; ++it) {
        int m, c;
        if (x_chunk(it, m, c)) {
            const unsigned ofs = (unsigned)(m * K + kb_begin * 128 + c * 8) * 2u;
            *reinterpret_cast<uint4_t*>(&xs[m * x_stride + c * 8]) =
                __builtin_bit_cast(uint4_t, __builtin_amdgcn_raw_buffer_load_b128(rx, ofs, 0, 0));
        }
    }
    __syncthreads();
    const half_t* xs_lane = xs + col * x_stride + 8 * kq;

    float4_t acc[RT][MT];
#pragma unroll
    for (int r = 0; r < RT; ++r)
#pragma unroll
        for (int t = 0; t < MT; ++t)
            acc[r][t] = float4_t{0.f, 0.f, 0.f, 0.f};

    auto consume = [&](int i, const Slot& s) {
        // a slot past the end reads the last valid k-block of LDS; its scale is zero
        const int kbl = min(i, cnt - 1);
        half8_t a[MT][4];
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                a[t][j] = *reinterpret_cast<const half8_t*>(xs_lane + 16 * t * x_stride + kbl * 128 + 32 * j);
#pragma unroll
        for (int r = 0; r < RT; ++r) {
            auto add_scaled = [&](int gi, const float4_t(&part)[MT]) {
                const uint32_t sbits = s.scale[r][gi >> 1] >> (16 * (gi & 1));
                const float scale = (float)__builtin_bit_cast(half_t, (uint16_t)sbits);
#pragma unroll
                for (int t = 0; t < MT; ++t) {
                    acc[r][t].x += scale * part[t].x;
                    acc[r][t].y += scale * part[t].y;
                    acc[r][t].z += scale * part[t].z;
                    acc[r][t].w += scale * part[t].w;
                }
            };
            if constexpr (BITS == 4) {
                const uint32_t wd[4] = {s.w[r][0].x, s.w[r][0].y, s.w[r][0].z, s.w[r][0].w};
                constexpr int kPerGroup = 4 / GPB;  // MFMAs per group
#pragma unroll
                for (int gi = 0; gi < GPB; ++gi) {
                    const float zpv = ZP_TABLE ? (float)((s.zp[r] >> (8 * gi)) & 0xFFu) : (float)zp_const;
                    const half2_t off_lo = splat(1024.f + zpv), off_hi = splat(64.f + zpv);
                    float4_t part[MT];
#pragma unroll
                    for (int t = 0; t < MT; ++t)
                        part[t] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int j = gi * kPerGroup; j < (gi + 1) * kPerGroup; ++j) {
                        Frag8 b;
                        unpack4(wd[j], off_lo, off_hi, b);
#pragma unroll
                        for (int t = 0; t < MT; ++t)
                            part[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[t][j], b.v, part[t], 0, 0, 0);
                    }
                    add_scaled(gi, part);
                }
            } else {
                const float zpv = ZP_TABLE ? (float)s.zp[r] : (float)zp_const;
                float4_t part0[MT];
#pragma unroll
                for (int t = 0; t < MT; ++t)
                    part0[t] = float4_t{0.f, 0.f, 0.f, 0.f};
                const half2_t off = splat(1024.f + zpv);
#pragma unroll
                for (int i2 = 0; i2 < 2; ++i2) {
                    const uint32_t wd[4] = {s.w[r][i2].x, s.w[r][i2].y, s.w[r][i2].z, s.w[r][i2].w};
#pragma unroll
                    for (int jj = 0; jj < 2; ++jj) {
                        Frag8 b;
                        unpack8(wd[2 * jj], wd[2 * jj + 1], off, b);
#pragma unroll
                        for (int t = 0; t < MT; ++t)
                            part0[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[t][2 * i2 + jj], b.v, part0[t], 0, 0, 0);
                    }
                }
                add_scaled(0, part0);
            }
        }
    };

    for (int i = 0; i < cnt; i += DEPTH) {
#pragma unroll
        for (int u = 0; u < DEPTH; ++u) {
            consume(i + u, slot[u]);
            issue(i + u + DEPTH, slot[u]);
        }
    }

    float sum[RT][MT][4];
#pragma unroll
    for (int r = 0; r < RT; ++r)
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            sum[r][t][0] = acc[r][t].x;
            sum[r][t][1] = acc[r][t].y;
            sum[r][t][2] = acc[r][t].z;
            sum[r][t][3] = acc[r][t].w;
        }

    if (split_k > 1) {
        // partial layout: [group][ks][wave][RT][MT][4 r][64 lanes] floats; only rows < M are written and read
        constexpr int kPart = RT * MT * 256;
        float* mine = ws + (((size_t)grp * split_k + ks) * nw + wave) * kPart;
#pragma unroll
        for (int r = 0; r < RT; ++r)
#pragma unroll
            for (int t = 0; t < MT; ++t)
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    if (r < tiles_here && 4 * kq + q + 16 * t < M)
                        __hip_atomic_store(mine + ((r * MT + t) * 4 + q) * 64 + lane, sum[r][t][q], __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_AGENT);
        // device-scope stores write through; once every wave's are acknowledged the ticket may be drawn
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (threadIdx.x == 0)
            ticket_s = __hip_atomic_fetch_add(counters + grp, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        if (ticket_s != (unsigned)(split_k - 1))
            return;
        // last arrival: every wave adds the partials of its own tiles in split order.  The loads are
        // device-scope buffer loads (they must not hit a stale line of this XCD's L2), eight splits in flight;
        // a split index past split_k falls outside the descriptor's range and reads zero.
        constexpr int kAuxDeviceScope = 16;  // sc1
        const unsigned s_stride = (unsigned)nw * kPart * 4u;
        const __amdgpu_buffer_rsrc_t rp = __builtin_amdgcn_make_buffer_rsrc(
            ws + ((size_t)grp * split_k * nw + wave) * kPart, 0, (split_k - 1) * (int)s_stride + kPart * 4, kRsrcFlags);
#pragma unroll
        for (int r = 0; r < RT; ++r)
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                float tot[4] = {0.f, 0.f, 0.f, 0.f};
                for (int s0 = 0; s0 < split_k; s0 += 8) {
                    float v[8][4];
#pragma unroll
                    for (int u = 0; u < 8; ++u)
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            const bool live = r < tiles_here && 4 * kq + q + 16 * t < M;
                            const unsigned ofs =
                                (unsigned)(s0 + u) * s_stride + (unsigned)(((r * MT + t) * 4 + q) * 64 + lane) * 4u;
                            v[u][q] = __builtin_bit_cast(
                                float, __builtin_amdgcn_raw_buffer_load_b32(rp, live ? ofs : kOob, 0, kAuxDeviceScope));
                        }
#pragma unroll
                    for (int u = 0; u < 8; ++u)
#pragma unroll
                        for (int q = 0; q < 4; ++q)
                            tot[q] += v[u][q];
                }
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    sum[r][t][q] = tot[q];
            }
        if (threadIdx.x == 0)
            __hip_atomic_store(counters + grp, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }

    if (glu) {
        // gated linear unit: the wave's two tiles are the gate and up channels 16 (tile0 / 2) .. of the
        // [M, N / 2] output
        if constexpr (RT == 1) {
            // one tile per wave: even waves own gate tiles, the next wave the matching up tile, handed over
            // through LDS (the staged activations are no longer needed once every wave is here)
            float* hand = reinterpret_cast<float*>(lds);  // [nw / 2][MT][4][64 lanes]
            const int n = tile0 * 16 + col;
            const float b = bias && tiles_here ? (float)bias[n] : 0.f;
            __syncthreads();
            if (wave & 1) {
#pragma unroll
                for (int t = 0; t < MT; ++t)
#pragma unroll
                    for (int q = 0; q < 4; ++q)
                        hand[(((wave >> 1) * MT + t) * 4 + q) * 64 + lane] = sum[0][t][q] + b;
            }
            __syncthreads();
            if (!(wave & 1) && tiles_here) {
#pragma unroll
                for (int t = 0; t < MT; ++t)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const int m = 4 * kq + q + 16 * t;
                        if (m < M)
                            store_out(y, (size_t)m * (N / 2) + (tile0 >> 1) * 16 + col,
                                      glu_value(glu, sum[0][t][q] + b,
                                                hand[(((wave >> 1) * MT + t) * 4 + q) * 64 + lane]),
                                      out_f32);
                    }
            }
        } else {
            if (tiles_here == 2) {
                const int n = tile0 * 16 + col;
                const float bg = bias ? (float)bias[n] : 0.f, bu = bias ? (float)bias[n + 16] : 0.f;
#pragma unroll
                for (int t = 0; t < MT; ++t)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const int m = 4 * kq + q + 16 * t;
                        if (m < M)
                            store_out(y, (size_t)m * (N / 2) + (tile0 >> 1) * 16 + col,
                                      glu_value(glu, sum[0][t][q] + bg, sum[1][t][q] + bu), out_f32);
                    }
            }
        }
        return;
    }
#pragma unroll
    for (int r = 0; r < RT; ++r) {
        if (r >= tiles_here)
            break;
        const int n = (tile0 + r) * 16 + col;
        const float b = bias ? (float)bias[n] : 0.f;
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int m = 4 * kq + q + 16 * t;
                if (m < M)
                    store_out(y, (size_t)m * N + n, sum[r][t][q] + b, out_f32);
            }
    }
}

template <int BITS, int MT, bool ZP_TABLE, int RT, int GPB>
__global__ __launch_bounds__(512) void fcc_batch_kernel(const uint4_t* __restrict__ wt, const half_t* __restrict__ st,
                                                        const uint8_t* __restrict__ zt, const half_t* __restrict__ x,
                                                        const half_t* __restrict__ bias, void* __restrict__ y,
                                                        float* __restrict__ ws, unsigned* __restrict__ counters,
                                                        int M, int N, int K, int kb_total, int kb_per_group, int ng,
                                                        int zp_const, int kb_per_split, int split_k, int n_tiles,
                                                        int out_f32, int glu) {
    batch_body<BITS, MT, ZP_TABLE, RT, GPB>(wt, st, zt, x, bias, y, ws, counters, M, N, K, kb_total, kb_per_group, ng,
                                       zp_const, kb_per_split, split_k, n_tiles, out_f32, glu);
}

// Grouped launch: blockIdx.z picks one of up to kMaxGroupItems independent problems that share N, K and the weight
// format (the experts of a mixture-of-experts layer, each with its own rows): one launch instead of one per expert.
// The table travels in the kernel arguments; every problem has its own slice of the split-K workspace and counters.
template <int BITS, int MT, bool ZP_TABLE, int RT, int GPB>
__global__ __launch_bounds__(512) void fcc_batch_grouped_kernel(BatchGroupTable tab, float* __restrict__ ws,
                                                                unsigned* __restrict__ counters, size_t ws_per_item,
                                                                int counters_per_item, int N, int K, int kb_total,
                                                                int kb_per_group, int ng, int zp_const,
                                                                int kb_per_split, int split_k, int n_tiles,
                                                                int out_f32) {
    const BatchGroupItem& it = tab.item[blockIdx.z];
    if (it.M == 0)
        return;
    batch_body<BITS, MT, ZP_TABLE, RT, GPB>(static_cast<const uint4_t*>(it.w), static_cast<const half_t*>(it.scale),
                                       static_cast<const uint8_t*>(it.zp), static_cast<const half_t*>(it.x),
                                       static_cast<const half_t*>(it.bias), it.y, ws + blockIdx.z * ws_per_item,
                                       counters + blockIdx.z * counters_per_item, it.M, N, K, kb_total, kb_per_group,
                                       ng, zp_const, kb_per_split, split_k, n_tiles, out_f32, 0);
}

template <int BITS, int MT, bool ZPT, int RT, int GPB>
static int launch_batch_gpb(const FcDeviceArgs& a, const LaunchPlan& p, hipStream_t s) {
    const Layout& L = a.layout;
    auto kern = fcc_batch_kernel<BITS, MT, ZPT, RT, GPB>;
    if (p.dynamic_lds > 48 * 1024) {
        static bool attr_set = false;  // per instantiation; the attribute is idempotent, a race only repeats it
        if (!attr_set) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024);
            if (e != hipSuccess)
                return (int)e;
            attr_set = true;
        }
    }
    hipLaunchKernelGGL(kern, dim3(p.grid[0], p.grid[1], 1), dim3(p.block), p.dynamic_lds, s, (const uint4_t*)a.w,
                       (const half_t*)a.scale, (const uint8_t*)a.zp, (const half_t*)a.x, (const half_t*)a.bias, a.y,
                       a.workspace, a.counters, (int)a.M, (int)a.N, (int)a.K, (int)L.k_blocks,
                       (int)L.kblocks_per_group, (int)L.groups, L.zp_const, p.kblocks_per_split, p.split_k,
                       (int)L.n_tiles, a.out_f32, L.glu);
    return (int)hipGetLastError();
}

template <int BITS, int MT, bool ZPT, int RT>
static int launch_batch_impl(const FcDeviceArgs& a, const LaunchPlan& p, hipStream_t s) {
    if constexpr (BITS == 4) {
        if (a.layout.groups_per_kblock == 2)
            return launch_batch_gpb<BITS, MT, ZPT, RT, 2>(a, p, s);
        if (a.layout.groups_per_kblock == 4)
            return launch_batch_gpb<BITS, MT, ZPT, RT, 4>(a, p, s);
    }
    return launch_batch_gpb<BITS, MT, ZPT, RT, 1>(a, p, s);
}

template <int BITS, bool ZPT>
static int launch_batch_bits(const FcDeviceArgs& a, const LaunchPlan& p, hipStream_t s) {
    const int mt = (int)(a.M + 15) / 16;
    const int rt = p.tiles_per_group;
    if (mt <= 1)
        return rt == 2 ? launch_batch_impl<BITS, 1, ZPT, 2>(a, p, s) : launch_batch_impl<BITS, 1, ZPT, 1>(a, p, s);
    if (mt == 2)
        return rt == 2 ? launch_batch_impl<BITS, 2, ZPT, 2>(a, p, s) : launch_batch_impl<BITS, 2, ZPT, 1>(a, p, s);
    return rt == 2 ? launch_batch_impl<BITS, 3, ZPT, 2>(a, p, s) : launch_batch_impl<BITS, 3, ZPT, 1>(a, p, s);
}

template <int BITS, int MT, bool ZPT, int GPB>
static int launch_grouped_gpb(const BatchGroupTable& tab, int n_items, const FcDeviceArgs& a, const LaunchPlan& p,
                              hipStream_t s) {
    const Layout& L = a.layout;
    auto kern = fcc_batch_grouped_kernel<BITS, MT, ZPT, 1, GPB>;
    if (p.dynamic_lds > 48 * 1024) {
        static bool attr_set = false;  // per instantiation; the attribute is idempotent, a race only repeats it
        if (!attr_set) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024);
            if (e != hipSuccess)
                return (int)e;
            attr_set = true;
        }
    }
    hipLaunchKernelGGL(kern, dim3(p.grid[0], p.grid[1], (unsigned)n_items), dim3(p.block), p.dynamic_lds, s, tab,
                       a.workspace, a.counters, p.workspace_bytes / sizeof(float), (int)p.counter_count, (int)a.N,
                       (int)a.K, (int)L.k_blocks, (int)L.kblocks_per_group, (int)L.groups, L.zp_const,
                       p.kblocks_per_split, p.split_k, (int)L.n_tiles, a.out_f32);
    return (int)hipGetLastError();
}

template <int BITS, int MT, bool ZPT>
static int launch_grouped_impl(const BatchGroupTable& tab, int n_items, const FcDeviceArgs& a, const LaunchPlan& p,
                               hipStream_t s) {
    if constexpr (BITS == 4) {
        if (a.layout.groups_per_kblock == 2)
            return launch_grouped_gpb<BITS, MT, ZPT, 2>(tab, n_items, a, p, s);
        if (a.layout.groups_per_kblock == 4)
            return launch_grouped_gpb<BITS, MT, ZPT, 4>(tab, n_items, a, p, s);
    }
    return launch_grouped_gpb<BITS, MT, ZPT, 1>(tab, n_items, a, p, s);
}

// `a` describes the shared shape (M = the largest row count of any item, at most 48); `p` is its small-batch plan
// with one channel tile per wave; workspace and counters hold n_items slices of p.workspace_bytes / p.counter_count.
int launch_batch_grouped(const BatchGroupTable& tab, int n_items, const FcDeviceArgs& a, const LaunchPlan& p,
                         void* stream) {
    hipStream_t s = static_cast<hipStream_t>(stream);
    const Layout& L = a.layout;
    if (L.glu || p.tiles_per_group != 1)
        return (int)hipErrorInvalidValue;  // the grouped kernel is built for one tile per wave
    if (L.groups_per_kblock != 1 && L.bits != 4)
        return (int)hipErrorInvalidValue;
    const int mt = (int)(a.M + 15) / 16;
#define OVFCC_GROUPED(B, Z)                                                         \
    (mt <= 1   ? launch_grouped_impl<B, 1, Z>(tab, n_items, a, p, s)                \
     : mt == 2 ? launch_grouped_impl<B, 2, Z>(tab, n_items, a, p, s)                \
               : launch_grouped_impl<B, 3, Z>(tab, n_items, a, p, s))
    if (L.bits == 4)
        return L.zp_table ? OVFCC_GROUPED(4, true) : OVFCC_GROUPED(4, false);
    return L.zp_table ? OVFCC_GROUPED(8, true) : OVFCC_GROUPED(8, false);
#undef OVFCC_GROUPED
}

int launch_batch(const FcDeviceArgs& a, const LaunchPlan& p, void* stream) {
    hipStream_t s = static_cast<hipStream_t>(stream);
    const Layout& L = a.layout;
    if (L.glu && ((p.tiles_per_group == 1 && ((p.block >> 6) & 1)) || p.dynamic_lds < (p.block >> 7) * (unsigned)p.tile_m * 64u))
        return (int)hipErrorInvalidValue;  // gate and up tile: one wave, or two neighbours with room for the hand-over
    if (L.groups_per_kblock != 1 && L.bits != 4)
        return (int)hipErrorInvalidValue;
    if (L.bits == 4)
        return L.zp_table ? launch_batch_bits<4, true>(a, p, s) : launch_batch_bits<4, false>(a, p, s);
    return L.zp_table ? launch_batch_bits<8, true>(a, p, s) : launch_batch_bits<8, false>(a, p, s);
}

}  // namespace ovfcc
