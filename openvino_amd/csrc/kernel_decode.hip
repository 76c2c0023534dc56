// Decode kernel (M <= 32) over the tiled layout: a split-K streaming kernel.
//
// grid = (N / (16 RT), split_k), block = 64 * NW (NW = 4, 8 or 16 waves).  Workgroup (g, ks) owns RT
// consecutive 16-channel tiles and k-blocks [ks * kb_per_split, min(KB, (ks + 1) * kb_per_split)); wave w
// takes k-blocks first + w, first + w + NW, ... of every one of the RT tiles.  A k-block of one tile is one
// (4-bit) or two (8-bit) 1 KiB tiles, read with one 128-bit load per lane; DEPTH k-blocks per wave are
// kept in flight in registers.  All global loads go through buffer descriptors with hardware range
// checking, so a slot past the end of a wave's share reads zeros without a branch and the loop's waits
// count exactly.
//
// Activations: for M <= 4 the workgroup stages X[0:M, its k-range] once in LDS and every wave reads its
// MFMA operand from there (all lanes of a row read the same address: a broadcast); rows >= M of the
// operand repeat row 0 and only produce output rows that are never stored.  For larger M the operand
// comes straight from global memory (L2) together with the weights.
//
// Arithmetic per k-block: nibbles/bytes are unpacked in registers to the exact halves bias + q and
// contracted against the activation rows on the matrix cores (A = activations, rows m; B = weights,
// columns n; v_mfma_f32_16x16x32_f16, f32 result: lane holds column n = lane & 15, rows 4 (lane >> 4) + r);
// one more MFMA per k-step against the constant fragment -(bias + zp) cancels bias and zero-point in the
// f32 accumulator, which keeps the vector ALU free for the unpack.  The group scale multiplies the f32
// partial sum of the k-block, so no weight is ever rounded.  Groups of 64 or 32 inputs (GPB = 2 or 4 groups
// per k-block, 4-bit weights) keep one partial sum per group: MFMA j of a k-block covers inputs 32 j ..+32.
//
// Reductions: the waves of a workgroup are summed through LDS in wave order.  With split_k > 1 every
// workgroup writes its partial tiles with device-scope stores, waits for them, and takes a ticket from a
// per-group arrival counter; the workgroup that draws the last ticket adds all partials in split order
// (the result does not depend on arrival order) and returns the counter to zero for the next launch.
#include "device_common.h"

namespace ovfcc {

template <int TPB, int MT, int RT, bool XLDS, int GPB>
struct DecodeSlot {
    uint4_t w[RT][TPB];
    half8_t a[XLDS ? 1 : MT][XLDS ? 1 : 4];  // unused when the activations come from LDS
    uint32_t scale[RT][GPB == 4 ? 2 : 1];    // GPB f16 scales, packed
    uint32_t zp[RT];                         // GPB zero-points, one per byte
};

// XLEAD (with XLDS): the activation loads go out before the first weight slot instead of right after it.
template <int BITS, int MT, bool ZP_TABLE, int RT, bool XLDS, int GPB, bool XLEAD>
__global__ __launch_bounds__(1024) void fcc_decode_kernel(const uint4_t* __restrict__ wt,
                                                          const half_t* __restrict__ st,
                                                          const uint8_t* __restrict__ zt,
                                                          const half_t* __restrict__ x,
                                                          const half_t* __restrict__ bias, void* __restrict__ y,
                                                          float* __restrict__ ws, unsigned* __restrict__ counters,
                                                          int M, int N, int K, int kb_total, int kb_per_group,
                                                          int ng, int zp_const, int kb_per_split, int split_k,
                                                          int out_f32, int glu) {
    static_assert(!XLDS || MT == 1, "LDS-staged activations serve one 16-row tile");
    static_assert(GPB == 1 || ((GPB == 2 || GPB == 4) && BITS == 4), "groups below 128 inputs: 4-bit weights only");
    constexpr int TPB = BITS == 4 ? 1 : 2;                                            // tiles per k-block
    constexpr int DEPTH = XLDS ? (RT * TPB >= 4 ? 2 : 4) : (MT == 1 ? 4 : 2) / TPB;  // k-blocks in flight
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];              // [red][xs]
    __shared__ unsigned ticket_s;

    const int grp = blockIdx.x;  // group of RT channel tiles
    const int ks = blockIdx.y;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nw = blockDim.x >> 6;
    const int col = lane & 15;
    const int kq = lane >> 4;
    float* red = reinterpret_cast<float*>(lds);  // [wave][RT][MT][4 r][64 lanes]
    half_t* xs = reinterpret_cast<half_t*>(lds + (size_t)nw * RT * MT * 256 * sizeof(float));

    const int kb_begin = ks * kb_per_split;
    const int kb_end = min(kb_total, kb_begin + kb_per_split);
    const int kb_first = kb_begin + wave;
    const int cnt = kb_first < kb_end ? (kb_end - kb_first + nw - 1) / nw : 0;
    const int x_stride = (kb_end - kb_begin) * 128 + 8;  // halves; +8 so rows start on different banks

    constexpr unsigned kOob = 0x80000000u;
    constexpr int kRsrcFlags = 0x00020000;
    const size_t tile0 = (size_t)grp * RT;
    const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint4_t*>(wt + tile0 * kb_total * TPB * 64), 0, RT * kb_total * TPB * kTileBytes, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t rs =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(st + tile0 * ng * 16), 0, RT * ng * 32, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t rz = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint8_t*>(ZP_TABLE ? zt + tile0 * ng * 16 : zt), 0, ZP_TABLE ? RT * ng * 16 : 0, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t rx =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(x), 0, M * K * 2, kRsrcFlags);
    // global activation operand of this lane: row m = col (+16 for the second tile), inputs 8 kq ..+8
    unsigned xbase[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        const int m = col + 16 * t;
        xbase[t] = m < M ? (unsigned)(m * K + 8 * kq) * 2u : kOob;
    }

    // group index of a k-block without a division in the loop: kb_per_group == 1 -> kb, else the high word of
    // kb * ceil(2^32 / kb_per_group) (exact for kb < 2^16)
    const unsigned g_mul = kb_per_group == 1 ? 0u : (unsigned)((0x100000000ull + kb_per_group - 1) / kb_per_group);
    using Slot = DecodeSlot<TPB, MT, RT, XLDS, GPB>;
    auto issue = [&](int i, Slot& s) {
        // bit 31 of every offset of a slot past the end of this wave's share is set: out of range, reads zero
        const unsigned oob = (unsigned)((cnt - 1 - i) >> 31) & kOob;
        const unsigned kb = (unsigned)(kb_first + nw * i);
        const unsigned g = kb_per_group == 1 ? kb : __umulhi(kb, g_mul);
#pragma unroll
        for (int r = 0; r < RT; ++r) {
            const unsigned wofs = ((r * kb_total + kb) * (unsigned)(TPB * kTileBytes) + lane * 16u) | oob;
#pragma unroll
            for (int t = 0; t < TPB; ++t)
                s.w[r][t] =
                    __builtin_bit_cast(uint4_t, __builtin_amdgcn_raw_buffer_load_b128(rw, wofs + t * kTileBytes, 0, 2));
        }
        if constexpr (!XLDS) {
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                const unsigned xofs = (xbase[t] + kb * 256u) | oob;  // an invalid row keeps bit 31 of its base
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    s.a[t][j] =
                        __builtin_bit_cast(half8_t, __builtin_amdgcn_raw_buffer_load_b128(rx, xofs + 64u * j, 0, 0));
            }
        }
#pragma unroll
        for (int r = 0; r < RT; ++r) {
            if constexpr (GPB == 1) {
                const unsigned sidx = (r * ng + g) * 16u + col;
                s.scale[r][0] = __builtin_amdgcn_raw_buffer_load_b16(rs, (sidx * 2u) | oob, 0, 0);
                if constexpr (ZP_TABLE)
                    s.zp[r] = __builtin_amdgcn_raw_buffer_load_b8(rz, sidx | oob, 0, 0);
            } else {
                // the GPB groups of this k-block for the lane's channel lie side by side
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

    // Stage X[0:M, k-range of this workgroup] in LDS once, in 16-byte chunks coalesced along k.  The loads go out
    // BEFORE most of the first weight loads: the memory counter retires in order, so a wave that asked for all
    // its weights first could not write (or read) the staged activations until all of those weights had landed,
    // and no workgroup would start computing before the first DEPTH k-blocks of every wave were in.
    constexpr int kXChunks = 10;  // per thread: 40 KiB of activations over at least 256 threads
    uint4_t xr[XLDS ? kXChunks : 1];
    const int x_cpr = (kb_end - kb_begin) * 16;  // chunks per row
    const int x_total = M * x_cpr;
    const int x_iters = (x_total + (int)blockDim.x - 1) / (int)blockDim.x;
    auto x_chunk = [&](int it, int& m, int& c) {
        const int idx = (int)threadIdx.x + it * (int)blockDim.x;
        m = (idx >= x_cpr) + (idx >= 2 * x_cpr) + (idx >= 3 * x_cpr);  // M <= 4
        c = idx - m * x_cpr;
        return idx < x_total;
    };
    // (When every wave's whole share of k-blocks is in flight from the start, the activations go out before all
    // of it -- XLEAD; with more k-blocks than slots the first weight slot, which is needed first in any case,
    // leads.  Measured: 2-4 % either way on the nodes of the other kind; the launcher picks.)
    Slot slot[DEPTH];
    if constexpr (!XLEAD)
        issue(0, slot[0]);
    if constexpr (XLDS) {
#pragma unroll
        for (int it = 0; it < kXChunks; ++it)
            if (it < x_iters) {
                int m, c;
                const bool ok = x_chunk(it, m, c);
                const unsigned ofs = ok ? (unsigned)(m * K + kb_begin * 128 + c * 8) * 2u : kOob;
                xr[it] = __builtin_bit_cast(uint4_t, __builtin_amdgcn_raw_buffer_load_b128(rx, ofs, 0, 0));
            }
    }
    if constexpr (XLEAD)
        issue(0, slot[0]);
#pragma unroll
    for (int u = 1; u < DEPTH; ++u)
        issue(u, slot[u]);

    if constexpr (XLDS) {
#pragma unroll
        for (int it = 0; it < kXChunks; ++it)
            if (it < x_iters) {
                int m, c;
                if (x_chunk(it, m, c))
                    *reinterpret_cast<uint4_t*>(&xs[m * x_stride + c * 8]) = xr[it];
            }
        __syncthreads();
    }
    // LDS operand address of this lane: rows >= M repeat row 0 (their output rows are never stored)
    const half_t* xs_lane = xs + (col < M ? col : 0) * x_stride + 8 * kq;

    float4_t acc[RT][MT];
#pragma unroll
    for (int r = 0; r < RT; ++r)
#pragma unroll
        for (int t = 0; t < MT; ++t)
            acc[r][t] = float4_t{0.f, 0.f, 0.f, 0.f};

    const Unpack4Consts uc = unpack4_consts();
    auto consume = [&](int i, const Slot& s) {
        half8_t a[MT][4];
        if constexpr (XLDS) {
            // a slot past the end reads some valid k-block of LDS; its weights and scale are zero
            const int kbl = i < cnt ? wave + nw * i : 0;
#pragma unroll
            for (int j = 0; j < 4; ++j)
                a[0][j] = *reinterpret_cast<const half8_t*>(xs_lane + kbl * 128 + 32 * j);
        } else {
#pragma unroll
            for (int t = 0; t < MT; ++t)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    a[t][j] = s.a[t][j];
        }
#pragma unroll
        for (int r = 0; r < RT; ++r) {
            // weights enter the matrix cores with their unpack bias (1024 + q, 64 + q); a second MFMA against
            // the constant fragment -(bias + zp) removes bias and zero-point inside the f32 accumulator
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
                    Frag8 bc;
                    bc.h2[0] = bc.h2[2] = splat(-(1024.f + zpv));
                    bc.h2[1] = bc.h2[3] = splat(-(64.f + zpv));
                    float4_t part[MT];
#pragma unroll
                    for (int t = 0; t < MT; ++t)
                        part[t] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int j = gi * kPerGroup; j < (gi + 1) * kPerGroup; ++j) {
                        Frag8 b;
                        unpack4_biased(wd[j], uc, b);
#pragma unroll
                        for (int t = 0; t < MT; ++t) {
                            part[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[t][j], b.v, part[t], 0, 0, 0);
                            part[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[t][j], bc.v, part[t], 0, 0, 0);
                        }
                    }
                    add_scaled(gi, part);
                }
            } else {
                const float zpv = ZP_TABLE ? (float)s.zp[r] : (float)zp_const;
                float4_t part0[MT];
#pragma unroll
                for (int t = 0; t < MT; ++t)
                    part0[t] = float4_t{0.f, 0.f, 0.f, 0.f};
                Frag8 bc;
                bc.h2[0] = bc.h2[1] = bc.h2[2] = bc.h2[3] = splat(-(1024.f + zpv));
#pragma unroll
                for (int i2 = 0; i2 < 2; ++i2) {
                    const uint32_t wd[4] = {s.w[r][i2].x, s.w[r][i2].y, s.w[r][i2].z, s.w[r][i2].w};
#pragma unroll
                    for (int jj = 0; jj < 2; ++jj) {
                        Frag8 b;
                        unpack8_biased(wd[2 * jj], wd[2 * jj + 1], b);
#pragma unroll
                        for (int t = 0; t < MT; ++t) {
                            part0[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[t][2 * i2 + jj], b.v, part0[t], 0, 0, 0);
                            part0[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[t][2 * i2 + jj], bc.v, part0[t], 0, 0, 0);
                        }
                    }
                }
                add_scaled(0, part0);
            }
        }
    };

    // slots past the end of this wave's share hold zero weights and a zero scale and add nothing
    for (int i = 0; i < cnt; i += DEPTH) {
#pragma unroll
        for (int u = 0; u < DEPTH; ++u) {
            consume(i + u, slot[u]);
            issue(i + u + DEPTH, slot[u]);
        }
    }

    // ---- reduce the waves through LDS, in wave order; only rows < M carry data ----
#pragma unroll
    for (int r = 0; r < RT; ++r)
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            const float v[4] = {acc[r][t].x, acc[r][t].y, acc[r][t].z, acc[r][t].w};
#pragma unroll
            for (int q = 0; q < 4; ++q)
                if (4 * kq + q + 16 * t < M)
                    red[((wave * RT + r) * MT + t) * 256 + q * 64 + lane] = v[q];
        }
    __syncthreads();
    if (wave != 0 && split_k == 1)
        return;

    float sum[RT][MT][4];
#pragma unroll
    for (int r = 0; r < RT; ++r)
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                sum[r][t][q] = 0.f;
                if (wave == 0 && 4 * kq + q + 16 * t < M)
                    for (int w = 0; w < nw; ++w)
                        sum[r][t][q] += red[((w * RT + r) * MT + t) * 256 + q * 64 + lane];
            }

    if (split_k > 1) {
        // partial layout: [group][ks][RT][MT][4 r][64 lanes] floats; only rows < M are written and read
        constexpr int kPart = RT * MT * 256;
        float* mine = ws + ((size_t)grp * split_k + ks) * kPart;
        if (wave == 0) {
#pragma unroll
            for (int r = 0; r < RT; ++r)
#pragma unroll
                for (int t = 0; t < MT; ++t)
#pragma unroll
                    for (int q = 0; q < 4; ++q)
                        if (4 * kq + q + 16 * t < M)
                            __hip_atomic_store(mine + ((r * MT + t) * 4 + q) * 64 + lane, sum[r][t][q],
                                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            // device-scope stores write through; once they are acknowledged the ticket may be drawn
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
        __syncthreads();
        if (threadIdx.x == 0)
            ticket_s = __hip_atomic_fetch_add(counters + grp, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        if (ticket_s != (unsigned)(split_k - 1) || wave != 0)
            return;
        // last arrival: add all partials in split order with device-scope loads
#pragma unroll
        for (int r = 0; r < RT; ++r)
#pragma unroll
            for (int t = 0; t < MT; ++t)
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    sum[r][t][q] = 0.f;
        for (int s = 0; s < split_k; ++s) {
            const float* p = ws + ((size_t)grp * split_k + s) * kPart;
#pragma unroll
            for (int r = 0; r < RT; ++r)
#pragma unroll
                for (int t = 0; t < MT; ++t)
#pragma unroll
                    for (int q = 0; q < 4; ++q)
                        if (4 * kq + q + 16 * t < M)
                            sum[r][t][q] += __hip_atomic_load(p + ((r * MT + t) * 4 + q) * 64 + lane, __ATOMIC_RELAXED,
                                                              __HIP_MEMORY_SCOPE_AGENT);
        }
        if (lane == 0)
            __hip_atomic_store(counters + grp, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }

    if (glu) {
        // gated linear unit: tiles 2 j and 2 j + 1 are the gate and up channels 16 j .. of the [M, N / 2] output
        if constexpr (RT % 2 == 0) {
#pragma unroll
            for (int r = 0; r < RT; r += 2) {
                const int n = (grp * RT + r) * 16 + col;
                const float bg = bias ? (float)bias[n] : 0.f, bu = bias ? (float)bias[n + 16] : 0.f;
#pragma unroll
                for (int t = 0; t < MT; ++t)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const int m = 4 * kq + q + 16 * t;
                        if (m < M)
                            store_out(y, (size_t)m * (N / 2) + (n >> 5) * 16 + col,
                                      glu_value(glu, sum[r][t][q] + bg, sum[r + 1][t][q] + bu), out_f32);
                    }
            }
        }
        return;
    }
#pragma unroll
    for (int r = 0; r < RT; ++r) {
        const int n = (grp * RT + r) * 16 + col;
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

template <int BITS, int MT, bool ZPT, int RT, bool XLDS, int GPB, bool XLEAD>
static void launch_decode_lead(const FcDeviceArgs& a, const LaunchPlan& p, hipStream_t s) {
    const Layout& L = a.layout;
    hipLaunchKernelGGL((fcc_decode_kernel<BITS, MT, ZPT, RT, XLDS, GPB, XLEAD>), dim3(p.grid[0], p.grid[1], 1),
                       dim3(p.block), p.dynamic_lds, s, (const uint4_t*)a.w, (const half_t*)a.scale,
                       (const uint8_t*)a.zp, (const half_t*)a.x, (const half_t*)a.bias, a.y, a.workspace, a.counters,
                       (int)a.M, (int)a.N, (int)a.K, (int)L.k_blocks, (int)L.kblocks_per_group, (int)L.groups,
                       L.zp_const, p.kblocks_per_split, p.split_k, a.out_f32, L.glu);
}

template <int BITS, int MT, bool ZPT, int RT, bool XLDS, int GPB>
static void launch_decode_gpb(const FcDeviceArgs& a, const LaunchPlan& p, hipStream_t s) {
    if constexpr (XLDS && RT == 1) {
        // four k-blocks per wave are in flight from the start: does a wave have more?
        const int waves = (int)p.block / 64;
        if ((p.kblocks_per_split + waves - 1) / waves > 4)
            return launch_decode_lead<BITS, MT, ZPT, RT, XLDS, GPB, false>(a, p, s);
    }
    launch_decode_lead<BITS, MT, ZPT, RT, XLDS, GPB, XLDS>(a, p, s);
}

template <int BITS, int MT, bool ZPT, int RT, bool XLDS>
static void launch_decode_impl(const FcDeviceArgs& a, const LaunchPlan& p, hipStream_t s) {
    if constexpr (BITS == 4) {
        if (a.layout.groups_per_kblock == 2)
            return launch_decode_gpb<BITS, MT, ZPT, RT, XLDS, 2>(a, p, s);
        if (a.layout.groups_per_kblock == 4)
            return launch_decode_gpb<BITS, MT, ZPT, RT, XLDS, 4>(a, p, s);
    }
    launch_decode_gpb<BITS, MT, ZPT, RT, XLDS, 1>(a, p, s);
}

template <int BITS, bool ZPT>
static void launch_decode_bits(const FcDeviceArgs& a, const LaunchPlan& p, hipStream_t s) {
    if (a.M > 16) {
        launch_decode_impl<BITS, 2, ZPT, 1, false>(a, p, s);
    } else if (!p.x_in_lds) {
        launch_decode_impl<BITS, 1, ZPT, 1, false>(a, p, s);
    } else {
        switch (p.tiles_per_group) {
        case 4:
            if constexpr (BITS == 4)  // four 8-bit tiles in flight would not fit the register budget
                launch_decode_impl<BITS, 1, ZPT, 4, true>(a, p, s);
            else
                launch_decode_impl<BITS, 1, ZPT, 2, true>(a, p, s);
            break;
        case 2:
            launch_decode_impl<BITS, 1, ZPT, 2, true>(a, p, s);
            break;
        default:
            launch_decode_impl<BITS, 1, ZPT, 1, true>(a, p, s);
        }
    }
}

int launch_decode(const FcDeviceArgs& a, const LaunchPlan& p, void* stream) {
    hipStream_t s = static_cast<hipStream_t>(stream);
    const Layout& L = a.layout;
    if (L.glu && (!p.x_in_lds || a.M > 16 || (p.tiles_per_group & 1)))
        return (int)hipErrorInvalidValue;  // gate and up tile must share a workgroup
    if (L.groups_per_kblock != 1 && (L.bits != 4 || (L.groups_per_kblock != 2 && L.groups_per_kblock != 4)))
        return (int)hipErrorInvalidValue;
    // the staged activations: at most four rows, at most ten 16-byte chunks per thread
    if (p.x_in_lds && (a.M > 4 || (int64_t)a.M * p.kblocks_per_split * 16 > (int64_t)10 * p.block))
        return (int)hipErrorInvalidValue;
    if (L.bits == 4)
        L.zp_table ? launch_decode_bits<4, true>(a, p, s) : launch_decode_bits<4, false>(a, p, s);
    else
        L.zp_table ? launch_decode_bits<8, true>(a, p, s) : launch_decode_bits<8, false>(a, p, s);
    return (int)hipGetLastError();
}

}  // namespace ovfcc
