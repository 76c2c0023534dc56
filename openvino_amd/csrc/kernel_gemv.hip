// Decode kernel for one to four rows (M <= 4) over 4-bit tiles with one group per k-block (G = 128): a lean
// streaming matrix-vector product.  A launch of this size lives for a few microseconds and every wave runs its
// whole life once, so what counts is the number of instructions between a wave's start and its last load and
// between its last byte and its end; the kernel keeps both short.
//
// grid = N / 16 channel tiles (N / 32 tile pairs with a gated linear unit), block = 64 * NWT * tiles per
// workgroup, NWT = K / (128 C): wave w of a tile owns the C k-blocks w, w + NWT, w + 2 NWT, ... of it, all C
// weight tiles in flight in registers from its first instructions on (C = 2, 4 or 8).  The stride matters: the
// memory system serves neighbouring kilobytes together, so a wave that asked for C consecutive tiles received
// them in one burst near the end of the launch and did all its arithmetic after it (gate/up 7.2 us); with the
// waves of a workgroup interleaved, every wave's tiles arrive spread over the launch and the arithmetic hides
// behind the stream (5.9 us, the time of a bare streaming kernel over the same bytes).
//
// Weights.  A nibble q left in the mantissa of a half is the subnormal q 2^-24 (the matrix cores keep subnormal
// operands), so a dword unpacks into its four operand registers with four ANDs and one shift, exactly and with no
// bias to remove: bits 3:0 of a half give q 2^-24, bits 7:4 give q 2^-20.  The activations that meet the second
// kind are staged multiplied by 2^-4 (exact unless |x| < 2^-10, where the error stays below 2^-21 absolute), so one
// MFMA chain per k-block yields P = 2^-24 sum_k x_k q_k.  Zero-points leave through the activations' group sums
// c = sum_k x_k, one f32 per row and k-block, which a wave computes from its own activations while its weights
// travel:  y = 2^24 sum_kb s_kb (P_kb - zp_kb 2^-24 c_kb),  two vector operations per row and k-block.
//
// The f32 arithmetic behind a partial sum is spelled out with explicit fused multiply-adds (left to the compiler,
// which products it fuses depends on the code around them, and the one-launch MLP kernel, kernel_mlp.hip, promises
// this kernel's bits).
//
// Activations.  A wave loads X[0:M, its k-range] itself (M x C x 256 bytes, before the weights, because loads
// retire in order), forms the group sums (four dot products and a 16-lane DPP reduction per load, read back into
// scalar registers), and parks the rows in its own slice of LDS in operand order; no workgroup barrier sits
// between a wave and its arithmetic.  Scales (and zero-points) come from a channel-major copy of the group
// parameters, [N/16][16][K/128], so that lanes 0-15 -- the lanes that hold output rows 0-3 of the MFMA result --
// fetch all C of them with one load; the table is stored in the order the waves use it, [tile][channel][wave][slot]
// with k-block = wave + NWT slot, which fixes C per node when the node is created.
//
// Reduction.  Each wave leaves its M x 16 partial sums in LDS; one wave adds them -- its four rows of sixteen lanes
// take every fourth wave's sums each and two register exchanges add the rows, a fixed order that does not depend on
// arrival -- applies bias, gated linear unit and output type, and stores.  Which wave: with TICKET the one that
// draws the last ticket from an LDS counter (the counter is zeroed behind a barrier that sits right after the loads
// have been issued, where it waits for no memory) -- best for small workgroups, whose waves then retire one by one;
// without TICKET wave 0 after a closing barrier -- best for workgroups of eight and more waves, which an early
// barrier would march in step (down projection: 6.5 against 5.7 us).
//
// What the compiler must not do to the ends of a wave's life (both seen in its output): sink the loads of the group
// parameters to their only use, the final sums, where they are one more trip to memory behind the last weight
// tile; and start on the activations after the first two of eight weight loads, so that six leave a round trip
// late.  Scheduling fences around the load block and an empty asm statement at the point of need prevent both.
#include "device_common.h"

namespace ovfcc {

namespace {

template <int N>
struct VecOf;
template <>
struct VecOf<2> {
    typedef uint32_t type;
};
template <>
struct VecOf<4> {
    typedef uint2_t type;
};
template <>
struct VecOf<8> {
    typedef uint4_t type;
};

// sum over the 16 lanes of a DPP row; lane 15 of every row ends with the row's total
__device__ __forceinline__ float row_sum16(float v) {
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

// The value is needed here: keeps the compiler from sinking the load that produced it to a later, conditional use
// (where it would be one more round trip to memory at the end of a wave's life).
__device__ __forceinline__ void needed_here(uint32_t& v) {
    asm volatile("" : "+v"(v));
}
__device__ __forceinline__ void needed_here(uint2_t& v) {
    uint32_t a = v.x, b = v.y;
    asm volatile("" : "+v"(a), "+v"(b));
    v = uint2_t{a, b};
}
__device__ __forceinline__ void needed_here(uint4_t& v) {
    uint32_t a = v.x, b = v.y, c = v.z, d = v.w;
    asm volatile("" : "+v"(a), "+v"(b), "+v"(c), "+v"(d));
    v = uint4_t{a, b, c, d};
}

}  // namespace

// C: k-blocks per wave; MR: rows the kernel carries (M <= MR); ZP_TABLE: zero-points per (channel, group)
template <int C, int MR, bool ZP_TABLE, bool TICKET>
__global__ __launch_bounds__(1024) void fcc_gemv_kernel(const uint4_t* __restrict__ wt,
                                                        const half_t* __restrict__ scale_cm,
                                                        const uint8_t* __restrict__ zp_cm,
                                                        const half_t* __restrict__ x, const half_t* __restrict__ bias,
                                                        void* __restrict__ y, int M, int N, int K, int kb_total,
                                                        int nwt, int zp_const, int out_f32, int glu) {
    constexpr int XL = (C + 3) / 4;                    // activation loads per row: four k-blocks each
    constexpr int kRowBytes = C * 256 + 64;            // one staged row; the pad keeps rows on different banks
    constexpr int kWaveBytes = MR * kRowBytes;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];  // [waves][MR rows] | partial sums
    __shared__ unsigned arrived;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int waves = blockDim.x >> 6;
    const int col = lane & 15;
    const int kq = lane >> 4;
    const int sub = wave >= nwt ? 1 : 0;               // tile of this workgroup the wave works on (0, or 0 / 1)
    const int part = wave - sub * nwt;                 // its share of K
    const int tile = blockIdx.x * (glu ? 2 : 1) + sub;
    // k-block of slot s: part + nwt * s

    if constexpr (TICKET)
        if (threadIdx.x == 0)
            arrived = 0;

    constexpr unsigned kOob = 0x80000000u;
    constexpr int kRsrcFlags = 0x00020000;
    const __amdgpu_buffer_rsrc_t rx =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(x), 0, M * K * 2, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint4_t*>(wt + ((size_t)tile * kb_total + part) * 64), 0, ((C - 1) * nwt + 1) * kTileBytes,
        kRsrcFlags);
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<half_t*>(scale_cm + (size_t)tile * 16 * kb_total), 0, 16 * kb_total * 2, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t rz = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint8_t*>(ZP_TABLE ? zp_cm + (size_t)tile * 16 * kb_total : zp_cm), 0,
        ZP_TABLE ? 16 * kb_total : 0, kRsrcFlags);

    // ---- loads, in the order their data is needed: activations, group parameters, weights ----
    uint4_t xr[MR][XL];
#pragma unroll
    for (int m = 0; m < MR; ++m)
#pragma unroll
        for (int i = 0; i < XL; ++i) {
            // lane: slot 4 i + kq of the wave, 16-byte chunk col of that k-block
            const bool ok = m < M && 4 * i + kq < C;
            const unsigned ofs = ok ? (unsigned)(m * K + (part + nwt * (4 * i + kq)) * 128 + col * 8) * 2u : kOob;
            xr[m][i] = __builtin_bit_cast(uint4_t, __builtin_amdgcn_raw_buffer_load_b128(rx, ofs, 0, 0));
        }
    // lanes 0-15: the C scales (zero-points) of channel col for this wave's k-blocks
    const unsigned pofs = kq == 0 ? (unsigned)(col * kb_total + part * C) : kOob;       // zero-points: one byte each
    const unsigned sofs = kq == 0 ? (unsigned)(col * kb_total + part * C) * 2u : kOob;  // scales: two bytes each
    typename VecOf<C>::type sv;
    if constexpr (C == 8)
        sv = __builtin_bit_cast(uint4_t, __builtin_amdgcn_raw_buffer_load_b128(rs, sofs, 0, 0));
    else if constexpr (C == 4)
        sv = __builtin_bit_cast(uint2_t, __builtin_amdgcn_raw_buffer_load_b64(rs, sofs, 0, 0));
    else
        sv = __builtin_amdgcn_raw_buffer_load_b32(rs, sofs, 0, 0);
    uint32_t zv[2] = {0u, 0u};
    if constexpr (ZP_TABLE) {
        if constexpr (C == 8) {
            const uint2_t v = __builtin_bit_cast(uint2_t, __builtin_amdgcn_raw_buffer_load_b64(rz, pofs, 0, 0));
            zv[0] = v.x, zv[1] = v.y;
        } else if constexpr (C == 4) {
            zv[0] = __builtin_amdgcn_raw_buffer_load_b32(rz, pofs, 0, 0);
        } else {
            zv[0] = __builtin_amdgcn_raw_buffer_load_b16(rz, pofs, 0, 0);
        }
    }
    // (activations and group parameters are requested before the weights: loads return in order)
    __builtin_amdgcn_sched_barrier(0);
    uint4_t wv[C];
#pragma unroll
    for (int i = 0; i < C; ++i)
        wv[i] = __builtin_bit_cast(uint4_t,
                                   __builtin_amdgcn_raw_buffer_load_b128(rw, (unsigned)(i * nwt * kTileBytes + lane * 16), 0, 2));
    // The output and bias pointers are wanted by one wave at the very end; fetched there, the kernel arguments would
    // be one more wait in the tail.
    uint64_t bias_bits = reinterpret_cast<uint64_t>(bias), y_bits = reinterpret_cast<uint64_t>(y);
    asm volatile("" : "+s"(bias_bits), "+s"(y_bits));
    typedef __attribute__((address_space(1))) const half_t* global_half_ptr;
    typedef __attribute__((address_space(1))) void* global_void_ptr;
    const global_half_ptr bias_k = reinterpret_cast<global_half_ptr>(bias_bits);
    const global_void_ptr y_k = reinterpret_cast<global_void_ptr>(y_bits);
    auto put = [&](size_t i, float v) {
        if (out_f32)
            static_cast<__attribute__((address_space(1))) float*>(y_k)[i] = v;
        else
            static_cast<__attribute__((address_space(1))) half_t*>(y_k)[i] = to_half_rne(v);
    };
    // Every load is on its way before anything waits for one: without the fence the compiler starts on the
    // activations after the first two weight loads and the others leave one memory round trip late.
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (TICKET) {
        // publishes the zeroed ticket counter; pinned here so that the barrier waits for nothing that has left the chip
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
    }

    // ---- stage the activations while the weights travel ----
    unsigned char* xs = lds + wave * kWaveBytes;
    float csum[MR][C];  // 2^-24 c (times -zp when the zero-point is one constant): wave-uniform
    const float cmul = ZP_TABLE ? 0x1p-24f : -(float)zp_const * 0x1p-24f;
    const half2_t ones = half2_t{(half_t)1.f, (half_t)1.f};
    const half2_t sixteenth = half2_t{(half_t)0.0625f, (half_t)0.0625f};
#pragma unroll
    for (int m = 0; m < MR; ++m)
#pragma unroll
        for (int i = 0; i < XL; ++i) {
            const uint4_t v = xr[m][i];
            float s = __builtin_amdgcn_fdot2(as_half2(v.x), ones, 0.f, false);
            s = __builtin_amdgcn_fdot2(as_half2(v.y), ones, s, false);
            s = __builtin_amdgcn_fdot2(as_half2(v.z), ones, s, false);
            s = __builtin_amdgcn_fdot2(as_half2(v.w), ones, s, false);
            s = row_sum16(s) * cmul;
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (4 * i + r < C)
                    csum[m][4 * i + r] =
                        __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, s), 16 * r + 15));
            // elements 2, 3, 6, 7 of a chunk meet nibbles that sit four bits up in their halves
            uint4_t p = v;
            p.y = as_u32(as_half2(v.y) * sixteenth);
            p.w = as_u32(as_half2(v.w) * sixteenth);
            if (4 * i + kq < C)
                *reinterpret_cast<uint4_t*>(xs + m * kRowBytes + (i * 64 + lane) * 16) = p;
        }

    // The group parameters arrived with the activations.  Their only use is the lanes' final sums; left alone, the
    // compiler moves the loads down to that use, behind the last weight tile.
    needed_here(sv);
    if constexpr (ZP_TABLE) {
        needed_here(zv[0]);
        if constexpr (C == 8)
            needed_here(zv[1]);
    }

    // operand address of this lane: row col (rows >= MR repeat row 0, their results are never stored), quarter kq
    const unsigned char* xs_lane = xs + (col < MR ? col : 0) * kRowBytes + kq * 16;
    const uint32_t mask_lo = 0x000F000Fu, mask_hi = 0x00F000F0u;
    float acc[MR];
#pragma unroll
    for (int r = 0; r < MR; ++r)
        acc[r] = 0.f;
#pragma unroll
    for (int i = 0; i < C; ++i) {
        const uint32_t wd[4] = {wv[i].x, wv[i].y, wv[i].z, wv[i].w};
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
        uint32_t sbits;
        if constexpr (C == 8)
            sbits = (i < 2 ? sv.x : i < 4 ? sv.y : i < 6 ? sv.z : sv.w) >> (16 * (i & 1));
        else if constexpr (C == 4)
            sbits = (i < 2 ? sv.x : sv.y) >> (16 * (i & 1));
        else
            sbits = sv >> (16 * (i & 1));
        const float scale = (float)__builtin_bit_cast(half_t, (uint16_t)sbits);
        const float pr[4] = {p.x, p.y, p.z, p.w};
        if constexpr (ZP_TABLE) {
            const float zpf = (float)((zv[i >> 2] >> (8 * (i & 3))) & 0xFFu);
#pragma unroll
            for (int r = 0; r < MR; ++r)
                acc[r] = __builtin_fmaf(scale, __builtin_fmaf(-zpf, csum[r][i], pr[r]), acc[r]);
        } else {
#pragma unroll
            for (int r = 0; r < MR; ++r)
                acc[r] = __builtin_fmaf(scale, pr[r] + csum[r][i], acc[r]);
        }
    }

    // ---- partial sums of the workgroup's waves meet in LDS; the last wave to arrive adds them in wave order ----
    float* red = reinterpret_cast<float*>(lds + waves * kWaveBytes);  // [wave][MR][16]
    if (kq == 0) {
#pragma unroll
        for (int r = 0; r < MR; ++r)
            red[(wave * MR + r) * 16 + col] = acc[r];
    }
    if constexpr (TICKET) {
        // release / acquire at workgroup scope: a wave's partial sums are in place before its ticket is drawn, and
        // the wave that draws the last ticket sees all of them
        unsigned ticket = 0;
        if (lane == 0)
            ticket = __hip_atomic_fetch_add(&arrived, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_WORKGROUP);
        ticket = __builtin_amdgcn_readfirstlane(ticket);
        if (ticket != (unsigned)(waves - 1))
            return;
    } else {
        __syncthreads();
        if (wave != 0)
            return;
    }

    // The reducing wave's four rows of sixteen lanes each add a quarter of the partial sums (waves g, g + 4, ...:
    // at most four reads per lane and row, all in flight together), then the rows are added across the wave with two
    // register exchanges: (g0 + g2) + (g1 + g3), the same order every time.
    // (The second result of an exchange passes through an empty asm statement: converted straight to a float, this
    // compiler reads the first result in its place.)
    auto across_rows = [](float v) {
        const uint32_t a = __builtin_bit_cast(uint32_t, v);
        const uint2_t h = __builtin_amdgcn_permlane32_swap(a, a, false, false);  // .x: lanes l & 31, .y: those + 32
        uint32_t hy = h.y;
        asm volatile("" : "+v"(hy));
        const float t = __builtin_bit_cast(float, h.x) + __builtin_bit_cast(float, hy);
        const uint32_t b = __builtin_bit_cast(uint32_t, t);
        const uint2_t q = __builtin_amdgcn_permlane16_swap(b, b, false, false);  // .x: even rows, .y: odd rows
        uint32_t qy = q.y;
        asm volatile("" : "+v"(qy));
        return __builtin_bit_cast(float, q.x) + __builtin_bit_cast(float, qy);
    };
    // sum over waves first, first + 1, ... first + count - 1 of row r, channel col
    auto tile_sum = [&](int first, int count, int r) {
        float s = 0.f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int w = kq + 4 * j;
            const float v = red[((first + (w < count ? w : 0)) * MR + r) * 16 + col];
            s += w < count ? v : 0.f;
        }
        return across_rows(s);
    };
    if (glu) {
        // waves 0 .. nwt-1 hold the gate tile, nwt .. 2 nwt-1 the up tile of channels 16 blockIdx.x ..
        const int n = blockIdx.x * 32 + col;  // position of the gate channel in the tiled bias order
        const float bg = bias_k ? (float)bias_k[n] : 0.f, bu = bias_k ? (float)bias_k[n + 16] : 0.f;
#pragma unroll
        for (int r = 0; r < MR; ++r) {
            const float g = tile_sum(0, nwt, r), u = tile_sum(nwt, nwt, r);
            if (r < M && kq == 0)
                put((size_t)r * (N / 2) + blockIdx.x * 16 + col, glu_value(glu, __builtin_fmaf(g, 0x1p24f, bg), __builtin_fmaf(u, 0x1p24f, bu)));
        }
        return;
    }
    const int n = tile * 16 + col;
    const float b = bias_k ? (float)bias_k[n] : 0.f;
#pragma unroll
    for (int r = 0; r < MR; ++r) {
        const float s = tile_sum(0, waves, r);
        if (r < M && kq == 0)
            put((size_t)r * N + n, __builtin_fmaf(s, 0x1p24f, b));
    }
}

// Channel-major copies of the tiled group parameters for the kernel above: [N/16][groups][16] ->
// [N/16][16][wave][slot] with group = wave + (groups / c) slot, c slots per wave.
__global__ __launch_bounds__(256) void fcc_gemv_params_kernel(const half_t* __restrict__ st,
                                                              const uint8_t* __restrict__ zt,
                                                              half_t* __restrict__ scale_cm,
                                                              uint8_t* __restrict__ zp_cm, int groups, int c_slots,
                                                              size_t total) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;  // index into the channel-major arrays
    if (i >= total)
        return;
    const size_t tile = i / ((size_t)16 * groups);
    const int rest = (int)(i - tile * 16 * groups);
    const int c = rest / groups, at = rest - c * groups;
    const int g = at / c_slots + (groups / c_slots) * (at % c_slots);
    const size_t from = (tile * groups + g) * 16 + c;
    scale_cm[i] = st[from];
    if (zt)
        zp_cm[i] = zt[from];
}

int launch_gemv_params(const void* scale_tiled, const void* zp_tiled, void* scale_cm, void* zp_cm, int64_t n_tiles,
                       int64_t groups, int c_slots, void* stream) {
    const size_t total = (size_t)n_tiles * 16 * groups;
    if (total == 0)
        return 0;
    if (c_slots <= 0 || groups % c_slots != 0)
        return (int)hipErrorInvalidValue;
    hipLaunchKernelGGL(fcc_gemv_params_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), (const half_t*)scale_tiled, (const uint8_t*)zp_tiled,
                       (half_t*)scale_cm, (uint8_t*)zp_cm, (int)groups, c_slots, total);
    return (int)hipGetLastError();
}

template <int C, int MR, bool ZPT, bool TICKET>
static void launch_gemv_ticket(const FcDeviceArgs& a, const LaunchPlan& p, hipStream_t s) {
    const Layout& L = a.layout;
    hipLaunchKernelGGL((fcc_gemv_kernel<C, MR, ZPT, TICKET>), dim3(p.grid[0]), dim3(p.block), p.dynamic_lds, s,
                       (const uint4_t*)a.w, (const half_t*)a.scale_cm, (const uint8_t*)a.zp_cm, (const half_t*)a.x,
                       (const half_t*)a.bias, a.y, (int)a.M, (int)a.N, (int)a.K, (int)L.k_blocks,
                       (int)(L.k_blocks / C), L.zp_const, a.out_f32, L.glu);
}

template <int C, int MR, bool ZPT>
static void launch_gemv_impl(const FcDeviceArgs& a, const LaunchPlan& p, hipStream_t s) {
    if (p.block <= 256)
        launch_gemv_ticket<C, MR, ZPT, true>(a, p, s);
    else
        launch_gemv_ticket<C, MR, ZPT, false>(a, p, s);
}

template <int C, bool ZPT>
static void launch_gemv_rows(const FcDeviceArgs& a, const LaunchPlan& p, hipStream_t s) {
    if (a.M == 1)
        launch_gemv_impl<C, 1, ZPT>(a, p, s);
    else if (a.M == 2)
        launch_gemv_impl<C, 2, ZPT>(a, p, s);
    else
        launch_gemv_impl<C, 4, ZPT>(a, p, s);
}

int launch_gemv(const FcDeviceArgs& a, const LaunchPlan& p, void* stream) {
    hipStream_t s = static_cast<hipStream_t>(stream);
    const Layout& L = a.layout;
    const int c = L.gemv_c;
    // what the kernel and its grid assume, checked against the operands before anything is launched
    if (!L.tiled || L.bits != 4 || L.groups_per_kblock != 1 || L.kblocks_per_group != 1 || !a.scale_cm ||
        (L.zp_table && !a.zp_cm) || a.M < 1 || a.M > 4 || (c != 2 && c != 4 && c != 8) || L.k_blocks % c != 0 ||
        p.gemv_c != c)
        return (int)hipErrorInvalidValue;
    const int nwt = (int)(L.k_blocks / c), tiles_per_wg = L.glu ? 2 : 1;
    if (nwt * tiles_per_wg > 16 || p.block != 64u * nwt * tiles_per_wg || (int64_t)p.grid[0] * tiles_per_wg != L.n_tiles ||
        p.dynamic_lds != gemv_lds_bytes(c, (int)a.M, nwt * tiles_per_wg) || a.M * a.K * 2 >= ((int64_t)1 << 31) ||
        (int64_t)16 * L.k_blocks * 2 >= ((int64_t)1 << 31))
        return (int)hipErrorInvalidValue;
    if (L.zp_table) {
        if (c == 8) launch_gemv_rows<8, true>(a, p, s);
        else if (c == 4) launch_gemv_rows<4, true>(a, p, s);
        else launch_gemv_rows<2, true>(a, p, s);
    } else {
        if (c == 8) launch_gemv_rows<8, false>(a, p, s);
        else if (c == 4) launch_gemv_rows<4, false>(a, p, s);
        else launch_gemv_rows<2, false>(a, p, s);
    }
    return (int)hipGetLastError();
}

}  // namespace ovfcc
