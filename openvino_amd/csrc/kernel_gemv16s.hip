// Decode kernel for five to sixteen rows of a 4-bit node (one group per k-block, G = 128) where the 16-row kernel with
// stationary activations (kernel_gemv16.hip: 16 rows x K must fit in LDS and, divided among the waves, in registers)
// has nothing to keep or cannot run: nodes whose workgroups visit one channel tile each, and K too long for LDS -- the
// down projection of an MLP, K = 14336: 448 KiB of activations per row tile.
//
// The structure is the matrix-vector kernel's (kernel_gemv.hip): one workgroup per channel tile, K / (128 C) waves,
// wave w owns the k-blocks w, w + NW, ... (C of them: one row of the node's channel-major tables), the waves' sums
// meet in LDS at the end.  Nothing is split along K through memory and no second launch adds partial sums.  What
// differs is how 16 rows of activations reach a wave: one k-block at a time (16 rows x 256 bytes = 4 KiB, four
// direct-to-LDS loads of 1 KiB) through a private double buffer in LDS -- no barrier, nobody else reads it -- and from
// there into MFMA operand order in registers, which the next k-block reuses.  A workgroup thus reads all of its row
// tile's activations (448 KiB for K = 14336) through the compute unit's 64 bytes per cycle from L2 while its 112 KiB
// of weights stream from memory; the former takes 3.3 us, the latter about 5, and they overlap.  A workgroup may take
// T = 2 or 4 neighbouring channel tiles instead of one: a k-block of activations in registers then meets T weight
// tiles, which divides that traffic by T for nodes with more channel tiles than compute units.
//
// One counter orders a wave's loads (vmcnt retires in order), so the issue order decides what a wait waits for:
// activations of k-blocks 0 and 1, then the weights of the first four k-blocks; after k-block s is multiplied, the
// activations of k-block s + 2 go into the buffer it has freed and the weights of k-block s + 4 are requested.  The
// wait before the LDS reads of k-block s counts the loads issued behind its activations (loads_after_x); scheduling
// barriers keep the compiler from moving loads across those points.  The count must not depend on M at run time: the
// kernel exists for 8, 12 and 16 rows of activations per k-block (two, three or four loads; a load costs its issue
// cycles wherever its lanes point), and within those, rows beyond M are loaded out of range (zeros) rather than
// skipped.  The compiler waits for the weight registers itself.
//
// LDS buffer of a wave, in 16-byte units: row r, chunk c of the k-block's 16 sits at 16 r + (c ^ r): the sixteen rows
// that one operand read touches lie in sixteen different bank groups.  Arithmetic as in the 16-row kernel: nibbles
// stay in the mantissa as subnormal halves, the activations that meet the nibbles four bits up are multiplied by 2^-4
// in their registers, zero-points leave through the activations' group sums (one MFMA chain against a constant
// operand), group scales multiply the f32 sums per k-block:  y = 2^24 sum_kb s_kb (P_kb - zp_kb 2^-24 c_kb).
#include <type_traits>
#include <utility>

#include "device_common.h"

namespace ovfcc {

namespace {
template <int N>
struct ParamWords;  // C scales (f16) and C zero-points (u8) of one channel, as loaded
template <>
struct ParamWords<2> {
    typedef uint32_t scales;
};
template <>
struct ParamWords<4> {
    typedef uint2_t scales;
};
template <>
struct ParamWords<8> {
    typedef uint4_t scales;
};

// weight k-blocks requested ahead of the one being multiplied
template <int C>
constexpr int weights_ahead() {
    return C < 4 ? C : 4;
}

// vector-memory loads a wave has issued behind the XL loads of k-block s's activations when it is about to read
// them: the order is X0, X1, W0 .. W(D-1), then after every k-block t: X(t+2), W(t+D); a W is T loads
template <int C, int XL, int T>
constexpr int loads_after_x(int s) {
    constexpr int D = weights_ahead<C>();
    int count = 0;
    bool seen = false;
    for (int i = 0; i < 2 && i < C; ++i) {
        if (seen)
            count += XL;
        if (i == s)
            seen = true;
    }
    for (int i = 0; i < D; ++i)
        if (seen)
            count += T;
    for (int t = 0; t < s; ++t) {
        if (t + 2 < C) {
            if (seen)
                count += XL;
            if (t + 2 == s)
                seen = true;
        }
        if (t + D < C && seen)
            count += T;
    }
    return count;
}

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>): the k-block slot is a constant in the body (the
// wait's immediate needs one)
template <class F, int... I>
__device__ __forceinline__ void for_each_slot(F&& f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}
}  // namespace

// XL: direct-to-LDS loads per k-block of activations, four rows each (2, 3 or 4: rows beyond 4 XL are never loaded --
// a load costs its 16 cycles of the address path wherever its lanes point -- and what is computed from them is
// never stored).  T: channel tiles per workgroup (tiles T blockIdx.x .. + T - 1): one k-block of activations in
// registers meets T weight tiles, so a node with more channel tiles than compute units moves its activations 1 / T
// times as often.
template <int C, bool ZP_TABLE, int XL, int T>
__global__ __launch_bounds__(1024) void fcc_gemv16s_kernel(const uint4_t* __restrict__ wt, const half_t* __restrict__ scale_cm,
                                                           const uint8_t* __restrict__ zp_cm, const half_t* __restrict__ x,
                                                           const half_t* __restrict__ bias, void* __restrict__ y, int M,
                                                           int N, int K, int kb_total, int n_tiles, int zp_const,
                                                           int out_f32) {
    constexpr int D = weights_ahead<C>();
    constexpr int kBufBytes = 4096;  // 16 rows x one k-block x 2 bytes
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];  // [waves][2] buffers
    const lds_byte_ptr lds3 = (lds_byte_ptr)lds_raw;
    typedef __attribute__((address_space(3))) const uint4_t* lds_u4_ptr;
    typedef __attribute__((address_space(3))) float* lds_f32_ptr;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int waves = blockDim.x >> 6;  // = kb_total / C: wave w reads row w of the channel-major tables
    const int col = lane & 15;
    const int kq = lane >> 4;
    const int t0 = T * blockIdx.x;  // first channel tile
    const int m0 = 16 * blockIdx.y;

    constexpr unsigned kOob = 0x80000000u;
    constexpr int kRsrcFlags = 0x00020000;
    const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(x), 0, M * K * 2, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t rw =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<uint4_t*>(wt), 0, n_tiles * kb_total * kTileBytes, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t rs =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(scale_cm), 0, n_tiles * 16 * kb_total * 2, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t rz = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(zp_cm), 0,
                                                                        ZP_TABLE ? n_tiles * 16 * kb_total : 0, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t rb =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(bias), 0, bias ? n_tiles * 32 : 0, kRsrcFlags);

    // ---- group parameters of channel col of every tile for the wave's C k-blocks, bias ----
    typename ParamWords<C>::scales sv[T];
    uint32_t zv[T][C == 8 ? 2 : 1] = {};
    uint32_t bias_bits[T];
#pragma unroll
    for (int u = 0; u < T; ++u) {
        const unsigned pofs = (unsigned)(((t0 + u) * 16 + col) * kb_total + wave * C);
        if constexpr (C == 8)
            sv[u] = __builtin_bit_cast(uint4_t, __builtin_amdgcn_raw_buffer_load_b128(rs, pofs * 2u, 0, 0));
        else if constexpr (C == 4)
            sv[u] = __builtin_bit_cast(uint2_t, __builtin_amdgcn_raw_buffer_load_b64(rs, pofs * 2u, 0, 0));
        else
            sv[u] = __builtin_amdgcn_raw_buffer_load_b32(rs, pofs * 2u, 0, 0);
        if constexpr (ZP_TABLE) {
            if constexpr (C == 8) {
                const uint2_t z = __builtin_bit_cast(uint2_t, __builtin_amdgcn_raw_buffer_load_b64(rz, pofs, 0, 0));
                zv[u][0] = z.x, zv[u][1] = z.y;
            } else if constexpr (C == 4) {
                zv[u][0] = __builtin_amdgcn_raw_buffer_load_b32(rz, pofs, 0, 0);
            } else {
                zv[u][0] = __builtin_amdgcn_raw_buffer_load_b16(rz, pofs, 0, 0);
            }
        }
        bias_bits[u] = __builtin_amdgcn_raw_buffer_load_b16(rb, (unsigned)(((t0 + u) * 16 + col) * 2), 0, 0);
    }
    __builtin_amdgcn_sched_barrier(0);

    // ---- activations of k-block slot s into buffer s & 1: load q fills units 64 q .. 64 q + 63 (rows 4 q .. 4 q + 3) ----
    auto load_x = [&](int s) {
        const int kb = wave + waves * s;
#pragma unroll
        for (int q = 0; q < XL; ++q) {
            const int row = 4 * q + kq;
            const int chunk = col ^ row;  // the chunk of the row that belongs in this lane's linear slot
            const unsigned ofs = ((unsigned)((m0 + row) * K + kb * 128 + chunk * 8) * 2u) |
                                 ((unsigned)((M - 1 - m0 - row) >> 31) & kOob);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(
                rx, (lds_void_ptr)(lds3 + wave * (2 * kBufBytes) + (s & 1) * kBufBytes + q * 1024), 16, ofs, 0, 0, 0);
        }
    };
    uint4_t wv[C][T];
    auto load_w = [&](int s) {
#pragma unroll
        for (int u = 0; u < T; ++u) {
            const unsigned wofs = (unsigned)((t0 + u) * kb_total + wave + waves * s) * kTileBytes + lane * 16;
            wv[s][u] = __builtin_bit_cast(uint4_t, __builtin_amdgcn_raw_buffer_load_b128(rw, wofs, 0, 2));
        }
    };
    load_x(0);
    if constexpr (C > 1)
        load_x(1);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int s = 0; s < D; ++s)
        load_w(s);
    __builtin_amdgcn_sched_barrier(0);

    Frag8 ones;  // 1 against the plain halves, 16 against the scaled ones
    ones.u[0] = ones.u[2] = 0x3C003C00u;
    ones.u[1] = ones.u[3] = 0x4C004C00u;
    const float cmul = ZP_TABLE ? 0x1p-24f : -(float)zp_const * 0x1p-24f;
    const half2_t sixteenth = half2_t{(half_t)0.0625f, (half_t)0.0625f};
    const uint32_t mask_lo = 0x000F000Fu, mask_hi = 0x00F000F0u;
    float acc[T][4];  // rows 4 kq .. + 3 of the row tile, channel col of tile u
#pragma unroll
    for (int u = 0; u < T; ++u)
#pragma unroll
        for (int q = 0; q < 4; ++q)
            acc[u][q] = 0.f;

    auto step = [&](auto slot) {
        constexpr int s = decltype(slot)::value;
        // the activations of this k-block have landed (and with them everything requested before them)
        __builtin_amdgcn_s_waitcnt(wait_vmcnt_imm(loads_after_x<C, XL, T>(s)));
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
        const lds_byte_ptr xs_lane = lds3 + wave * (2 * kBufBytes) + (s & 1) * kBufBytes + col * 256;
        Frag8 xa[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint4_t v = *(lds_u4_ptr)(xs_lane + (((4 * j + kq) ^ col) << 4));
            xa[j].u[0] = v.x, xa[j].u[1] = v.y, xa[j].u[2] = v.z, xa[j].u[3] = v.w;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            xa[j].u[1] = as_u32(as_half2(xa[j].u[1]) * sixteenth);
            xa[j].u[3] = as_u32(as_half2(xa[j].u[3]) * sixteenth);
        }
        float4_t c4 = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < 4; ++j)
            c4 = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[j].v, ones.v, c4, 0, 0, 0);
        const float cz[4] = {c4.x * cmul, c4.y * cmul, c4.z * cmul, c4.w * cmul};
#pragma unroll
        for (int u = 0; u < T; ++u) {
            const uint32_t wd[4] = {wv[s][u].x, wv[s][u].y, wv[s][u].z, wv[s][u].w};
            float4_t p = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t w8 = wd[j] >> 8;
                Frag8 b;  // element e of the dword's eight: nibble (e >> 1) + 4 (e & 1)
                b.u[0] = wd[j] & mask_lo;
                b.u[1] = wd[j] & mask_hi;
                b.u[2] = w8 & mask_lo;
                b.u[3] = w8 & mask_hi;
                p = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[j].v, b.v, p, 0, 0, 0);
            }
            uint32_t sbits;
            if constexpr (C == 8)
                sbits = (s < 2 ? sv[u].x : s < 4 ? sv[u].y : s < 6 ? sv[u].z : sv[u].w) >> (16 * (s & 1));
            else if constexpr (C == 4)
                sbits = (s < 2 ? sv[u].x : sv[u].y) >> (16 * (s & 1));
            else
                sbits = sv[u] >> (16 * (s & 1));
            const float scale = (float)__builtin_bit_cast(half_t, (uint16_t)sbits);
            const float pr[4] = {p.x, p.y, p.z, p.w};
            if constexpr (ZP_TABLE) {
                const float zpf = (float)((zv[u][s >> 2] >> (8 * (s & 3))) & 0xFFu);
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    acc[u][q] = __builtin_fmaf(scale, __builtin_fmaf(-zpf, cz[q], pr[q]), acc[u][q]);
            } else {
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    acc[u][q] = __builtin_fmaf(scale, pr[q] + cz[q], acc[u][q]);
            }
        }
        // the buffer is free (its reads fed the MFMAs above): the activations of k-block s + 2, the weights of s + D
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (s + 2 < C)
            load_x(s + 2);
        if constexpr (s + D < C)
            load_w(s + D);
        __builtin_amdgcn_sched_barrier(0);
    };
    for_each_slot(step, std::make_integer_sequence<int, C>{});

    // ---- the waves' partial sums meet in LDS, each wave's in its own activation buffers (its last loads have
    // landed and been read; nobody else writes there): 16 rows x 16 channels per tile with the 16-float pieces of a
    // row group rotated by the group (no two lanes of a write or a read share a bank); waves 0-3 add one group of
    // four rows each, in wave order, apply the bias and store ----
    static_assert(T * 1024 <= 2 * kBufBytes, "a wave's partial sums fit in its buffers");
    constexpr int kWaveFloats = 2 * kBufBytes / 4;
    const lds_f32_ptr red = (lds_f32_ptr)lds3;
#pragma unroll
    for (int u = 0; u < T; ++u)
#pragma unroll
        for (int q = 0; q < 4; ++q)
            red[wave * kWaveFloats + u * 256 + (((4 * kq + q) * 16 + col) ^ (kq << 4))] = acc[u][q];
    __syncthreads();
#pragma unroll
    for (int gi = 0; gi < 4; ++gi) {
        const int g = wave + gi * waves;  // wave-uniform
        if (g < 4) {
            const int at = ((4 * g + kq) * 16 + col) ^ (g << 4);  // this lane: row 4 g + kq of the tile, channel col
            const int row = m0 + 4 * g + kq;
#pragma unroll
            for (int u = 0; u < T; ++u) {
                float sum = 0.f;
#pragma unroll 4
                for (int w = 0; w < waves; ++w)
                    sum += red[w * kWaveFloats + u * 256 + at];
                sum = __builtin_fmaf(sum, 0x1p24f, (float)__builtin_bit_cast(half_t, (uint16_t)bias_bits[u]));
                if (row < M)
                    store_out(y, (size_t)row * N + (t0 + u) * 16 + col, sum, out_f32);
            }
        }
    }
}

// Dynamic LDS: two 4 KiB activation buffers per wave, which hold the wave's partial sums (1 KiB per tile) at the end.
size_t gemv16s_lds_bytes(int waves, int tiles) {
    return tiles >= 1 && tiles <= 8 ? (size_t)waves * (2 * 4096) : (size_t)-1;
}

template <int C, bool ZPT, int XL, int T>
static int launch_gemv16s_tiles(const FcDeviceArgs& a, const LaunchPlan& p, hipStream_t s) {
    const Layout& L = a.layout;
    auto kern = fcc_gemv16s_kernel<C, ZPT, XL, T>;
    static bool attr_set = false;  // per instantiation; the attribute is idempotent, a race only repeats it
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                           160 * 1024 - 64);
        if (e != hipSuccess)
            return (int)e;
        attr_set = true;
    }
    hipLaunchKernelGGL(kern, dim3(p.grid[0], p.grid[1], 1), dim3(p.block), p.dynamic_lds, s, (const uint4_t*)a.w,
                       (const half_t*)a.scale_cm, (const uint8_t*)a.zp_cm, (const half_t*)a.x, (const half_t*)a.bias, a.y,
                       (int)a.M, (int)a.N, (int)a.K, (int)L.k_blocks, (int)L.n_tiles, L.zp_const, a.out_f32);
    return (int)hipGetLastError();
}

template <int C, bool ZPT, int XL>
static int launch_gemv16s_rows(const FcDeviceArgs& a, const LaunchPlan& p, hipStream_t s) {
    return p.tiles_per_group == 4   ? launch_gemv16s_tiles<C, ZPT, XL, 4>(a, p, s)
           : p.tiles_per_group == 2 ? launch_gemv16s_tiles<C, ZPT, XL, 2>(a, p, s)
                                    : launch_gemv16s_tiles<C, ZPT, XL, 1>(a, p, s);
}

template <int C, bool ZPT>
static int launch_gemv16s_impl(const FcDeviceArgs& a, const LaunchPlan& p, hipStream_t s) {
    // one row tile: as many four-row loads as M needs; several row tiles: all four
    const int xl = a.M > 12 ? 4 : a.M > 8 ? 3 : 2;
    return xl == 4 ? launch_gemv16s_rows<C, ZPT, 4>(a, p, s)
                   : xl == 3 ? launch_gemv16s_rows<C, ZPT, 3>(a, p, s) : launch_gemv16s_rows<C, ZPT, 2>(a, p, s);
}

int launch_gemv16_stream(const FcDeviceArgs& a, const LaunchPlan& p, void* stream) {
    hipStream_t s = static_cast<hipStream_t>(stream);
    const Layout& L = a.layout;
    const int c = L.gemv_c;
    // what the kernel and its grid assume, checked against the operands before anything is launched
    if (!L.tiled || L.bits != 4 || L.groups_per_kblock != 1 || L.kblocks_per_group != 1 || L.glu || !a.scale_cm ||
        (L.zp_table && !a.zp_cm) || a.M < 1 || a.M > kDecodeMaxRows || (c != 2 && c != 4 && c != 8) || L.k_blocks % c != 0 ||
        p.gemv_c != c || (!L.zp_table && (L.zp_const < 0 || L.zp_const > 255)))
        return (int)hipErrorInvalidValue;
    const int waves = (int)(L.k_blocks / c);
    const int tiles = p.tiles_per_group;
    if (waves < 1 || waves > 16 || p.block != 64u * waves || (tiles != 1 && tiles != 2 && tiles != 4) ||
        (int64_t)p.grid[0] * tiles != L.n_tiles || p.grid[1] != (unsigned)((a.M + 15) / 16) || p.grid[2] != 1 ||
        p.split_k != 1 || p.dynamic_lds != gemv16s_lds_bytes(waves, tiles) || p.dynamic_lds > 160 * 1024 - 64 ||
        a.M * a.K * 2 >= ((int64_t)1 << 31) || L.n_tiles * L.k_blocks * kTileBytes >= ((int64_t)1 << 31))
        return (int)hipErrorInvalidValue;
    if (L.zp_table)
        return c == 8 ? launch_gemv16s_impl<8, true>(a, p, s)
                      : c == 4 ? launch_gemv16s_impl<4, true>(a, p, s) : launch_gemv16s_impl<2, true>(a, p, s);
    return c == 8 ? launch_gemv16s_impl<8, false>(a, p, s)
                  : c == 4 ? launch_gemv16s_impl<4, false>(a, p, s) : launch_gemv16s_impl<2, false>(a, p, s);
}

}  // namespace ovfcc
