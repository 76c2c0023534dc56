// Decode kernel for five to forty-eight rows over 4-bit tiles with one group per k-block (G = 128): the matrix-vector
// kernel's structure (kernel_gemv.hip) carried to whole 16-row MFMA tiles, with the activations stationary.
//
// A workgroup has K / (128 C) waves; wave w owns the k-blocks w, w + NWT, ... (C of them) of every channel tile the
// workgroup visits.  At its start every wave brings its own k-range of 16 rows of the activations through its own
// slice of LDS (direct-to-LDS loads of whole kilobytes, 16 x C x 256 bytes; no barrier, nobody else reads the
// slice) into registers, in MFMA operand order, and keeps them there: 16 C registers per lane.  (Loading them
// straight into operand order, 64 contiguous bytes per row and load, costs a microsecond more at 16 rows.)  Then the
// workgroup walks the channel tiles blockIdx.x, blockIdx.x + gridDim.x, ... streaming only weights: three register
// sets in turn hold the weight tiles and group parameters of this visit and the next two, so two visits' loads
// travel while one is multiplied, and a visit reads nothing but registers.  The waves' partial sums of a tile meet
// in LDS behind one barrier per visit, where four waves add them in wave order (four rows each), apply the bias
// and store.  Nothing is split along K through memory -- which is what the small-batch kernel
// (kernel_batch.hip) pays five dependent round trips for -- and the activations travel from L2 once per workgroup,
// not once per channel tile.  Rows 16-31 and 32-47 are further workgroup rows (blockIdx.y).  The price: 16 rows x K x 2
// bytes of LDS for the hand-over, so K <= 4096 or so, and registers (16 C for the activations, 4 C for their group
// sums, 3 (4 C + 4) for the weights), which bound the workgroup at 8 and 16 waves for C = 4 and 2.  A node whose
// channel-major tables were laid out for eight k-blocks per wave runs with two waves per table row, four k-blocks
// each.  With a gated linear unit a workgroup visits the gate tile and the up tile of 16 channels in turn; the
// waves that add the sums keep the gate values in a register for the visit between.  Where 16 rows x K do not fit
// (K = 14336), K is cut in parts across blockIdx.z -- every workgroup then takes a share of each table row's slots --
// the parts leave f32 partial sums in a workspace and a second, small launch adds them: two launches and plain
// stores instead of the tickets and fences of a split-K epilogue inside one.
//
// LDS slice of a wave, in 16-byte units: row r, slot s (k-block w + NWT s), chunk c of the k-block's 16 sits at
// r (16 C) + 16 s + (c ^ r): the sixteen rows that one operand read touches lie in sixteen different bank groups.
//
// Arithmetic as in the matrix-vector kernel: nibbles stay in the mantissa as subnormal halves q 2^-24 / q 2^-20 (the
// matrix cores keep subnormal operands), the activations that meet the second kind are multiplied by 2^-4 once, in
// their registers; group scales multiply the f32 sums per k-block.  Zero-points leave through the activations'
// group sums c = sum_k x_k per row and k-block, which one MFMA chain per k-block against a constant operand
// leaves in exactly the registers that hold the products' rows:  y = 2^24 sum_kb s_kb (P_kb - zp_kb 2^-24 c_kb).
#include <type_traits>

#include "device_common.h"

namespace ovfcc {

namespace {
template <int N>
struct Vec16Of;
template <>
struct Vec16Of<2> {
    typedef uint32_t type;
};
template <>
struct Vec16Of<4> {
    typedef uint2_t type;
};

// group parameters and weight tiles of one channel tile, as one wave holds them
template <int C>
struct TileRegs {
    typename Vec16Of<C>::type sv;  // C scales (f16) of channel col
    uint32_t zv;                   // C zero-points (u8) of channel col
    uint32_t bias;                 // bias (f16) of channel col; 0 without one
    uint4_t wv[C];                 // the wave's C weight tiles
};
}  // namespace

// C: k-blocks per wave (the node's channel-major tables may be laid out for 2 C: then two waves share a table
// row, `parts` = k_blocks / c_table of them side by side, and a wave takes half of its slots); ZP_TABLE: zero-points
// per (channel, group); MULTI: workgroups visit more than one channel tile; GLU: tiles 2 j and 2 j + 1 hold the gate
// and up channels 16 j .. of a gated linear unit and a workgroup visits them one after the other; KSPLIT: the
// workgroups of one blockIdx.z take the same share of every table row's slots (K cut in gridDim.z parts, so that a
// part's 16 rows of activations fit in LDS) and leave f32 partial sums [gridDim.z][16 gridDim.y][N] without bias
// in `y`, which fcc_gemv16_sum_kernel adds up
template <int C, bool ZP_TABLE, bool MULTI, bool GLU, bool KSPLIT>
__global__ __launch_bounds__(C == 4 ? 512 : 1024) void fcc_gemv16_kernel(
    const uint4_t* __restrict__ wt, const half_t* __restrict__ scale_cm, const uint8_t* __restrict__ zp_cm,
    const half_t* __restrict__ x, const half_t* __restrict__ bias, void* __restrict__ y, int M, int N, int K,
    int kb_total, int parts, int c_table, int n_tiles, int zp_const, int out_f32, int red_bufs, int glu) {
    static_assert(!GLU || MULTI, "a gated linear unit takes two visits");
    static_assert(!GLU || !KSPLIT, "partial sums cannot pass through a gated linear unit");
    constexpr int kWaveBytes = C * 4096;   // 16 rows x C k-blocks x 256 bytes
    constexpr int kDepth = MULTI ? 3 : 1;  // visits whose weights are in registers or on their way
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];  // [waves] slices | partial sums
    const lds_byte_ptr lds3 = (lds_byte_ptr)lds_raw;
    typedef __attribute__((address_space(3))) const uint4_t* lds_u4_ptr;
    typedef __attribute__((address_space(3))) float* lds_f32_ptr;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int waves = blockDim.x >> 6;  // parts * c_table / C (/ gridDim.z with KSPLIT)
    const int part = wave % parts;      // the table row this wave reads: k-blocks part, part + parts, ...
    // ... of which it takes slots slot0 .. slot0 + C - 1
    const int slot0 = (wave / parts + (KSPLIT ? (int)blockIdx.z * ((int)(blockDim.x >> 6) / parts) : 0)) * C;
    const int col = lane & 15;
    const int kq = lane >> 4;
    const int m0 = 16 * blockIdx.y;
    // visit v of this workgroup
    auto tile_of = [&](int v) {
        return GLU ? 2 * ((int)blockIdx.x + (v >> 1) * (int)gridDim.x) + (v & 1) : (int)blockIdx.x + v * (int)gridDim.x;
    };

    constexpr unsigned kOob = 0x80000000u;
    constexpr int kRsrcFlags = 0x00020000;
    const __amdgpu_buffer_rsrc_t rx =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(x), 0, M * K * 2, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint4_t*>(wt), 0,
                                                                        n_tiles * kb_total * kTileBytes, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(scale_cm), 0,
                                                                        n_tiles * 16 * kb_total * 2, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t rz = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint8_t*>(zp_cm), 0, ZP_TABLE ? n_tiles * 16 * kb_total : 0, kRsrcFlags);
    // fetched with the weights, so that the waves that store never wait for a load younger than their prefetches
    const __amdgpu_buffer_rsrc_t rb =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t*>(bias), 0, bias ? n_tiles * 32 : 0, kRsrcFlags);

    // ---- one channel tile's parameters and weights ----
    auto load_tile = [&](int t, TileRegs<C>& r) {
        // no branch (the compiler counts the loads in flight only along straight code); a load sent out of range
        // still costs its issue cycles, which is why workgroups with one visit run the kernel without prefetches
        const unsigned oob = (unsigned)((n_tiles - 1 - t) >> 31) & kOob;
        const unsigned pofs = (unsigned)((t * 16 + col) * kb_total + part * c_table + slot0);
        if constexpr (C == 4)
            r.sv = __builtin_bit_cast(uint2_t, __builtin_amdgcn_raw_buffer_load_b64(rs, (pofs * 2u) | oob, 0, 0));
        else
            r.sv = __builtin_amdgcn_raw_buffer_load_b32(rs, (pofs * 2u) | oob, 0, 0);
        r.bias = __builtin_amdgcn_raw_buffer_load_b16(rb, (unsigned)((t * 16 + col) * 2) | oob, 0, 0);
        r.zv = 0u;
        if constexpr (ZP_TABLE) {
            if constexpr (C == 4)
                r.zv = __builtin_amdgcn_raw_buffer_load_b32(rz, pofs | oob, 0, 0);
            else
                r.zv = __builtin_amdgcn_raw_buffer_load_b16(rz, pofs | oob, 0, 0);
        }
        const unsigned wofs = (unsigned)(t * kb_total + part + parts * slot0) * kTileBytes + lane * 16;
#pragma unroll
        for (int i = 0; i < C; ++i)
            r.wv[i] = __builtin_bit_cast(
                uint4_t, __builtin_amdgcn_raw_buffer_load_b128(rw, (wofs + (unsigned)(i * parts) * kTileBytes) | oob, 0, 2));
    };

    // ---- loads: the first two visits' weights, then the activations: load q of the wave fills units 64 q ..
    // 64 q + 63 of its slice.  The wait below is for everything in flight -- the compiler cannot see that the LDS
    // reads depend on these loads -- so that it holds wherever the loads whose results the compiler tracks itself
    // end up. ----
    TileRegs<C> ring[kDepth];
#pragma unroll
    for (int u = 0; u < (MULTI ? kDepth - 1 : 1); ++u)
        load_tile(tile_of(u), ring[u]);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int q = 0; q < 4 * C; ++q) {
        const int unit = 64 * q + lane;
        const int row = unit / (16 * C), in_row = unit % (16 * C);
        const int slot = in_row >> 4, chunk = (in_row & 15) ^ row;
        const unsigned ofs = ((unsigned)((m0 + row) * K + (part + parts * (slot0 + slot)) * 128 + chunk * 8) * 2u) |
                             ((unsigned)((M - 1 - m0 - row) >> 31) & kOob);
        // a load whose rows all lie beyond M is left out (it would cost its issue cycles all the same): those rows
        // of the slice keep what LDS held, and what is computed from them is never stored
        if (m0 + (64 * q) / (16 * C) < M)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, (lds_void_ptr)(lds3 + wave * kWaveBytes + q * 1024), 16, ofs,
                                                     0, 0, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(wait_vmcnt_imm(0));
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);

    // ---- activations into registers, in operand order: row col, chunk (4 j + kq) ^ col of slot i ----
    const lds_byte_ptr xs_lane = lds3 + wave * kWaveBytes + col * (C * 256);
    Frag8 xa[C][4];
#pragma unroll
    for (int i = 0; i < C; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint4_t v = *(lds_u4_ptr)(xs_lane + i * 256 + (((4 * j + kq) ^ col) << 4));
            xa[i][j].u[0] = v.x, xa[i][j].u[1] = v.y, xa[i][j].u[2] = v.z, xa[i][j].u[3] = v.w;
        }
    // the halves that meet nibbles four bits up (elements 2, 3, 6, 7 of a chunk) times 2^-4
    const half2_t sixteenth = half2_t{(half_t)0.0625f, (half_t)0.0625f};
#pragma unroll
    for (int i = 0; i < C; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            xa[i][j].u[1] = as_u32(as_half2(xa[i][j].u[1]) * sixteenth);
            xa[i][j].u[3] = as_u32(as_half2(xa[i][j].u[3]) * sixteenth);
        }
    // group sums, 2^-24 c (times -zp when the zero-point is one constant), for rows 4 kq .. + 3 and every slot
    float cz[C][4];
    {
        Frag8 ones;  // 1 against the plain halves, 16 against the scaled ones
        ones.u[0] = ones.u[2] = 0x3C003C00u;
        ones.u[1] = ones.u[3] = 0x4C004C00u;
        const float cmul = ZP_TABLE ? 0x1p-24f : -(float)zp_const * 0x1p-24f;
#pragma unroll
        for (int i = 0; i < C; ++i) {
            float4_t p = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j = 0; j < 4; ++j)
                p = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[i][j].v, ones.v, p, 0, 0, 0);
            cz[i][0] = p.x * cmul, cz[i][1] = p.y * cmul, cz[i][2] = p.z * cmul, cz[i][3] = p.w * cmul;
        }
    }

    const uint32_t mask_lo = 0x000F000Fu, mask_hi = 0x00F000F0u;
    int buf = 0;
    float gate[4] = {0.f, 0.f, 0.f, 0.f};  // gated linear unit: what the gate tile's visit left for the up tile's

    // ---- one visit: multiply the channel tile held in `cur`, meet the other waves, store ----
    auto visit = [&](const TileRegs<C>& cur, int t) {
        float acc[4] = {0.f, 0.f, 0.f, 0.f};  // rows 4 kq .. + 3 of the row tile, channel col
#pragma unroll
        for (int i = 0; i < C; ++i) {
            const uint32_t wd[4] = {cur.wv[i].x, cur.wv[i].y, cur.wv[i].z, cur.wv[i].w};
            float4_t p = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t w8 = wd[j] >> 8;
                Frag8 b;  // element e of the dword's eight: nibble (e >> 1) + 4 (e & 1)
                b.u[0] = wd[j] & mask_lo;
                b.u[1] = wd[j] & mask_hi;
                b.u[2] = w8 & mask_lo;
                b.u[3] = w8 & mask_hi;
                p = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[i][j].v, b.v, p, 0, 0, 0);
            }
            uint32_t sbits;
            if constexpr (C == 4)
                sbits = (i < 2 ? cur.sv.x : cur.sv.y) >> (16 * (i & 1));
            else
                sbits = cur.sv >> (16 * (i & 1));
            const float scale = (float)__builtin_bit_cast(half_t, (uint16_t)sbits);
            const float pr[4] = {p.x, p.y, p.z, p.w};
            if constexpr (ZP_TABLE) {
                const float zpf = (float)((cur.zv >> (8 * i)) & 0xFFu);
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    acc[q] += scale * (pr[q] - zpf * cz[i][q]);
            } else {
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    acc[q] += scale * (pr[q] + cz[i][q]);
            }
        }
        // Partial sums of the workgroup's waves meet in LDS, 16 rows x 16 channels per wave with the 16-float
        // pieces of a row group rotated by the group (no two lanes of a write or a read share a bank); waves 0-3
        // add one group of four rows each, in wave order, apply the bias and store.  With two buffers in turn, the
        // barrier of the next visit stands between a buffer's readers and its next writers.
        const lds_f32_ptr red = (lds_f32_ptr)(lds3 + waves * kWaveBytes + buf * (waves * 1024));
#pragma unroll
        for (int q = 0; q < 4; ++q)
            red[wave * 256 + (((4 * kq + q) * 16 + col) ^ (kq << 4))] = acc[q];
        __syncthreads();
#pragma unroll
        for (int gi = 0; gi < 4; ++gi) {
            const int g = wave + gi * waves;  // wave-uniform
            if (g < 4) {
                const int at = ((4 * g + kq) * 16 + col) ^ (g << 4);  // this lane: row 4 g + kq of the tile, channel col
                float s = 0.f;
#pragma unroll 4
                for (int w = 0; w < waves; ++w)
                    s += red[w * 256 + at];
                const int row = m0 + 4 * g + kq;
                if constexpr (KSPLIT) {
                    // rows >= M of the last row tile are stored too: the partial buffer has whole row tiles
                    static_cast<float*>(y)[((size_t)blockIdx.z * (16 * gridDim.y) + row) * N + t * 16 + col] = s * 0x1p24f;
                    continue;
                }
                s = s * 0x1p24f + (float)__builtin_bit_cast(half_t, (uint16_t)cur.bias);
                if constexpr (GLU) {
                    if (t & 1) {
                        if (row < M)
                            store_out(y, (size_t)row * (N / 2) + (t >> 1) * 16 + col, glu_value(glu, gate[gi], s), out_f32);
                    } else {
                        gate[gi] = s;
                    }
                } else {
                    if (row < M)
                        store_out(y, (size_t)row * N + t * 16 + col, s, out_f32);
                }
            }
        }
        buf = buf + 1 == red_bufs ? 0 : buf + 1;
    };

    if constexpr (!MULTI) {
        visit(ring[0], tile_of(0));
    } else {
        // kDepth register sets in turn: the set multiplied last is refilled for the visit kDepth - 1 from now
        for (int v = 0;; v += kDepth) {
#pragma unroll
            for (int u = 0; u < kDepth; ++u) {
                load_tile(tile_of(v + u + kDepth - 1), ring[(u + kDepth - 1) % kDepth]);
                visit(ring[u], tile_of(v + u));
                if (tile_of(v + u + 1) >= n_tiles)
                    return;
            }
        }
    }
}

// y[m][n] = sum over z of partial[z][m][n] + bias[n], in the order of z; partial has rows_pad rows per part
__global__ __launch_bounds__(256) void fcc_gemv16_sum_kernel(const float* __restrict__ partial, const half_t* __restrict__ bias,
                                                             void* __restrict__ y, int M, int N, int rows_pad, int parts,
                                                             int out_f32) {
    const int i = blockIdx.x * 256 + threadIdx.x;  // four neighbouring channels of one row
    const int per_row = N / 4;
    if (i >= M * per_row)
        return;
    const int m = i / per_row, n = (i - m * per_row) * 4;
    float4_t s = float4_t{0.f, 0.f, 0.f, 0.f};
    for (int z = 0; z < parts; ++z)
        s += *reinterpret_cast<const float4_t*>(partial + ((size_t)z * rows_pad + m) * N + n);
    const float v[4] = {s.x, s.y, s.z, s.w};
#pragma unroll
    for (int j = 0; j < 4; ++j)
        store_out(y, (size_t)m * N + n + j, v[j] + (bias ? (float)bias[n + j] : 0.f), out_f32);
}

// Dynamic LDS: every wave hands over 16 rows of its c k-blocks and leaves 16 x 16 partial sums per buffer.
size_t gemv16_lds_bytes(int c, int waves, int red_bufs) {
    return (size_t)waves * c * 4096 + (size_t)red_bufs * waves * 1024;
}

// k-blocks per wave that the kernel runs a node with: tables laid out for eight are read by two waves per row; with
// K cut in split_k parts a wave takes its share of the row's slots
int gemv16_kblocks_per_wave(int c_table, int split_k) {
    if (split_k > 1)
        return c_table / split_k;
    return c_table == 2 ? 2 : 4;
}

template <int C, bool ZPT, bool MULTI, bool GLU, bool KSPLIT>
static int launch_gemv16_impl(const FcDeviceArgs& a, const LaunchPlan& p, int red_bufs, hipStream_t s) {
    const Layout& L = a.layout;
    auto kern = fcc_gemv16_kernel<C, ZPT, MULTI, GLU, KSPLIT>;
    static bool attr_set = false;  // per instantiation; the attribute is idempotent, a race only repeats it
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024 - 64);
        if (e != hipSuccess)
            return (int)e;
        attr_set = true;
    }
    hipLaunchKernelGGL(kern, dim3(p.grid[0], p.grid[1], p.grid[2]), dim3(p.block), p.dynamic_lds, s, (const uint4_t*)a.w,
                       (const half_t*)a.scale_cm, (const uint8_t*)a.zp_cm, (const half_t*)a.x, (const half_t*)a.bias,
                       KSPLIT ? (void*)a.workspace : a.y, (int)a.M, (int)a.N, (int)a.K, (int)L.k_blocks,
                       (int)(L.k_blocks / L.gemv_c), L.gemv_c, (int)L.n_tiles, L.zp_const, a.out_f32, red_bufs, L.glu);
    if constexpr (KSPLIT) {
        const int64_t quads = a.M * (a.N / 4);
        hipLaunchKernelGGL(fcc_gemv16_sum_kernel, dim3((unsigned)((quads + 255) / 256)), dim3(256), 0, s,
                           (const float*)a.workspace, (const half_t*)a.bias, a.y, (int)a.M, (int)a.N, (int)(16 * p.grid[1]),
                           (int)p.grid[2], a.out_f32);
    }
    return (int)hipGetLastError();
}

int launch_gemv16(const FcDeviceArgs& a, const LaunchPlan& p, void* stream) {
    hipStream_t s = static_cast<hipStream_t>(stream);
    const Layout& L = a.layout;
    const int ct = L.gemv_c;
    // what the kernel and its grid assume, checked against the operands before anything is launched
    if (!L.tiled || L.bits != 4 || L.groups_per_kblock != 1 || L.kblocks_per_group != 1 || !a.scale_cm ||
        (L.zp_table && !a.zp_cm) || a.M < 1 || a.M > kDecodeMaxRows || (ct != 2 && ct != 4 && ct != 8) || L.k_blocks % ct != 0 ||
        p.gemv_c != ct || (!L.zp_table && (L.zp_const < 0 || L.zp_const > 255)) || (L.glu && (L.n_tiles & 1)))
        return (int)hipErrorInvalidValue;
    const int split = p.split_k;
    if (split < 1 || (split > 1 && (L.glu || ct % split != 0 || !a.workspace || (a.N & 3) ||
                                    p.workspace_bytes != (size_t)split * 16 * p.grid[1] * a.N * sizeof(float))))
        return (int)hipErrorInvalidValue;
    const int c = gemv16_kblocks_per_wave(ct, split);
    if (c != 2 && c != 4)
        return (int)hipErrorInvalidValue;
    const int waves = (int)(L.k_blocks / c / split);
    const int64_t units = L.glu ? L.n_tiles / 2 : L.n_tiles;  // what a workgroup visits in one go: tiles or tile pairs
    if (waves < 1 || waves > (c == 4 ? 8 : 16) || p.block != 64u * waves || p.grid[0] < 1 || (int64_t)p.grid[0] > units ||
        p.grid[1] != (unsigned)((a.M + 15) / 16) || p.grid[2] != (unsigned)split)
        return (int)hipErrorInvalidValue;
    const int red_bufs = (L.glu || (int64_t)p.grid[0] < units) ? 2 : 1;
    if (p.dynamic_lds != gemv16_lds_bytes(c, waves, red_bufs) || p.dynamic_lds > 160 * 1024 - 64 ||
        a.M * a.K * 2 >= ((int64_t)1 << 31) || (L.n_tiles + 2 * (int64_t)p.grid[0]) * L.k_blocks * kTileBytes >= ((int64_t)1 << 32) ||
        L.n_tiles * L.k_blocks * kTileBytes >= ((int64_t)1 << 31))
        return (int)hipErrorInvalidValue;
    const bool multi = red_bufs == 2;
    auto go = [&](auto zpt, auto mul, auto gl) {
        constexpr bool Z = decltype(zpt)::value, U = decltype(mul)::value, G = decltype(gl)::value;
        if constexpr (!G) {
            if (split > 1)
                return c == 4 ? launch_gemv16_impl<4, Z, U, false, true>(a, p, red_bufs, s)
                              : launch_gemv16_impl<2, Z, U, false, true>(a, p, red_bufs, s);
        }
        return c == 4 ? launch_gemv16_impl<4, Z, U, G, false>(a, p, red_bufs, s)
                      : launch_gemv16_impl<2, Z, U, G, false>(a, p, red_bufs, s);
    };
    const std::true_type yes{};
    const std::false_type no{};
    if (L.glu)
        return L.zp_table ? go(yes, yes, yes) : go(no, yes, yes);
    if (L.zp_table)
        return multi ? go(yes, yes, no) : go(yes, no, no);
    return multi ? go(no, yes, no) : go(no, no, no);
}

}  // namespace ovfcc
