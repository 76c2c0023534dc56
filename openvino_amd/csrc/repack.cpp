// Host-side descriptor validation and the compile-time weight repacker.
//
// Stands in for what the OpenVINO plugins do once per FullyConnectedCompressed node:
//   - the support gate FullyConnected::isSupportedCompressedOperation
//     (src/plugins/intel_cpu/src/nodes/fullyconnected.cpp:143-218),
//   - the one-time weight re-layout (CPU: utils::prepareWeightsMemory,
//     src/plugins/intel_cpu/src/nodes/executors/dnnl/dnnl_utils.cpp:49-122;
//     Intel GPU: cl_kernels/reorder_weights_int4.cl),
//   - the signed -> unsigned shift of i4/i8 weights (dnnl_utils.cpp:70-97).
// The element order inside a byte is OpenVINO's: even element in the low nibble
// (src/core/dev_api/openvino/core/type/element_iterator.hpp:76,161-176).
#include <algorithm>
#include <cstring>
#include <thread>
#include <vector>

#include "ovfcc_internal.h"

namespace ovfcc {

static thread_local std::string g_error;

void set_error(const std::string& msg) {
    g_error = msg;
}

int fail(int code, const std::string& msg) {
    g_error = msg;
    return code;
}

const std::string& last_error_string() {
    return g_error;
}

static inline bool is4(int t) {
    return t == OVFCC_U4 || t == OVFCC_I4;
}

int validate_desc(const ovfcc_fc_desc* d) {
    if (!d)
        return fail(OVFCC_EINVAL, "descriptor is null");
    if (d->N <= 0 || d->K <= 0)
        return fail(OVFCC_EINVAL, "N and K must be positive");
    if (d->group_size <= 0 || d->K % d->group_size != 0)
        return fail(OVFCC_EINVAL, "group_size must be positive and divide K");
    switch (d->w_type) {
    case OVFCC_U4:
    case OVFCC_I4:
    case OVFCC_U8:
    case OVFCC_I8:
        break;
    default:
        return fail(OVFCC_EUNSUPPORTED, "weight type must be u4, i4, u8 or i8");
    }
    if (d->scale_type != OVFCC_F16)
        return fail(OVFCC_EUNSUPPORTED, "scales must be f16");
    if (d->zp_type != OVFCC_NONE && d->zp_type != OVFCC_U4 && d->zp_type != OVFCC_U8)
        return fail(OVFCC_EUNSUPPORTED, "zero-points must be absent, u4 or u8");
    if (d->bias_type != OVFCC_NONE && d->bias_type != OVFCC_F16)
        return fail(OVFCC_EUNSUPPORTED, "bias must be absent or f16");
    if (d->act_type != OVFCC_F16)
        return fail(OVFCC_EUNSUPPORTED, "activations must be f16");
    if (d->out_type != OVFCC_F16 && d->out_type != OVFCC_F32)
        return fail(OVFCC_EUNSUPPORTED, "output must be f16 or f32");
    if (d->flags & ~(OVFCC_GLU_TYPE_MASK | OVFCC_GLU_GATE_SECOND | OVFCC_DYNQUANT_I8 | OVFCC_DYNQUANT_PER_GROUP | OVFCC_DYNQUANT_ASYM |
                     OVFCC_W_INPUT_MAJOR))
        return fail(OVFCC_EINVAL, "unknown bits in flags");
    if ((d->flags & OVFCC_DYNQUANT_PER_GROUP) && !(d->flags & OVFCC_DYNQUANT_I8))
        return fail(OVFCC_EINVAL, "OVFCC_DYNQUANT_PER_GROUP without OVFCC_DYNQUANT_I8");
    if ((d->flags & OVFCC_DYNQUANT_ASYM) && (!(d->flags & OVFCC_DYNQUANT_I8) || (d->flags & OVFCC_DYNQUANT_PER_GROUP)))
        return fail(OVFCC_EINVAL, "OVFCC_DYNQUANT_ASYM goes with OVFCC_DYNQUANT_I8 and per-token quantisation only");
    if ((d->flags & OVFCC_GLU_GATE_SECOND) && (d->flags & OVFCC_GLU_TYPE_MASK) == OVFCC_GLU_NONE)
        return fail(OVFCC_EINVAL, "OVFCC_GLU_GATE_SECOND without a gated-linear-unit type");
    if ((d->flags & OVFCC_GLU_TYPE_MASK) != OVFCC_GLU_NONE && (d->N % 2) != 0)
        return fail(OVFCC_EINVAL, "a gated linear unit splits N in two: N must be even");
    if (d->N > (int64_t)1 << 24 || d->K > (int64_t)1 << 24)
        return fail(OVFCC_EUNSUPPORTED, "N and K are limited to 2^24");
    return OVFCC_OK;
}

Layout make_layout(const ovfcc_fc_desc& d) {
    Layout L;
    L.bits = is4(d.w_type) ? 4 : 8;
    L.groups = d.K / d.group_size;
    L.zp_offset = d.w_type == OVFCC_I4 ? 8 : (d.w_type == OVFCC_I8 ? 128 : 0);
    L.zp_table = d.zp_type != OVFCC_NONE && !d.zp_scalar;
    L.zp_const = L.zp_offset;
    // K / 128 < 2^16 keeps the kernels' 32-bit offsets and reciprocal group index exact
    L.dynquant = (d.flags & OVFCC_DYNQUANT_I8) != 0;
    L.dynquant_grouped = L.dynquant && (d.flags & OVFCC_DYNQUANT_PER_GROUP) != 0;
    L.dynquant_asym = L.dynquant && (d.flags & OVFCC_DYNQUANT_ASYM) != 0;
    L.glu = d.flags & OVFCC_GLU_TYPE_MASK;
    L.glu_gate_second = (d.flags & OVFCC_GLU_GATE_SECOND) != 0;
    const bool small_groups = L.bits == 4 && (d.group_size == 32 || d.group_size == 64);
    // The tiled zero-point table holds zp + zp_offset in one byte: signed weights with 8-bit zero-points per group
    // (up to 255 + 8 or 255 + 128) do not fit and keep OpenVINO's layout, which the plain kernel runs.
    const bool zp_fits = !L.zp_table || L.zp_offset + (d.zp_type == OVFCC_U4 ? 15 : 255) <= 255;
    L.tiled = (d.N % (L.glu ? 2 * kTileRows : kTileRows) == 0) && (d.K % kBlockK == 0) &&
              (d.group_size % kBlockK == 0 || small_groups) && (d.K / kBlockK < 65536) && zp_fits;
    if (L.tiled) {
        L.n_tiles = d.N / kTileRows;
        L.k_blocks = d.K / kBlockK;
        L.tiles_per_kblock = L.bits == 4 ? 1 : 2;
        L.kblocks_per_group = small_groups ? 1 : d.group_size / kBlockK;
        L.groups_per_kblock = small_groups ? kBlockK / (int)d.group_size : 1;
        L.w_bytes = (size_t)L.n_tiles * L.k_blocks * L.tiles_per_kblock * kTileBytes;
        L.scale_bytes = (size_t)L.n_tiles * L.groups * kTileRows * 2;
        L.zp_bytes = L.zp_table ? (size_t)L.n_tiles * L.groups * kTileRows : 0;
    }
    return L;
}

static inline unsigned nibble(const uint8_t* p, size_t i) {
    return (i & 1) ? (p[i >> 1] >> 4) : (p[i >> 1] & 0x0F);
}

int scalar_zero_point(const ovfcc_fc_desc& d, const void* zp) {
    if (d.zp_type == OVFCC_NONE || !zp)
        return 0;
    const uint8_t* p = static_cast<const uint8_t*>(zp);
    return d.zp_type == OVFCC_U4 ? (int)(p[0] & 0x0F) : (int)p[0];
}

template <class F>
static void parallel_for(int64_t n, F&& body) {
    unsigned hw = std::max(1u, std::min(16u, std::thread::hardware_concurrency()));
    if (n < 64 || hw == 1) {
        for (int64_t i = 0; i < n; ++i)
            body(i);
        return;
    }
    std::vector<std::thread> pool;
    const int64_t chunk = (n + hw - 1) / hw;
    for (unsigned t = 0; t < hw; ++t) {
        const int64_t lo = t * chunk, hi = std::min<int64_t>(n, lo + chunk);
        if (lo >= hi)
            break;
        pool.emplace_back([lo, hi, &body] {
            for (int64_t i = lo; i < hi; ++i)
                body(i);
        });
    }
    for (auto& th : pool)
        th.join();
}

// source dword holds elements e = 0..7 at bits 4e; tile dword holds element e at nibble (e>>1) + 4*(e&1)
static inline uint32_t permute_nibbles_to_tile(uint32_t s) {
    uint32_t out = 0;
    for (int e = 0; e < 8; ++e) {
        const int p = (e >> 1) + 4 * (e & 1);
        out |= ((s >> (4 * e)) & 0xFu) << (4 * p);
    }
    return out;
}

static inline uint32_t permute_nibbles_from_tile(uint32_t t) {
    uint32_t out = 0;
    for (int e = 0; e < 8; ++e) {
        const int p = (e >> 1) + 4 * (e & 1);
        out |= ((t >> (4 * p)) & 0xFu) << (4 * e);
    }
    return out;
}

static inline void set_nibble(uint8_t* p, size_t i, unsigned v) {
    uint8_t& b = p[i >> 1];
    b = (i & 1) ? (uint8_t)((b & 0x0F) | (v << 4)) : (uint8_t)((b & 0xF0) | v);
}

// rows x cols (row-major, `bits` per element, packed over the flattened index) -> cols x rows
static void transpose_elements(const uint8_t* src, uint8_t* dst, int64_t rows, int64_t cols, int bits) {
    if (bits == 4) {
        // Two output rows share a byte where `rows` is odd, so workers own pairs of output rows.
        parallel_for((cols + 1) / 2, [&](int64_t pair) {
            for (int64_t c = 2 * pair; c < std::min(cols, 2 * pair + 2); ++c)
                for (int64_t r = 0; r < rows; ++r)
                    set_nibble(dst, (size_t)(c * rows + r), nibble(src, (size_t)(r * cols + c)));
        });
    } else {
        const int bytes = bits / 8;
        parallel_for(cols, [&](int64_t c) {
            for (int64_t r = 0; r < rows; ++r)
                std::memcpy(dst + (size_t)(c * rows + r) * bytes, src + (size_t)(r * cols + c) * bytes, bytes);
        });
    }
}

void transpose_input_major(const ovfcc_fc_desc& d, const void* w, const void* scales, const void* zp,
                           OutputMajorCopy* out) {
    const int64_t N = d.N, K = d.K, ng = K / d.group_size;
    const int wbits = is4(d.w_type) ? 4 : 8;
    out->w.assign(((size_t)N * K * wbits + 7) / 8, 0);
    transpose_elements(static_cast<const uint8_t*>(w), out->w.data(), K, N, wbits);
    out->scales.assign((size_t)N * ng, 0);
    transpose_elements(static_cast<const uint8_t*>(scales), reinterpret_cast<uint8_t*>(out->scales.data()), ng, N, 16);
    out->zp.clear();
    if (d.zp_type != OVFCC_NONE && zp) {
        const int zbits = d.zp_type == OVFCC_U4 ? 4 : 8;
        if (d.zp_scalar) {
            out->zp.assign(1, static_cast<const uint8_t*>(zp)[0]);
        } else {
            out->zp.assign(((size_t)N * ng * zbits + 7) / 8, 0);
            transpose_elements(static_cast<const uint8_t*>(zp), out->zp.data(), ng, N, zbits);
        }
    }
}

void repack_weights(const ovfcc_fc_desc& d, const Layout& L, const void* w, void* w_tiled) {
    const uint8_t* src = static_cast<const uint8_t*>(w);
    uint8_t* dst = static_cast<uint8_t*>(w_tiled);
    const int64_t K = d.K;
    if (L.bits == 4) {
        const uint32_t flip = d.w_type == OVFCC_I4 ? 0x88888888u : 0u;
        parallel_for(L.n_tiles, [&](int64_t nt) {
            for (int64_t kb = 0; kb < L.k_blocks; ++kb) {
                uint8_t* tile = dst + (size_t)(nt * L.k_blocks + kb) * kTileBytes;
                for (int lane = 0; lane < 64; ++lane) {
                    const int64_t n = L.source_tile(nt) * kTileRows + (lane & 15);
                    const int kq = lane >> 4;
                    for (int j = 0; j < 4; ++j) {
                        const int64_t k = kb * kBlockK + 32 * j + 8 * kq;
                        uint32_t s;
                        std::memcpy(&s, src + (size_t)(n * K + k) / 2, 4);
                        const uint32_t t = permute_nibbles_to_tile(s ^ flip);
                        std::memcpy(tile + lane * 16 + j * 4, &t, 4);
                    }
                }
            }
        });
    } else {
        const uint8_t flip = d.w_type == OVFCC_I8 ? 0x80 : 0;
        const int64_t k_tiles = L.k_blocks * 2;
        parallel_for(L.n_tiles, [&](int64_t nt) {
            for (int64_t kt = 0; kt < k_tiles; ++kt) {
                uint8_t* tile = dst + (size_t)(nt * k_tiles + kt) * kTileBytes;
                for (int lane = 0; lane < 64; ++lane) {
                    const int64_t n = L.source_tile(nt) * kTileRows + (lane & 15);
                    const int kq = lane >> 4;
                    for (int dw = 0; dw < 4; ++dw) {
                        const int64_t k = kt * 64 + 32 * (dw >> 1) + 8 * kq + 4 * (dw & 1);
                        for (int b = 0; b < 4; ++b)
                            tile[lane * 16 + dw * 4 + b] = (uint8_t)(src[(size_t)(n * K + k + b)] ^ flip);
                    }
                }
            }
        });
    }
}

void unrepack_weights(const ovfcc_fc_desc& d, const Layout& L, const void* w_tiled, void* w) {
    const uint8_t* src = static_cast<const uint8_t*>(w_tiled);
    uint8_t* dst = static_cast<uint8_t*>(w);
    const int64_t K = d.K;
    if (L.bits == 4) {
        const uint32_t flip = d.w_type == OVFCC_I4 ? 0x88888888u : 0u;
        parallel_for(L.n_tiles, [&](int64_t nt) {
            for (int64_t kb = 0; kb < L.k_blocks; ++kb) {
                const uint8_t* tile = src + (size_t)(nt * L.k_blocks + kb) * kTileBytes;
                for (int lane = 0; lane < 64; ++lane) {
                    const int64_t n = L.source_tile(nt) * kTileRows + (lane & 15);
                    const int kq = lane >> 4;
                    for (int j = 0; j < 4; ++j) {
                        const int64_t k = kb * kBlockK + 32 * j + 8 * kq;
                        uint32_t t;
                        std::memcpy(&t, tile + lane * 16 + j * 4, 4);
                        const uint32_t s = permute_nibbles_from_tile(t) ^ flip;
                        std::memcpy(dst + (size_t)(n * K + k) / 2, &s, 4);
                    }
                }
            }
        });
    } else {
        const uint8_t flip = d.w_type == OVFCC_I8 ? 0x80 : 0;
        const int64_t k_tiles = L.k_blocks * 2;
        parallel_for(L.n_tiles, [&](int64_t nt) {
            for (int64_t kt = 0; kt < k_tiles; ++kt) {
                const uint8_t* tile = src + (size_t)(nt * k_tiles + kt) * kTileBytes;
                for (int lane = 0; lane < 64; ++lane) {
                    const int64_t n = L.source_tile(nt) * kTileRows + (lane & 15);
                    const int kq = lane >> 4;
                    for (int dw = 0; dw < 4; ++dw) {
                        const int64_t k = kt * 64 + 32 * (dw >> 1) + 8 * kq + 4 * (dw & 1);
                        for (int b = 0; b < 4; ++b)
                            dst[(size_t)(n * K + k + b)] = (uint8_t)(tile[lane * 16 + dw * 4 + b] ^ flip);
                    }
                }
            }
        });
    }
}

void repack_params(const ovfcc_fc_desc& d, const Layout& L, const void* scales, const void* zp, void* scale_tiled,
                   void* zp_tiled) {
    const uint16_t* s = static_cast<const uint16_t*>(scales);
    uint16_t* st = static_cast<uint16_t*>(scale_tiled);
    const uint8_t* z = static_cast<const uint8_t*>(zp);
    uint8_t* zt = static_cast<uint8_t*>(zp_tiled);
    const int64_t ng = L.groups;
    for (int64_t nt = 0; nt < L.n_tiles; ++nt)
        for (int64_t g = 0; g < ng; ++g)
            for (int r = 0; r < kTileRows; ++r) {
                const int64_t n = L.source_tile(nt) * kTileRows + r;
                const size_t o = L.param_index(nt, g, r);
                st[o] = s[n * ng + g];
                if (L.zp_table) {
                    const unsigned v = d.zp_type == OVFCC_U4 ? nibble(z, (size_t)(n * ng + g)) : z[n * ng + g];
                    zt[o] = (uint8_t)(v + L.zp_offset);
                }
            }
}

void unrepack_params(const ovfcc_fc_desc& d, const Layout& L, const void* scale_tiled, const void* zp_tiled,
                     void* scales, void* zp) {
    const uint16_t* st = static_cast<const uint16_t*>(scale_tiled);
    uint16_t* s = static_cast<uint16_t*>(scales);
    const uint8_t* zt = static_cast<const uint8_t*>(zp_tiled);
    uint8_t* z = static_cast<uint8_t*>(zp);
    const int64_t ng = L.groups;
    if (L.zp_table && d.zp_type == OVFCC_U4)
        std::memset(z, 0, (size_t)(d.N * ng + 1) / 2);
    for (int64_t nt = 0; nt < L.n_tiles; ++nt)
        for (int64_t g = 0; g < ng; ++g)
            for (int r = 0; r < kTileRows; ++r) {
                const int64_t n = L.source_tile(nt) * kTileRows + r;
                const size_t o = L.param_index(nt, g, r);
                s[n * ng + g] = st[o];
                if (L.zp_table) {
                    const unsigned v = (unsigned)zt[o] - L.zp_offset;
                    const size_t i = (size_t)(n * ng + g);
                    if (d.zp_type == OVFCC_U4)
                        z[i >> 1] |= (uint8_t)((v & 0xF) << ((i & 1) * 4));
                    else
                        z[i] = (uint8_t)v;
                }
            }
}

}  // namespace ovfcc

// ---- C ABI: host-only entry points ---------------------------------------------------------------

namespace ovfcc {
const std::string& last_error_string();
}

extern "C" {

const char* ovfcc_last_error(void) {
    return ovfcc::last_error_string().c_str();
}

const char* ovfcc_version(void) {
    return "ovfcc 0.1 (gfx950)";
}

int ovfcc_desc_validate(const ovfcc_fc_desc* desc) {
    return ovfcc::validate_desc(desc);
}

int ovfcc_tiled_sizes(const ovfcc_fc_desc* desc, size_t* w_bytes, size_t* scale_bytes, size_t* zp_bytes) {
    if (!w_bytes || !scale_bytes || !zp_bytes)
        return ovfcc::fail(OVFCC_EINVAL, "size outputs are null");
    int rc = ovfcc::validate_desc(desc);
    if (rc != OVFCC_OK)
        return rc;
    const ovfcc::Layout L = ovfcc::make_layout(*desc);
    *w_bytes = L.w_bytes;
    *scale_bytes = L.scale_bytes;
    *zp_bytes = L.zp_bytes;
    return OVFCC_OK;
}

int ovfcc_repack_host(const ovfcc_fc_desc* desc, const void* w, const void* scales, const void* zp, void* w_tiled,
                      void* scale_tiled, void* zp_tiled) {
    int rc = ovfcc::validate_desc(desc);
    if (rc != OVFCC_OK)
        return rc;
    const ovfcc::Layout L = ovfcc::make_layout(*desc);
    if (!L.tiled)
        return ovfcc::fail(OVFCC_EUNSUPPORTED, "shape keeps the OpenVINO layout (needs N%16==0, K%128==0, G%128==0 or 4-bit weights with G of 32 or 64)");
    if (!w || !scales || !w_tiled || !scale_tiled || (L.zp_table && (!zp || !zp_tiled)))
        return ovfcc::fail(OVFCC_EINVAL, "null buffer");
    ovfcc::OutputMajorCopy nk;
    if (desc->flags & OVFCC_W_INPUT_MAJOR) {
        ovfcc::transpose_input_major(*desc, w, scales, zp, &nk);
        w = nk.w.data(), scales = nk.scales.data(), zp = nk.zp.empty() ? zp : nk.zp.data();
    }
    ovfcc::repack_weights(*desc, L, w, w_tiled);
    ovfcc::repack_params(*desc, L, scales, zp, scale_tiled, zp_tiled);
    return OVFCC_OK;
}

int ovfcc_unrepack_host(const ovfcc_fc_desc* desc, const void* w_tiled, const void* scale_tiled, const void* zp_tiled,
                        void* w, void* scales, void* zp) {
    int rc = ovfcc::validate_desc(desc);
    if (rc != OVFCC_OK)
        return rc;
    if (desc->flags & OVFCC_W_INPUT_MAJOR)
        return ovfcc::fail(OVFCC_EINVAL, "tiles unpack to the [N, K] order; clear OVFCC_W_INPUT_MAJOR");
    const ovfcc::Layout L = ovfcc::make_layout(*desc);
    if (!L.tiled)
        return ovfcc::fail(OVFCC_EUNSUPPORTED, "shape keeps the OpenVINO layout (needs N%16==0, K%128==0, G%128==0 or 4-bit weights with G of 32 or 64)");
    if (!w || !scales || !w_tiled || !scale_tiled || (L.zp_table && (!zp || !zp_tiled)))
        return ovfcc::fail(OVFCC_EINVAL, "null buffer");
    ovfcc::unrepack_weights(*desc, L, w_tiled, w);
    ovfcc::unrepack_params(*desc, L, scale_tiled, zp_tiled, scales, zp);
    return OVFCC_OK;
}

int ovfcc_unpack_u4(const void* src, size_t n, uint8_t* dst) {
    if ((!src || !dst) && n)
        return ovfcc::fail(OVFCC_EINVAL, "null buffer");
    const uint8_t* p = static_cast<const uint8_t*>(src);
    for (size_t i = 0; i < n; ++i)
        dst[i] = (uint8_t)ovfcc::nibble(p, i);
    return OVFCC_OK;
}

int ovfcc_unpack_i4(const void* src, size_t n, int8_t* dst) {
    if ((!src || !dst) && n)
        return ovfcc::fail(OVFCC_EINVAL, "null buffer");
    const uint8_t* p = static_cast<const uint8_t*>(src);
    for (size_t i = 0; i < n; ++i) {
        const int v = (int)ovfcc::nibble(p, i);
        dst[i] = (int8_t)(v >= 8 ? v - 16 : v);
    }
    return OVFCC_OK;
}

}  // extern "C"
