/*
 * CPU oracle for the weight-compressed FullyConnected path.
 *
 * TEST INFRASTRUCTURE ONLY.  This file restates, in plain C, the arithmetic the
 * OpenVINO reference performs for FullyConnectedCompressed.  It is linked only by
 * the tests, by the smoke check and by the benchmark's cpu_baseline leg; the
 * product library never calls it.
 *
 * Reference files restated (paths relative to the OpenVINO source tree):
 *   - nibble order of u4/i4 buffers, sign extension of i4:
 *       src/core/dev_api/openvino/core/type/element_iterator.hpp:76,161-176,248-259
 *   - IEEE binary16 <-> binary32, round-to-nearest-even:
 *       src/core/src/type/float16.cpp:32-110 (to half), :112-140 (to float)
 *   - per-element FullyConnected-with-decompression formula
 *       y[m,n] = sum_k x[m,k] * ((q[n,k] - zp[n,k/G]) * s[n,k/G]) (+ bias[n]):
 *       src/plugins/intel_gpu/src/kernel_selector/cl_kernels/fully_connected_gpu_bfyx_ref.cl:88-160
 *   - weights are [N,K] (MatMul with transpose_b = true):
 *       src/common/transformations/src/ov_ops/fully_connected.cpp:40-57
 *   - the dot product itself is the textbook triple loop of
 *       src/core/reference/include/openvino/reference/matmul.hpp:19-46
 *
 * How each function is pinned (see tests/test_oracle_*.py):
 *   unpack/pack      known-answer bytes of src/core/tests/element_iterator_test.cpp,
 *                    uint4.cpp, int4.cpp; the reference's own element_iterator.hpp
 *                    compiled into oracle/_ref where the reference tree is present
 *   f16 conversion   exhaustive 65536-pattern round trip + numpy.float16 on random and
 *                    edge values; the reference's float16.cpp compiled into oracle/_ref
 *   fc_reference     exact golden vectors of fully_connected_gpu_test.cpp
 *                    (:1425-1481, :2842-2909, :3014-3066, :3068-3119, :3121-3180,
 *                    :1819-1877), an independent numpy float64 restatement, and
 *                    algebraic invariants (zp == q gives 0, scale linearity, unit-vector
 *                    probes, i4 == u4 xor 8 with zp 8, row permutation)
 *
 *   glu              the stand-alone formula of the Intel-GPU plugin,
 *                    src/plugins/intel_gpu/src/kernel_selector/cl_kernels/swiglu_gpu_ref.cl:46-90
 *                    (split form, GATE_IDX, the three GLU_TYPEs), the op's attributes
 *                    src/common/transformations/include/ov_ops/glu.hpp:16-40 and the host
 *                    restatement in the reference's own test,
 *                    src/plugins/intel_gpu/tests/unit/test_cases/swiglu_gpu_test.cpp:55-72.
 *                    The reference holds no numeric vector for it (its tests recompute the
 *                    formula); pinned against library routines (torch silu / gelu, exact and
 *                    tanh form), the identities act(x) - act(-x) = x, act(0) = 0, and the
 *                    roles of the two halves on one-hot inputs.
 *
 *   dynquant         per-token symmetric int8 quantisation of activations and the integer
 *                    FullyConnected on top of it, as the Intel-GPU plugin does for large batches:
 *                    src/plugins/intel_gpu/src/kernel_selector/cl_kernels/dynamic_quantize_gpu_ref.cl:100-250
 *                    (max |x| clamped below at 0.003, scale = 127 / max in half, q = rte(half(x * scale)),
 *                    stored scale 1 / scale, sum of q), fully_connected_gpu_bf_tiled.cl:1283-1284
 *                    ((acc - zp * sum) * weight scale * stored scale); attributes
 *                    src/common/transformations/include/ov_ops/dynamic_quantize.hpp:16-60.  The reference
 *                    holds no numeric vector for it (its tests compare against the unquantised result with
 *                    absolute tolerances 0.1-0.2).  Pinned by: exact round trip on rows that are integer
 *                    multiples of max / 127; |x - q * stored scale| <= stored scale / 2 (+ half rounding);
 *                    sum and range of q; an independent numpy restatement; and, for the FC, equality with
 *                    ovo_fc_reference applied to the dequantised activations q * stored scale.
 *
 *   dynquant_asym    the same with the reference's asymmetric form (unsigned 8-bit activations, a zero-point per
 *                    token): dynamic_quantize_gpu_ref.cl:100-250 under ASYMMETRIC_QUANTIZATION and UNSIGNED_OUTPUT
 *                    (d = max - min in half, 0.003 if equal; scale = half(255 / d); zp = half(-min * (255 / d));
 *                    q = convert_uchar_rte(half(x * scale) + zp); stored scale 1 / scale; stored zero-point
 *                    convert_uchar_rte(zp)), chosen by src/plugins/intel_gpu/src/plugin/transformations/
 *                    dynamic_quantize_fully_connected.cpp:109-117 and consumed as the source zero-point of the
 *                    product (graph/impls/onednn/fully_connected_onednn.cpp:83-88,325-329; oneDNN itself is a
 *                    third-party dependency absent from the tree: its documented meaning, src = (q - zp) * scale,
 *                    is what is restated).  The conversions saturate here where OpenCL leaves them undefined.
 *                    The reference holds no numeric vector for it (its test compares two of its own kernels on
 *                    inputs in [-16, 20]).  Pinned by: minimum -> 0 and maximum -> 255 on rows that straddle zero;
 *                    |x - (q - za) * stored scale| bounded by half a step plus the half roundings; a constant row
 *                    (d = 0.003); an independent numpy restatement in numpy's own half arithmetic; and, for the
 *                    FC, equality with ovo_fc_reference applied to the dequantised activations (q - za) * stored
 *                    scale (which fixes every cross term of the integer form).
 *
 * Parity unpinned: the CPU plugin's numbers come from the oneDNN fork's decompression
 * inner-product kernel (openvinotoolkit/oneDNN, a submodule whose commit the tree does
 * not record and whose sources are absent).  Its summation order and intermediate
 * roundings are not restated here; the reference's own tests hold only tolerance checks
 * at that boundary, and so does this oracle's use (fp32 accumulation in k order).
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

/* element type tags shared with oracle.py */
enum {
    OVO_NONE = 0,
    OVO_U4 = 1,
    OVO_I4 = 2,
    OVO_U8 = 3,
    OVO_I8 = 4,
    OVO_F16 = 5,
    OVO_F32 = 6
};

/* ---- 4-bit packing: element i lives in byte i/2, low nibble when i is even ---- */

static inline uint8_t nibble_at(const uint8_t* bytes, size_t i) {
    uint8_t b = bytes[i >> 1];
    return (i & 1) ? (uint8_t)(b >> 4) : (uint8_t)(b & 0x0F);
}

static inline int8_t sext4(uint8_t v) {
    return (int8_t)((v & 0x8) ? (int)v - 16 : (int)v);
}

void ovo_unpack_u4(const uint8_t* src, size_t n, uint8_t* dst) {
    for (size_t i = 0; i < n; ++i)
        dst[i] = nibble_at(src, i);
}

void ovo_unpack_i4(const uint8_t* src, size_t n, int8_t* dst) {
    for (size_t i = 0; i < n; ++i)
        dst[i] = sext4(nibble_at(src, i));
}

/* dst has (n+1)/2 bytes; a trailing unused high nibble is left zero */
void ovo_pack_u4(const uint8_t* src, size_t n, uint8_t* dst) {
    memset(dst, 0, (n + 1) / 2);
    for (size_t i = 0; i < n; ++i) {
        uint8_t v = (uint8_t)(src[i] & 0x0F);
        dst[i >> 1] |= (i & 1) ? (uint8_t)(v << 4) : v;
    }
}

void ovo_pack_i4(const int8_t* src, size_t n, uint8_t* dst) {
    memset(dst, 0, (n + 1) / 2);
    for (size_t i = 0; i < n; ++i) {
        uint8_t v = (uint8_t)((uint8_t)src[i] & 0x0F);
        dst[i >> 1] |= (i & 1) ? (uint8_t)(v << 4) : v;
    }
}

/* ---- binary16 <-> binary32 ---- */

uint16_t ovo_f32_to_f16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    const uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    const uint32_t e32 = (u >> 23) & 0xFFu;
    const uint32_t m32 = u & 0x7FFFFFu;

    if (e32 == 0xFFu) { /* inf / nan: keep the top payload bits, never turn a nan into inf */
        if (m32 == 0)
            return (uint16_t)(sign | 0x7C00u);
        uint16_t payload = (uint16_t)(m32 >> 13);
        if (payload == 0)
            payload = 1;
        return (uint16_t)(sign | 0x7C00u | payload);
    }
    if (e32 == 0) /* float zero or float subnormal: far below half's smallest subnormal */
        return sign;

    const int e = (int)e32 - 127; /* unbiased */
    if (e > 15)
        return (uint16_t)(sign | 0x7C00u);

    if (e >= -14) { /* normal half unless rounding carries out */
        uint32_t mant = m32 >> 13; /* 10 kept bits */
        const uint32_t rest = m32 & 0x1FFFu;
        uint32_t h = ((uint32_t)(e + 15) << 10) | mant;
        if (rest > 0x1000u || (rest == 0x1000u && (mant & 1u)))
            h += 1; /* a carry walks into the exponent, up to inf, which is what RNE wants */
        return (uint16_t)(sign | h);
    }

    /* subnormal half: value = full * 2^(e-23), target unit 2^-24 */
    if (e < -25)
        return sign; /* below half of the smallest subnormal */
    const uint32_t full = m32 | 0x800000u;
    const int shift = -e - 1; /* 14..24 */
    uint32_t mant = full >> shift;
    const uint32_t rest = full & ((1u << shift) - 1u);
    const uint32_t half = 1u << (shift - 1);
    if (rest > half || (rest == half && (mant & 1u)))
        mant += 1; /* may become 0x400 = smallest normal, encoded correctly */
    return (uint16_t)(sign | mant);
}

float ovo_f16_to_f32(uint16_t h) {
    const uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    const uint32_t e = (h >> 10) & 0x1Fu;
    uint32_t m = h & 0x3FFu;
    uint32_t u;
    if (e == 0x1Fu) {
        u = sign | 0x7F800000u | (m << 13);
    } else if (e != 0) {
        u = sign | ((e + 112u) << 23) | (m << 13);
    } else if (m == 0) {
        u = sign;
    } else { /* subnormal: renormalise */
        int k = 0;
        while (!(m & 0x400u)) {
            m <<= 1;
            ++k;
        }
        u = sign | ((uint32_t)(113 - k) << 23) | ((m & 0x3FFu) << 13);
    }
    float f;
    memcpy(&f, &u, 4);
    return f;
}

void ovo_f32_to_f16_n(const float* src, size_t n, uint16_t* dst) {
    for (size_t i = 0; i < n; ++i)
        dst[i] = ovo_f32_to_f16(src[i]);
}

void ovo_f16_to_f32_n(const uint16_t* src, size_t n, float* dst) {
    for (size_t i = 0; i < n; ++i)
        dst[i] = ovo_f16_to_f32(src[i]);
}

/* ---- FullyConnected with weight decompression ---- */

typedef struct {
    int64_t M, N, K;
    int64_t group_size;  /* along K; == K for per-output-channel parameters */
    int32_t w_type;      /* OVO_U4 / OVO_I4 / OVO_U8 / OVO_I8, row-major [N,K] */
    int32_t scale_type;  /* OVO_F16 / OVO_F32, [N, K/group_size] */
    int32_t zp_type;     /* OVO_NONE / OVO_U4 / OVO_U8 / OVO_F32, [N, K/group_size] or one element */
    int32_t zp_scalar;   /* non-zero: zp holds exactly one element used everywhere */
    int32_t bias_type;   /* OVO_NONE / OVO_F16 / OVO_F32, [N] */
    int32_t x_type;      /* OVO_F16 / OVO_F32, [M,K] */
    int32_t acc_f64;     /* 0: float accumulator, k ascending (the reference kernel's order); 1: double */
    int32_t reserved;
    const void* w;
    const void* scale;
    const void* zp;
    const void* bias;
    const void* x;
    const int64_t* n_index; /* optional subset of output channels (NULL = all) */
    int64_t n_count;        /* length of n_index; y is then [M, n_count] */
} ovo_fc_args;

static inline float load_real(const void* p, int32_t type, size_t i) {
    if (type == OVO_F32)
        return ((const float*)p)[i];
    return ovo_f16_to_f32(((const uint16_t*)p)[i]);
}

static inline float load_weight(const void* w, int32_t type, size_t i) {
    switch (type) {
    case OVO_U4: return (float)nibble_at((const uint8_t*)w, i);
    case OVO_I4: return (float)sext4(nibble_at((const uint8_t*)w, i));
    case OVO_U8: return (float)((const uint8_t*)w)[i];
    default:     return (float)((const int8_t*)w)[i];
    }
}

static inline float load_zp(const void* zp, int32_t type, size_t i) {
    switch (type) {
    case OVO_NONE: return 0.0f;
    case OVO_U4:   return (float)nibble_at((const uint8_t*)zp, i);
    case OVO_U8:   return (float)((const uint8_t*)zp)[i];
    default:       return ((const float*)zp)[i];
    }
}

/* Returns 0 on success, a negative number naming the bad argument otherwise.
 * y is float [M, n_count or N]; bias is added after the accumulation, before any output cast
 * (fully_connected_gpu_bfyx_ref.cl:139-156); the cast to the output type is the caller's. */
int ovo_fc_reference(const ovo_fc_args* a, float* y) {
    if (!a || !y || !a->w || !a->scale || !a->x) return -1;
    if (a->M < 0 || a->N <= 0 || a->K <= 0) return -2;
    if (a->group_size <= 0 || a->K % a->group_size) return -3;
    if (a->w_type < OVO_U4 || a->w_type > OVO_I8) return -4;
    if (a->scale_type != OVO_F16 && a->scale_type != OVO_F32) return -5;
    if (a->zp_type != OVO_NONE && a->zp_type != OVO_U4 && a->zp_type != OVO_U8 && a->zp_type != OVO_F32) return -6;
    if (a->zp_type != OVO_NONE && !a->zp) return -6;
    if (a->bias_type != OVO_NONE && a->bias_type != OVO_F16 && a->bias_type != OVO_F32) return -7;
    if (a->bias_type != OVO_NONE && !a->bias) return -7;
    if (a->x_type != OVO_F16 && a->x_type != OVO_F32) return -8;

    const int64_t M = a->M, N = a->N, K = a->K, G = a->group_size, ng = K / G;
    const int64_t ncols = a->n_index ? a->n_count : N;
    int status = 0;

    /* activations as float, converted once */
    float* xf = (float*)__builtin_malloc((size_t)(M > 0 ? M : 1) * (size_t)K * sizeof(float));
    if (!xf) return -10;
    for (int64_t i = 0; i < M * K; ++i)
        xf[i] = load_real(a->x, a->x_type, (size_t)i);

#pragma omp parallel
    {
        float* wrow = (float*)__builtin_malloc((size_t)K * sizeof(float));
#pragma omp for schedule(dynamic, 4)
        for (int64_t c = 0; c < ncols; ++c) {
            const int64_t n = a->n_index ? a->n_index[c] : c;
            if (n < 0 || n >= N || !wrow) {
                status = -9;
                continue;
            }
            /* dequantise one weight row: (q - zp) * s, all in float */
            for (int64_t k = 0; k < K; ++k) {
                const int64_t g = k / G;
                const float q = load_weight(a->w, a->w_type, (size_t)(n * K + k));
                const float z = load_zp(a->zp, a->zp_type, a->zp_scalar ? 0 : (size_t)(n * ng + g));
                const float s = load_real(a->scale, a->scale_type, (size_t)(n * ng + g));
                wrow[k] = (q - z) * s;
            }
            const float b = a->bias_type == OVO_NONE ? 0.0f : load_real(a->bias, a->bias_type, (size_t)n);
            for (int64_t m = 0; m < M; ++m) {
                const float* xrow = xf + m * K;
                if (a->acc_f64) {
                    double acc = 0.0;
                    for (int64_t k = 0; k < K; ++k)
                        acc += (double)xrow[k] * (double)wrow[k];
                    y[m * ncols + c] = (float)(acc + (double)b);
                } else {
                    float acc = 0.0f;
                    for (int64_t k = 0; k < K; ++k)
                        acc += xrow[k] * wrow[k];
                    y[m * ncols + c] = acc + b;
                }
            }
        }
        __builtin_free(wrow);
    }
    __builtin_free(xf);
    return status;
}

/* Gated linear unit over the last axis of y [M, 2 L]: out[m, f] = act(y[m, g + f]) * y[m, u + f] with
 * (g, u) = (0, L), or (L, 0) when gate_second (the op's split_to_glu_idx = 1).  type: 1 Swish (beta = 1),
 * 2 Gelu (erf), 3 Gelu_Tanh.  Evaluated in double, returned as float. */
int ovo_glu(const float* y, int64_t M, int64_t L, int32_t type, int32_t gate_second, float* out) {
    if (!y || !out || M < 0 || L <= 0 || type < 1 || type > 3)
        return -1;
    const int64_t g0 = gate_second ? L : 0, u0 = gate_second ? 0 : L;
    for (int64_t m = 0; m < M; ++m)
        for (int64_t f = 0; f < L; ++f) {
            const double gate = y[m * 2 * L + g0 + f], up = y[m * 2 * L + u0 + f];
            double a;
            if (type == 1)
                a = gate / (1.0 + exp(-gate));
            else if (type == 2)
                a = 0.5 * gate * (1.0 + erf(gate * 0.70710678118654752440));
            else
                a = 0.5 * gate * (1.0 + tanh(0.79788456080286535588 * gate * (1.0 + 0.044715 * gate * gate)));
            out[m * L + f] = (float)(a * up);
        }
    return 0;
}

/* Per-token symmetric int8 quantisation of x [M, K] (f16 bit patterns): q [M, K], inv_scale [M] (the f16 value
 * the reference stores, returned as float), qsum [M] = sum_k q.  Half arithmetic as in the reference kernel:
 * max and product are exact half operations; 127 / max is one f32 division rounded to half, which equals the half
 * division (a quotient of two 11-bit significands cannot lie within 2^-24 of a 12-bit tie). */
int ovo_dynquant_rows(const uint16_t* x, int64_t M, int64_t K, int8_t* q, float* inv_scale, int32_t* qsum) {
    if (!x || !q || !inv_scale || !qsum || M < 0 || K <= 0)
        return -1;
    for (int64_t m = 0; m < M; ++m) {
        float mx = ovo_f16_to_f32(ovo_f32_to_f16(0.003f));
        for (int64_t k = 0; k < K; ++k) {
            const float a = fabsf(ovo_f16_to_f32(x[m * K + k]));
            if (a > mx)
                mx = a;
        }
        const float scale = ovo_f16_to_f32(ovo_f32_to_f16(127.0f / mx));
        int32_t sum = 0;
        for (int64_t k = 0; k < K; ++k) {
            const float v = ovo_f16_to_f32(ovo_f32_to_f16(ovo_f16_to_f32(x[m * K + k]) * scale));
            const float r = nearbyintf(v);  /* round to nearest even, the default mode */
            const int32_t i = (int32_t)(r > 127.f ? 127.f : (r < -128.f ? -128.f : r));
            q[m * K + k] = (int8_t)i;
            sum += i;
        }
        inv_scale[m] = ovo_f16_to_f32(ovo_f32_to_f16(1.0f / scale));
        qsum[m] = sum;
    }
    return 0;
}

/* FullyConnected over dynamically quantised activations, 8-bit weights, one scale (and zero-point) per output
 * channel: y[m, n] = (sum_k q[m, k] w[n, k] - zp[n] qsum[m]) * (scale[n] * inv_scale[m]) (+ bias[n]), integers
 * exact, the rest in f32.  w_signed: weights are i8 instead of u8.  zp may be null (0), bias may be null. */
int ovo_fc_dynquant_reference(const int8_t* q, const float* inv_scale, const int32_t* qsum, int64_t M, int64_t K,
                              int64_t N, const uint8_t* w, int32_t w_signed, const float* scale, const float* zp,
                              const float* bias, float* y) {
    if (!q || !inv_scale || !qsum || !w || !scale || !y || M < 0 || K <= 0 || N <= 0)
        return -1;
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; ++n)
        for (int64_t m = 0; m < M; ++m) {
            int64_t acc = 0;
            for (int64_t k = 0; k < K; ++k) {
                const int32_t wv = w_signed ? (int32_t)(int8_t)w[n * K + k] : (int32_t)w[n * K + k];
                acc += (int32_t)q[m * K + k] * wv;
            }
            acc -= (int64_t)(zp ? (int32_t)zp[n] : 0) * qsum[m];
            y[m * N + n] = (float)(int32_t)acc * (scale[n] * inv_scale[m]) + (bias ? bias[n] : 0.f);
        }
    return 0;
}

/* double -> f16 bits, round to nearest even (the exact sum of two halves fits a double; rounding it through float
 * first could round twice). */
static uint16_t ovo_f64_to_f16(double v) {
    if (v != v)
        return 0x7E00;
    const uint16_t sign = signbit(v) ? 0x8000 : 0;
    const double a = fabs(v);
    if (a >= 65520.0)
        return (uint16_t)(sign | 0x7C00);
    if (a < 6.103515625e-05) /* below the smallest normal: a multiple of 2^-24 */
        return (uint16_t)(sign | (uint16_t)nearbyint(a * 16777216.0));
    int e;
    (void)frexp(a, &e); /* a = f * 2^e, f in [0.5, 1): exponent of a is e - 1 */
    int ex = e - 1;
    double m = nearbyint(ldexp(a, 10 - ex)); /* 1024 .. 2048 */
    if (m >= 2048.0) {
        m = 1024.0;
        ++ex;
    }
    if (ex > 15)
        return (uint16_t)(sign | 0x7C00);
    return (uint16_t)(sign | ((uint16_t)(ex + 15) << 10) | ((uint16_t)m - 1024));
}

static int32_t ovo_sat_u8_rte(float v) {
    if (v != v)
        return 0;
    const float r = nearbyintf(v);
    return (int32_t)(r > 255.f ? 255.f : (r < 0.f ? 0.f : r));
}

/* Per-token asymmetric quantisation of x [M, K] (f16 bit patterns) to unsigned bytes: q [M, K], inv_scale [M] (the
 * f16 value the reference stores, as float), za [M] the stored zero-point, qsum [M] = sum_k q.  Half arithmetic as in
 * the reference kernel: max, min exact; max - min one half subtraction; 255 / d and -min * (255 / d) in f32, each
 * rounded to half; x * scale a half product (exact in f32, rounded once); + zp a half sum (exact in double, rounded
 * once). */
int ovo_dynquant_rows_asym(const uint16_t* x, int64_t M, int64_t K, uint8_t* q, float* inv_scale, int32_t* za,
                           int32_t* qsum) {
    if (!x || !q || !inv_scale || !za || !qsum || M < 0 || K <= 0)
        return -1;
    for (int64_t m = 0; m < M; ++m) {
        float mx = -65504.f, mn = 65504.f;
        for (int64_t k = 0; k < K; ++k) {
            const float a = ovo_f16_to_f32(x[m * K + k]);
            if (a > mx)
                mx = a;
            if (a < mn)
                mn = a;
        }
        const float range = ovo_f16_to_f32(ovo_f64_to_f16((double)mx - (double)mn));
        const float diff = mx == mn ? ovo_f16_to_f32(ovo_f32_to_f16(0.003f)) : range;
        const float scale_f = 255.0f / diff;
        const float scale = ovo_f16_to_f32(ovo_f32_to_f16(scale_f));
        const float zp = ovo_f16_to_f32(ovo_f32_to_f16(-mn * scale_f));
        int32_t sum = 0;
        for (int64_t k = 0; k < K; ++k) {
            const float p = ovo_f16_to_f32(ovo_f32_to_f16(ovo_f16_to_f32(x[m * K + k]) * scale));
            const float v = ovo_f16_to_f32(ovo_f64_to_f16((double)p + (double)zp));
            const int32_t i = ovo_sat_u8_rte(v);
            q[m * K + k] = (uint8_t)i;
            sum += i;
        }
        inv_scale[m] = ovo_f16_to_f32(ovo_f32_to_f16(1.0f / scale));
        za[m] = ovo_sat_u8_rte(zp);
        qsum[m] = sum;
    }
    return 0;
}

/* FullyConnected over asymmetrically quantised activations, 8-bit weights, one scale (and zero-point) per output
 * channel: y[m, n] = sum_k (q[m, k] - za[m]) (w[n, k] - zp[n]) * (scale[n] * inv_scale[m]) (+ bias[n]), the sum
 * exact, the rest in f32.  w_signed: weights are i8 instead of u8.  zp may be null (0), bias may be null. */
int ovo_fc_dynquant_asym_reference(const uint8_t* q, const float* inv_scale, const int32_t* za, int64_t M, int64_t K,
                                   int64_t N, const uint8_t* w, int32_t w_signed, const float* scale, const float* zp,
                                   const float* bias, float* y) {
    if (!q || !inv_scale || !za || !w || !scale || !y || M < 0 || K <= 0 || N <= 0)
        return -1;
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; ++n)
        for (int64_t m = 0; m < M; ++m) {
            const int32_t zw = zp ? (int32_t)zp[n] : 0;
            int64_t acc = 0;
            for (int64_t k = 0; k < K; ++k) {
                const int32_t wv = w_signed ? (int32_t)(int8_t)w[n * K + k] : (int32_t)w[n * K + k];
                acc += (int64_t)((int32_t)q[m * K + k] - za[m]) * (wv - zw);
            }
            y[m * N + n] = (float)(int32_t)acc * (scale[n] * inv_scale[m]) + (bias ? bias[n] : 0.f);
        }
    return 0;
}

/* The same quantisation over groups of G consecutive inputs of a row instead of whole rows (the reference's
 * DynamicQuantize with group_sizes = {1, .., G}, src/plugins/intel_gpu/src/kernel_selector/cl_kernels/
 * dynamic_quantize_gpu_ref.cl:100-250 with GROUP_SIZE_DIM3 = G; on the CPU the source group of
 * src/plugins/intel_cpu/src/nodes/executors/dnnl/dnnl_fullyconnected_primitive.cpp:161-241,284-298):
 * q [M, K], inv_scale [M, K / G], qsum [M, K / G].  G = K is ovo_dynquant_rows. */
int ovo_dynquant_groups(const uint16_t* x, int64_t M, int64_t K, int64_t G, int8_t* q, float* inv_scale,
                        int32_t* qsum) {
    if (!x || !q || !inv_scale || !qsum || M < 0 || K <= 0 || G <= 0 || K % G)
        return -1;
    /* a [M, K] matrix cut into groups of G along K is a [M K / G, G] matrix cut into rows */
    return ovo_dynquant_rows(x, M * (K / G), G, q, inv_scale, qsum);
}

/* FullyConnected over activations quantised in groups of Ga inputs, 4- or 8-bit weights with scales (and
 * zero-points) per group of Gw inputs; Ga and Gw divide K and one of them divides the other.  With
 * g = min(Ga, Gw):
 *     y[m, n] = sum_blocks-of-g ( sum_{k in block} q[m, k] (w[n, k] - zp[n, k / Gw]) ) * scale[n, k / Gw]
 *               * inv_scale[m, k / Ga]  (+ bias[n]),
 * the integer sums exact, the sum over blocks in double.  w holds one code per byte ([N, K], already unpacked;
 * w_signed: two's complement), zp one value per (n, group) or null (0); scale [N, K / Gw] f32. */
int ovo_fc_dynquant_grouped_reference(const int8_t* q, const float* inv_scale, int64_t M, int64_t K, int64_t Ga,
                                      int64_t N, const uint8_t* w, int32_t w_signed, int64_t Gw, const float* scale,
                                      const float* zp, const float* bias, float* y) {
    if (!q || !inv_scale || !w || !scale || !y || M < 0 || K <= 0 || N <= 0 || Ga <= 0 || Gw <= 0 || K % Ga || K % Gw ||
        (Ga % Gw && Gw % Ga))
        return -1;
    const int64_t g = Ga < Gw ? Ga : Gw, nga = K / Ga, ngw = K / Gw;
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; ++n)
        for (int64_t m = 0; m < M; ++m) {
            double sum = 0.0;
            for (int64_t k0 = 0; k0 < K; k0 += g) {
                const int32_t z = zp ? (int32_t)zp[n * ngw + k0 / Gw] : 0;
                int64_t acc = 0;
                for (int64_t k = k0; k < k0 + g; ++k) {
                    const int32_t wv = w_signed ? (int32_t)(int8_t)w[n * K + k] : (int32_t)w[n * K + k];
                    acc += (int32_t)q[m * K + k] * (wv - z);
                }
                sum += (double)acc * ((double)scale[n * ngw + k0 / Gw] * (double)inv_scale[m * nga + k0 / Ga]);
            }
            y[m * N + n] = (float)(sum + (bias ? (double)bias[n] : 0.0));
        }
    return 0;
}

int ovo_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

void ovo_set_num_threads(int n) {
#ifdef _OPENMP
    if (n > 0) omp_set_num_threads(n);
#else
    (void)n;
#endif
}
