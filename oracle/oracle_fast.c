/* TEST / BENCHMARK INFRASTRUCTURE ONLY -- never linked into or loaded by the product.
 *
 * A faster CPU statement of the same FullyConnected with weight decompression as ovo_fc_reference
 * (oracle.c), used as the CPU baseline that the benchmark times beside the GPU figures: what a
 * straightforward blocked, vectorised host implementation reaches on the box's cores.  The reference's
 * own CPU path for this node is a oneDNN brgemm JIT kernel (src/plugins/intel_cpu/src/nodes/executors/
 * dnnl/dnnl_fullyconnected_primitive.cpp:243-301 creates it; oneDNN itself is a submodule that the
 * reference tree here does not hold), so this is a port of the algorithm -- dequantise (q - zp) * s in
 * float, accumulate in float, add the bias -- not the reference's code.
 *
 * Differences from ovo_fc_reference: the sum over k runs in 16 interleaved partial sums per output
 * (so that it vectorises without reassociation flags) and uses fused multiply-add; results agree with the
 * oracle to f32 summation-order effects (checked in tests/test_oracle_fast.py), not bit for bit.
 * Few rows (M <= 4): one pass over the weights, every row dequantised once and used for all rows.
 * Many rows: blocks of 32 channels are dequantised into a float panel that stays in cache and is then
 * multiplied with all rows by a 4 x 4 register-blocked micro-kernel.
 */
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define OVO_NONE 0
#define OVO_U4 1
#define OVO_I4 2
#define OVO_U8 3
#define OVO_I8 4
#define OVO_F16 5
#define OVO_F32 6

typedef struct {
    int64_t M, N, K;
    int64_t group_size;
    int32_t w_type, scale_type, zp_type, zp_scalar, bias_type, x_type, acc_f64, reserved;
    const void* w;
    const void* scale;
    const void* zp;
    const void* bias;
    const void* x;
    const int64_t* n_index;
    int64_t n_count;
} ovo_fc_args; /* the layout of oracle.c's struct */

float ovo_f16_to_f32(uint16_t h); /* oracle.c */

#define LANES 16
#define HOT __attribute__((target_clones("default", "avx2,fma", "avx512f")))

static inline float real_at(const void* p, int32_t type, size_t i) {
    return type == OVO_F32 ? ((const float*)p)[i] : ovo_f16_to_f32(((const uint16_t*)p)[i]);
}

static inline float zp_at(const ovo_fc_args* a, size_t i) {
    if (a->zp_type == OVO_NONE)
        return 0.f;
    if (a->zp_scalar)
        i = 0;
    if (a->zp_type == OVO_U4) {
        const uint8_t b = ((const uint8_t*)a->zp)[i >> 1];
        return (float)((i & 1) ? (b >> 4) : (b & 15));
    }
    if (a->zp_type == OVO_U8)
        return (float)((const uint8_t*)a->zp)[i];
    return ((const float*)a->zp)[i];
}

/* codes of `count` consecutive elements starting at element index i0 (even for 4-bit types), as float */
HOT static void codes_to_float(const void* w, int32_t type, size_t i0, int64_t count, float* out) {
    if (type == OVO_U4 || type == OVO_I4) {
        const uint8_t* p = (const uint8_t*)w + (i0 >> 1);
        if (type == OVO_U4) {
            for (int64_t j = 0; j < count / 2; ++j) {
                out[2 * j] = (float)(p[j] & 15);
                out[2 * j + 1] = (float)(p[j] >> 4);
            }
        } else {
            for (int64_t j = 0; j < count / 2; ++j) {
                out[2 * j] = (float)((int8_t)(p[j] << 4) >> 4);
                out[2 * j + 1] = (float)((int8_t)p[j] >> 4);
            }
        }
    } else if (type == OVO_U8) {
        const uint8_t* p = (const uint8_t*)w + i0;
        for (int64_t j = 0; j < count; ++j)
            out[j] = (float)p[j];
    } else {
        const int8_t* p = (const int8_t*)w + i0;
        for (int64_t j = 0; j < count; ++j)
            out[j] = (float)p[j];
    }
}

/* row n dequantised: out[k] = (q - zp) * s */
HOT static void dequantise_row(const ovo_fc_args* a, int64_t n, float* out) {
    const int64_t K = a->K, G = a->group_size, ng = K / G;
    codes_to_float(a->w, a->w_type, (size_t)(n * K), K, out);
    for (int64_t g = 0; g < ng; ++g) {
        const float s = real_at(a->scale, a->scale_type, (size_t)(n * ng + g));
        const float z = zp_at(a, (size_t)(n * ng + g));
        float* o = out + g * G;
        for (int64_t k = 0; k < G; ++k)
            o[k] = (o[k] - z) * s;
    }
}

HOT static float dot(const float* x, const float* w, int64_t K) {
    float acc[LANES] = {0};
    int64_t k = 0;
    for (; k + LANES <= K; k += LANES)
        for (int j = 0; j < LANES; ++j)
            acc[j] += x[k + j] * w[k + j];
    float s = 0.f;
    for (int j = 0; j < LANES; ++j)
        s += acc[j];
    for (; k < K; ++k)
        s += x[k] * w[k];
    return s;
}

/* 4 rows x 4 channels at once: 16 outputs, each 16 partial sums wide */
HOT static void micro_4x4(const float* x, int64_t ldx, const float* w, int64_t ldw, int64_t K, float* out /* [4][4] */) {
    float acc[4][4][LANES];
    memset(acc, 0, sizeof(acc));
    int64_t k = 0;
    for (; k + LANES <= K; k += LANES)
        for (int m = 0; m < 4; ++m)
            for (int n = 0; n < 4; ++n)
                for (int j = 0; j < LANES; ++j)
                    acc[m][n][j] += x[m * ldx + k + j] * w[n * ldw + k + j];
    for (int m = 0; m < 4; ++m)
        for (int n = 0; n < 4; ++n) {
            float s = 0.f;
            for (int j = 0; j < LANES; ++j)
                s += acc[m][n][j];
            for (int64_t kk = k; kk < K; ++kk)
                s += x[m * ldx + kk] * w[n * ldw + kk];
            out[m * 4 + n] = s;
        }
}

#define PANEL 32 /* channels dequantised together for the many-row case */

/* Same arguments and result layout as ovo_fc_reference (n_index is not supported: all channels).  4-bit weights
 * need an even K.  Returns 0, or a negative number naming the bad argument. */
int ovo_fc_blocked(const ovo_fc_args* a, float* y) {
    if (!a || !y || !a->w || !a->scale || !a->x) return -1;
    if (a->M < 0 || a->N <= 0 || a->K <= 0) return -2;
    if (a->group_size <= 0 || a->K % a->group_size) return -3;
    if (a->w_type < OVO_U4 || a->w_type > OVO_I8) return -4;
    if ((a->w_type == OVO_U4 || a->w_type == OVO_I4) && (a->K & 1)) return -4;
    if (a->zp_type != OVO_NONE && !a->zp) return -6;
    if (a->bias_type != OVO_NONE && !a->bias) return -7;
    if (a->n_index) return -9;
    const int64_t M = a->M, N = a->N, K = a->K;
    float* xf = (float*)malloc((size_t)(M > 0 ? M : 1) * (size_t)K * sizeof(float));
    if (!xf) return -10;
    for (int64_t i = 0; i < M * K; ++i)
        xf[i] = real_at(a->x, a->x_type, (size_t)i);
    int status = 0;
    const int64_t panels = (N + PANEL - 1) / PANEL;
#pragma omp parallel
    {
        float* wp = (float*)malloc((size_t)PANEL * (size_t)K * sizeof(float));
#pragma omp for schedule(dynamic, 1)
        for (int64_t p = 0; p < panels; ++p) {
            if (!wp) {
                status = -10;
                continue;
            }
            const int64_t n0 = p * PANEL, nn = N - n0 < PANEL ? N - n0 : PANEL;
            for (int64_t i = 0; i < nn; ++i)
                dequantise_row(a, n0 + i, wp + i * K);
            int64_t m = 0;
            for (; m + 4 <= M; m += 4) {
                int64_t i = 0;
                for (; i + 4 <= nn; i += 4) {
                    float o[16];
                    micro_4x4(xf + m * K, K, wp + i * K, K, K, o);
                    for (int mm = 0; mm < 4; ++mm)
                        for (int ii = 0; ii < 4; ++ii)
                            y[(m + mm) * N + n0 + i + ii] = o[mm * 4 + ii];
                }
                for (; i < nn; ++i)
                    for (int mm = 0; mm < 4; ++mm)
                        y[(m + mm) * N + n0 + i] = dot(xf + (m + mm) * K, wp + i * K, K);
            }
            for (; m < M; ++m)
                for (int64_t i = 0; i < nn; ++i)
                    y[m * N + n0 + i] = dot(xf + m * K, wp + i * K, K);
            if (a->bias_type != OVO_NONE)
                for (int64_t i = 0; i < nn; ++i) {
                    const float b = real_at(a->bias, a->bias_type, (size_t)(n0 + i));
                    for (int64_t mm = 0; mm < M; ++mm)
                        y[mm * N + n0 + i] += b;
                }
        }
        free(wp);
    }
    free(xf);
    return status;
}
