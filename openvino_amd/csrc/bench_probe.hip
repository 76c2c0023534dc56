// Benchmark probes (no part of the FullyConnected path): what a graph node costs with nothing in it, how fast the
// matrix cores run a loop of nothing but v_mfma_f32_16x16x32_f16 (the chip lowers its clock under that load, so
// the figure lies below the nominal peak), and how
// fast a bare streaming kernel -- loads only, the access pattern of the decode kernels, no arithmetic, no
// reduction, no store -- reads a buffer of a given size under graph replay.  The decode kernels are measured
// against these: a node cannot finish sooner than an empty one starts and stops, nor move its weights faster
// than a kernel that does nothing else.
#include "bench_probe.h"
#include "device_common.h"

namespace ovfcc {

// Plain 128-bit copy: the yardstick for bandwidth figures and for the scaling of the HBM traffic counters.
__global__ __launch_bounds__(256) void fcc_copy_kernel(uint4_t* __restrict__ dst, const uint4_t* __restrict__ src,
                                                       size_t n16) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n16; i += stride)
        dst[i] = __builtin_nontemporal_load(src + i);
}

int launch_copy(void* dst, const void* src, size_t bytes, void* stream) {
    const size_t n16 = bytes / 16;
    hipLaunchKernelGGL(fcc_copy_kernel, dim3(256 * 8), dim3(256), 0, static_cast<hipStream_t>(stream), (uint4_t*)dst,
                       (const uint4_t*)src, n16);
    return (int)hipGetLastError();
}

__global__ void fcc_empty_kernel(unsigned* out) {
    if (out && threadIdx.x == 9999)
        out[0] = 1;
}

// Workgroup g owns the 1 KiB chunks [g cpw, (g + 1) cpw); wave w reads chunks w, w + nw, ..., DEPTH in flight.
template <int DEPTH>
__global__ __launch_bounds__(1024) void fcc_stream_probe_kernel(const uint4_t* __restrict__ base, unsigned total_chunks,
                                                                unsigned cpw, unsigned* __restrict__ out) {
    const unsigned lane = threadIdx.x & 63;
    const unsigned wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const unsigned nw = blockDim.x >> 6;
    const __amdgpu_buffer_rsrc_t r =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<uint4_t*>(base), 0, total_chunks * 1024u, 0x00020000);
    const unsigned first = blockIdx.x * cpw + wave;
    const unsigned cnt = wave < cpw ? (cpw - wave + nw - 1) / nw : 0;
    uint4_t slot[DEPTH];
    auto issue = [&](unsigned i, uint4_t& s) {
        const unsigned oob = i < cnt ? 0u : 0x80000000u;
        s = __builtin_bit_cast(uint4_t, __builtin_amdgcn_raw_buffer_load_b128(r, ((first + nw * i) * 1024u + lane * 16u) | oob, 0, 2));
    };
#pragma unroll
    for (int u = 0; u < DEPTH; ++u)
        issue(u, slot[u]);
    uint4_t acc = {0, 0, 0, 0};
    for (unsigned i = 0; i < cnt; i += DEPTH) {
#pragma unroll
        for (int u = 0; u < DEPTH; ++u) {
            acc ^= slot[u];
            issue(i + u + DEPTH, slot[u]);
        }
    }
    const unsigned v = acc.x ^ acc.y ^ acc.z ^ acc.w;
    if (v == 0x12345678u)  // keeps the loads alive; the buffers never hold this pattern
        out[0] = v;
}

// Operands of the matrix-core loops: four A and four B registers sets per lane, filled from a hash of lane and index
// with halves of random sign and mantissa and magnitudes between 1/4 and 4 -- on constant operands nothing toggles
// between consecutive instructions and the chip holds a clock that no real kernel sees.
__device__ __forceinline__ half8_t probe_operand(unsigned seed) {
    Frag8 f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        unsigned h = (seed * 4u + i) * 2654435761u;
        h ^= h >> 15, h *= 2246822519u, h ^= h >> 13;
        // per half: sign, exponent 13..16 (2^-2 .. 2^1), ten random mantissa bits
        const unsigned lo = (h & 0x83FFu) | ((13u + ((h >> 10) & 3u)) << 10);
        const unsigned hi = ((h >> 16) & 0x83FFu) | ((13u + ((h >> 26) & 3u)) << 10);
        f.u[i] = lo | (hi << 16);
    }
    return f.v;
}

// Every wave runs `iters` rounds of eight independent MFMAs (eight accumulators, operands in registers, no
// memory traffic), each followed by VALU packed-f16 multiplications on registers the MFMAs do not touch.
template <int VALU>
__global__ __launch_bounds__(512) void fcc_mfma_probe_kernel(float* __restrict__ sink, int iters) {
    half8_t a[4], b[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
        a[i] = probe_operand(threadIdx.x * 8u + i), b[i] = probe_operand(threadIdx.x * 8u + 4u + i);
    float4_t acc[8];
    uint32_t r[8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
        acc[i] = float4_t{0.f, 0.f, 0.f, 0.f}, r[i] = 0x3c003c00u + (uint32_t)i;
    const uint32_t c = 0x3c003c00u;  // 1.0 in both halves
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(acc[j]) : "v"(a[j & 3]), "v"(b[(j >> 1) & 3]));
#pragma unroll
            for (int v = 0; v < VALU; ++v)
                asm volatile("v_pk_mul_f16 %0, %0, %1" : "+v"(r[(j + v) & 7]) : "v"(c));
        }
    }
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i)
        s += acc[i].x + acc[i].y + acc[i].z + acc[i].w + (float)r[i];
    sink[blockIdx.x * blockDim.x + threadIdx.x] = s;
}

// The same loop with v_mfma_f32_32x32x16_f16: four independent accumulators of sixteen registers, so that one round
// is the same matrix-core work as the eight 16 x 16 x 32 instructions above (VALU multiplications after each: twice
// as many, to keep the ratio of vector work to matrix work).
template <int VALU>
__global__ __launch_bounds__(512) void fcc_mfma32_probe_kernel(float* __restrict__ sink, int iters) {
    half8_t a[4], b[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
        a[i] = probe_operand(threadIdx.x * 8u + i), b[i] = probe_operand(threadIdx.x * 8u + 4u + i);
    float16_t acc[4];
    uint32_t r[8];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int e = 0; e < 16; ++e)
            acc[i][e] = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i)
        r[i] = 0x3c003c00u + (uint32_t)i;
    const uint32_t c = 0x3c003c00u;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(acc[j]) : "v"(a[j]), "v"(b[(j + 1) & 3]));
#pragma unroll
            for (int v = 0; v < 2 * VALU; ++v)
                asm volatile("v_pk_mul_f16 %0, %0, %1" : "+v"(r[(2 * j + v) & 7]) : "v"(c));
        }
    }
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int e = 0; e < 16; ++e)
            s += acc[i][e];
#pragma unroll
    for (int i = 0; i < 8; ++i)
        s += (float)r[i];
    sink[blockIdx.x * blockDim.x + threadIdx.x] = s;
}

// What the weight operand looks like to the matrix cores, with the activation operand random as above: PATTERN 1
// small integers -8 .. 7 as halves (a 4-bit weight minus its zero-point, unscaled), 2 the integers 0 .. 15 in the low
// mantissa bits of subnormal halves (what the decode kernels feed), 3 integers -8 .. 7 times a scale between 0.002 and
// 0.02 rounded to half (what the prefill kernels feed).  The chip's clock under this load depends on how many operand
// bits toggle.
__device__ __forceinline__ half8_t probe_weight_operand(unsigned seed, int pattern) {
    half8_t v;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        unsigned h = (seed * 8u + e) * 2654435761u;
        h ^= h >> 15, h *= 2246822519u, h ^= h >> 13;
        const int w = (int)(h & 15u);
        if (pattern == 1)
            v[e] = (half_t)(float)(w - 8);
        else if (pattern == 2)
            v[e] = __builtin_bit_cast(half_t, (uint16_t)w);
        else
            v[e] = (half_t)((float)(w - 8) * (0.002f + 0.018f * (float)((seed >> 3) & 63u) / 63.f));
    }
    return v;
}

__global__ __launch_bounds__(512) void fcc_mfma_pattern_probe_kernel(float* __restrict__ sink, int iters, int pattern) {
    half8_t a[4], b[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        a[i] = probe_operand(threadIdx.x * 8u + i);
        b[i] = probe_weight_operand(threadIdx.x * 8u + 4u + i, pattern);
    }
    float4_t acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
        acc[i] = float4_t{0.f, 0.f, 0.f, 0.f};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int j = 0; j < 8; ++j)
            asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(acc[j]) : "v"(a[j & 3]), "v"(b[(j >> 1) & 3]));
    }
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i)
        s += acc[i].x + acc[i].y + acc[i].z + acc[i].w;
    sink[blockIdx.x * blockDim.x + threadIdx.x] = s;
}

// sink: 4 * workgroups * 64 * waves bytes.  valu: 0 to 4 multiplications after every MFMA.  shape 0: 16 x 16 x 32
// instructions, shape 1: 32 x 32 x 16; shapes 2, 3, 4: 16 x 16 x 32 with weight-operand pattern 1, 2, 3 (valu = 0).
int launch_mfma_probe(float* sink, int workgroups, int waves, int valu, int shape, int iters, void* stream) {
    if (!sink || workgroups < 1 || (waves != 4 && waves != 8) || valu < 0 || valu > 4 || iters < 1 || shape < 0 || shape > 4 ||
        (shape >= 2 && valu != 0))
        return (int)hipErrorInvalidValue;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const dim3 g((unsigned)workgroups), b(64u * waves);
    if (shape >= 2) {
        hipLaunchKernelGGL(fcc_mfma_pattern_probe_kernel, g, b, 0, s, sink, iters, shape - 1);
        return (int)hipGetLastError();
    }
    if (shape == 1) {
        switch (valu) {
        case 0: hipLaunchKernelGGL(fcc_mfma32_probe_kernel<0>, g, b, 0, s, sink, iters); break;
        case 1: hipLaunchKernelGGL(fcc_mfma32_probe_kernel<1>, g, b, 0, s, sink, iters); break;
        case 2: hipLaunchKernelGGL(fcc_mfma32_probe_kernel<2>, g, b, 0, s, sink, iters); break;
        case 3: hipLaunchKernelGGL(fcc_mfma32_probe_kernel<3>, g, b, 0, s, sink, iters); break;
        default: hipLaunchKernelGGL(fcc_mfma32_probe_kernel<4>, g, b, 0, s, sink, iters); break;
        }
        return (int)hipGetLastError();
    }
    switch (valu) {
    case 0: hipLaunchKernelGGL(fcc_mfma_probe_kernel<0>, g, b, 0, s, sink, iters); break;
    case 1: hipLaunchKernelGGL(fcc_mfma_probe_kernel<1>, g, b, 0, s, sink, iters); break;
    case 2: hipLaunchKernelGGL(fcc_mfma_probe_kernel<2>, g, b, 0, s, sink, iters); break;
    case 3: hipLaunchKernelGGL(fcc_mfma_probe_kernel<3>, g, b, 0, s, sink, iters); break;
    default: hipLaunchKernelGGL(fcc_mfma_probe_kernel<4>, g, b, 0, s, sink, iters); break;
    }
    return (int)hipGetLastError();
}

// How one SIMD overlaps matrix-core and vector instructions, in shader cycles: the loop of fcc_mfma_probe_kernel with
// the vector instructions after each MFMA arranged by MODE -- 0: independent packed-f16 multiplications; 1: one
// dependent chain of them; 2: the first one writes a register of the B operand that the MFMA has just read; 3: as 0,
// with MFMAs whose destination is the next accumulator slot instead of their own input (what the compiler emits where
// it is free to).  Lane 0 of every workgroup leaves its tick counts (shader clock, 100 MHz wall clock) in ticks[].
template <int MODE, int VALU>
__global__ __launch_bounds__(512) void fcc_issue_probe_kernel(float* __restrict__ sink, long long* __restrict__ ticks,
                                                              int iters) {
    half8_t a[4], b[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
        a[i] = probe_operand(threadIdx.x * 8u + i), b[i] = probe_operand(threadIdx.x * 8u + 4u + i);
    float4_t acc[8];
    uint32_t r[8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
        acc[i] = float4_t{0.f, 0.f, 0.f, 0.f}, r[i] = 0x3c003c00u + (uint32_t)i;
    const uint32_t c = 0x3c003c00u, m = 0x000f000fu;
    __syncthreads();
    const long long t0 = clock64(), w0 = wall_clock64();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            if constexpr (MODE == 3)
                asm volatile("v_mfma_f32_16x16x32_f16 %0, %2, %3, %1"
                             : "=&v"(acc[(j + 1) & 7])
                             : "v"(acc[j]), "v"(a[j & 3]), "v"(b[(j >> 1) & 3]));
            else
                asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(acc[j]) : "v"(a[j & 3]), "v"(b[(j >> 1) & 3]));
#pragma unroll
            for (int v = 0; v < VALU; ++v) {
                if constexpr (MODE == 1)
                    asm volatile("v_pk_mul_f16 %0, %0, %1" : "+v"(r[j & 7]) : "v"(c));
                else if (MODE == 2 && v == 0)
                    asm volatile("v_and_or_b32 %0, %0, %1, %2"
                                 : "+v"(reinterpret_cast<uint32_t*>(&b[(j >> 1) & 3])[0])
                                 : "v"(m), "v"(c));
                else
                    asm volatile("v_pk_mul_f16 %0, %0, %1" : "+v"(r[(j + v) & 7]) : "v"(c));
            }
        }
    }
    const long long t1 = clock64(), w1 = wall_clock64();
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i)
        s += acc[i].x + acc[i].y + acc[i].z + acc[i].w + (float)r[i];
#pragma unroll
    for (int i = 0; i < 4; ++i)
        s += (float)b[i][0];
    sink[blockIdx.x * blockDim.x + threadIdx.x] = s;
    if (threadIdx.x == 0)
        ticks[2 * blockIdx.x] = t1 - t0, ticks[2 * blockIdx.x + 1] = w1 - w0;
}

int launch_issue_probe(float* sink, long long* ticks, int workgroups, int waves, int mode, int valu, int iters, void* stream) {
    if (!sink || !ticks || workgroups < 1 || (waves != 4 && waves != 8) || iters < 1)
        return (int)hipErrorInvalidValue;
    const dim3 g((unsigned)workgroups), b(64u * waves);
    hipStream_t s = static_cast<hipStream_t>(stream);
#define OVFCC_ISSUE(MODE, VALU) hipLaunchKernelGGL((fcc_issue_probe_kernel<MODE, VALU>), g, b, 0, s, sink, ticks, iters)
    if (mode == 0 && valu == 0) OVFCC_ISSUE(0, 0);
    else if (mode == 0 && valu == 2) OVFCC_ISSUE(0, 2);
    else if (mode == 0 && valu == 3) OVFCC_ISSUE(0, 3);
    else if (mode == 0 && valu == 4) OVFCC_ISSUE(0, 4);
    else if (mode == 0 && valu == 6) OVFCC_ISSUE(0, 6);
    else if (mode == 1 && valu == 3) OVFCC_ISSUE(1, 3);
    else if (mode == 2 && valu == 3) OVFCC_ISSUE(2, 3);
    else if (mode == 3 && valu == 3) OVFCC_ISSUE(3, 3);
    else return (int)hipErrorInvalidValue;
#undef OVFCC_ISSUE
    return (int)hipGetLastError();
}

int launch_empty(unsigned* out, void* stream) {
    hipLaunchKernelGGL(fcc_empty_kernel, dim3(256), dim3(256), 0, static_cast<hipStream_t>(stream), out);
    return (int)hipGetLastError();
}

int launch_stream_probe(const void* src, size_t bytes, int waves, int kib_per_wave, unsigned* out, void* stream) {
    const size_t chunks = bytes >> 10;
    const size_t cpw = (size_t)waves * kib_per_wave;
    if (!src || !out || bytes == 0 || (bytes & 1023) || waves < 1 || waves > 16 || kib_per_wave < 8 || chunks % cpw ||
        chunks >= ((size_t)1 << 21))
        return (int)hipErrorInvalidValue;
    hipLaunchKernelGGL(fcc_stream_probe_kernel<8>, dim3((unsigned)(chunks / cpw)), dim3(64u * waves), 0,
                       static_cast<hipStream_t>(stream), (const uint4_t*)src, (unsigned)chunks, (unsigned)cpw, out);
    return (int)hipGetLastError();
}

}  // namespace ovfcc
