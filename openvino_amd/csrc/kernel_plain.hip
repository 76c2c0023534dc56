// Fallback kernel for shapes that keep OpenVINO's constant layout, and the small helper kernels of the routed calls.
// Semantics: the scalar reference kernel of the OpenVINO Intel-GPU plugin
// (src/plugins/intel_gpu/src/kernel_selector/cl_kernels/fully_connected_gpu_bfyx_ref.cl:88-160).
#include "device_common.h"

namespace ovfcc {

// ------------------------------------------------------------------------------------------------
// Plain kernel: OpenVINO layout, any N/K/G.  One wave per (n, m); lanes stride over k.
// ------------------------------------------------------------------------------------------------
__device__ __forceinline__ float plain_dot(const uint8_t* __restrict__ w, const half_t* __restrict__ s,
                                           const uint8_t* __restrict__ zp, const half_t* __restrict__ x, int n, int m,
                                           int K, int G, int w_type, int zp_type, int zp_scalar) {
    const int lane = threadIdx.x;
    const int ng = K / G;
    float acc = 0.f;
    for (int k = lane; k < K; k += 64) {
        const size_t wi = (size_t)n * K + k;
        float q;
        if (w_type == OVFCC_U4 || w_type == OVFCC_I4) {
            const unsigned b = w[wi >> 1];
            int v = (wi & 1) ? (b >> 4) : (b & 0xF);
            if (w_type == OVFCC_I4 && v >= 8)
                v -= 16;
            q = (float)v;
        } else if (w_type == OVFCC_U8) {
            q = (float)w[wi];
        } else {
            q = (float)(int8_t)w[wi];
        }
        const int g = k / G;
        float z = 0.f;
        if (zp_type != OVFCC_NONE) {
            const size_t zi = zp_scalar ? 0 : (size_t)n * ng + g;
            if (zp_type == OVFCC_U4) {
                const unsigned b = zp[zi >> 1];
                z = (float)((zi & 1) ? (b >> 4) : (b & 0xF));
            } else {
                z = (float)zp[zi];
            }
        }
        const float sc = (float)s[(size_t)n * ng + g];
        acc += (float)x[(size_t)m * K + k] * ((q - z) * sc);
    }
    for (int off = 32; off > 0; off >>= 1)
        acc += __shfl_down(acc, off, 64);
    return acc;  // lane 0 holds the sum
}

// grid = (output channels, M).  With a gated linear unit (glu != 0) output channel f is
// act(channel gate_offset + f) * (channel up_offset + f) and N_out = N / 2.
__global__ __launch_bounds__(64) void fcc_plain_kernel(const uint8_t* __restrict__ w, const half_t* __restrict__ s,
                                                       const uint8_t* __restrict__ zp,
                                                       const half_t* __restrict__ bias,
                                                       const half_t* __restrict__ x, void* __restrict__ y, int M,
                                                       int N_out, int K, int G, int w_type, int zp_type, int zp_scalar,
                                                       int out_f32, int glu, int gate_offset, int up_offset) {
    const int f = blockIdx.x;
    const int m = blockIdx.y;
    const int n = glu ? gate_offset + f : f;
    float acc = plain_dot(w, s, zp, x, n, m, K, G, w_type, zp_type, zp_scalar);
    if (bias)
        acc += (float)bias[n];
    if (glu) {
        float up = plain_dot(w, s, zp, x, up_offset + f, m, K, G, w_type, zp_type, zp_scalar);
        if (bias)
            up += (float)bias[up_offset + f];
        acc = glu_value(glu, acc, up);
    }
    if (threadIdx.x == 0)
        store_out(y, (size_t)m * N_out + f, acc, out_f32);
}

// ------------------------------------------------------------------------------------------------
// Row gather / scatter for the mixture-of-experts entry point: dst row r = src row src_row[r] (gather, dst_row
// null) or dst row dst_row[r] = src row r (scatter, src_row null); rows of row_bytes (a multiple of 16) bytes.
// A negative map entry skips the row.  One workgroup per row.
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void fcc_rows_kernel(uint4_t* __restrict__ dst, const uint4_t* __restrict__ src,
                                                       const int* __restrict__ src_row,
                                                       const int* __restrict__ dst_row, int row_bytes) {
    const int r = blockIdx.x;
    const int named = src_row ? src_row[r] : dst_row[r];
    if (named < 0)
        return;  // a slot that the routing left empty
    const size_t from = (size_t)(src_row ? named : r) * (row_bytes / 16);
    const size_t to = (size_t)(dst_row ? named : r) * (row_bytes / 16);
    for (int i = threadIdx.x; i < row_bytes / 16; i += blockDim.x)
        dst[to + i] = src[from + i];
}

int launch_rows(void* dst, const void* src, const int* src_row, const int* dst_row, int rows, int row_bytes,
                void* stream) {
    if (rows <= 0)
        return 0;
    if (row_bytes <= 0 || (row_bytes & 15) || (!src_row == !dst_row))
        return (int)hipErrorInvalidValue;
    hipLaunchKernelGGL(fcc_rows_kernel, dim3((unsigned)rows), dim3(256), 0, static_cast<hipStream_t>(stream),
                       (uint4_t*)dst, (const uint4_t*)src, src_row, dst_row, row_bytes);
    return (int)hipGetLastError();
}

// ------------------------------------------------------------------------------------------------
// Last step of a mixture-of-experts block: y[m, :] = sum_j routing[m, j] * d[pos[m, j], :] over the top_k experts
// of row m, in the order j = 0, 1, ... (the Multiply by the routing weights and the ReduceSum over the expert
// axis that MOE fuses, src/common/transformations/src/transformations/common_optimizations/moe_op_fusion.cpp:97-104).
// d holds one result row per (row, expert) pair in bucket order, pos maps (m, j) to it.  f32 sums; one workgroup
// per row, four channels per thread and step.
// ------------------------------------------------------------------------------------------------
template <bool IN_F32>
__global__ __launch_bounds__(256) void fcc_moe_combine_kernel(void* __restrict__ y, const void* __restrict__ d,
                                                              const half_t* __restrict__ routing,
                                                              const int* __restrict__ pos, int top_k, int H,
                                                              int out_f32) {
    const int m = blockIdx.x;
    for (int c = 4 * threadIdx.x; c < H; c += 4 * blockDim.x) {
        float acc[4] = {0.f, 0.f, 0.f, 0.f};
        for (int j = 0; j < top_k; ++j) {
            const int slot = pos[(size_t)m * top_k + j];
            if (slot < 0)
                continue;  // an index outside the experts selects nothing
            const float wgt = (float)routing[(size_t)m * top_k + j];
            const size_t row = (size_t)slot * H + c;
            if constexpr (IN_F32) {
                const float4_t v = *reinterpret_cast<const float4_t*>(static_cast<const float*>(d) + row);
                acc[0] += wgt * v.x, acc[1] += wgt * v.y, acc[2] += wgt * v.z, acc[3] += wgt * v.w;
            } else {
                const half4_t v = *reinterpret_cast<const half4_t*>(static_cast<const half_t*>(d) + row);
                acc[0] += wgt * (float)v[0], acc[1] += wgt * (float)v[1], acc[2] += wgt * (float)v[2],
                    acc[3] += wgt * (float)v[3];
            }
        }
        if (out_f32)
            *reinterpret_cast<float4_t*>(static_cast<float*>(y) + (size_t)m * H + c) =
                float4_t{acc[0], acc[1], acc[2], acc[3]};
        else
            *reinterpret_cast<half4_t*>(static_cast<half_t*>(y) + (size_t)m * H + c) =
                half4_t{(half_t)acc[0], (half_t)acc[1], (half_t)acc[2], (half_t)acc[3]};
    }
}

// ------------------------------------------------------------------------------------------------
// Mixture-of-experts routing on the device (the reference's GPU plugin builds its expert masks there too,
// src/plugins/intel_gpu/src/graph/impls/ocl_v2/moe_mask_gen.cl; the bucket order is that of the CPU executor,
// src/plugins/intel_cpu/src/nodes/executors/dnnl/dnnl_gathermatmul_executor.cpp:492-509).  One workgroup per
// expert, no communication between workgroups: every workgroup counts all experts' pairs (a histogram in LDS over
// the R indices), derives its own bucket's first slot and first slice from the counts of the experts before it,
// and then places its own pairs in ascending order with a block-wide prefix sum.
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void fcc_moe_route_kernel(const int* __restrict__ indices, int R, int M, int top_k,
                                                            int n_experts, int a_batches, int inverse, int cap,
                                                            int x_mapped, ExpertPointers experts, const char* x_base,
                                                            size_t x_row_bytes, char* y_base, size_t y_row_bytes,
                                                            int* __restrict__ first, int* __restrict__ second,
                                                            BatchGroupItem* __restrict__ table, int n_slices_max,
                                                            RoutedHeader* __restrict__ header, int tiles_x,
                                                            int kb_total, int n_cus, SecondTable t2,
                                                            char* unrouted_y, size_t unrouted_row_bytes) {
    __shared__ int hist[kMaxGroupItems];
    __shared__ int wave_total[4];
    __shared__ int start_s, slice_s, total_slices_s, total_pairs_s;
    const int e = blockIdx.x;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (tid < kMaxGroupItems)
        hist[tid] = 0;
    __syncthreads();
    for (int j = tid; j < R; j += 256) {
        const int v = indices[j];
        if (v >= 0 && v < n_experts) {
            atomicAdd(&hist[v], 1);
        } else if (e == 0) {
            if (inverse)
                second[j] = -1;
            if (unrouted_y) {
                // no expert computes this pair's row of the result [top_k, M, .]: it reads as zeros
                const int m = j / top_k, i = j - m * top_k;
                uint4_t* row = reinterpret_cast<uint4_t*>(unrouted_y + (size_t)(i * M + m) * unrouted_row_bytes);
                for (size_t c = 0; c < unrouted_row_bytes / 16; ++c)
                    row[c] = uint4_t{0u, 0u, 0u, 0u};
            }
        }
    }
    __syncthreads();
    if (tid == 0) {
        int start = 0, slice = 0, total = 0, pairs = 0;
        for (int k = 0; k < n_experts; ++k) {
            const int slices = (hist[k] + cap - 1) / cap;
            if (k < e)
                start += hist[k], slice += slices;
            total += slices;
            pairs += hist[k];
        }
        start_s = start, slice_s = slice, total_slices_s = total, total_pairs_s = pairs;
    }
    __syncthreads();
    const int start = start_s, count = hist[e];
    // this expert's pairs, in ascending order of (row, selection)
    int placed = 0;
    for (int j0 = 0; j0 < R; j0 += 256) {
        const int j = j0 + tid;
        const bool mine = j < R && indices[j] == e;
        const unsigned long long ballot = __ballot(mine);
        const int before = __popcll(ballot & ((1ull << lane) - 1ull));
        if (lane == 0)
            wave_total[wave] = __popcll(ballot);
        __syncthreads();
        int base = placed;
        for (int w = 0; w < wave; ++w)
            base += wave_total[w];
        if (mine) {
            const int slot = start + base + before;
            const int m = j / top_k, i = j - m * top_k;
            first[slot] = a_batches == 1 ? m : i * M + m;
            if (inverse)
                second[j] = slot;
            else
                second[slot] = i * M + m;
        }
        placed += wave_total[0] + wave_total[1] + wave_total[2] + wave_total[3];
        __syncthreads();
    }
    // the bucket cut into equal slices of at most cap rows
    const int slices = (count + cap - 1) / cap;
    const int step = slices ? (count + slices - 1) / slices : 0;
    for (int t = tid; t < slices; t += 256) {
        BatchGroupItem it;
        it.w = experts.w[e], it.scale = experts.scale[e], it.zp = experts.zp[e], it.bias = experts.bias[e];
        it.x = x_mapped ? x_base : x_base + (size_t)(start + t * step) * x_row_bytes;
        it.y = y_base + (size_t)(start + t * step) * y_row_bytes;
        it.M = min(step, count - t * step);
        it.reserved = x_mapped ? start + t * step : 0;
        table[slice_s + t] = it;
        if (t2.table) {
            it.w = t2.w[e], it.scale = t2.scale[e], it.zp = t2.zp[e], it.bias = t2.bias[e];
            it.x = static_cast<const char*>(t2.x_base) + (size_t)(start + t * step) * t2.x_row_bytes;
            it.y = static_cast<char*>(t2.y_base) + (size_t)(start + t * step) * t2.y_row_bytes;
            it.reserved = 0;
            t2.table[slice_s + t] = it;
        }
    }
    // the last workgroup closes what no bucket owns: the slices beyond the last one, and the slots beyond the
    // last pair (there are some when an index named no expert)
    if (e == n_experts - 1) {
        if (tid == 0) {
            *header = routed_header(tiles_x, total_slices_s, kb_total, n_cus);
            if (t2.table)
                *t2.header = routed_header(t2.tiles_x, total_slices_s, t2.kb_total, n_cus);
        }
        for (int t = total_slices_s + tid; t < n_slices_max; t += 256) {
            BatchGroupItem it{};
            table[t] = it;
            if (t2.table)
                t2.table[t] = it;
        }
        for (int slot = total_pairs_s + tid; slot < R; slot += 256) {
            first[slot] = -1;
            if (!inverse)
                second[slot] = -1;
        }
    }
}

int launch_moe_route(const int* indices_dev, int64_t M, int top_k, int n_experts, int a_batches, int inverse, int cap,
                     int x_mapped, const ExpertPointers& experts, const void* x_base, size_t x_row_bytes, void* y_base,
                     size_t y_row_bytes, int* first, int* second, BatchGroupItem* table, int n_slices_max,
                     RoutedHeader* header, int tiles_x, int kb_total, int n_cus, void* stream,
                     const SecondTable* second_table, void* unrouted_y, size_t unrouted_row_bytes) {
    const int64_t R = M * top_k;
    if (unrouted_y && (unrouted_row_bytes == 0 || (unrouted_row_bytes & 15)))
        return (int)hipErrorInvalidValue;
    SecondTable t2{};
    if (second_table) {
        t2 = *second_table;
        if (n_experts > kMaxSecondTableItems || !t2.table || !t2.header || t2.tiles_x < 1 || t2.kb_total < 1)
            return (int)hipErrorInvalidValue;
    }
    if (R <= 0 || R > ((int64_t)1 << 24) || n_experts < 1 || n_experts > kMaxGroupItems || cap < 1 ||
        n_slices_max < (R + cap - 1) / cap + n_experts || (a_batches != 1 && a_batches != top_k) || !header ||
        tiles_x < 1 || kb_total < 1 || n_cus < 1)
        return (int)hipErrorInvalidValue;
    hipLaunchKernelGGL(fcc_moe_route_kernel, dim3((unsigned)n_experts), dim3(256), 0, static_cast<hipStream_t>(stream),
                       indices_dev, (int)R, (int)M, top_k, n_experts, a_batches, inverse, cap, x_mapped, experts,
                       static_cast<const char*>(x_base), x_row_bytes, static_cast<char*>(y_base), y_row_bytes, first,
                       second, table, n_slices_max, header, tiles_x, kb_total, n_cus, t2, static_cast<char*>(unrouted_y),
                       unrouted_row_bytes);
    return (int)hipGetLastError();
}

// ------------------------------------------------------------------------------------------------
// GroupedMatMul with its offsets in device memory: the slice table of the grouped prefill launch from the
// cumulative row ends offsets[0 .. n_groups) of rows that are already contiguous per group (group g owns rows
// [offsets[g-1], offsets[g]) of x and y).  One workgroup.  Offsets are read as the reference's loop reads them
// (start = previous end), clamped to [previous end, rows], so that a bad value can empty a group but never reach
// outside the buffers.  tail[0] receives the first row that belongs to no group.
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void fcc_offsets_table_kernel(const int* __restrict__ offsets, int n_groups, int rows,
                                                                int cap, ExpertPointers groups, const char* x_base,
                                                                size_t x_row_bytes, char* y_base, size_t y_row_bytes,
                                                                BatchGroupItem* __restrict__ table, int n_slices_max,
                                                                RoutedHeader* __restrict__ header, int* __restrict__ tail,
                                                                int tiles_x, int kb_total, int n_cus) {
    __shared__ int start_s[kMaxGroupItems], count_s[kMaxGroupItems], slice_s[kMaxGroupItems];
    __shared__ int total_s;
    const int tid = threadIdx.x;
    if (tid == 0) {
        int start = 0, slice = 0;
        for (int g = 0; g < n_groups; ++g) {
            const int end = min(max(offsets[g], start), rows);
            start_s[g] = start, count_s[g] = end - start, slice_s[g] = slice;
            slice += (end - start + cap - 1) / cap;
            start = end;
        }
        total_s = slice;
        *tail = start;
        *header = routed_header(tiles_x, slice, kb_total, n_cus);
    }
    __syncthreads();
    for (int g = 0; g < n_groups; ++g) {
        const int count = count_s[g], slices = (count + cap - 1) / cap;
        const int step = slices ? (count + slices - 1) / slices : 0;  // equal slices of at most cap rows
        for (int t = tid; t < slices; t += 256) {
            BatchGroupItem it;
            it.w = groups.w[g], it.scale = groups.scale[g], it.zp = groups.zp[g], it.bias = groups.bias[g];
            it.x = x_base + (size_t)(start_s[g] + t * step) * x_row_bytes;
            it.y = y_base + (size_t)(start_s[g] + t * step) * y_row_bytes;
            it.M = min(step, count - t * step);
            it.reserved = 0;
            table[slice_s[g] + t] = it;
        }
    }
    for (int t = total_s + tid; t < n_slices_max; t += 256) {
        BatchGroupItem it{};
        table[t] = it;
    }
}

// rows [tail[0], rows) of y, row_bytes each (a multiple of 4): zeros.  One workgroup per row.
__global__ __launch_bounds__(256) void fcc_zero_tail_kernel(unsigned* __restrict__ y, const int* __restrict__ tail,
                                                            int row_words) {
    const int row = blockIdx.x;
    if (row < tail[0])
        return;
    unsigned* p = y + (size_t)row * row_words;
    for (int i = threadIdx.x; i < row_words; i += 256)
        p[i] = 0u;
}

int launch_offsets_table(const int* offsets_dev, int n_groups, int64_t rows, int cap, const ExpertPointers& groups,
                         const void* x_base, size_t x_row_bytes, void* y_base, size_t y_row_bytes,
                         BatchGroupItem* table, int n_slices_max, RoutedHeader* header, int* tail, int tiles_x,
                         int kb_total, int n_cus, void* stream) {
    if (!offsets_dev || rows <= 0 || rows > ((int64_t)1 << 24) || n_groups < 1 || n_groups > kMaxGroupItems || cap < 1 ||
        n_slices_max < (rows + cap - 1) / cap + n_groups || !header || !tail || tiles_x < 1 || kb_total < 1 ||
        n_cus < 1 || (y_row_bytes & 3))
        return (int)hipErrorInvalidValue;
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(fcc_offsets_table_kernel, dim3(1), dim3(256), 0, s, offsets_dev, n_groups, (int)rows, cap, groups,
                       static_cast<const char*>(x_base), x_row_bytes, static_cast<char*>(y_base), y_row_bytes, table,
                       n_slices_max, header, tail, tiles_x, kb_total, n_cus);
    hipLaunchKernelGGL(fcc_zero_tail_kernel, dim3((unsigned)rows), dim3(256), 0, s, static_cast<unsigned*>(y_base), tail,
                       (int)(y_row_bytes / 4));
    return (int)hipGetLastError();
}

int launch_moe_combine(void* y, const void* d, const void* routing, const int* pos, int rows, int top_k, int H,
                       int d_f32, int out_f32, void* stream) {
    if (rows <= 0)
        return 0;
    if (top_k <= 0 || H <= 0 || (H & 3))
        return (int)hipErrorInvalidValue;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (d_f32)
        hipLaunchKernelGGL(fcc_moe_combine_kernel<true>, dim3((unsigned)rows), dim3(256), 0, s, y, d,
                           (const half_t*)routing, pos, top_k, H, out_f32);
    else
        hipLaunchKernelGGL(fcc_moe_combine_kernel<false>, dim3((unsigned)rows), dim3(256), 0, s, y, d,
                           (const half_t*)routing, pos, top_k, H, out_f32);
    return (int)hipGetLastError();
}

int launch_plain(const FcDeviceArgs& a, const LaunchPlan& p, void* stream) {
    hipLaunchKernelGGL(fcc_plain_kernel, dim3(p.grid[0], p.grid[1], 1), dim3(64), 0, static_cast<hipStream_t>(stream),
                       (const uint8_t*)a.w, (const half_t*)a.scale, (const uint8_t*)a.zp, (const half_t*)a.bias,
                       (const half_t*)a.x, a.y, (int)a.M, (int)a.N_out, (int)a.K, (int)a.group_size, a.w_type,
                       a.zp_type, a.zp_scalar, a.out_f32, a.layout.glu, a.gate_offset, a.up_offset);
    return (int)hipGetLastError();
}

}  // namespace ovfcc
