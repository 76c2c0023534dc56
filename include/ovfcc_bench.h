/*
 * ovfcc_bench -- timing helpers of the benchmark driver, exported by libovfcc_bench.so (built beside libovfcc.so,
 * which it links; the product library carries none of them and none of their probe kernels).  Not part of the
 * drop-in boundary: nothing in the OpenVINO sources corresponds to them and an integration does not bind them.
 * They are native code because the timed region has to be bracketed by HIP events on the very stream the kernels
 * are launched on, which a host without HIP (the Python benchmark) cannot do itself.
 */
#ifndef OVFCC_BENCH_H
#define OVFCC_BENCH_H

#include "ovfcc.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Timed back-to-back launches: runs `iters` passes over the `n_layers` nodes in order (layer i reads x_dev,
 * writes y_dev; buffers must fit the largest layer), all on the request's stream, bracketed by HIP events on
 * that stream.  Returns elapsed milliseconds of the whole timed region.  use_graph != 0 captures one pass into
 * a HIP graph and replays it. */
int ovfcc_bench_layers(ovfcc_request* req, const ovfcc_weights* const* layers, int n_layers, const void* x_dev,
                       void* y_dev, int64_t M, int warmup, int iters, int use_graph, float* elapsed_ms);

/* The same for grouped runs: `iters` eager calls of ovfcc_fc_run_grouped_device on the request's stream,
 * bracketed by HIP events on that stream. */
int ovfcc_bench_grouped(ovfcc_request* req, const ovfcc_group_item* items, int n_items, int warmup, int iters,
                        float* elapsed_ms);

/* Plain device-to-device copy kernel of `bytes` (multiple of 16) repeated `iters` times, timed with HIP
 * events: the yardstick the HBM counters and the achieved-bandwidth figures are scaled by. */
int ovfcc_bench_copy(ovfcc_ctx* ctx, void* dst_dev, const void* src_dev, size_t bytes, int iters, float* elapsed_ms);

/* Launch floors under graph replay: a graph of n_nodes launches of a probe kernel is replayed `iters` times and
 * timed with events.  node_bytes = 0: empty kernels (what a graph node costs with nothing in it).  Otherwise a
 * loads-only streaming kernel over node_bytes (a multiple of waves * kib_per_wave KiB; workgroups of `waves` waves,
 * kib_per_wave >= 8 KiB per wave, eight 1 KiB loads in flight per wave), node i reading slice i mod
 * (arena_bytes / node_bytes) of arena_dev so that the caches do not serve it: how fast a kernel that only reads can
 * move that many bytes. */
int ovfcc_bench_floor(ovfcc_ctx* ctx, const void* arena_dev, size_t arena_bytes, size_t node_bytes, int n_nodes, int waves,
                      int kib_per_wave, int iters, float* elapsed_ms);

/* Matrix-core ceiling: one workgroup per compute unit with `waves` waves (4 or 8: one or two per SIMD), every
 * wave `rounds` times eight independent v_mfma_f32_16x16x32_f16 (shape 0) or four independent
 * v_mfma_f32_32x32x16_f16 (shape 1; the same matrix-core work) on registers, each followed by `valu` (0..4; twice
 * that for shape 1) packed-f16 vector multiplications on other registers; no memory traffic.  Timed with HIP
 * events; *flops is the matrix-core work of the timed launch.  What the chip sustains under that load (it lowers
 * its clock) is the ceiling the prefill kernels are measured against beside the nominal peak.  Both operands are
 * random halves; shapes 2, 3 and 4 (valu = 0) are shape 0 with the second operand looking like weights instead:
 * integers -8 .. 7 as halves, the integers 0 .. 15 as subnormal halves, integers -8 .. 7 times a scale rounded to
 * half -- the sustained rate depends on how many operand bits toggle. */
int ovfcc_bench_mfma(ovfcc_ctx* ctx, int waves, int valu, int shape, int rounds, float* elapsed_ms, double* flops);

/* How one SIMD overlaps matrix-core and vector instructions: `workgroups` workgroups (1: one compute unit alone, no
 * power limit; the number of compute units: the whole chip) of `waves` waves (4 or 8) run the loop of
 * ovfcc_bench_mfma with `valu` vector instructions after every v_mfma_f32_16x16x32_f16, arranged by `mode` -- 0:
 * independent packed-f16 multiplications (valu 0, 2, 3, 4 or 6); 1: one dependent chain (valu 3); 2: the first one
 * writes a register of the B operand the MFMA has just read (valu 3); 3: as 0 with MFMAs whose destination is not
 * their accumulator input (valu 3).  Measured inside the kernel: *cycles_per_mfma = shader-clock ticks per MFMA and
 * SIMD, *ns_per_mfma = the same from the 100 MHz wall clock (their ratio is the clock the loop ran at). */
int ovfcc_bench_issue(ovfcc_ctx* ctx, int workgroups, int waves, int mode, int valu, int rounds, double* cycles_per_mfma,
                      double* ns_per_mfma);

#ifdef __cplusplus
}
#endif
#endif /* OVFCC_BENCH_H */
