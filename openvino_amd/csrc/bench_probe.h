// Launchers of the benchmark probes (bench_probe.hip), used by the benchmark library only.
#pragma once

#include <cstddef>

namespace ovfcc {

int launch_copy(void* dst, const void* src, size_t bytes, void* stream);
// an empty kernel, and a loads-only streaming kernel (workgroups of `waves` waves, kib_per_wave KiB per wave, eight
// loads in flight per wave) over `bytes`
int launch_empty(unsigned* out, void* stream);
int launch_stream_probe(const void* src, size_t bytes, int waves, int kib_per_wave, unsigned* out, void* stream);
// matrix-core loop on registers: shape 0 = v_mfma_f32_16x16x32_f16, 1 = v_mfma_f32_32x32x16_f16
int launch_mfma_probe(float* sink, int workgroups, int waves, int valu, int shape, int iters, void* stream);
// issue probe: shader-clock and wall-clock ticks of the loop, two per workgroup, in ticks[]
int launch_issue_probe(float* sink, long long* ticks, int workgroups, int waves, int mode, int valu, int iters, void* stream);

}  // namespace ovfcc
