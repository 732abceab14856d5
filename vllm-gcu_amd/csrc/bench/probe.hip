// Benchmark helper, not part of the product library (built into libmi355q_bench.so, loaded by
// bench.py only): a plain streaming read of a buffer, the floor against which the weight-streaming
// kernels are quoted (same bytes, no arithmetic, nothing stored).
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

typedef uint32_t u4 __attribute__((ext_vector_type(4)));

// grid-stride: consecutive workgroups read consecutive 4 KiB pieces, eight 16-byte loads per lane in flight
__global__ void __launch_bounds__(256) probe_read_kernel(const u4* p, long total_words, u4* sink) {
  u4 acc = {0u, 0u, 0u, 0u};
  const long stride = (long)gridDim.x * 256;
  long i = (long)blockIdx.x * 256 + threadIdx.x;
  for (; i + 7 * stride < total_words; i += 8 * stride) {
    u4 v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = __builtin_nontemporal_load(p + i + u * stride);
#pragma unroll
    for (int u = 0; u < 8; ++u) acc ^= v[u];
  }
  for (; i < total_words; i += stride) acc ^= __builtin_nontemporal_load(p + i);
  // never true for the benchmark's data; keeps the loads alive
  if ((acc.x & acc.y & acc.z & acc.w) == 0x9e3779b9u) sink[0] = acc;
}

// 0 on success.  bytes a multiple of 16; sink is 16 writable bytes (never written in practice).
extern "C" int mi355q_bench_stream_read(const void* src, size_t bytes, int workgroups, void* sink, void* stream) {
  if (!src || !sink || workgroups <= 0 || workgroups > 65536 || bytes % 16) return 1;
  hipLaunchKernelGGL(probe_read_kernel, dim3(workgroups), dim3(256), 0, (hipStream_t)stream, (const u4*)src,
                     (long)(bytes / 16), (u4*)sink);
  return hipGetLastError() == hipSuccess ? 0 : 2;
}
