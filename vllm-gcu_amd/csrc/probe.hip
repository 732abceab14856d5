// Measurement probe: a plain streaming read of a buffer, the floor against
// which the weight-streaming kernels are judged (same bytes, no arithmetic).
#include "common.h"

namespace mi355q {

template <int UNR>
__global__ void __launch_bounds__(256) probe_read_kernel(const u4* p, long words_per_wg, u4* sink) {
  const u4* q = p + (long)blockIdx.x * words_per_wg + threadIdx.x;
  u4 acc = {0u, 0u, 0u, 0u};
  for (long i = 0; i < words_per_wg; i += 256 * UNR) {
    u4 v[UNR];
#pragma unroll
    for (int u = 0; u < UNR; ++u) v[u] = __builtin_nontemporal_load(q + i + u * 256);
#pragma unroll
    for (int u = 0; u < UNR; ++u) acc ^= v[u];
  }
  // never true for the benchmark's data; keeps the loads alive
  if ((acc.x & acc.y & acc.z & acc.w) == 0x9e3779b9u) sink[0] = acc;
}

}  // namespace mi355q

using namespace mi355q;

extern "C" int mi355q_probe_stream_read(const void* src, size_t bytes, int workgroups, void* sink,
                                        void* stream) {
  MQ_REQUIRE(src && sink, "probe_stream_read: null pointer");
  MQ_REQUIRE(workgroups > 0 && workgroups <= 65536, "probe_stream_read: bad workgroup count %d", workgroups);
  const size_t chunk = (size_t)workgroups * 256 * 8 * 16;      // bytes per trip of the whole grid
  MQ_REQUIRE(bytes >= chunk && bytes % chunk == 0,
             "probe_stream_read: bytes=%zu must be a positive multiple of %zu (workgroups * 32 KiB)", bytes, chunk);
  const long words_per_wg = (long)(bytes / 16 / workgroups);
  hipLaunchKernelGGL((probe_read_kernel<8>), dim3(workgroups), dim3(256), 0, as_stream(stream),
                     (const u4*)src, words_per_wg, (u4*)sink);
  MQ_LAUNCH_CHECK("probe_stream_read");
  return 0;
}
