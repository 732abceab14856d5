// Benchmark helpers, not part of the product library (built into libmi355q_bench.so, loaded by
// bench.py only): a plain streaming read of a buffer, the floor against which the weight-streaming
// kernels are quoted (same bytes, no arithmetic, nothing stored); and a loop of matrix instructions
// on register-resident operands, the rate the matrix pipes sustain on the caller's data when
// nothing else is asked of the chip (the published peak assumes the nominal clock, which the
// power limit does not grant under this load).
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

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef int i4 __attribute__((ext_vector_type(4)));

// KIND 0: v_mfma_f32_16x16x32_f16, 1: v_mfma_i32_16x16x64_i8.  Each wavefront loads 8 A operands from the
// first 2 MiB of `src` and 4 B operands from the second 2 MiB once (whatever the caller put there: the
// rate depends on the data, the chip being power-limited) and runs iters x 32 independent accumulations.
template <int KIND>
__global__ void __launch_bounds__(256) probe_mfma_kernel(const u4* src, int iters, u4* sink, unsigned long long* clk) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  // core-clock ticks and 100 MHz reference ticks around the loop: the clock the chip grants under this load
  const unsigned long long c0 = __builtin_amdgcn_s_memtime(), r0 = __builtin_amdgcn_s_memrealtime();
  u4 a[8], b[4];
#pragma unroll
  for (int i = 0; i < 8; ++i) a[i] = src[((blockIdx.x * 4 + wave) * 8 + i) % 2048 * 64 + lane];
#pragma unroll
  for (int i = 0; i < 4; ++i) b[i] = src[(2048 + ((blockIdx.x * 4 + wave) * 4 + i) % 2048) * 64 + lane];
  f4 accf[32];
  i4 acci[32];
#pragma unroll
  for (int c = 0; c < 32; ++c) {
    accf[c] = (f4){0.f, 0.f, 0.f, 0.f};
    acci[c] = (i4){0, 0, 0, 0};
  }
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int c = 0; c < 32; ++c) {
      // written as assembly so that every accumulation is in place (left to itself the compiler
      // rotates the accumulators through the loop, and a result that overlaps its addend without
      // coinciding with it runs at about half rate)
      if (KIND == 0)
        asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(accf[c]) : "v"(a[c & 7]), "v"(b[c >> 3]));
      else
        asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" : "+v"(acci[c]) : "v"(a[c & 7]), "v"(b[c >> 3]));
    }
  }
  if (clk && blockIdx.x == gridDim.x / 2 && threadIdx.x == 0) {
    clk[0] = __builtin_amdgcn_s_memtime() - c0;
    clk[1] = __builtin_amdgcn_s_memrealtime() - r0;
  }
  f4 rf = {0.f, 0.f, 0.f, 0.f};
  i4 ri = {0, 0, 0, 0};
#pragma unroll
  for (int c = 0; c < 32; ++c) {
    rf += accf[c];
    ri += acci[c];
  }
  // never true for the benchmark's data; keeps the accumulators alive
  if (rf.x == 12345.678f || ri.x == 0x12345678) sink[0] = (u4){(uint32_t)ri.x, (uint32_t)ri.y, 0u, 0u};
}

// 0 on success.  src: 2 MiB of A then 2 MiB of B operand data (fp16 values or int8 values); one workgroup of four
// wavefronts per launch slot, `workgroups` of them; operations done = workgroups * 4 * iters * 32 *
// (2 * 16 * 16 * 32 for kind 0, 2 * 16 * 16 * 64 for kind 1).
// clk (optional): two 64-bit words, core-clock and 100 MHz reference ticks one wavefront spent in the loop.
extern "C" int mi355q_bench_mfma_rate(const void* src, int kind, int workgroups, int iters, void* sink, void* clk,
                                      void* stream) {
  if (!src || !sink || workgroups <= 0 || workgroups > 65536 || iters <= 0 || (kind != 0 && kind != 1)) return 1;
  if (kind == 0)
    hipLaunchKernelGGL(probe_mfma_kernel<0>, dim3(workgroups), dim3(256), 0, (hipStream_t)stream, (const u4*)src, iters, (u4*)sink,
                       (unsigned long long*)clk);
  else
    hipLaunchKernelGGL(probe_mfma_kernel<1>, dim3(workgroups), dim3(256), 0, (hipStream_t)stream, (const u4*)src, iters, (u4*)sink,
                       (unsigned long long*)clk);
  return hipGetLastError() == hipSuccess ? 0 : 2;
}
