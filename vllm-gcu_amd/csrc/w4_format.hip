// int4 weight-format kernels: checkpoint / reference layouts -> slab layout,
// zero-point repack, and the slab -> byte-per-value unpack used for parity.
//
// Slab layout (flat int32 stream): [N/128][K/128][8 tiles][64 lanes][4 words].
// Word s of lane l (c = l % 16, kq = l / 16) of tile t in (slab S, group g)
// holds, in nibble NIB[j], the weight at k = 128g + 32s + 8kq + j and
// n = 128S + 8c + t, with NIB = {0,4,1,5,2,6,3,7}.
#include "common.h"

namespace mi355q {

__device__ __forceinline__ int nib_of_j(int j) { return (j >> 1) + ((j & 1) << 2); }

// one thread per destination word
__global__ void __launch_bounds__(256)
w4_repack_kernel(const void* __restrict__ src, int fmt, uint32_t* __restrict__ dst,
                 int K, int N, long words_per_matrix, long total_words) {
  long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total_words) return;
  long b = idx / words_per_matrix;
  long w = idx - b * words_per_matrix;
  int s = (int)(w & 3);
  int lane = (int)((w >> 2) & 63);
  int t = (int)((w >> 8) & 7);
  long sg = w >> 11;                       // S * (K/128) + g
  int G = K >> 7;
  int g = (int)(sg % G);
  int S = (int)(sg / G);
  int c = lane & 15, kq = lane >> 4;
  int n = 128 * S + 8 * c + t;
  int k0 = 128 * g + 32 * s + 8 * kq;
  uint32_t out = 0;
  if (fmt == MI355Q_W4_SRC_GPTQ) {
    // the 8 k values are the 8 nibbles of one source word
    const uint32_t* q = (const uint32_t*)src + b * ((long)(K >> 3) * N);
    uint32_t v = q[(long)(k0 >> 3) * N + n];
#pragma unroll
    for (int j = 0; j < 8; ++j) out |= ((v >> (4 * j)) & 15u) << (4 * nib_of_j(j));
  } else if (fmt == MI355Q_W4_SRC_AWQ) {
    const uint32_t* q = (const uint32_t*)src + b * ((long)K * (N >> 3));
    const int order[8] = {0, 4, 1, 5, 2, 6, 3, 7};
    int sh = 4 * order[n & 7];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      uint32_t v = q[(long)(k0 + j) * (N >> 3) + (n >> 3)];
      out |= ((v >> sh) & 15u) << (4 * nib_of_j(j));
    }
  } else if (fmt == MI355Q_W4_SRC_REF_KN_G64S) {
    // half-groups of 32 rows, signed nibbles (w - 8 in two's complement): group-of-64-local
    // row i < 32 in the low nibble, i >= 32 in the high nibble of byte row 32 G64 + (i & 31)
    const uint8_t* q = (const uint8_t*)src + b * ((long)(K >> 1) * N);
    const int k = k0 & 63, hi = k >= 32;
    const long row0 = 32 * (long)(k0 >> 6) + (k & 31);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const uint8_t v = q[(row0 + j) * N + n];
      const uint32_t nib = ((hi ? (v >> 4) : (v & 15u)) ^ 8u) & 15u;
      out |= nib << (4 * nib_of_j(j));
    }
  } else {
    // reference half-group bytes: group-local row i < 64 in the low nibble,
    // i >= 64 in the high nibble of byte row 64g + (i & 63)
    const uint8_t* q = (const uint8_t*)src + b * ((long)(K >> 1) * N);
    int i0 = 32 * s + 8 * kq;              // group-local k of j = 0
    int hi = i0 >= 64;
    int row0 = 64 * g + (i0 & 63);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      uint8_t v = (fmt == MI355Q_W4_SRC_REF_KN) ? q[(long)(row0 + j) * N + n]
                                                : q[(long)n * (K >> 1) + row0 + j];
      uint32_t nib = hi ? (v >> 4) : (v & 15u);
      out |= nib << (4 * nib_of_j(j));
    }
  }
  dst[idx] = out;
}

__global__ void __launch_bounds__(256)
w4_repack_zeros_kernel(const uint32_t* __restrict__ src, int fmt, uint32_t* __restrict__ dst,
                       long total_words) {
  long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total_words) return;
  uint32_t v = src[idx];
  uint32_t out;
  if (fmt == MI355Q_W4_SRC_GPTQ) {
    uint32_t lo = ((v & 0x0f0f0f0fu) + 0x01010101u) & 0x0f0f0f0fu;
    uint32_t hi = (((v >> 4) & 0x0f0f0f0fu) + 0x01010101u) & 0x0f0f0f0fu;
    out = lo | (hi << 4);
  } else {
    const int order[8] = {0, 4, 1, 5, 2, 6, 3, 7};
    out = 0;
#pragma unroll
    for (int j = 0; j < 8; ++j) out |= ((v >> (4 * order[j])) & 15u) << (4 * j);
  }
  dst[idx] = out;
}

// one thread per source word -> 8 bytes
__global__ void __launch_bounds__(256)
w4_unpack_kernel(const uint32_t* __restrict__ packed, uint8_t* __restrict__ dst, int K, int N,
                 long words_per_matrix, long total_words) {
  long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total_words) return;
  long b = idx / words_per_matrix;
  long w = idx - b * words_per_matrix;
  int s = (int)(w & 3);
  int lane = (int)((w >> 2) & 63);
  int t = (int)((w >> 8) & 7);
  long sg = w >> 11;
  int G = K >> 7;
  int g = (int)(sg % G);
  int S = (int)(sg / G);
  int c = lane & 15, kq = lane >> 4;
  int n = 128 * S + 8 * c + t;
  int k0 = 128 * g + 32 * s + 8 * kq;
  uint32_t v = packed[idx];
  uint8_t* o = dst + b * ((long)K * N);
#pragma unroll
  for (int j = 0; j < 8; ++j) o[(long)(k0 + j) * N + n] = (uint8_t)((v >> (4 * nib_of_j(j))) & 15u);
}

}  // namespace mi355q

using namespace mi355q;

extern "C" int mi355q_w4_repack(const void* src, int src_format, int32_t* dst, int batch, int K,
                                int N, void* stream) {
  MQ_REQUIRE(src && dst, "w4_repack: null pointer");
  MQ_REQUIRE(src_format >= MI355Q_W4_SRC_GPTQ && src_format <= MI355Q_W4_SRC_REF_KN_G64S,
             "w4_repack: unknown source format %d", src_format);
  MQ_REQUIRE(batch >= 0 && K > 0 && N > 0 && K % 128 == 0 && N % 128 == 0,
             "w4_repack: K=%d and N=%d must be positive multiples of 128", K, N);
  long wpm = (long)(K / 8) * N;
  long total = wpm * batch;
  if (total == 0) return 0;
  unsigned blocks = (unsigned)((total + 255) / 256);
  hipLaunchKernelGGL(w4_repack_kernel, dim3(blocks), dim3(256), 0, as_stream(stream), src,
                     src_format, (uint32_t*)dst, K, N, wpm, total);
  MQ_LAUNCH_CHECK("w4_repack");
  return 0;
}

extern "C" int mi355q_w4_repack_zeros(const int32_t* src, int src_format, int32_t* dst, int batch,
                                      int G, int N, void* stream) {
  MQ_REQUIRE(src && dst, "w4_repack_zeros: null pointer");
  MQ_REQUIRE(src_format == MI355Q_W4_SRC_GPTQ || src_format == MI355Q_W4_SRC_AWQ,
             "w4_repack_zeros: source format must be GPTQ or AWQ, got %d", src_format);
  MQ_REQUIRE(batch >= 0 && G > 0 && N > 0 && N % 8 == 0, "w4_repack_zeros: bad shape G=%d N=%d", G, N);
  long total = (long)batch * G * (N / 8);
  if (total == 0) return 0;
  unsigned blocks = (unsigned)((total + 255) / 256);
  hipLaunchKernelGGL(w4_repack_zeros_kernel, dim3(blocks), dim3(256), 0, as_stream(stream),
                     (const uint32_t*)src, src_format, (uint32_t*)dst, total);
  MQ_LAUNCH_CHECK("w4_repack_zeros");
  return 0;
}

extern "C" int mi355q_w4_unpack(const int32_t* packed, uint8_t* dst, int batch, int K, int N,
                                void* stream) {
  MQ_REQUIRE(packed && dst, "w4_unpack: null pointer");
  MQ_REQUIRE(batch >= 0 && K > 0 && N > 0 && K % 128 == 0 && N % 128 == 0,
             "w4_unpack: K=%d and N=%d must be positive multiples of 128", K, N);
  long wpm = (long)(K / 8) * N;
  long total = wpm * batch;
  if (total == 0) return 0;
  unsigned blocks = (unsigned)((total + 255) / 256);
  hipLaunchKernelGGL(w4_unpack_kernel, dim3(blocks), dim3(256), 0, as_stream(stream),
                     (const uint32_t*)packed, dst, K, N, wpm, total);
  MQ_LAUNCH_CHECK("w4_unpack");
  return 0;
}
