// W8A8 int8 GEMM on the gfx950 int8 MFMA (v_mfma_i32_16x16x64_i8) with the
// per-token x per-channel scales (and bias) fused into the epilogue, plus the
// per-token / static int8 activation quantisers that feed it.
//
// GEMM: out[M, N] = (xq[M, K] . wq[N, K]^T in int32) * x_scale[m] * w_scale[n].
// Both operands are K-contiguous (that is what the MFMA lanes consume: 16
// consecutive k per lane).  Workgroup tile 256 x 256, K step 128, four
// wavefronts 2 x 2, each 128 x 128 = 8 x 8 MFMA tiles (256 int32 accumulator
// registers).  Tiles are staged in LDS with a 16-byte-chunk XOR swizzle so the
// 8-lane groups of a 128-bit LDS read hit 8 different bank groups; LDS is
// double buffered and the next tile's global loads are issued before the
// current tile's MFMAs.  The weights take the A operand slot so that each lane
// ends up with 4 consecutive output columns (one 8-byte store).
#include "common.h"

namespace mi355q {
namespace {

constexpr int TM = 256, TN = 256, TK = 128;
constexpr int TILE_BYTES = 256 * TK;              // one operand tile (32 KiB)
constexpr int STAGE_BYTES = 2 * TILE_BYTES;       // x tile + w tile

struct I8Args {
  void* out;                // [M, N] f16 / bf16 / f32, row stride ldo elements
  int32_t* acc_out;         // optional raw accumulators [M, N]
  const int8_t* x;          // [M, K], row stride ldx bytes
  const int8_t* w;          // [N, K], row stride ldw bytes
  const float* x_scale;     // [M] or [1]
  const float* w_scale;     // [N] or [1]
  const void* bias;         // [N] in out dtype (or f32 when bias_f32) or null
  int M, N, K;
  long ldx, ldw, ldo;
  int x_scale_per_row, w_scale_per_col, bias_f32;
  int n_panels_swizzle;     // non-zero: XCD-aware tile order
};

__device__ __forceinline__ int swz(int row, int chunk) { return chunk ^ (row & 7); }

template <int DT>
__device__ __forceinline__ void store4(void* out, long idx, const float* v) {
  if (DT == MI355Q_F32) {
    *(f4*)((float*)out + idx) = (f4){v[0], v[1], v[2], v[3]};
  } else {
    u2 o;
    o.x = (uint32_t)Elem<DT == MI355Q_F32 ? MI355Q_F16 : DT>::from_f32(v[0]) |
          ((uint32_t)Elem<DT == MI355Q_F32 ? MI355Q_F16 : DT>::from_f32(v[1]) << 16);
    o.y = (uint32_t)Elem<DT == MI355Q_F32 ? MI355Q_F16 : DT>::from_f32(v[2]) |
          ((uint32_t)Elem<DT == MI355Q_F32 ? MI355Q_F16 : DT>::from_f32(v[3]) << 16);
    *(u2*)((uint16_t*)out + idx) = o;
  }
}

template <int DT>
__device__ __forceinline__ float load_bias(const void* bias, int bias_f32, int n) {
  if (bias_f32 || DT == MI355Q_F32) return ((const float*)bias)[n];
  return Elem<DT == MI355Q_F32 ? MI355Q_F16 : DT>::to_f32(((const uint16_t*)bias)[n]);
}

template <int DT>
__global__ void __launch_bounds__(256, 1)
w8a8_int8_gemm_kernel(I8Args a) {
  extern __shared__ __align__(16) unsigned char lds[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l16 = lane & 15, kq = lane >> 4;
  const int wm = wave >> 1, wn = wave & 1;
  const int M = a.M, N = a.N, K = a.K;

  // tile coordinates; with the swizzle, the workgroups that land on one XCD
  // (ids congruent mod 8) sweep all row tiles of the same weight panels
  const int mtiles = (M + TM - 1) / TM, ntiles = (N + TN - 1) / TN;
  int pid = blockIdx.x, tm, tn;
  if (a.n_panels_swizzle) {
    const int x = pid & 7, j = pid >> 3;
    tm = j % mtiles;
    tn = (j / mtiles) * 8 + x;
  } else {
    tm = pid % mtiles;
    tn = pid / mtiles;
  }
  (void)ntiles;
  const int m0 = tm * TM, n0 = tn * TN;

  i4 acc[8][8];      // [n tile][m tile]: weights are the MFMA "A" operand
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[i][j] = (i4){0, 0, 0, 0};

  // global -> LDS staging: each operand tile is 256 rows x 8 chunks of 16 B;
  // thread t copies chunks t, t + 256, ... (8 per operand)
  u4 xr[8], wr[8];
  const int srow = tid >> 3, schunk = tid & 7;
  auto gload = [&](int k0) {
#pragma unroll
    for (int p = 0; p < 8; ++p) {
      const int r = p * 32 + srow;
      const int xm = min(m0 + r, M - 1), wn_ = min(n0 + r, N - 1);
      xr[p] = *(const u4*)(a.x + (long)xm * a.ldx + k0 + 16 * schunk);
      wr[p] = *(const u4*)(a.w + (long)wn_ * a.ldw + k0 + 16 * schunk);
    }
  };
  auto lstore = [&](int stage) {
    unsigned char* xs = lds + stage * STAGE_BYTES;
    unsigned char* ws = xs + TILE_BYTES;
#pragma unroll
    for (int p = 0; p < 8; ++p) {
      const int r = p * 32 + srow;
      const int off = r * TK + swz(r, schunk) * 16;
      *(u4*)(xs + off) = xr[p];
      *(u4*)(ws + off) = wr[p];
    }
  };

  gload(0);
  lstore(0);
  __syncthreads();

  const int nk = K / TK;
  for (int kt = 0; kt < nk; ++kt) {
    const int stage = kt & 1;
    gload(min(kt + 1, nk - 1) * TK);
    const unsigned char* xs = lds + stage * STAGE_BYTES;
    const unsigned char* ws = xs + TILE_BYTES;
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      i4 bx[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int r = wm * 128 + j * 16 + l16;
        bx[j] = *(const i4*)(xs + r * TK + swz(r, 4 * s + kq) * 16);
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int r = wn * 128 + i * 16 + l16;
        const i4 aw = *(const i4*)(ws + r * TK + swz(r, 4 * s + kq) * 16);
#pragma unroll
        for (int j = 0; j < 8; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(aw, bx[j], acc[i][j], 0, 0, 0);
      }
    }
    lstore(stage ^ 1);
    __syncthreads();
  }

  // ---- epilogue: lane holds, per (n tile i, m tile j), output row
  // m = .. + l16 and columns n = .. + 4 kq + {0..3}
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int m = m0 + wm * 128 + j * 16 + l16;
    if (m >= M) continue;
    const float xsc = a.x_scale ? a.x_scale[a.x_scale_per_row ? m : 0] : 1.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int n = n0 + wn * 128 + i * 16 + 4 * kq;
      if (n >= N) continue;                     // N is a multiple of 4
      if (a.acc_out) *(i4*)(a.acc_out + (long)m * N + n) = acc[i][j];
      float v[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float wsc = a.w_scale ? a.w_scale[a.w_scale_per_col ? n + e : 0] : 1.0f;
        v[e] = ((float)acc[i][j][e] * xsc) * wsc;
        if (a.bias) v[e] += load_bias<DT>(a.bias, a.bias_f32, n + e);
      }
      store4<DT>(a.out, (long)m * a.ldo + n, v);
    }
  }
}

// ---- activation quantisers -------------------------------------------------
template <int DT>
__device__ __forceinline__ float ld_act(const void* p, long i) {
  if (DT == MI355Q_F32) return ((const float*)p)[i];
  return Elem<DT == MI355Q_F32 ? MI355Q_F16 : DT>::to_f32(((const uint16_t*)p)[i]);
}

__device__ __forceinline__ int8_t sat_rne_s8(float y) {
  y = __builtin_rintf(y);                       // round half to even
  y = fminf(fmaxf(y, -128.0f), 127.0f);
  return (int8_t)(int)y;
}

// one workgroup per token row: absmax -> scale = absmax / 127 -> q = rne(x * (127 / absmax))
template <int DT>
__global__ void __launch_bounds__(256)
dynamic_int8_quant_kernel(int8_t* out, float* scales, const void* x, int K, const int* valid_rows) {
  const int row = blockIdx.x;
  if (valid_rows && row >= *valid_rows) return;
  __shared__ float red[4];
  float mx = 0.f;
  for (int k = threadIdx.x; k < K; k += 256) mx = fmaxf(mx, fabsf(ld_act<DT>(x, (long)row * K + k)));
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = mx;
  __syncthreads();
  mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  if (threadIdx.x == 0) scales[row] = mx / 127.0f;
  const float inv = 127.0f / mx;                // inf for an all-zero row
  for (int k = threadIdx.x; k < K; k += 256) {
    float y = ld_act<DT>(x, (long)row * K + k) * inv;
    if (y != y) y = 0.f;                        // 0 * inf
    out[(long)row * K + k] = sat_rne_s8(y);
  }
}

// static: the reciprocal of the scale is rounded to the input dtype first
template <int DT>
__global__ void __launch_bounds__(256)
static_int8_quant_kernel(int8_t* out, const void* x, const float* scale, int per_channel, long total, int K) {
  long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  float inv = 1.0f / scale[per_channel ? (int)(i % K) : 0];
  if (DT != MI355Q_F32) inv = Elem<DT == MI355Q_F32 ? MI355Q_F16 : DT>::to_f32(Elem<DT == MI355Q_F32 ? MI355Q_F16 : DT>::from_f32(inv));
  out[i] = sat_rne_s8(ld_act<DT>(x, i) * inv);
}

template <int DT>
int launch_gemm(const I8Args& a, hipStream_t st) {
  const int mtiles = (a.M + TM - 1) / TM, ntiles = (a.N + TN - 1) / TN;
  I8Args b = a;
  b.n_panels_swizzle = (ntiles % 8 == 0) ? 1 : 0;
  const size_t shmem = 2 * STAGE_BYTES;          // 128 KiB
  static hipError_t attr = hipFuncSetAttribute((const void*)w8a8_int8_gemm_kernel<DT>,
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
  MQ_REQUIRE(attr == hipSuccess, "w8a8_int8_gemm: cannot reserve %zu bytes of LDS: %s", shmem,
             hipGetErrorString(attr));
  hipLaunchKernelGGL((w8a8_int8_gemm_kernel<DT>), dim3(mtiles * ntiles), dim3(256), shmem, st, b);
  MQ_LAUNCH_CHECK("w8a8_int8_gemm");
  return 0;
}

}  // namespace
}  // namespace mi355q

using namespace mi355q;

extern "C" int mi355q_w8a8_int8_gemm(void* out, int32_t* acc_out, const int8_t* x, const int8_t* w,
                                     const float* x_scale, int x_scale_per_row, const float* w_scale,
                                     int w_scale_per_col, const void* bias, int bias_f32, int M, int N,
                                     int K, long ldx, long ldw, long ldo, int out_dtype, void* stream) {
  MQ_REQUIRE(M >= 0 && N > 0 && K > 0, "w8a8_int8_gemm: bad shape M=%d N=%d K=%d", M, N, K);
  if (M == 0) return 0;
  MQ_REQUIRE(out && x && w, "w8a8_int8_gemm: null pointer");
  MQ_REQUIRE(K % TK == 0, "w8a8_int8_gemm: K=%d must be a multiple of %d", K, TK);
  MQ_REQUIRE(N % 4 == 0, "w8a8_int8_gemm: N=%d must be a multiple of 4", N);
  MQ_REQUIRE(ldx % 16 == 0 && ldw % 16 == 0 && ldx >= K && ldw >= K,
             "w8a8_int8_gemm: operand row strides (%ld, %ld) must be >= K and multiples of 16", ldx, ldw);
  MQ_REQUIRE(ldo >= N && ldo % 4 == 0, "w8a8_int8_gemm: output row stride %ld must be >= N and a multiple of 4", ldo);
  MQ_REQUIRE(out_dtype >= MI355Q_F16 && out_dtype <= MI355Q_F32, "w8a8_int8_gemm: bad out dtype %d", out_dtype);
  I8Args a;
  a.out = out; a.acc_out = acc_out; a.x = x; a.w = w; a.x_scale = x_scale; a.w_scale = w_scale;
  a.bias = bias; a.M = M; a.N = N; a.K = K; a.ldx = ldx; a.ldw = ldw; a.ldo = ldo;
  a.x_scale_per_row = x_scale_per_row; a.w_scale_per_col = w_scale_per_col; a.bias_f32 = bias_f32;
  a.n_panels_swizzle = 0;
  if (out_dtype == MI355Q_F16) return launch_gemm<MI355Q_F16>(a, as_stream(stream));
  if (out_dtype == MI355Q_BF16) return launch_gemm<MI355Q_BF16>(a, as_stream(stream));
  return launch_gemm<MI355Q_F32>(a, as_stream(stream));
}

extern "C" int mi355q_dynamic_int8_quant(int8_t* out, float* scales, const void* x, int M, int K,
                                         int dtype, const int32_t* valid_rows, void* stream) {
  MQ_REQUIRE(M >= 0 && K > 0, "dynamic_int8_quant: bad shape M=%d K=%d", M, K);
  if (M == 0) return 0;
  MQ_REQUIRE(out && scales && x, "dynamic_int8_quant: null pointer");
  hipStream_t st = as_stream(stream);
  if (dtype == MI355Q_F16)
    hipLaunchKernelGGL((dynamic_int8_quant_kernel<MI355Q_F16>), dim3(M), dim3(256), 0, st, out, scales, x, K, valid_rows);
  else if (dtype == MI355Q_BF16)
    hipLaunchKernelGGL((dynamic_int8_quant_kernel<MI355Q_BF16>), dim3(M), dim3(256), 0, st, out, scales, x, K, valid_rows);
  else if (dtype == MI355Q_F32)
    hipLaunchKernelGGL((dynamic_int8_quant_kernel<MI355Q_F32>), dim3(M), dim3(256), 0, st, out, scales, x, K, valid_rows);
  else
    MQ_REQUIRE(false, "dynamic_int8_quant: bad dtype %d", dtype);
  MQ_LAUNCH_CHECK("dynamic_int8_quant");
  return 0;
}

extern "C" int mi355q_static_int8_quant(int8_t* out, const void* x, const float* scale, int per_channel,
                                        int M, int K, int dtype, void* stream) {
  MQ_REQUIRE(M >= 0 && K > 0, "static_int8_quant: bad shape M=%d K=%d", M, K);
  if (M == 0) return 0;
  MQ_REQUIRE(out && scale && x, "static_int8_quant: null pointer");
  const long total = (long)M * K;
  const unsigned blocks = (unsigned)((total + 255) / 256);
  hipStream_t st = as_stream(stream);
  if (dtype == MI355Q_F16)
    hipLaunchKernelGGL((static_int8_quant_kernel<MI355Q_F16>), dim3(blocks), dim3(256), 0, st, out, x, scale, per_channel, total, K);
  else if (dtype == MI355Q_BF16)
    hipLaunchKernelGGL((static_int8_quant_kernel<MI355Q_BF16>), dim3(blocks), dim3(256), 0, st, out, x, scale, per_channel, total, K);
  else if (dtype == MI355Q_F32)
    hipLaunchKernelGGL((static_int8_quant_kernel<MI355Q_F32>), dim3(blocks), dim3(256), 0, st, out, x, scale, per_channel, total, K);
  else
    MQ_REQUIRE(false, "static_int8_quant: bad dtype %d", dtype);
  MQ_LAUNCH_CHECK("static_int8_quant");
  return 0;
}
