// Elementwise glue between the GEMMs: SiLU-gate, fp8-e4m3fn activation
// quantisers (per token group, per token, static), the fused SiLU-gate + group
// quantiser, and the top-k sum.  All are HBM-bound: 16-byte loads per lane,
// fp32 arithmetic, one pass over the data.  Every kernel takes an optional
// device int32 `valid_rows` so padded (graph-captured) batches skip dead rows
// without a host synchronisation.
#include "common.h"

namespace mi355q {
namespace {

constexpr float FP8_MAX = 448.0f;

template <int DT> struct E16 { typedef Elem<DT> T; };

template <int DT>
__device__ __forceinline__ void unpack8(const u4& v, float* f) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f[2 * i] = Elem<DT>::to_f32((uint16_t)(v[i] & 0xffffu));
    f[2 * i + 1] = Elem<DT>::to_f32((uint16_t)(v[i] >> 16));
  }
}
template <int DT>
__device__ __forceinline__ u4 pack8(const float* f) {
  u4 v;
#pragma unroll
  for (int i = 0; i < 4; ++i)
    v[i] = (uint32_t)Elem<DT>::from_f32(f[2 * i]) | ((uint32_t)Elem<DT>::from_f32(f[2 * i + 1]) << 16);
  return v;
}
template <int DT>
__device__ __forceinline__ float round_act(float f) {
  return Elem<DT>::to_f32(Elem<DT>::from_f32(f));
}

__device__ __forceinline__ float silu_mul(float a, float b) {
  return a * (1.0f / (1.0f + expf(-a))) * b;      // left * sigmoid(left) * right
}

// 8 floats (already within +-448) -> 8 e4m3fn codes, round to nearest even
__device__ __forceinline__ u2 to_fp8x8(const float* y) {
  u2 r;
  int w0 = 0, w1 = 0;
  w0 = __builtin_amdgcn_cvt_pk_fp8_f32(y[0], y[1], w0, false);
  w0 = __builtin_amdgcn_cvt_pk_fp8_f32(y[2], y[3], w0, true);
  w1 = __builtin_amdgcn_cvt_pk_fp8_f32(y[4], y[5], w1, false);
  w1 = __builtin_amdgcn_cvt_pk_fp8_f32(y[6], y[7], w1, true);
  r.x = (uint32_t)w0;
  r.y = (uint32_t)w1;
  return r;
}

__device__ __forceinline__ float clamp448(float y) { return fminf(fmaxf(y, -FP8_MAX), FP8_MAX); }

// a / s for many a and one s, with the result of the IEEE division: the reciprocal estimate and
// its Newton step are made once per divisor, the quotient estimate and its two residual
// corrections once per dividend -- the same fused multiply-adds the division expands to, without
// the operand scaling that only matters when s, 1 / s, a / s or a residual leave the normal range.
// For the dynamic scales here s = max(absmax, 1e-10) / 448 is normal, |a / s| <= 448, and a
// residual can only underflow where the quotient is far below the smallest fp8 step.
struct SharedDivisor {
  float s, y;
  __device__ __forceinline__ explicit SharedDivisor(float s_) : s(s_) {
    const float y0 = __builtin_amdgcn_rcpf(s_);
    y = __builtin_fmaf(__builtin_fmaf(-s_, y0, 1.0f), y0, y0);
  }
  __device__ __forceinline__ float div(float a) const {
    const float q0 = a * y;
    const float q1 = __builtin_fmaf(__builtin_fmaf(-s, q0, a), y, q0);
    // the division's own last instruction: signed zeros, infinities and NaN as IEEE has them
    return __builtin_amdgcn_div_fixupf(__builtin_fmaf(__builtin_fmaf(-s, q1, a), y, q1), s, a);
  }
};

// ---- silu_and_mul: out[r, :d] = silu(x[r, :d]) * x[r, d:] -------------------
template <int DT>
__global__ void __launch_bounds__(256)
silu_and_mul_kernel(uint16_t* out, const uint16_t* x, long rows, int d, const int* valid_rows, int rpc) {
  const long nrow = valid_rows ? min(rows, (long)max(0, *valid_rows) * rpc) : rows;
  const int chunks = d / 8;
  const long total = nrow * chunks;
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < total; i += (long)gridDim.x * 256) {
    const long r = i / chunks;
    const int c = (int)(i - r * chunks);
    float a[8], b[8], y[8];
    unpack8<DT>(*(const u4*)(x + r * 2 * d + 8 * c), a);
    unpack8<DT>(*(const u4*)(x + r * 2 * d + d + 8 * c), b);
#pragma unroll
    for (int e = 0; e < 8; ++e) y[e] = silu_mul(a[e], b[e]);
    *(u4*)(out + r * d + 8 * c) = pack8<DT>(y);
  }
}

// ---- per-token-group fp8 quantisation (optionally fused behind SiLU-gate) ---
// A group of `gs` elements is handled by gs/8 adjacent lanes (gs in 64,128,256,512).
template <int DT, bool SILU>
__global__ void __launch_bounds__(256)
group_fp8_quant_kernel(uint8_t* out, float* scales, const uint16_t* x, long rows, int K, int gs,
                       const int* valid_rows, int rpc) {
  const long nrow = valid_rows ? min(rows, (long)max(0, *valid_rows) * rpc) : rows;
  const int chunks = K / 8;                      // 8-element chunks per output row
  const int lpg = gs / 8;                        // lanes per group (power of two <= 64)
  const long total = nrow * chunks;
  const long stride = (long)gridDim.x * 256;
  for (long i0 = (long)blockIdx.x * 256; i0 < total; i0 += stride) {
    const long i = i0 + threadIdx.x;
    const bool live = i < total;
    const long r = live ? i / chunks : 0;
    const int c = live ? (int)(i - r * chunks) : 0;
    float y[8];
    if (SILU) {
      float a[8], b[8];
      unpack8<DT>(*(const u4*)(x + r * 2 * K + 8 * c), a);
      unpack8<DT>(*(const u4*)(x + r * 2 * K + K + 8 * c), b);
      // the unfused sequence stores the gate output in the activation dtype
#pragma unroll
      for (int e = 0; e < 8; ++e) y[e] = round_act<DT>(silu_mul(a[e], b[e]));
    } else {
      unpack8<DT>(*(const u4*)(x + r * K + 8 * c), y);
    }
    float mx = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) mx = fmaxf(mx, fabsf(y[e]));
    if (!live) mx = 0.f;
    mx = lane_group_max(mx, lpg);
    const float s = fmaxf(mx, 1e-10f) / FP8_MAX;
    const SharedDivisor by_s(s);
    float q[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) q[e] = clamp448(by_s.div(y[e]));
    if (live) {
      *(u2*)(out + r * K + 8 * c) = to_fp8x8(q);
      if ((c % lpg) == 0) scales[r * (K / gs) + c / lpg] = s;
    }
  }
}

// ---- per-token fp8 (one workgroup per row) and static fp8 --------------------
template <int DT>
__global__ void __launch_bounds__(256)
token_fp8_quant_kernel(uint8_t* out, float* scales, const uint16_t* x, int K, const int* valid_rows) {
  const long row = blockIdx.x;
  if (valid_rows && row >= *valid_rows) return;
  __shared__ float red[4];
  float mx = 0.f;
  for (int k = threadIdx.x; k < K; k += 256) mx = fmaxf(mx, fabsf(Elem<DT>::to_f32(x[row * K + k])));
  mx = wave_max(mx);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = mx;
  __syncthreads();
  mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  const float s = fmaxf(mx, 1e-10f) / FP8_MAX;
  if (threadIdx.x == 0) scales[row] = s;
  const SharedDivisor by_s(s);
  for (int k = threadIdx.x; k < K; k += 256) {
    const float y = clamp448(by_s.div(Elem<DT>::to_f32(x[row * K + k])));
    int w = __builtin_amdgcn_cvt_pk_fp8_f32(y, y, 0, false);
    out[row * K + k] = (uint8_t)(w & 0xff);
  }
}

// FUSE: 0 = quantise x; 1 = silu(x[:, :K]) * x[:, K:] first; 2 = x[:, :K] * x[:, K:] first
template <int DT, int FUSE>
__global__ void __launch_bounds__(256)
static_fp8_quant_kernel(uint8_t* out, const uint16_t* x, const float* scale, long rows, int K,
                        const int* valid_rows, int rpc) {
  const long nrow = valid_rows ? min(rows, (long)max(0, *valid_rows) * rpc) : rows;
  const float s = *scale;
  if ((K & 7) == 0) {
    // 8 elements per lane and step: 16-byte loads, 8-byte stores
    const int chunks = K / 8;
    const long total = nrow * chunks;
    for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < total; i += (long)gridDim.x * 256) {
      const long r = i / chunks;
      const int c = (int)(i - r * chunks);
      float v[8];
      if (FUSE) {
        float l[8], g[8];
        unpack8<DT>(*(const u4*)(x + r * 2 * K + 8 * c), l);
        unpack8<DT>(*(const u4*)(x + r * 2 * K + K + 8 * c), g);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = round_act<DT>(FUSE == 1 ? silu_mul(l[e], g[e]) : l[e] * g[e]);
      } else {
        unpack8<DT>(*(const u4*)(x + r * K + 8 * c), v);
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = clamp448(v[e] / s);
      *(u2*)(out + r * K + 8 * c) = to_fp8x8(v);
    }
    return;
  }
  const long total = nrow * K;
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < total; i += (long)gridDim.x * 256) {
    float v;
    if (FUSE) {
      const long r = i / K;
      const int c = (int)(i - r * K);
      const float l = Elem<DT>::to_f32(x[r * 2 * K + c]), g = Elem<DT>::to_f32(x[r * 2 * K + K + c]);
      v = round_act<DT>(FUSE == 1 ? silu_mul(l, g) : l * g);
    } else {
      v = Elem<DT>::to_f32(x[i]);
    }
    const float y = clamp448(v / s);
    int w = __builtin_amdgcn_cvt_pk_fp8_f32(y, y, 0, false);
    out[i] = (uint8_t)(w & 0xff);
  }
}

// ---- moe_sum: out[m, :] = sum_t in[m, t, :] in fp32 --------------------------
template <int DT_IN, int DT_OUT>
__global__ void __launch_bounds__(256)
moe_sum_kernel(void* out, const uint16_t* in, long rows, int T, int K, const int* valid_rows) {
  const long nrow = valid_rows ? min(rows, (long)max(0, *valid_rows)) : rows;
  const int chunks = K / 8;
  const long total = nrow * chunks;
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < total; i += (long)gridDim.x * 256) {
    const long r = i / chunks;
    const int c = (int)(i - r * chunks);
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (int t = 0; t < T; ++t) {
      float v[8];
      unpack8<DT_IN>(*(const u4*)(in + (r * T + t) * K + 8 * c), v);
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] += v[e];
    }
    if (DT_OUT == MI355Q_F32) {
      float* o = (float*)out + r * K + 8 * c;
      *(f4*)o = (f4){acc[0], acc[1], acc[2], acc[3]};
      *(f4*)(o + 4) = (f4){acc[4], acc[5], acc[6], acc[7]};
    } else {
      *(u4*)((uint16_t*)out + r * K + 8 * c) = pack8<DT_OUT == MI355Q_F32 ? MI355Q_F16 : DT_OUT>(acc);
    }
  }
}

// ---- RMS norm (+ residual add) (+ quantisation of the normalised row) -------
// One workgroup per row, two passes over it (the second one hits the L2):
//   z = x (+ residual, rounded to the activation type and written back to residual)
//   n = act(z * rsqrt(mean(z^2) + eps)),  o = act(n * weight)
// then QM 0: o; 1: e4m3fn(clamp(o / scale)); 2: e4m3fn per group of gs with its own scale
// absmax / 448; 3: int8 rne(o * act(1 / scale)) -- each exactly what the separate
// quantisation operator makes of the stored o.
template <int DT, bool ADD, int QM>
__global__ void __launch_bounds__(256)
rms_norm_kernel(void* out, float* out_scales, const uint16_t* x, uint16_t* residual, const uint16_t* weight,
                const float* scale, float eps, int K, int gs) {
  const long row = blockIdx.x;
  const int chunks = K / 8;
  const uint16_t* xr = x + row * K;
  uint16_t* rr = ADD ? residual + row * K : nullptr;
  __shared__ float red[4];
  float ss = 0.f;
  for (int c = threadIdx.x; c < chunks; c += 256) {
    float v[8];
    unpack8<DT>(*(const u4*)(xr + 8 * c), v);
    if (ADD) {
      float r[8];
      unpack8<DT>(*(const u4*)(rr + 8 * c), r);
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = round_act<DT>(v[e] + r[e]);
      *(u4*)(rr + 8 * c) = pack8<DT>(v);
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) ss += v[e] * v[e];
  }
  ss = wave_sum(ss);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
  __syncthreads();
  ss = (red[0] + red[1]) + (red[2] + red[3]);
  const float rs = rsqrtf(ss / (float)K + eps);
  float qs = 1.f;
  if (QM == 1) qs = *scale;
  if (QM == 3) qs = round_act<DT>(1.0f / *scale);
  const int lpg = QM == 2 ? gs / 8 : 1;
  const int padded = (chunks + 255) / 256 * 256;       // every lane stays in the loop for the group shuffles
  for (int c0 = threadIdx.x; c0 < padded; c0 += 256) {
    const bool live = c0 < chunks;
    const int c = live ? c0 : 0;
    float v[8], w[8];
    // a thread re-reads only what it wrote itself in the first pass
    unpack8<DT>(*(const u4*)((ADD ? (const uint16_t*)rr : xr) + 8 * c), v);
    unpack8<DT>(*(const u4*)(weight + 8 * c), w);
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = round_act<DT>(round_act<DT>(v[e] * rs) * w[e]);
    if (QM == 0) {
      if (live) *(u4*)((uint16_t*)out + row * K + 8 * c) = pack8<DT>(v);
    } else if (QM == 1) {
      float q[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) q[e] = clamp448(v[e] / qs);
      if (live) *(u2*)((uint8_t*)out + row * K + 8 * c) = to_fp8x8(q);
    } else if (QM == 2) {
      float mx = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) mx = fmaxf(mx, fabsf(v[e]));
      if (!live) mx = 0.f;
      mx = lane_group_max(mx, lpg);
      const float sg = fmaxf(mx, 1e-10f) / FP8_MAX;
      const SharedDivisor by_sg(sg);
      float q[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) q[e] = clamp448(by_sg.div(v[e]));
      if (live) {
        *(u2*)((uint8_t*)out + row * K + 8 * c) = to_fp8x8(q);
        if ((c % lpg) == 0) out_scales[row * (K / gs) + c / lpg] = sg;
      }
    } else {
      uint32_t lo = 0, hi = 0;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float a = fminf(fmaxf(__builtin_rintf(v[e] * qs), -128.f), 127.f);
        float b = fminf(fmaxf(__builtin_rintf(v[4 + e] * qs), -128.f), 127.f);
        lo |= ((uint32_t)(int)a & 0xffu) << (8 * e);
        hi |= ((uint32_t)(int)b & 0xffu) << (8 * e);
      }
      if (live) *(u2*)((uint8_t*)out + row * K + 8 * c) = (u2){lo, hi};
    }
  }
}

// The same operator for rows of up to 8192 elements: the row (and the weight vector) is loaded once,
// up to four 16-byte pieces per lane with all loads in flight together, and both passes run from
// registers -- the loop version above waits for one piece at a time and reads the row twice.  Same
// arithmetic in the same order per element; the sum of squares adds the lane's pieces in the same
// order too, so the results are bit-identical.
template <int DT, bool ADD, int QM>
__global__ void __launch_bounds__(256)
rms_norm_row_kernel(void* out, float* out_scales, const uint16_t* x, uint16_t* residual, const uint16_t* weight,
                    const float* scale, float eps, int K, int gs) {
  const long row = blockIdx.x;
  const int chunks = K / 8;
  const uint16_t* xr = x + row * K;
  uint16_t* rr = ADD ? residual + row * K : nullptr;
  __shared__ float red[4];
  u4 xv[4], rv[4], wv[4];
  bool live[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int c0 = threadIdx.x + 256 * i;
    live[i] = c0 < chunks;
    const int c = live[i] ? c0 : 0;
    xv[i] = *(const u4*)(xr + 8 * c);
    if (ADD) rv[i] = *(const u4*)(rr + 8 * c);
    wv[i] = *(const u4*)(weight + 8 * c);
  }
  float v[4][8];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    unpack8<DT>(xv[i], v[i]);
    if (ADD) {
      float r[8];
      unpack8<DT>(rv[i], r);
#pragma unroll
      for (int e = 0; e < 8; ++e) v[i][e] = round_act<DT>(v[i][e] + r[e]);
      if (live[i]) *(u4*)(rr + 8 * (threadIdx.x + 256 * i)) = pack8<DT>(v[i]);
    }
    if (live[i]) {
#pragma unroll
      for (int e = 0; e < 8; ++e) ss += v[i][e] * v[i][e];
    }
  }
  ss = wave_sum(ss);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
  __syncthreads();
  ss = (red[0] + red[1]) + (red[2] + red[3]);
  const float rs = rsqrtf(ss / (float)K + eps);
  float qs = 1.f;
  if (QM == 1) qs = *scale;
  if (QM == 3) qs = round_act<DT>(1.0f / *scale);
  const int lpg = QM == 2 ? gs / 8 : 1;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if (256 * i >= chunks) break;                       // (uniform: every lane stays for the group shuffles)
    const int c = threadIdx.x + 256 * i;
    float w[8];
    unpack8<DT>(wv[i], w);
    float* y = v[i];
#pragma unroll
    for (int e = 0; e < 8; ++e) y[e] = round_act<DT>(round_act<DT>(y[e] * rs) * w[e]);
    if (QM == 0) {
      if (live[i]) *(u4*)((uint16_t*)out + row * K + 8 * c) = pack8<DT>(y);
    } else if (QM == 1) {
      float q[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) q[e] = clamp448(y[e] / qs);
      if (live[i]) *(u2*)((uint8_t*)out + row * K + 8 * c) = to_fp8x8(q);
    } else if (QM == 2) {
      float mx = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) mx = fmaxf(mx, fabsf(y[e]));
      if (!live[i]) mx = 0.f;
      mx = lane_group_max(mx, lpg);
      const float sg = fmaxf(mx, 1e-10f) / FP8_MAX;
      const SharedDivisor by_sg(sg);
      float q[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) q[e] = clamp448(by_sg.div(y[e]));
      if (live[i]) {
        *(u2*)((uint8_t*)out + row * K + 8 * c) = to_fp8x8(q);
        if ((c % lpg) == 0) out_scales[row * (K / gs) + c / lpg] = sg;
      }
    } else {
      uint32_t lo = 0, hi = 0;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float a = fminf(fmaxf(__builtin_rintf(y[e] * qs), -128.f), 127.f);
        float b = fminf(fmaxf(__builtin_rintf(y[4 + e] * qs), -128.f), 127.f);
        lo |= ((uint32_t)(int)a & 0xffu) << (8 * e);
        hi |= ((uint32_t)(int)b & 0xffu) << (8 * e);
      }
      if (live[i]) *(u2*)((uint8_t*)out + row * K + 8 * c) = (u2){lo, hi};
    }
  }
}

template <int DT, bool ADD>
void launch_rms(int qm, long rows, hipStream_t st, void* out, float* out_scales, const uint16_t* x,
                uint16_t* residual, const uint16_t* weight, const float* scale, float eps, int K, int gs) {
  const dim3 grid((unsigned)rows);
  if (K <= 8192) {
    switch (qm) {
      case 0: hipLaunchKernelGGL((rms_norm_row_kernel<DT, ADD, 0>), grid, dim3(256), 0, st, out, out_scales, x, residual, weight, scale, eps, K, gs); break;
      case 1: hipLaunchKernelGGL((rms_norm_row_kernel<DT, ADD, 1>), grid, dim3(256), 0, st, out, out_scales, x, residual, weight, scale, eps, K, gs); break;
      case 2: hipLaunchKernelGGL((rms_norm_row_kernel<DT, ADD, 2>), grid, dim3(256), 0, st, out, out_scales, x, residual, weight, scale, eps, K, gs); break;
      default: hipLaunchKernelGGL((rms_norm_row_kernel<DT, ADD, 3>), grid, dim3(256), 0, st, out, out_scales, x, residual, weight, scale, eps, K, gs); break;
    }
    return;
  }
  switch (qm) {
    case 0: hipLaunchKernelGGL((rms_norm_kernel<DT, ADD, 0>), grid, dim3(256), 0, st, out, out_scales, x, residual, weight, scale, eps, K, gs); break;
    case 1: hipLaunchKernelGGL((rms_norm_kernel<DT, ADD, 1>), grid, dim3(256), 0, st, out, out_scales, x, residual, weight, scale, eps, K, gs); break;
    case 2: hipLaunchKernelGGL((rms_norm_kernel<DT, ADD, 2>), grid, dim3(256), 0, st, out, out_scales, x, residual, weight, scale, eps, K, gs); break;
    default: hipLaunchKernelGGL((rms_norm_kernel<DT, ADD, 3>), grid, dim3(256), 0, st, out, out_scales, x, residual, weight, scale, eps, K, gs); break;
  }
}

inline unsigned grid_for(long items) {
  long b = (items + 255) / 256;
  long cap = (long)device_cu_count() * 16;
  return (unsigned)(b < 1 ? 1 : (b > cap ? cap : b));
}

}  // namespace
}  // namespace mi355q

using namespace mi355q;

#define MQ_DISPATCH_16(dtype, CALL_F16, CALL_BF16, what)             \
  do {                                                               \
    if ((dtype) == MI355Q_F16) { CALL_F16; }                         \
    else if ((dtype) == MI355Q_BF16) { CALL_BF16; }                  \
    else MQ_REQUIRE(false, what ": dtype %d must be f16 or bf16", (int)(dtype)); \
  } while (0)

extern "C" int mi355q_silu_and_mul(void* out, const void* x, long rows, int d, int dtype,
                                   const int32_t* valid_rows, int rows_per_count, void* stream) {
  if (rows_per_count < 1) rows_per_count = 1;
  MQ_REQUIRE(rows >= 0 && d > 0 && d % 8 == 0, "silu_and_mul: bad shape rows=%ld d=%d (d %% 8 == 0)", rows, d);
  if (rows == 0) return 0;
  MQ_REQUIRE(out && x, "silu_and_mul: null pointer");
  hipStream_t st = as_stream(stream);
  unsigned g = grid_for(rows * (d / 8));
  MQ_DISPATCH_16(dtype,
    hipLaunchKernelGGL((silu_and_mul_kernel<MI355Q_F16>), dim3(g), dim3(256), 0, st, (uint16_t*)out, (const uint16_t*)x, rows, d, valid_rows, rows_per_count),
    hipLaunchKernelGGL((silu_and_mul_kernel<MI355Q_BF16>), dim3(g), dim3(256), 0, st, (uint16_t*)out, (const uint16_t*)x, rows, d, valid_rows, rows_per_count),
    "silu_and_mul");
  MQ_LAUNCH_CHECK("silu_and_mul");
  return 0;
}

extern "C" int mi355q_fp8_group_quant(uint8_t* out, float* scales, const void* x, long rows, int K,
                                      int group_size, int fuse_silu_mul, int dtype,
                                      const int32_t* valid_rows, int rows_per_count, void* stream) {
  if (rows_per_count < 1) rows_per_count = 1;
  MQ_REQUIRE(rows >= 0 && K > 0, "fp8_group_quant: bad shape rows=%ld K=%d", rows, K);
  if (rows == 0) return 0;
  MQ_REQUIRE(out && scales && x, "fp8_group_quant: null pointer");
  MQ_REQUIRE(group_size == 64 || group_size == 128 || group_size == 256 || group_size == 512,
             "fp8_group_quant: group_size=%d must be 64, 128, 256 or 512", group_size);
  MQ_REQUIRE(K % group_size == 0, "fp8_group_quant: K=%d must be a multiple of group_size=%d", K, group_size);
  hipStream_t st = as_stream(stream);
  // whole groups must sit inside one workgroup pass: 256 lanes cover 2048 elements
  unsigned g = grid_for(rows * (K / 8));
  if (fuse_silu_mul) {
    MQ_DISPATCH_16(dtype,
      hipLaunchKernelGGL((group_fp8_quant_kernel<MI355Q_F16, true>), dim3(g), dim3(256), 0, st, out, scales, (const uint16_t*)x, rows, K, group_size, valid_rows, rows_per_count),
      hipLaunchKernelGGL((group_fp8_quant_kernel<MI355Q_BF16, true>), dim3(g), dim3(256), 0, st, out, scales, (const uint16_t*)x, rows, K, group_size, valid_rows, rows_per_count),
      "fp8_group_quant");
  } else {
    MQ_DISPATCH_16(dtype,
      hipLaunchKernelGGL((group_fp8_quant_kernel<MI355Q_F16, false>), dim3(g), dim3(256), 0, st, out, scales, (const uint16_t*)x, rows, K, group_size, valid_rows, rows_per_count),
      hipLaunchKernelGGL((group_fp8_quant_kernel<MI355Q_BF16, false>), dim3(g), dim3(256), 0, st, out, scales, (const uint16_t*)x, rows, K, group_size, valid_rows, rows_per_count),
      "fp8_group_quant");
  }
  MQ_LAUNCH_CHECK("fp8_group_quant");
  return 0;
}

extern "C" int mi355q_fp8_token_quant(uint8_t* out, float* scales, const void* x, int rows, int K, int dtype,
                                      const int32_t* valid_rows, void* stream) {
  MQ_REQUIRE(rows >= 0 && K > 0, "fp8_token_quant: bad shape rows=%d K=%d", rows, K);
  if (rows == 0) return 0;
  MQ_REQUIRE(out && scales && x, "fp8_token_quant: null pointer");
  hipStream_t st = as_stream(stream);
  MQ_DISPATCH_16(dtype,
    hipLaunchKernelGGL((token_fp8_quant_kernel<MI355Q_F16>), dim3(rows), dim3(256), 0, st, out, scales, (const uint16_t*)x, K, valid_rows),
    hipLaunchKernelGGL((token_fp8_quant_kernel<MI355Q_BF16>), dim3(rows), dim3(256), 0, st, out, scales, (const uint16_t*)x, K, valid_rows),
    "fp8_token_quant");
  MQ_LAUNCH_CHECK("fp8_token_quant");
  return 0;
}

extern "C" int mi355q_fp8_static_quant(uint8_t* out, const void* x, const float* scale, long rows, int K,
                                       int fuse_silu_mul, int dtype, const int32_t* valid_rows,
                                       int rows_per_count, void* stream) {
  if (rows_per_count < 1) rows_per_count = 1;
  MQ_REQUIRE(rows >= 0 && K > 0, "fp8_static_quant: bad shape rows=%ld K=%d", rows, K);
  if (rows == 0) return 0;
  MQ_REQUIRE(out && scale && x, "fp8_static_quant: null pointer");
  hipStream_t st = as_stream(stream);
  unsigned g = grid_for((K & 7) == 0 ? rows * (K / 8) : rows * K);
  MQ_REQUIRE(fuse_silu_mul >= 0 && fuse_silu_mul <= 2, "fp8_static_quant: unknown fusion %d", fuse_silu_mul);
  if (fuse_silu_mul == 1) {
    MQ_DISPATCH_16(dtype,
      hipLaunchKernelGGL((static_fp8_quant_kernel<MI355Q_F16, 1>), dim3(g), dim3(256), 0, st, out, (const uint16_t*)x, scale, rows, K, valid_rows, rows_per_count),
      hipLaunchKernelGGL((static_fp8_quant_kernel<MI355Q_BF16, 1>), dim3(g), dim3(256), 0, st, out, (const uint16_t*)x, scale, rows, K, valid_rows, rows_per_count),
      "fp8_static_quant");
  } else if (fuse_silu_mul == 2) {
    MQ_DISPATCH_16(dtype,
      hipLaunchKernelGGL((static_fp8_quant_kernel<MI355Q_F16, 2>), dim3(g), dim3(256), 0, st, out, (const uint16_t*)x, scale, rows, K, valid_rows, rows_per_count),
      hipLaunchKernelGGL((static_fp8_quant_kernel<MI355Q_BF16, 2>), dim3(g), dim3(256), 0, st, out, (const uint16_t*)x, scale, rows, K, valid_rows, rows_per_count),
      "fp8_static_quant");
  } else {
    MQ_DISPATCH_16(dtype,
      hipLaunchKernelGGL((static_fp8_quant_kernel<MI355Q_F16, 0>), dim3(g), dim3(256), 0, st, out, (const uint16_t*)x, scale, rows, K, valid_rows, rows_per_count),
      hipLaunchKernelGGL((static_fp8_quant_kernel<MI355Q_BF16, 0>), dim3(g), dim3(256), 0, st, out, (const uint16_t*)x, scale, rows, K, valid_rows, rows_per_count),
      "fp8_static_quant");
  }
  MQ_LAUNCH_CHECK("fp8_static_quant");
  return 0;
}

extern "C" int mi355q_moe_sum(void* out, const void* in, long rows, int topk, int K, int in_dtype,
                              int out_dtype, const int32_t* valid_rows, void* stream) {
  MQ_REQUIRE(rows >= 0 && topk > 0 && K > 0 && K % 8 == 0, "moe_sum: bad shape rows=%ld topk=%d K=%d (K %% 8 == 0)", rows, topk, K);
  if (rows == 0) return 0;
  MQ_REQUIRE(out && in, "moe_sum: null pointer");
  MQ_REQUIRE(in_dtype == MI355Q_F16 || in_dtype == MI355Q_BF16, "moe_sum: input dtype %d must be f16 or bf16", in_dtype);
  MQ_REQUIRE(out_dtype == in_dtype || out_dtype == MI355Q_F32, "moe_sum: output dtype %d must equal the input's or be f32", out_dtype);
  hipStream_t st = as_stream(stream);
  unsigned g = grid_for(rows * (K / 8));
  const uint16_t* p = (const uint16_t*)in;
  if (in_dtype == MI355Q_F16 && out_dtype == MI355Q_F16)
    hipLaunchKernelGGL((moe_sum_kernel<MI355Q_F16, MI355Q_F16>), dim3(g), dim3(256), 0, st, out, p, rows, topk, K, valid_rows);
  else if (in_dtype == MI355Q_F16)
    hipLaunchKernelGGL((moe_sum_kernel<MI355Q_F16, MI355Q_F32>), dim3(g), dim3(256), 0, st, out, p, rows, topk, K, valid_rows);
  else if (out_dtype == MI355Q_BF16)
    hipLaunchKernelGGL((moe_sum_kernel<MI355Q_BF16, MI355Q_BF16>), dim3(g), dim3(256), 0, st, out, p, rows, topk, K, valid_rows);
  else
    hipLaunchKernelGGL((moe_sum_kernel<MI355Q_BF16, MI355Q_F32>), dim3(g), dim3(256), 0, st, out, p, rows, topk, K, valid_rows);
  MQ_LAUNCH_CHECK("moe_sum");
  return 0;
}

// ---- fp8-e4m3fn -> f16 / bf16, exact (every e4m3fn value is representable in both) ----
template <int DT>
__global__ void __launch_bounds__(256)
fp8_to_half_kernel(uint16_t* out, const uint32_t* in, long words) {
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < words; i += (long)gridDim.x * 256) {
    const int w = (int)in[i];
    const f2 lo = __builtin_amdgcn_cvt_pk_f32_fp8(w, false), hi = __builtin_amdgcn_cvt_pk_f32_fp8(w, true);
    uint2 o;
    o.x = (uint32_t)Elem<DT>::from_f32(lo.x) | ((uint32_t)Elem<DT>::from_f32(lo.y) << 16);
    o.y = (uint32_t)Elem<DT>::from_f32(hi.x) | ((uint32_t)Elem<DT>::from_f32(hi.y) << 16);
    *(uint2*)(out + 4 * i) = o;
  }
}

extern "C" int mi355q_fp8_to_half(void* out, const uint8_t* in, long n, int out_dtype, void* stream) {
  MQ_REQUIRE(n >= 0 && n % 4 == 0, "fp8_to_half: element count %ld must be a multiple of 4", n);
  if (n == 0) return 0;
  MQ_REQUIRE(out && in, "fp8_to_half: null pointer");
  MQ_REQUIRE(out_dtype == MI355Q_F16 || out_dtype == MI355Q_BF16, "fp8_to_half: output dtype %d must be f16 or bf16", out_dtype);
  hipStream_t st = as_stream(stream);
  const unsigned g = grid_for(n / 4);
  if (out_dtype == MI355Q_F16)
    hipLaunchKernelGGL((fp8_to_half_kernel<MI355Q_F16>), dim3(g), dim3(256), 0, st, (uint16_t*)out, (const uint32_t*)in, n / 4);
  else
    hipLaunchKernelGGL((fp8_to_half_kernel<MI355Q_BF16>), dim3(g), dim3(256), 0, st, (uint16_t*)out, (const uint32_t*)in, n / 4);
  MQ_LAUNCH_CHECK("fp8_to_half");
  return 0;
}

extern "C" int mi355q_rms_norm(void* out, float* out_scales, const void* x, void* residual, const void* weight,
                               const float* scale, float eps, long rows, int K, int quant_mode, int group_size,
                               int dtype, void* stream) {
  MQ_REQUIRE(rows >= 0 && K > 0 && K % 8 == 0, "rms_norm: bad shape rows=%ld K=%d (K %% 8 == 0)", rows, K);
  if (rows == 0) return 0;
  MQ_REQUIRE(out && x && weight, "rms_norm: null pointer");
  MQ_REQUIRE(rows <= 0x7fffffffL, "rms_norm: too many rows");
  MQ_REQUIRE(quant_mode >= 0 && quant_mode <= 3, "rms_norm: quant_mode %d must be 0..3", quant_mode);
  MQ_REQUIRE(dtype == MI355Q_F16 || dtype == MI355Q_BF16, "rms_norm: dtype %d must be f16 or bf16", dtype);
  if (quant_mode == 1 || quant_mode == 3) MQ_REQUIRE(scale, "rms_norm: static scale missing");
  if (quant_mode == 2) {
    MQ_REQUIRE(out_scales, "rms_norm: group scales output missing");
    MQ_REQUIRE((group_size == 64 || group_size == 128 || group_size == 256 || group_size == 512) && K % group_size == 0,
               "rms_norm: group_size %d must be 64..512 (a power of two) and divide K=%d", group_size, K);
  }
  hipStream_t st = as_stream(stream);
  const long grid = rows;
  const uint16_t* xp = (const uint16_t*)x;
  uint16_t* rp = (uint16_t*)residual;
  const uint16_t* wp = (const uint16_t*)weight;
  if (dtype == MI355Q_F16) {
    if (residual) launch_rms<MI355Q_F16, true>(quant_mode, grid, st, out, out_scales, xp, rp, wp, scale, eps, K, group_size);
    else launch_rms<MI355Q_F16, false>(quant_mode, grid, st, out, out_scales, xp, rp, wp, scale, eps, K, group_size);
  } else {
    if (residual) launch_rms<MI355Q_BF16, true>(quant_mode, grid, st, out, out_scales, xp, rp, wp, scale, eps, K, group_size);
    else launch_rms<MI355Q_BF16, false>(quant_mode, grid, st, out, out_scales, xp, rp, wp, scale, eps, K, group_size);
  }
  MQ_LAUNCH_CHECK("rms_norm");
  return 0;
}
