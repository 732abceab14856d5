// W8A8 int8 GEMM on the gfx950 int8 MFMA (v_mfma_i32_16x16x64_i8) with the
// per-token x per-channel scales (and bias) fused into the epilogue, plus the
// per-token / static int8 activation quantisers that feed it.
//
// GEMM: out[M, N] = (xq[M, K] . wq[N, K]^T in int32) * x_scale[m] * w_scale[n].
// Both operands are K-contiguous (that is what the MFMA lanes consume: 16
// consecutive k per lane).  Workgroup tile 256 x 256, K step 64, eight
// wavefronts 2 (M) x 4 (N), each 128 rows x 64 columns = 8 x 4 MFMA tiles (128
// int32 accumulator registers, two wavefronts per SIMD so one's LDS reads hide
// behind the other's MFMAs).  Tiles go from global memory straight into LDS (global_load ...
// lds, 16 B per lane, no staging registers) with a 16-byte-chunk XOR swizzle
// so a 128-bit LDS operand read hits 16 different bank groups; LDS is a ring
// of 4 K tiles of 64, three of them in flight while one feeds the MFMAs.  The weights take the A operand slot so that each lane
// ends up with 4 consecutive output columns (one 8-byte store).
#include "common.h"

namespace mi355q {
namespace {

constexpr int TM = 256, TN = 256, TK = 64;
constexpr int NSTAGE = 4;                         // LDS ring: 3 K tiles in flight behind the one in use
constexpr int TILE_BYTES = 256 * TK;              // one operand tile (16 KiB)
constexpr int STAGE_BYTES = 2 * TILE_BYTES;       // x tile + w tile
constexpr int CHUNKS = TK / 16;                   // 16-byte chunks per tile row
constexpr int ROWS_PER_COPY = 64 / CHUNKS;        // tile rows moved by one wavefront copy

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

// 16-byte chunk `chunk` of a 64-byte tile row lives in slot chunk ^ ((row >> 1) & 3).
// Measured on MI355X with a 16-wavefront ds_read_b128 loop: the MFMA operand
// read (lane = row + 16 * chunk) runs at the full 230 B/clk/CU with this
// swizzle and at half that with none or with (row >> 2) & 3.
__device__ __forceinline__ int swz(int row, int chunk) { return chunk ^ ((row >> 1) & 3); }

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

// one wavefront instruction copies 64 x 16 B from global memory straight into
// 1 KiB of LDS (lane l lands at base + 16 l); no registers, no LDS store
__device__ __forceinline__ void dma16(const void* gptr, void* lds_wave_base) {
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)gptr,
                                   (__attribute__((address_space(3))) void*)lds_wave_base, 16, 0, 0);
}

#ifndef MQ_I8_WAVES_N
#define MQ_I8_WAVES_N 4
#endif
constexpr int WAVES_N = MQ_I8_WAVES_N;            // wavefronts along N (2 along M)
constexpr int GEMM_THREADS = 128 * WAVES_N;
constexpr int NI = 16 / WAVES_N, NJ = 8;          // MFMA tiles per wavefront: NI*16 columns x 128 rows

template <int DT>
__global__ void __launch_bounds__(GEMM_THREADS, 1)
w8a8_int8_gemm_kernel(I8Args a) {
  extern __shared__ __align__(16) unsigned char lds[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l16 = lane & 15, kq = lane >> 4;
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  if (NI * NJ * 4 > 128) use_agpr_accumulators();
  const int M = a.M, N = a.N, K = a.K;

  // tile coordinates; with the swizzle, the workgroups that land on one XCD
  // (ids congruent mod 8) sweep all row tiles of the same weight panels
  const int mtiles = (M + TM - 1) / TM;
  int pid = blockIdx.x, tm, tn;
  if (a.n_panels_swizzle) {
    const int x = pid & 7, j = pid >> 3;
    tm = j % mtiles;
    tn = (j / mtiles) * 8 + x;
  } else {
    tm = pid % mtiles;
    tn = pid / mtiles;
  }
  const int m0 = tm * TM, n0 = tn * TN;

  i4 acc[NI][NJ];    // [n tile][m tile]: weights are the MFMA "A" operand
#pragma unroll
  for (int i = 0; i < NI; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j) acc[i][j] = (i4){0, 0, 0, 0};

  // global -> LDS: an operand tile is 256 rows x TK bytes; one wavefront copy
  // moves 1 KiB = ROWS_PER_COPY rows (lane = CHUNKS * row + slot); slot p of
  // row r holds the 16-byte chunk swz(r, p) of that row, which makes the MFMA
  // operand reads below bank-conflict free.
  constexpr int COPIES = 256 / ROWS_PER_COPY / (2 * WAVES_N);   // per wavefront and operand
  const int crow = lane / CHUNKS, cslot = lane % CHUNKS;
  // 32-bit byte offsets from the tile's first row (rows past the matrix edge
  // re-read the last row; their results are never stored)
  uint32_t xo[COPIES], wo[COPIES];
#pragma unroll
  for (int p = 0; p < COPIES; ++p) {
    const int r = (wave * COPIES + p) * ROWS_PER_COPY + crow;   // row of the tile, 0..255
    const int chunk = swz(r, cslot);
    xo[p] = (uint32_t)((min(m0 + r, M - 1) - m0) * a.ldx + 16 * chunk);
    wo[p] = (uint32_t)((min(n0 + r, N - 1) - n0) * a.ldw + 16 * chunk);
  }
  const int8_t* xtile = a.x + (long)m0 * a.ldx;
  const int8_t* wtile = a.w + (long)n0 * a.ldw;
  auto issue = [&](int stage, int k0) {
    unsigned char* xs = lds + stage * STAGE_BYTES + wave * COPIES * 1024;
    unsigned char* ws = xs + TILE_BYTES;
    const int8_t* xk = xtile + k0;
    const int8_t* wk = wtile + k0;
#pragma unroll
    for (int p = 0; p < COPIES; ++p) {
      dma16(xk + xo[p], xs + p * 1024);
      dma16(wk + wo[p], ws + p * 1024);
    }
  };

  // per-lane LDS read address: row l16 of a 16-row tile, logical chunk kq; the
  // swizzle term only depends on the row modulo 16, so it is the same for
  // every tile and tiles differ by a compile-time offset
  const uint32_t lo = (uint32_t)(l16 * TK + swz(l16, kq) * 16);
  const uint32_t xwave = wm * (16 * NJ) * TK, wwave = TILE_BYTES + wn * (16 * NI) * TK;

  // Ring of NSTAGE K tiles in LDS and two register sets of MFMA operands.
  // Iteration kt multiplies tile kt (already in registers) while it reads
  // tile kt+1 from LDS into the other register set and starts the copy of
  // tile kt+3; tile kt+2 is in flight.  The barrier at the top guarantees that
  // everybody's copies of tile kt+1 have landed and that the buffer refilled
  // next (tile kt-1's) is no longer read.  Every iteration issues exactly one
  // tile (the tail re-reads the last one into a buffer nobody uses), so the
  // wait counts below are constants.
  static_assert(NSTAGE == 4 && (COPIES == 2 || COPIES == 4), "wait counts assume 2 * COPIES copy instructions per tile");
  const int nk = K / TK;
  struct Frag { i4 bx[NJ]; i4 aw[NI]; };
  auto read_bx = [&](Frag& f, int tile) {
    const unsigned char* xb = lds + (tile % NSTAGE) * STAGE_BYTES + xwave + lo;
#pragma unroll
    for (int j = 0; j < NJ; ++j) f.bx[j] = *(const i4*)(xb + j * 16 * TK);
  };
  auto read_aw = [&](Frag& f, int tile) {
    const unsigned char* wb = lds + (tile % NSTAGE) * STAGE_BYTES + wwave + lo;
#pragma unroll
    for (int i = 0; i < NI; ++i) f.aw[i] = *(const i4*)(wb + i * 16 * TK);
  };
  auto mma = [&](const Frag& f, int ib, int ie) {
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      if (i < ib || i >= ie) continue;
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        if (NI * NJ * 4 > 128) {
          // 256 accumulator registers = the whole accumulation register file:
          // the in-place AGPR form is spelled out so that no accumulator is
          // ever copied (each one is next touched 64 MFMAs later)
          asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" : "+a"(acc[i][j]) : "v"(f.aw[i]), "v"(f.bx[j]));
        } else {
          acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(f.aw[i], f.bx[j], acc[i][j], 0, 0, 0);
        }
      }
    }
  };
  // The LDS reads of the next tile are issued in two batches of at most 8,
  // each followed by half of the current tile's MFMAs: the wait for the
  // current operands can then leave the newer reads outstanding (the LDS
  // counter only counts to 15).
  auto step = [&](const Frag& cur, Frag& nxt, int kt) {
    __builtin_amdgcn_s_waitcnt(COPIES == 2 ? 0x0f74 : 0x0f78);   // vmcnt(2 * COPIES): my copies of tile kt+1 landed
    __builtin_amdgcn_s_barrier();                  // bare barrier: a fence would drain the ring
    issue((kt + 3) % NSTAGE, min(kt + 3, nk - 1) * TK);
    if (NI * NJ * 4 > 128) {
      read_bx(nxt, kt + 1);
      __builtin_amdgcn_sched_barrier(0);
      mma(cur, 0, NI / 2);
      __builtin_amdgcn_sched_barrier(0);
      read_aw(nxt, kt + 1);
      __builtin_amdgcn_sched_barrier(0);
      mma(cur, NI / 2, NI);
      __builtin_amdgcn_sched_barrier(0);
    } else {
      // two wavefronts per SIMD: the instruction scheduler is free to mix the
      // next tile's LDS reads into this tile's MFMAs
      read_bx(nxt, kt + 1);
      read_aw(nxt, kt + 1);
      mma(cur, 0, NI);
    }
  };

#pragma unroll
  for (int p = 0; p < 3; ++p) issue(p, min(p, nk - 1) * TK);
  Frag f0, f1;
  __builtin_amdgcn_s_waitcnt(COPIES == 2 ? 0x0f78 : 0x4f70);    // vmcnt(4 * COPIES): tile 0 landed
  __builtin_amdgcn_s_barrier();
  read_bx(f0, 0);
  read_aw(f0, 0);
  for (int kt = 0; kt < nk; kt += 2) {             // nk is even (K % 128 == 0)
    step(f0, f1, kt);
    step(f1, f0, kt + 1);
  }
  // no copy may still be writing LDS when the workgroup retires
  __builtin_amdgcn_s_waitcnt(0x0f70);              // vmcnt(0)
  if (NI * NJ * 4 > 128) asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");   // last MFMA results settle before they are read

  // ---- epilogue: lane holds, per (n tile i, m tile j), output row
  // m = .. + l16 and columns n = .. + 4 kq + {0..3}
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    const int m = m0 + wm * (16 * NJ) + j * 16 + l16;
    if (m >= M) continue;
    const float xsc = a.x_scale ? a.x_scale[a.x_scale_per_row ? m : 0] : 1.0f;
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int n = n0 + wn * (16 * NI) + i * 16 + 4 * kq;
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
  const size_t shmem = NSTAGE * STAGE_BYTES;     // 128 KiB
  static hipError_t attr = hipFuncSetAttribute((const void*)w8a8_int8_gemm_kernel<DT>,
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
  MQ_REQUIRE(attr == hipSuccess, "w8a8_int8_gemm: cannot reserve %zu bytes of LDS: %s", shmem,
             hipGetErrorString(attr));
  hipLaunchKernelGGL((w8a8_int8_gemm_kernel<DT>), dim3(mtiles * ntiles), dim3(GEMM_THREADS), shmem, st, b);
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
  MQ_REQUIRE(K % 128 == 0, "w8a8_int8_gemm: K=%d must be a multiple of 128", K);
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
