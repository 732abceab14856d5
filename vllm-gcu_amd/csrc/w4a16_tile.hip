// W4A16 LDS-staged MFMA GEMM for large M (prefill-shaped) on gfx950.
//
// Workgroup tile 128 (M) x 256 (N), K step 128 (one slab K block), 4
// wavefronts side by side along N: wave w owns 64 columns (four 16-column
// tiles of one slab) for all 128 rows.  Because the slab layout already stores
// each lane's MFMA B operand contiguously, a wavefront dequantises its own
// columns straight into B operands in registers -- (q - z) * s rounded once to
// the activation type -- and every operand is reused for the 8 row tiles, so no
// weight is dequantised twice in a workgroup.  The activation tile is shared
// by the 4 wavefronts through LDS (double buffered, rows padded by 16 B so
// the 16-lane x 16 B operand reads are bank-conflict free).  fp32 accumulate.
#include "common.h"

namespace mi355q {

namespace {

constexpr int BM = 128, BN = 256, BK = 128;
constexpr int A_ROW = BK * 2 + 16;                 // bytes per LDS row (padded)
constexpr int A_BUF = BM * A_ROW;                  // bytes per buffer

struct TileArgs {
  uint16_t* out;
  const uint16_t* x;
  const u4* qw;
  const uint16_t* scales;
  const void* zeros;
  const uint16_t* bias;
  int M, K, N, gs;
};

template <int DT> struct TileMma;
template <> struct TileMma<MI355Q_F16> {
  typedef h8 vec;
  static __device__ __forceinline__ f4 run(vec a, vec b, f4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
  // one packed word -> 8 weights (q - z) * s in fp16
  //   zlo = (1024 + z) x2, zhi = (64 + z) x2, sc = s x2
  static __device__ __forceinline__ vec dequant(uint32_t w, float z, float s) {
    const uint32_t MAGIC = 0x64006400u;
    const h2 sixteenth = {(_Float16)0.0625f, (_Float16)0.0625f};
    const _Float16 zl = (_Float16)(1024.0f + z), zh = (_Float16)(64.0f + z), sh = (_Float16)s;
    const h2 zlo = {zl, zl}, zhi = {zh, zh}, sc = {sh, sh};
    uint32_t w8 = w >> 8;
    h2 a0 = bitcast<h2>((w & 0x000f000fu) | MAGIC);
    h2 a1 = bitcast<h2>((w & 0x00f000f0u) | MAGIC);
    h2 a2 = bitcast<h2>((w8 & 0x000f000fu) | MAGIC);
    h2 a3 = bitcast<h2>((w8 & 0x00f000f0u) | MAGIC);
    h2 r0 = (a0 - zlo) * sc;
    h2 r1 = __builtin_elementwise_fma(a1, sixteenth, -zhi) * sc;
    h2 r2 = (a2 - zlo) * sc;
    h2 r3 = __builtin_elementwise_fma(a3, sixteenth, -zhi) * sc;
    return (h8){r0.x, r0.y, r1.x, r1.y, r2.x, r2.y, r3.x, r3.y};
  }
};
template <> struct TileMma<MI355Q_BF16> {
  typedef b8 vec;
  static __device__ __forceinline__ f4 run(vec a, vec b, f4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack(float lo, float hi) {
    return (uint32_t)f32_to_bf16(lo) | ((uint32_t)f32_to_bf16(hi) << 16);
  }
  static __device__ __forceinline__ vec dequant(uint32_t w, float z, float s) {
    float v[8];
#pragma unroll
    for (int p = 0; p < 8; ++p) v[p] = ((float)((w >> (4 * p)) & 15u) - z) * s;
    // nibble order {0,4,1,5,2,6,3,7} = k offsets 0..7
    u4 r = {pack(v[0], v[4]), pack(v[1], v[5]), pack(v[2], v[6]), pack(v[3], v[7])};
    return bitcast<vec>(r);
  }
};

template <int DT, int ZK>
__global__ void __launch_bounds__(256, 1)
w4a16_tile_kernel(TileArgs a) {
  typedef TileMma<DT> MM;
  typedef typename MM::vec vec;
  extern __shared__ __align__(16) unsigned char lds[];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int c = lane & 15, kq = lane >> 4;
  const int N = a.N, K = a.K, M = a.M;
  const int G = K >> 7;
  const int m0 = blockIdx.y * BM;
  // N may end in the middle of the 256-column tile: the two wavefronts of a
  // missing slab compute on the previous one and skip the epilogue
  const bool live = (blockIdx.x * 2 + (wave >> 1)) < (N >> 7);
  const int slab = live ? blockIdx.x * 2 + (wave >> 1) : (N >> 7) - 1;
  const int t0 = (wave & 1) * 4;
  const int ncol = 128 * slab + 8 * c + t0;          // first of this lane's 4 columns

  f4 acc[8][4];
#pragma unroll
  for (int mt = 0; mt < 8; ++mt)
#pragma unroll
    for (int t = 0; t < 4; ++t) acc[mt][t] = (f4){0.f, 0.f, 0.f, 0.f};

  // global -> register staging of the next activation tile: thread tid loads
  // 8 chunks of 16 B: row = pass * 16 + tid / 16, chunk = tid % 16
  const int arow = tid >> 4, achunk = tid & 15;
  u4 areg[8];
  auto load_a = [&](int g) {
#pragma unroll
    for (int p = 0; p < 8; ++p) {
      const int row = min(m0 + p * 16 + arow, M - 1);
      areg[p] = *(const u4*)(a.x + (size_t)row * K + 128 * g + 8 * achunk);
    }
  };
  auto store_a = [&](int buf) {
    unsigned char* base = lds + buf * A_BUF;
#pragma unroll
    for (int p = 0; p < 8; ++p) *(u4*)(base + (p * 16 + arow) * A_ROW + achunk * 16) = areg[p];
  };

  const u4* wbase = a.qw + ((size_t)slab * G * 8 + t0) * 64 + lane;
  u4 wreg[4];
  uint2 sreg;
  uint32_t zreg = 0x88888888u;
  uint2 zsreg = {0u, 0u};
  auto load_b = [&](int g) {
    const u4* p = wbase + (size_t)g * 512;
#pragma unroll
    for (int t = 0; t < 4; ++t) wreg[t] = p[t * 64];
    const int qrow = (128 * g) / a.gs;
    sreg = *(const uint2*)(a.scales + (size_t)qrow * N + ncol);
    if (ZK == MI355Q_ZP_PACKED) zreg = ((const uint32_t*)a.zeros)[(size_t)qrow * (N >> 3) + (ncol >> 3)] >> (4 * t0);
    if (ZK == MI355Q_ZP_PRESCALED) zsreg = *(const uint2*)((const uint16_t*)a.zeros + (size_t)qrow * N + ncol);
  };

  load_a(0);
  load_b(0);
  store_a(0);
  __syncthreads();

  for (int g = 0; g < G; ++g) {
    const int buf = g & 1;
    // operands of this K block, then start the next block's loads
    u4 wcur[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) wcur[t] = wreg[t];
    float sc[4], zf[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const uint32_t sw = (t < 2) ? sreg.x : sreg.y;
      sc[t] = Elem<DT>::to_f32((uint16_t)((t & 1) ? (sw >> 16) : (sw & 0xffffu)));
      if (ZK == MI355Q_ZP_PRESCALED) {
        const uint32_t zw = (t < 2) ? zsreg.x : zsreg.y;
        // z * s was pre-multiplied by the loader; recover the real-valued zero-point
        zf[t] = Elem<DT>::to_f32((uint16_t)((t & 1) ? (zw >> 16) : (zw & 0xffffu))) / sc[t];
      } else {
        zf[t] = (float)((zreg >> (4 * t)) & 15u);
      }
    }
    const int gn = min(g + 1, G - 1);
    load_a(gn);
    load_b(gn);

    const unsigned char* abase = lds + buf * A_BUF + c * A_ROW + kq * 16;
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      vec bv[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) bv[t] = MM::dequant(wcur[t][s], zf[t], sc[t]);
#pragma unroll
      for (int mt = 0; mt < 8; ++mt) {
        const vec av = bitcast<vec>(*(const u4*)(abase + mt * 16 * A_ROW + s * 64));
#pragma unroll
        for (int t = 0; t < 4; ++t) acc[mt][t] = MM::run(av, bv[t], acc[mt][t]);
      }
    }
    // the other buffer was last read one iteration ago: every wavefront has
    // passed the barrier below since, so it can be overwritten now
    store_a(buf ^ 1);
    __syncthreads();
  }

  // ---- epilogue: 4 adjacent columns per (row tile, i) ----
  if (!live) return;
  float bs[4] = {0.f, 0.f, 0.f, 0.f};
  if (a.bias) {
#pragma unroll
    for (int t = 0; t < 4; ++t) bs[t] = Elem<DT>::to_f32(a.bias[ncol + t]);
  }
#pragma unroll
  for (int mt = 0; mt < 8; ++mt)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = m0 + mt * 16 + 4 * kq + i;
      if (m < M) {
        uint2 o;
        o.x = (uint32_t)Elem<DT>::from_f32(acc[mt][0][i] + bs[0]) |
              ((uint32_t)Elem<DT>::from_f32(acc[mt][1][i] + bs[1]) << 16);
        o.y = (uint32_t)Elem<DT>::from_f32(acc[mt][2][i] + bs[2]) |
              ((uint32_t)Elem<DT>::from_f32(acc[mt][3][i] + bs[3]) << 16);
        *(uint2*)(a.out + (size_t)m * N + ncol) = o;
      }
    }
}

template <int DT, int ZK>
hipError_t launch_one(const TileArgs& a, hipStream_t st) {
  dim3 grid((a.N + BN - 1) / BN, (a.M + BM - 1) / BM), block(256);
  const size_t shmem = 2 * A_BUF;                  // 68 KiB: above the 64 KiB default
  static hipError_t attr = hipFuncSetAttribute((const void*)w4a16_tile_kernel<DT, ZK>,
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
  if (attr != hipSuccess) return attr;
  hipLaunchKernelGGL((w4a16_tile_kernel<DT, ZK>), grid, block, shmem, st, a);
  return hipSuccess;
}

template <int DT>
hipError_t launch_zk(const TileArgs& a, int zk, hipStream_t st) {
  if (zk == MI355Q_ZP_NONE) return launch_one<DT, MI355Q_ZP_NONE>(a, st);
  if (zk == MI355Q_ZP_PACKED) return launch_one<DT, MI355Q_ZP_PACKED>(a, st);
  return launch_one<DT, MI355Q_ZP_PRESCALED>(a, st);
}

}  // namespace

int w4a16_tile_launch(void* out, const void* x, const int32_t* qweight, const void* scales,
                      const void* zeros, int zeros_kind, const void* bias, int M, int K, int N,
                      int group_size, int dtype, hipStream_t st) {
  MQ_REQUIRE(group_size % 128 == 0,
             "w4a16_gemm: the MFMA kernel needs group_size %% 128 == 0, got %d", group_size);
  TileArgs a;
  a.out = (uint16_t*)out;
  a.x = (const uint16_t*)x;
  a.qw = (const u4*)qweight;
  a.scales = (const uint16_t*)scales;
  a.zeros = zeros;
  a.bias = (const uint16_t*)bias;
  a.M = M; a.K = K; a.N = N; a.gs = group_size;
  hipError_t e = (dtype == MI355Q_F16) ? launch_zk<MI355Q_F16>(a, zeros_kind, st)
                                       : launch_zk<MI355Q_BF16>(a, zeros_kind, st);
  MQ_REQUIRE(e == hipSuccess, "w4a16_gemm(tile): cannot reserve LDS: %s", hipGetErrorString(e));
  MQ_LAUNCH_CHECK("w4a16_gemm(tile)");
  return 0;
}

}  // namespace mi355q
