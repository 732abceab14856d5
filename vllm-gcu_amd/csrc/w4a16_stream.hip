// W4A16 streaming (decode-shaped) GEMM for M <= 64 on gfx950.
//
// The kernel is bound by the HBM stream of packed int4 weights.  One
// workgroup (4 wavefronts) owns one 128-column slab and a contiguous range of
// 128-row K blocks; its wavefronts take K blocks round-robin, so every
// wavefront load instruction reads one tile = 1 KiB of contiguous memory
// (64 lanes x 16 B).  Weights are turned into exact small integers (q - z) in
// the activation type in registers, multiplied on the 16x16x32 MFMA with fp32
// accumulation, and the group scale is applied once per group to the fp32
// partial sum.  Wavefront partials are reduced through LDS; workgroups that
// split K publish fp32 partial tiles and the last one to arrive adds them in
// split order, so the result does not depend on scheduling.
#include "common.h"

namespace mi355q {

struct StreamArgs {
  uint16_t* out;
  const uint16_t* x;
  const u4* qw;
  const uint16_t* scales;
  const void* zeros;
  const uint16_t* bias;
  int M, K, N;
  int gs;            // quantisation group size (rows of K per scale row)
  int splits;
  float* partial;    // [splits][16*MT][N]
  int* counters;     // [N/128], zero between launches
};

template <int DT> struct Mma;
template <> struct Mma<MI355Q_F16> {
  typedef h8 vec;
  static __device__ __forceinline__ f4 run(vec a, vec b, f4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ vec from_h2(h2 r0, h2 r1, h2 r2, h2 r3) {
    return (h8){r0.x, r0.y, r1.x, r1.y, r2.x, r2.y, r3.x, r3.y};
  }
  static __device__ __forceinline__ vec splat_one() {
    const _Float16 o = (_Float16)1.0f;
    return (h8){o, o, o, o, o, o, o, o};
  }
};
template <> struct Mma<MI355Q_BF16> {
  typedef b8 vec;
  static __device__ __forceinline__ f4 run(vec a, vec b, f4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
  // small integers held exactly in fp16 -> the same integers in bf16
  static __device__ __forceinline__ uint32_t cvt(h2 r) {
    uint32_t lo = bitcast<uint32_t>((float)r.x), hi = bitcast<uint32_t>((float)r.y);
    return __builtin_amdgcn_perm(hi, lo, 0x07060302u);
  }
  static __device__ __forceinline__ vec from_h2(h2 r0, h2 r1, h2 r2, h2 r3) {
    u4 v = {cvt(r0), cvt(r1), cvt(r2), cvt(r3)};
    return bitcast<vec>(v);
  }
  static __device__ __forceinline__ vec splat_one() {
    u4 v = {0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u};
    return bitcast<vec>(v);
  }
};

// one 32-bit word (8 nibbles) -> four packed pairs of exact (q - z)
// zlo = (1024 + z, 1024 + z), zhi = (64 + z, 64 + z)
__device__ __forceinline__ void dequant_word(uint32_t w, h2 zlo, h2 zhi, h2& r0, h2& r1, h2& r2,
                                             h2& r3) {
  const uint32_t MAGIC = 0x64006400u;            // fp16 1024.0 twice
  const h2 sixteenth = {(_Float16)0.0625f, (_Float16)0.0625f};
  uint32_t w8 = w >> 8;
  h2 a0 = bitcast<h2>((w & 0x000f000fu) | MAGIC);    // 1024 + q
  h2 a1 = bitcast<h2>((w & 0x00f000f0u) | MAGIC);    // 1024 + 16 q
  h2 a2 = bitcast<h2>((w8 & 0x000f000fu) | MAGIC);
  h2 a3 = bitcast<h2>((w8 & 0x00f000f0u) | MAGIC);
  r0 = a0 - zlo;
  r1 = __builtin_elementwise_fma(a1, sixteenth, -zhi);
  r2 = a2 - zlo;
  r3 = __builtin_elementwise_fma(a3, sixteenth, -zhi);
}

template <int DT, int MT, int ZK, int SPF>
__global__ void __launch_bounds__(256)
w4a16_stream_kernel(StreamArgs a) {
  typedef typename Mma<DT>::vec vec;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c = lane & 15, kq = lane >> 4;
  const int slab = blockIdx.x, split = blockIdx.y;
  const int G = a.K >> 7;
  const int per = (G + a.splits - 1) / a.splits;
  const int gb = split * per;
  const int ge = min(G, gb + per);
  const int N = a.N, K = a.K;

  f4 acc[MT][8];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int t = 0; t < 8; ++t) acc[mt][t] = (f4){0.f, 0.f, 0.f, 0.f};

  const u4* wbase = a.qw + (size_t)slab * G * 512 + lane;
  const int ncol = 128 * slab + 8 * c;               // first of this lane's 8 columns

  struct Block {
    u4 w[8];
    vec av[MT == 1 ? 4 : 1];
  };
  auto load_block = [&](Block& b, int g) {
    const u4* p = wbase + (size_t)g * 512;
#pragma unroll
    for (int t = 0; t < 8; ++t) b.w[t] = __builtin_nontemporal_load(p + t * 64);
    if (MT == 1) {
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        u4 v = {0u, 0u, 0u, 0u};
        if (c < a.M) v = *(const u4*)(a.x + (size_t)c * K + 128 * g + 32 * s + 8 * kq);
        b.av[s] = bitcast<vec>(v);
      }
    }
  };

  auto compute_block = [&](const Block& b, int g) {
    vec av[MT][4];
    if (MT == 1) {
#pragma unroll
      for (int s = 0; s < 4; ++s) av[0][s] = b.av[s];
    } else {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          u4 v = {0u, 0u, 0u, 0u};
          int row = 16 * mt + c;
          if (row < a.M) v = *(const u4*)(a.x + (size_t)row * K + 128 * g + 32 * s + 8 * kq);
          av[mt][s] = bitcast<vec>(v);
        }
    }
#pragma unroll
    for (int f = 0; f < 4 / SPF; ++f) {
      const int qrow = (128 * g + 32 * SPF * f) / a.gs;
      // 8 scales, 8 zero-points for this lane's columns
      u4 sraw = *(const u4*)(a.scales + (size_t)qrow * N + ncol);
      float sc[8];
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        uint32_t word = sraw[t >> 1];
        sc[t] = Elem<DT>::to_f32((uint16_t)((t & 1) ? (word >> 16) : (word & 0xffffu)));
      }
      uint32_t zword = 0x88888888u;
      float zs[8];
      if (ZK == MI355Q_ZP_PACKED) zword = ((const uint32_t*)a.zeros)[(size_t)qrow * (N >> 3) + (ncol >> 3)];
      if (ZK == MI355Q_ZP_PRESCALED) {
        zword = 0u;
        u4 zraw = *(const u4*)((const uint16_t*)a.zeros + (size_t)qrow * N + ncol);
#pragma unroll
        for (int t = 0; t < 8; ++t) {
          uint32_t word = zraw[t >> 1];
          zs[t] = Elem<DT>::to_f32((uint16_t)((t & 1) ? (word >> 16) : (word & 0xffffu)));
        }
      }
      // row sums of x over this scale group (only the pre-scaled-zero form needs them)
      f4 xsum[MT];
      if (ZK == MI355Q_ZP_PRESCALED) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          xsum[mt] = (f4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int s = 0; s < SPF; ++s)
            xsum[mt] = Mma<DT>::run(av[mt][SPF * f + s], Mma<DT>::splat_one(), xsum[mt]);
        }
      }
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        const float zf = (float)((zword >> (4 * t)) & 15u);
        const _Float16 zl = (_Float16)(1024.0f + zf), zh = (_Float16)(64.0f + zf);
        const h2 zlo = {zl, zl}, zhi = {zh, zh};
        f4 part[MT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) part[mt] = (f4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < SPF; ++s) {
          h2 r0, r1, r2, r3;
          dequant_word(b.w[t][SPF * f + s], zlo, zhi, r0, r1, r2, r3);
          vec bv = Mma<DT>::from_h2(r0, r1, r2, r3);
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) part[mt] = Mma<DT>::run(av[mt][SPF * f + s], bv, part[mt]);
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          if (ZK == MI355Q_ZP_PRESCALED)
            acc[mt][t] += sc[t] * part[mt] - zs[t] * xsum[mt];
          else
            acc[mt][t] += sc[t] * part[mt];
        }
      }
    }
  };

  {
    Block b0, b1;
    int g = gb + wave;
    if (g < ge) {
      load_block(b0, g);
      while (true) {
        if (g + 4 < ge) load_block(b1, g + 4);
        compute_block(b0, g);
        g += 4;
        if (g >= ge) break;
        if (g + 4 < ge) load_block(b0, g + 4);
        compute_block(b1, g);
        g += 4;
        if (g >= ge) break;
      }
    }
  }

  // ---- reduce the 4 wavefronts through LDS; wave w finishes rows 4*kq + w ----
  __shared__ float red[4][32][64];
  const int Mpad = 16 * MT;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
    for (int t = 0; t < 8; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) red[wave][i * 8 + t][lane] = acc[mt][t][i];
    __syncthreads();
    float v[8];
#pragma unroll
    for (int t = 0; t < 8; ++t)
      v[t] = ((red[0][wave * 8 + t][lane] + red[1][wave * 8 + t][lane]) +
              red[2][wave * 8 + t][lane]) + red[3][wave * 8 + t][lane];
    __syncthreads();
    const int m = 16 * mt + 4 * kq + wave;
    if (a.splits == 1) {
      if (m < a.M) {
        u4 o;
#pragma unroll
        for (int t = 0; t < 8; t += 2) {
          float v0 = v[t], v1 = v[t + 1];
          if (a.bias) {
            v0 += Elem<DT>::to_f32(a.bias[ncol + t]);
            v1 += Elem<DT>::to_f32(a.bias[ncol + t + 1]);
          }
          o[t >> 1] = (uint32_t)Elem<DT>::from_f32(v0) | ((uint32_t)Elem<DT>::from_f32(v1) << 16);
        }
        *(u4*)(a.out + (size_t)m * N + ncol) = o;
      }
    } else {
      float* p = a.partial + ((size_t)split * Mpad + m) * N + ncol;
      *(f4*)p = (f4){v[0], v[1], v[2], v[3]};
      *(f4*)(p + 4) = (f4){v[4], v[5], v[6], v[7]};
    }
  }
  if (a.splits == 1) return;

  // ---- cross-workgroup split-K: last arriver adds the partial tiles in order ----
  __shared__ int is_last;
  __threadfence();
  __syncthreads();
  if (threadIdx.x == 0) {
    int old = __hip_atomic_fetch_add(a.counters + slab, 1, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
    is_last = (old == a.splits - 1);
  }
  __syncthreads();
  if (!is_last) return;
  __threadfence();
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = 16 * mt + 4 * kq + wave;
    if (m >= a.M) continue;
    f4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
    for (int sp = 0; sp < a.splits; ++sp) {
      const float* p = a.partial + ((size_t)sp * Mpad + m) * N + ncol;
      s0 += __builtin_nontemporal_load((const f4*)p);
      s1 += __builtin_nontemporal_load((const f4*)(p + 4));
    }
    float v[8] = {s0[0], s0[1], s0[2], s0[3], s1[0], s1[1], s1[2], s1[3]};
    u4 o;
#pragma unroll
    for (int t = 0; t < 8; t += 2) {
      float v0 = v[t], v1 = v[t + 1];
      if (a.bias) {
        v0 += Elem<DT>::to_f32(a.bias[ncol + t]);
        v1 += Elem<DT>::to_f32(a.bias[ncol + t + 1]);
      }
      o[t >> 1] = (uint32_t)Elem<DT>::from_f32(v0) | ((uint32_t)Elem<DT>::from_f32(v1) << 16);
    }
    *(u4*)(a.out + (size_t)m * N + ncol) = o;
  }
  if (threadIdx.x == 0) a.counters[slab] = 0;
}

template <int DT, int MT, int ZK>
static void launch_spf(const StreamArgs& a, hipStream_t st) {
  dim3 grid(a.N / 128, a.splits), block(256);
  if (a.gs % 128 == 0)
    hipLaunchKernelGGL((w4a16_stream_kernel<DT, MT, ZK, 4>), grid, block, 0, st, a);
  else
    hipLaunchKernelGGL((w4a16_stream_kernel<DT, MT, ZK, 1>), grid, block, 0, st, a);
}

template <int DT, int MT>
static void launch_zk(const StreamArgs& a, int zk, hipStream_t st) {
  if (zk == MI355Q_ZP_NONE) launch_spf<DT, MT, MI355Q_ZP_NONE>(a, st);
  else if (zk == MI355Q_ZP_PACKED) launch_spf<DT, MT, MI355Q_ZP_PACKED>(a, st);
  else launch_spf<DT, MT, MI355Q_ZP_PRESCALED>(a, st);
}

template <int DT>
static void launch_mt(const StreamArgs& a, int zk, hipStream_t st) {
  if (a.M <= 16) launch_zk<DT, 1>(a, zk, st);
  else if (a.M <= 32) launch_zk<DT, 2>(a, zk, st);
  else launch_zk<DT, 4>(a, zk, st);
}

// split-K choice: enough workgroups to cover the CUs about twice while every
// wavefront still streams at least two K blocks
int w4a16_stream_auto_splits(int M, int K, int N) {
  const int slabs = N / 128, G = K / 128;
  const int cus = device_cu_count();
  int want = (2 * cus + slabs - 1) / slabs;
  int maxs = G / 8 > 0 ? G / 8 : 1;        // >= 8 K blocks (2 per wavefront) per workgroup
  int s = want < maxs ? want : maxs;
  if (s < 1) s = 1;
  if (s > 32) s = 32;
  (void)M;
  return s;
}

size_t w4a16_stream_workspace_bytes(int M, int N) {
  const int Mpad = M <= 16 ? 16 : (M <= 32 ? 32 : 64);
  return (size_t)(N / 128) * sizeof(int) + 256 + (size_t)32 * Mpad * N * sizeof(float);
}

int w4a16_stream_launch(void* out, const void* x, const int32_t* qweight, const void* scales,
                        const void* zeros, int zeros_kind, const void* bias, int M, int K, int N,
                        int group_size, int dtype, void* workspace, size_t workspace_bytes,
                        int split_k, hipStream_t st) {
  StreamArgs a;
  a.out = (uint16_t*)out;
  a.x = (const uint16_t*)x;
  a.qw = (const u4*)qweight;
  a.scales = (const uint16_t*)scales;
  a.zeros = zeros;
  a.bias = (const uint16_t*)bias;
  a.M = M; a.K = K; a.N = N;
  a.gs = group_size;
  int G = K / 128;
  int splits = split_k > 0 ? split_k : w4a16_stream_auto_splits(M, K, N);
  if (splits > G) splits = G;
  if (splits > 32) splits = 32;
  // no empty splits: ceil(G / splits) * (splits - 1) < G
  while (splits > 1 && ((G + splits - 1) / splits) * (splits - 1) >= G) --splits;
  a.splits = splits;
  a.partial = nullptr;
  a.counters = nullptr;
  if (splits > 1) {
    const int Mpad = M <= 16 ? 16 : (M <= 32 ? 32 : 64);
    size_t cbytes = ((size_t)(N / 128) * sizeof(int) + 255) / 256 * 256;
    size_t need = cbytes + (size_t)splits * Mpad * N * sizeof(float);
    MQ_REQUIRE(workspace && workspace_bytes >= need,
               "w4a16_gemm: workspace of %zu bytes needed for split_k=%d, got %zu", need, splits,
               workspace_bytes);
    a.counters = (int*)workspace;
    a.partial = (float*)((char*)workspace + cbytes);
  }
  if (dtype == MI355Q_F16) launch_mt<MI355Q_F16>(a, zeros_kind, st);
  else launch_mt<MI355Q_BF16>(a, zeros_kind, st);
  MQ_LAUNCH_CHECK("w4a16_gemm(stream)");
  return 0;
}

}  // namespace mi355q
