// W4A16 streaming (decode-shaped) GEMM for M <= 64 on gfx950.
//
// The kernel is bound by the HBM stream of packed int4 weights.  One
// workgroup (4 wavefronts) owns NT of the 8 tiles of one 128-column slab and a
// contiguous range of 128-row K blocks; its wavefronts take K blocks
// round-robin, so every wavefront load instruction reads one tile = 1 KiB of
// contiguous memory (64 lanes x 16 B).  Narrow matrices use NT < 8: more
// workgroups without splitting K across workgroups (whose exchange costs
// dependent round trips to memory), at the price of re-reading activations
// from L2 once per tile group.  Weights are turned into exact small integers (q - z) in
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
  int* counters;     // one per blockIdx.x (<= N/16), zero between launches
};

// (a & mask) | orv.  Callers launder `mask` into an SGPR and `orv` into a VGPR
// (see launder_*) so the compiler cannot fold them into literals and selects
// the single VOP3 v_and_or_b32 instead of an and + or pair.
__device__ __forceinline__ uint32_t and_or(uint32_t a, uint32_t mask, uint32_t orv) {
  return (a & mask) | orv;
}
__device__ __forceinline__ uint32_t launder_sgpr(uint32_t v) {
  asm volatile("" : "+s"(v));
  return v;
}
__device__ __forceinline__ uint32_t launder_vgpr(uint32_t v) {
  asm volatile("" : "+v"(v));
  return v;
}

// Per activation type: the MFMA, and how packed nibbles become B operands
// WITHOUT per-weight arithmetic.  A nibble q is OR-ed into the mantissa of a
// constant, giving base + q (or base + 16 q for the odd nibble of a byte in
// fp16, whose A elements are pre-multiplied by 1/16).  The MFMA therefore
// accumulates  sum_k x_k q_k + CORR  where CORR depends only on row sums of x;
// CORR and the zero-point term z * sum_k x_k are removed once per group from
// the fp32 accumulator.
template <int DT> struct Mma;
template <> struct Mma<MI355Q_F16> {
  typedef h8 vec;
  static constexpr bool kScaledA = true;      // needs the separate correction MFMA
  static constexpr float kBase = 1024.0f;
  static __device__ __forceinline__ f4 run(vec a, vec b, f4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ vec splat(float v) {
    const _Float16 o = (_Float16)v;
    return (h8){o, o, o, o, o, o, o, o};
  }
  // elements (2,3) and (6,7) meet the "16 q" nibbles: scale them by 1/16
  static __device__ __forceinline__ vec prep_a(u4 raw) {
    const h2 sixteenth = {(_Float16)0.0625f, (_Float16)0.0625f};
    raw[1] = bitcast<uint32_t>(bitcast<h2>(raw[1]) * sixteenth);
    raw[3] = bitcast<uint32_t>(bitcast<h2>(raw[3]) * sixteenth);
    return bitcast<vec>(raw);
  }
  static __device__ __forceinline__ vec make_b(uint32_t w, uint32_t magic, uint32_t mlo, uint32_t mhi) {
    uint32_t w8 = w >> 8;
    u4 v = {and_or(w, mlo, magic), and_or(w, mhi, magic), and_or(w8, mlo, magic), and_or(w8, mhi, magic)};
    return bitcast<vec>(v);
  }
  static __device__ __forceinline__ uint32_t magic() { return 0x64006400u; }   // 1024.0 x2
};
template <> struct Mma<MI355Q_BF16> {
  typedef b8 vec;
  static constexpr bool kScaledA = false;
  static constexpr float kBase = 128.0f;
  static __device__ __forceinline__ f4 run(vec a, vec b, f4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ vec splat(float v) {
    uint32_t h = bitcast<uint32_t>(v) >> 16;
    h |= h << 16;
    u4 r = {h, h, h, h};
    return bitcast<vec>(r);
  }
  static __device__ __forceinline__ vec prep_a(u4 raw) { return bitcast<vec>(raw); }
  static __device__ __forceinline__ vec make_b(uint32_t w, uint32_t magic, uint32_t mlo, uint32_t) {
    u4 v = {and_or(w, mlo, magic), and_or(w >> 4, mlo, magic), and_or(w >> 8, mlo, magic),
            and_or(w >> 12, mlo, magic)};
    return bitcast<vec>(v);
  }
  static __device__ __forceinline__ uint32_t magic() { return 0x43004300u; }   // 128.0 x2
};

template <int NT>
__device__ __forceinline__ void store_partial(float* p, const float* v) {
  // device-scope relaxed stores: written through to memory, no cache flush
  if (NT == 1) {
    __hip_atomic_store((uint32_t*)p, bitcast<uint32_t>(v[0]), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return;
  }
#pragma unroll
  for (int t = 0; t + 1 < NT; t += 2) {
    uint64_t bits = (uint64_t)bitcast<uint32_t>(v[t]) | ((uint64_t)bitcast<uint32_t>(v[t + 1]) << 32);
    __hip_atomic_store((uint64_t*)(p + t), bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}
template <int NT>
__device__ __forceinline__ void load_partial_add(const float* p, float* v) {
  if (NT == 1) {
    uint32_t bits = __hip_atomic_load((const uint32_t*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    v[0] += bitcast<float>(bits);
    return;
  }
#pragma unroll
  for (int t = 0; t + 1 < NT; t += 2) {
    uint64_t bits = __hip_atomic_load((const uint64_t*)(p + t), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    v[t] += bitcast<float>((uint32_t)bits);
    v[t + 1] += bitcast<float>((uint32_t)(bits >> 32));
  }
}

// NT consecutive output columns of one row (ncol = the first of them)
template <int DT, int NT>
__device__ __forceinline__ void store_out_row(uint16_t* out, const uint16_t* bias, int ncol, const float* v) {
  uint16_t h[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    float f = v[t];
    if (bias) f += Elem<DT>::to_f32(bias[ncol + t]);
    h[t] = Elem<DT>::from_f32(f);
  }
  if (NT == 1) {
    *out = h[0];
  } else {
    constexpr int P = NT >= 2 ? NT / 2 : 1;
    uint32_t o[P];
#pragma unroll
    for (int t = 0; t < NT / 2; ++t) o[t] = (uint32_t)h[2 * t] | ((uint32_t)h[2 * t + 1] << 16);
    if (NT == 8) *(u4*)out = (u4){o[0], o[P > 1 ? 1 : 0], o[P > 2 ? 2 : 0], o[P > 3 ? 3 : 0]};
    else if (NT == 4) *(u2*)out = (u2){o[0], o[P > 1 ? 1 : 0]};
    else *(uint32_t*)out = o[0];
  }
}

// NT consecutive 16-bit values (scales or pre-scaled zeros) as packed pairs
template <int NT>
__device__ __forceinline__ void load_halves(const uint16_t* p, uint32_t* dst) {
  if (NT == 8) { u4 v = *(const u4*)p; dst[0] = v[0]; dst[NT > 2 ? 1 : 0] = v[1]; dst[NT > 4 ? 2 : 0] = v[2]; dst[NT > 6 ? 3 : 0] = v[3]; }
  else if (NT == 4) { u2 v = *(const u2*)p; dst[0] = v[0]; dst[NT > 2 ? 1 : 0] = v[1]; }
  else if (NT == 2) dst[0] = *(const uint32_t*)p;
  else dst[0] = *p;
}

template <int DT, int MT, int ZK, int SPF, int NT>
__global__ void __launch_bounds__(256, (MT == 1 || (MT == 2 && NT <= 4)) ? 2 : 1)
w4a16_stream_kernel(StreamArgs a) {
  typedef Mma<DT> MM;
  typedef typename MM::vec vec;
  // the wavefront index is made visibly uniform: K-block indices and loop control then live in scalar registers
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int c = lane & 15, kq = lane >> 4;
  constexpr int TG = 8 / NT;                          // tile groups per slab
  constexpr int HW = NT >= 2 ? NT / 2 : 1;            // packed 16-bit pairs per lane
  const int slab = blockIdx.x / TG, t0 = (blockIdx.x % TG) * NT, split = blockIdx.y;
  const int G = a.K >> 7;
  const int per = (G + a.splits - 1) / a.splits;
  const int gb = split * per;
  const int ge = min(G, gb + per);
  const int N = a.N, K = a.K;

  f4 acc[MT][NT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[mt][t] = (f4){0.f, 0.f, 0.f, 0.f};

  const u4* wbase = a.qw + (size_t)slab * G * 512 + t0 * 64 + lane;
  const int ncol8 = 128 * slab + 8 * c;              // first of this lane's 8 slab columns
  const int ncol = ncol8 + t0;                       // first of the NT columns this workgroup owns
  const uint32_t magic = launder_vgpr(MM::magic());
  const uint32_t mlo = launder_sgpr(0x000f000fu), mhi = launder_sgpr(0x00f000f0u);

  // Everything a block's arithmetic needs is loaded together and one block
  // ahead, so the only memory wait inside the compute phase is for the block
  // being consumed while the next block's loads stay in flight (the wait
  // counter retires in order: a late load would drain the prefetch too).
  // activations ride along one block ahead up to 32 rows (16 for the small-group variant, which has no registers to spare)
  constexpr bool XA = MT == 1 || (MT == 2 && SPF == 4);
  struct Block {
    u4 w[NT];
    uint32_t sraw[4 / SPF][HW];
    uint32_t zraw[ZK == MI355Q_ZP_PRESCALED ? 4 / SPF : 1][HW];
    uint32_t zword[4 / SPF];
    u4 xr[XA ? 4 * MT : 1];
  };
  auto load_block = [&](Block& b, int g) {
    const u4* p = wbase + (size_t)g * 512;
#pragma unroll
    for (int t = 0; t < NT; ++t) b.w[t] = __builtin_nontemporal_load(p + t * 64);
#pragma unroll
    for (int f = 0; f < 4 / SPF; ++f) {
      const int qrow = (128 * g + 32 * SPF * f) / a.gs;
      load_halves<NT>(a.scales + (size_t)qrow * N + ncol, b.sraw[f]);
      b.zword[f] = 0x88888888u;
      if (ZK == MI355Q_ZP_PACKED) b.zword[f] = ((const uint32_t*)a.zeros)[(size_t)qrow * (N >> 3) + (ncol8 >> 3)];
      if (ZK == MI355Q_ZP_PRESCALED) load_halves<NT>((const uint16_t*)a.zeros + (size_t)qrow * N + ncol, b.zraw[f]);
    }
    if (XA) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          // rows past M repeat the last row: output rows are independent and
          // rows >= M are never stored, so no predicated load is needed
          b.xr[XA ? 4 * mt + s : 0] =
              *(const u4*)(a.x + (size_t)min(16 * mt + c, a.M - 1) * K + 128 * g + 32 * s + 8 * kq);
        }
    }
  };
  // activations of block g for 64-row launches (too many registers to carry a block ahead)
  struct Acts { u4 xr[XA ? 1 : MT][4]; };
  auto load_acts = [&](Acts& x, int g) {
    if (XA) return;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        const int row = min(16 * mt + c, a.M - 1);
        x.xr[mt][s] = *(const u4*)(a.x + (size_t)row * K + 128 * g + 32 * s + 8 * kq);
      }
  };

  auto compute_block = [&](const Block& b, const Acts& xa) {
#pragma unroll
    for (int f = 0; f < 4 / SPF; ++f) {
      const uint32_t zword = b.zword[f] >> (4 * t0);
      // per row of x over this scale group: xs = sum x, corr = what the
      // mantissa trick added to the accumulator
      vec av[MT][SPF];
      f4 xs[MT], corr[MT];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        xs[mt] = (f4){0.f, 0.f, 0.f, 0.f};
        corr[mt] = (f4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < SPF; ++s) {
          const u4 raw = XA ? b.xr[XA ? 4 * mt + SPF * f + s : 0] : xa.xr[XA ? 0 : mt][SPF * f + s];
          av[mt][s] = MM::prep_a(raw);
          xs[mt] = MM::run(bitcast<vec>(raw), MM::splat(1.0f), xs[mt]);
          if (MM::kScaledA) corr[mt] = MM::run(av[mt][s], MM::splat(MM::kBase), corr[mt]);
        }
        if (!MM::kScaledA) corr[mt] = MM::kBase * xs[mt];
      }
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        const uint32_t sword = b.sraw[f][t >> 1];
        const float sc = Elem<DT>::to_f32((uint16_t)((t & 1) ? (sword >> 16) : (sword & 0xffffu)));
        f4 part[MT];
        if (ZK == MI355Q_ZP_PRESCALED) {
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) part[mt] = -corr[mt];
        } else {
          const float zf = (float)((zword >> (4 * t)) & 15u);
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) part[mt] = -zf * xs[mt] - corr[mt];
        }
#pragma unroll
        for (int s = 0; s < SPF; ++s) {
          vec bv = MM::make_b(b.w[t][SPF * f + s], magic, mlo, mhi);
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) part[mt] = MM::run(av[mt][s], bv, part[mt]);
        }
        if (ZK == MI355Q_ZP_PRESCALED) {
          const uint32_t zw = b.zraw[ZK == MI355Q_ZP_PRESCALED ? f : 0][t >> 1];
          const float zsf = Elem<DT>::to_f32((uint16_t)((t & 1) ? (zw >> 16) : (zw & 0xffffu)));
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) acc[mt][t] += sc * part[mt] - zsf * xs[mt];
        } else {
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) acc[mt][t] += sc * part[mt];
        }
      }
    }
  };

  {
    // Two block buffers: the next K block of this wavefront is in flight while
    // one is consumed (deeper rings were measured and are slower).  The
    // prefetch is unconditional (past the end it re-reads a block of this
    // wavefront) and every step leaves the loop through a plain break, so the
    // body is straight-line code and the compiler waits for exactly the block
    // being consumed.
    //
    // K order: the wavefront's nb blocks are visited starting at a
    // workgroup-dependent position.  All workgroups read the same activation
    // rows, and a K block of them (16 rows x 256 B at a pitch of 2 K bytes)
    // sits in very few L2 channels: in a common order every workgroup of an XCD
    // would hammer those channels at the same moment.  (The order is fixed per
    // workgroup, so results stay run-to-run identical.)
    Block ring[2];
    Acts xa;
    const int g0 = gb + wave;
    const int nb = (ge - g0 + 3) >> 2;               // K blocks of this wavefront
    if (nb > 0) {
      const int rot = (int)((blockIdx.x >> 3) * 5u % (unsigned)nb);
      auto blk = [&](int i) {                        // i-th block in this workgroup's order
        int j = i + rot;
        if (j >= nb) j -= nb;
        if (j >= nb) j -= nb;                        // i may run one past the end
        return g0 + 4 * j;
      };
      load_block(ring[0], blk(0));
      int i = 0;
      while (true) {
        // sched_barrier: keep the prefetch ahead of the arithmetic, the
        // instruction scheduler would otherwise sink the loads next to
        // their first use one iteration later
        load_acts(xa, blk(i));
        load_block(ring[1], blk(i + 1));
        __builtin_amdgcn_sched_barrier(0);
        compute_block(ring[0], xa);
        __builtin_amdgcn_sched_barrier(0);
        if (++i >= nb) break;
        load_acts(xa, blk(i));
        load_block(ring[0], blk(i + 1));
        __builtin_amdgcn_sched_barrier(0);
        compute_block(ring[1], xa);
        __builtin_amdgcn_sched_barrier(0);
        if (++i >= nb) break;
      }
    }
  }

  // ---- reduce the 4 wavefronts through LDS; wave w finishes rows 4*kq + w ----
  __shared__ float red[4][4 * NT][64];
  const int Mpad = 16 * MT;
  float fin[MT][NT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) red[wave][i * NT + t][lane] = acc[mt][t][i];
    __syncthreads();
#pragma unroll
    for (int t = 0; t < NT; ++t)
      fin[mt][t] = ((red[0][wave * NT + t][lane] + red[1][wave * NT + t][lane]) +
                    red[2][wave * NT + t][lane]) + red[3][wave * NT + t][lane];
    __syncthreads();
    const int m = 16 * mt + 4 * kq + wave;
    if (m < a.M) {
      if (a.splits == 1)
        store_out_row<DT, NT>(a.out + (size_t)m * N + ncol, a.bias, ncol, fin[mt]);
      else
        store_partial<NT>(a.partial + ((size_t)split * Mpad + m) * N + ncol, fin[mt]);
    }
  }
  if (a.splits == 1) return;

  // ---- cross-workgroup split-K ---------------------------------------------
  // Partial tiles travel as device-scope relaxed accesses (they bypass the
  // per-XCD L2 instead of flushing it); the barrier's wait for outstanding
  // stores orders them before the arrival count.  The last workgroup to
  // arrive adds the tiles in split order, so the sum is reproducible.
  __shared__ int is_last;
  __syncthreads();
  if (threadIdx.x == 0) {
    int old = __hip_atomic_fetch_add(a.counters + blockIdx.x, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    is_last = (old == a.splits - 1);
  }
  __syncthreads();
  if (!is_last) return;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = 16 * mt + 4 * kq + wave;
    if (m >= a.M) continue;
    float v[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) v[t] = 0.f;
    for (int sp = 0; sp < a.splits; ++sp)
      load_partial_add<NT>(a.partial + ((size_t)sp * Mpad + m) * N + ncol, v);
    store_out_row<DT, NT>(a.out + (size_t)m * N + ncol, a.bias, ncol, v);
  }
  if (threadIdx.x == 0)
    __hip_atomic_store(a.counters + blockIdx.x, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

struct StreamPlan { int nt, splits; };

template <int DT, int MT, int ZK>
static void launch_spf(const StreamArgs& a, int nt, hipStream_t st) {
  dim3 grid(a.N / 128 * (8 / nt), a.splits), block(256);
#define MQ_STREAM_LAUNCH(SPF, NT) \
  hipLaunchKernelGGL((w4a16_stream_kernel<DT, MT, ZK, SPF, NT>), grid, block, 0, st, a)
  if (a.gs % 128 != 0) MQ_STREAM_LAUNCH(1, 8);
  else if (nt == 8) MQ_STREAM_LAUNCH(4, 8);
  else if (nt == 4) MQ_STREAM_LAUNCH(4, 4);
  else if (nt == 2) MQ_STREAM_LAUNCH(4, 2);
  else MQ_STREAM_LAUNCH(4, 1);
#undef MQ_STREAM_LAUNCH
}

template <int DT, int MT>
static void launch_zk(const StreamArgs& a, int zk, int nt, hipStream_t st) {
  if (zk == MI355Q_ZP_NONE) launch_spf<DT, MT, MI355Q_ZP_NONE>(a, nt, st);
  else if (zk == MI355Q_ZP_PACKED) launch_spf<DT, MT, MI355Q_ZP_PACKED>(a, nt, st);
  else launch_spf<DT, MT, MI355Q_ZP_PRESCALED>(a, nt, st);
}

template <int DT>
static void launch_mt(const StreamArgs& a, int zk, int nt, hipStream_t st) {
  if (a.M <= 16) launch_zk<DT, 1>(a, zk, nt, st);
  else if (a.M <= 32) launch_zk<DT, 2>(a, zk, nt, st);
  else launch_zk<DT, 4>(a, zk, nt, st);
}

// Work split, fitted to measurements on MI355X at M = 16 and 64.  Narrowing
// the tile group (NT = 8, 4, 2) multiplies the workgroups without any
// exchange, but every workgroup re-reads its K range of the activations from
// L2, so long K stops at NT = 4.  Splitting K costs dependent round trips to
// memory for the partial tiles; the split factor is the one that brings the
// grid closest to one workgroup per CU with at least 8 K blocks each.
StreamPlan w4a16_stream_auto_plan(int M, int K, int N, int gs) {
  const int slabs = N / 128, G = K / 128, cus = device_cu_count();
  StreamPlan p = {8, 1};
  if (gs % 128 == 0) {
    if (M > 32) p.nt = 4;          // 64 rows x 8 tiles of accumulators do not fit the register file
    const int floor_nt = K > 8192 ? 4 : 2;
    while (p.nt > floor_nt && slabs * (8 / p.nt) < cus / 2) p.nt >>= 1;
  }
  const int wgs = slabs * (8 / p.nt);
  const int maxs = G / 8 > 0 ? (G / 8 < 32 ? G / 8 : 32) : 1;
  int best = 1, best_d = abs(wgs - cus);
  for (int s = 2; s <= maxs; ++s) {
    const int d = abs(wgs * s - cus);
    if (d < best_d) { best = s; best_d = d; }
  }
  p.splits = best;
  return p;
}

size_t w4a16_stream_workspace_bytes(int M, int N) {
  const int Mpad = M <= 16 ? 16 : (M <= 32 ? 32 : 64);
  return ((size_t)(N / 16) * sizeof(int) + 255) / 256 * 256 + (size_t)32 * Mpad * N * sizeof(float);
}

// split_k: bits 0..7 force the split factor, bits 8..15 the tiles per
// workgroup (1, 2, 4 or 8); 0 in a field = automatic.
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
  StreamPlan plan = w4a16_stream_auto_plan(M, K, N, group_size);
  const int force_s = split_k & 0xff, force_nt = (split_k >> 8) & 0xff;
  if (force_nt) {
    MQ_REQUIRE(force_nt == 1 || force_nt == 2 || force_nt == 4 || force_nt == 8,
               "w4a16_gemm: tiles per workgroup must be 1, 2, 4 or 8, got %d", force_nt);
    MQ_REQUIRE(force_nt == 8 || group_size % 128 == 0,
               "w4a16_gemm: tile groups below 8 need group_size %% 128 == 0");
    plan.nt = force_nt;
    if (!force_s) plan.splits = 1;
  }
  int splits = force_s ? force_s : plan.splits;
  if (splits > G) splits = G;
  if (splits > 32) splits = 32;
  // no empty splits: ceil(G / splits) * (splits - 1) < G
  while (splits > 1 && ((G + splits - 1) / splits) * (splits - 1) >= G) --splits;
  a.splits = splits;
  a.partial = nullptr;
  a.counters = nullptr;
  if (splits > 1) {
    const int Mpad = M <= 16 ? 16 : (M <= 32 ? 32 : 64);
    size_t cbytes = ((size_t)(N / 16) * sizeof(int) + 255) / 256 * 256;
    size_t need = cbytes + (size_t)splits * Mpad * N * sizeof(float);
    MQ_REQUIRE(workspace && workspace_bytes >= need,
               "w4a16_gemm: workspace of %zu bytes needed for split_k=%d, got %zu", need, splits,
               workspace_bytes);
    a.counters = (int*)workspace;
    a.partial = (float*)((char*)workspace + cbytes);
  }
  if (dtype == MI355Q_F16) launch_mt<MI355Q_F16>(a, zeros_kind, plan.nt, st);
  else launch_mt<MI355Q_BF16>(a, zeros_kind, plan.nt, st);
  MQ_LAUNCH_CHECK("w4a16_gemm(stream)");
  return 0;
}

}  // namespace mi355q
