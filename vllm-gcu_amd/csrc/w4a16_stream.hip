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
  uint32_t gs_magic; // ceil(2^32 / gs): k / gs == umulhi(k, gs_magic) for every k < K
  int splits;
  int per;           // K blocks per split: ceil(K / 128 / splits) (host-side: no division in the kernel's prologue)
  int qrows;         // K / gs
  float* partial;    // [splits][16*MT][N]
  int* counters;     // four per blockIdx.x (<= N/16 workgroups, one per wavefront), zero between launches
  // grouped (fused-MoE) launches: blockIdx.z = block of 16 sorted token slots, all of one expert
  const int32_t* sorted_ids;    // [.. padded ..] slot ids, pads >= numel
  const int32_t* expert_ids;    // [blocks]
  const int32_t* npp;           // device scalar: slots after padding
  const float* topk_weights;    // [numel] or null
  int numel, topk, E;
  long w_stride, s_stride, z_stride;   // per expert, in elements of the respective arrays (weights: 16-byte units)
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
__device__ __forceinline__ void load_partial(const float* p, float* v) {
  if (NT == 1) {
    uint32_t bits = __hip_atomic_load((const uint32_t*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    v[0] = bitcast<float>(bits);
    return;
  }
#pragma unroll
  for (int t = 0; t + 1 < NT; t += 2) {
    uint64_t bits = __hip_atomic_load((const uint64_t*)(p + t), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    v[t] = bitcast<float>((uint32_t)bits);
    v[t + 1 < NT ? t + 1 : t] = bitcast<float>((uint32_t)(bits >> 32));
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
  // Written through to memory (sc0 sc1) instead of left dirty in this XCD's L2: the kernel ends a little
  // sooner (nothing to write back at its end) -- 0.1-0.2 us per launch, 1.8 % of the four-layer decode step.
  if (NT == 1) {
    const uint32_t val = h[0];
    asm volatile("global_store_short %0, %1, off sc0 sc1" ::"v"(out), "v"(val) : "memory");
  } else {
    constexpr int P = NT >= 2 ? NT / 2 : 1;
    uint32_t o[P];
#pragma unroll
    for (int t = 0; t < NT / 2; ++t) o[t] = (uint32_t)h[2 * t] | ((uint32_t)h[2 * t + 1] << 16);
    if (NT == 8) {
      const u4 val = (u4){o[0], o[P > 1 ? 1 : 0], o[P > 2 ? 2 : 0], o[P > 3 ? 3 : 0]};
      asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1" ::"v"(out), "v"(val) : "memory");
    } else if (NT == 4) {
      const u2 val = (u2){o[0], o[P > 1 ? 1 : 0]};
      asm volatile("global_store_dwordx2 %0, %1, off sc0 sc1" ::"v"(out), "v"(val) : "memory");
    } else {
      const uint32_t val = o[0];
      asm volatile("global_store_dword %0, %1, off sc0 sc1" ::"v"(out), "v"(val) : "memory");
    }
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

template <int NT>
__device__ __forceinline__ void buf_load_halves(rsrc_t r, uint32_t off, uint32_t* dst) {
  if (NT == 8) { u4 v = buf_load16(r, off); dst[0] = v[0]; dst[NT > 2 ? 1 : 0] = v[1]; dst[NT > 4 ? 2 : 0] = v[2]; dst[NT > 6 ? 3 : 0] = v[3]; }
  else if (NT == 4) { u2 v = bitcast<u2>(__builtin_amdgcn_raw_buffer_load_b64(r, (int)off, 0, 0)); dst[0] = v[0]; dst[NT > 2 ? 1 : 0] = v[1]; }
  else if (NT == 2) dst[0] = __builtin_amdgcn_raw_buffer_load_b32(r, (int)off, 0, 0);
  else dst[0] = __builtin_amdgcn_raw_buffer_load_b16(r, (int)off, 0, 0);
}

// GR: fused-MoE grouped launch -- the 16 MT rows of a workgroup are the token slots of block
// blockIdx.z (gathered from x by slot id / topk, scattered to out by slot id, optionally times the
// routing weight) and the weights are those of the block's expert.  The same stream as a dense
// decode launch: a decode-sized MoE layer is bound by the experts' weights in exactly the same way.
template <int DT, int MT, int ZK, int SPF, int NT, bool GR = false>
__global__ void __launch_bounds__(256, (MT == 1 || (MT == 2 && NT <= 4)) ? 2 : 1)
w4a16_stream_kernel(StreamArgs a) {
  typedef Mma<DT> MM;
  typedef typename MM::vec vec;
  static_assert(!GR || MT <= 2, "grouped launches take blocks of 16 or 32 slots");
  if (GR) {
    if ((int)blockIdx.z * 16 * MT >= *a.npp) return;
    const long e = a.expert_ids[blockIdx.z];
    if (e < 0 || e >= a.E) {
      // not one of this rank's experts (-1 under an expert map): zero the block's valid slot rows in this
      // workgroup's columns and read no weights
      const int zr = threadIdx.x >> 4, zc = threadIdx.x & 15;
      const float zero[NT] = {};
      const int col = 128 * (int)(blockIdx.x / (8 / NT)) + 8 * zc + (int)(blockIdx.x % (8 / NT)) * NT;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const int id = a.sorted_ids[(int)blockIdx.z * 16 * MT + 16 * mt + zr];
        if (id < a.numel) store_out_row<DT, NT>(a.out + (size_t)id * a.N + col, nullptr, col, zero);
      }
      return;
    }
    a.qw += e * a.w_stride;
    a.scales += e * a.s_stride;
    if (ZK == MI355Q_ZP_PACKED) a.zeros = (const uint32_t*)a.zeros + e * a.z_stride;
    if (ZK == MI355Q_ZP_PRESCALED) a.zeros = (const uint16_t*)a.zeros + e * a.z_stride;
  }
  // the wavefront index is made visibly uniform: K-block indices and loop control then live in scalar registers
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int c = lane & 15, kq = lane >> 4;
  constexpr int TG = 8 / NT;                          // tile groups per slab
  constexpr int HW = NT >= 2 ? NT / 2 : 1;            // packed 16-bit pairs per lane
  const int slab = blockIdx.x / TG, t0 = (blockIdx.x % TG) * NT, split = blockIdx.y;
  const int G = a.K >> 7;
  const int per = a.per;
  const int gb = split * per;
  const int ge = min(G, gb + per);
  const int N = a.N, K = a.K;

  f4 acc[MT][NT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[mt][t] = (f4){0.f, 0.f, 0.f, 0.f};

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
  constexpr int W = 4;                                // wavefronts per workgroup (8 and 16 were measured: not faster)
  // K blocks of this wavefront: gb + wave, + W, ... in order (starting each workgroup at a different
  // block of its range was measured equal, and the modulo sat in front of the first loads)
  const int g0 = gb + wave;
  const int nb = (ge - g0 + W - 1) / W;
  auto blk = [&](int i) { return g0 + W * i; };      // i-th block of this wavefront, i < nb
  const rsrc_t wres = make_rsrc(a.qw + (size_t)slab * G * 512, (uint32_t)G * 8192u);
  const rsrc_t sres = make_rsrc(a.scales, (uint32_t)a.qrows * N * 2u);
  const rsrc_t zres = make_rsrc(a.zeros, ZK == MI355Q_ZP_PACKED ? (uint32_t)a.qrows * (N >> 3) * 4u
                                                                 : (uint32_t)a.qrows * N * 2u);
  const rsrc_t xres = make_rsrc(a.x, (uint32_t)a.M * K * 2u);
  const uint32_t wlane = (uint32_t)(t0 * 64 + lane) * 16u;
  uint32_t xlane[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
    // Activations are fetched with 4 consecutive lanes on 64 contiguous bytes of one row (lane =
    // 4 * row + chunk): the MFMA wants lane 16 * chunk + row, whose neighbours sit a whole row
    // pitch apart, and 64 single 16-byte requests per instruction cost the L1 more than the weight
    // stream itself.  compute_block moves each register to its MFMA lane (xperm).
    // rows past M repeat the last row: output rows are independent and rows >= M are never stored
    if (GR) {
      // slot id -> row of x (pads repeat the last valid slot: their results are never stored)
      const int id = a.sorted_ids[(int)blockIdx.z * 16 * MT + 16 * mt + (lane >> 2)];
      xlane[mt] = ((uint32_t)(min(id, a.numel - 1) / a.topk) * K + 8 * (lane & 3)) * 2u;
    } else
    xlane[mt] = ((uint32_t)min(16 * mt + (lane >> 2), a.M - 1) * K + 8 * (lane & 3)) * 2u;
  // block i of this wavefront's order; i >= nb loads nothing (zeros, no memory traffic)
  auto load_block = [&](Block& b, int i) {
    const bool have = i < nb;
    const uint32_t oob = have ? 0u : 0x80000000u;
    const int g = have ? blk(i) : g0;
    const uint32_t wo = wlane + (uint32_t)g * 8192u + oob;
#pragma unroll
    for (int t = 0; t < NT; ++t) b.w[t] = buf_load16_nt(wres, wo + t * 1024);
#pragma unroll
    for (int f = 0; f < 4 / SPF; ++f) {
      const uint32_t krow = 128 * g + 32 * SPF * f;
      const uint32_t qrow = __umulhi(krow, a.gs_magic);
      buf_load_halves<NT>(sres, (qrow * N + ncol) * 2u + oob, b.sraw[f]);
      b.zword[f] = 0x88888888u;
      if (ZK == MI355Q_ZP_PACKED)
        b.zword[f] = __builtin_amdgcn_raw_buffer_load_b32(zres, (int)((qrow * (N >> 3) + (ncol8 >> 3)) * 4u + oob), 0, 0);
      if (ZK == MI355Q_ZP_PRESCALED) buf_load_halves<NT>(zres, (qrow * N + ncol) * 2u + oob, b.zraw[f]);
    }
    if (XA) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int s = 0; s < 4; ++s)
          b.xr[XA ? 4 * mt + s : 0] = buf_load16(xres, xlane[mt] + (uint32_t)(128 * g + 32 * s) * 2u + oob);
    }
  };
  // activations of block i for launches that cannot carry them a block ahead (no registers to spare)
  struct Acts { u4 xr[XA ? 1 : MT][4]; };
  auto load_acts = [&](Acts& x, int i) {
    if (XA) return;
    const int g = blk(i);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int s = 0; s < 4; ++s) x.xr[mt][s] = buf_load16(xres, xlane[mt] + (uint32_t)(128 * g + 32 * s) * 2u);
  };

  const int xperm = 4 * (4 * c + kq);                // byte index of the lane that fetched this lane's MFMA chunk
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
          const u4 got = XA ? b.xr[XA ? 4 * mt + SPF * f + s : 0] : xa.xr[XA ? 0 : mt][SPF * f + s];
          u4 raw;
#pragma unroll
          for (int d = 0; d < 4; ++d) raw[d] = (uint32_t)__builtin_amdgcn_ds_bpermute(xperm, (int)got[d]);
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
    // one is consumed (deeper rings were measured and are not faster).  The
    // prefetch is unconditional (past the end it is a descriptor-range miss:
    // zeros, no traffic) and every step leaves the loop through a plain break,
    // so the body is straight-line code and the compiler waits for exactly
    // the block being consumed.
    //
    // K order: the wavefront's nb blocks are visited starting at a
    // workgroup-dependent position.  All workgroups read the same activation
    // rows, and a K block of them (16 rows x 256 B at a pitch of 2 K bytes)
    // sits in very few L2 channels: in a common order every workgroup of an XCD
    // would hammer those channels at the same moment.  (The order is fixed per
    // workgroup, so results stay run-to-run identical.)
    Block ring[2];
    Acts xa;
    if (nb > 0) {
      load_block(ring[0], 0);
      int i = 0;
      while (true) {
        // sched_barrier: keep the prefetch ahead of the arithmetic, the
        // instruction scheduler would otherwise sink the loads next to
        // their first use one iteration later
        load_acts(xa, i);
        load_block(ring[1], i + 1);
        __builtin_amdgcn_sched_barrier(0);
        compute_block(ring[0], xa);
        __builtin_amdgcn_sched_barrier(0);
        if (++i >= nb) break;
        load_acts(xa, i);
        load_block(ring[0], i + 1);
        __builtin_amdgcn_sched_barrier(0);
        compute_block(ring[1], xa);
        __builtin_amdgcn_sched_barrier(0);
        if (++i >= nb) break;
      }
    }
  }

  // ---- reduce the W wavefronts through LDS.  A lane holds 4 rows (4 kq + i)
  // x NT columns per 16-row tile; wavefront w sums and stores CW of those
  // 4 NT values: row i = w CW / NT, columns (w CW) % NT .. + CW ----
  constexpr int CW = 4 * NT / W > 0 ? 4 * NT / W : 1;
  __shared__ float red[W][4 * NT][64];
  const int Mpad = 16 * MT;
  const bool fin_wave = wave * CW < 4 * NT;          // NT = 1 with 8 wavefronts: the upper four only contribute
  const int q0 = fin_wave ? wave * CW : 0, ri = q0 / NT, tc = q0 % NT;
  float fin[MT][CW];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) red[wave][i * NT + t][lane] = acc[mt][t][i];
    __syncthreads();
#pragma unroll
    for (int t = 0; t < CW; ++t) {
      float v = red[0][q0 + t][lane];
#pragma unroll
      for (int w = 1; w < W; ++w) v += red[w][q0 + t][lane];
      fin[mt][t] = v;
    }
    __syncthreads();
    const int m = 16 * mt + 4 * kq + ri;
    if (GR) {
      if (fin_wave) {
        const int id = a.sorted_ids[(int)blockIdx.z * 16 * MT + m];
        if (id < a.numel) {
          if (a.topk_weights) {
            const float rw = a.topk_weights[id];
#pragma unroll
            for (int t = 0; t < CW; ++t) fin[mt][t] *= rw;
          }
          store_out_row<DT, CW>(a.out + (size_t)id * N + ncol + tc, nullptr, ncol + tc, fin[mt]);
        }
      }
      continue;
    }
    if (fin_wave && m < a.M) {
      if (a.splits == 1)
        store_out_row<DT, CW>(a.out + (size_t)m * N + ncol + tc, a.bias, ncol + tc, fin[mt]);
      else
        store_partial<CW>(a.partial + ((size_t)split * Mpad + m) * N + ncol + tc, fin[mt]);
    }
  }
  if (GR || a.splits == 1) return;

  // ---- cross-workgroup split-K ---------------------------------------------
  // Partial tiles travel as device-scope relaxed accesses (they bypass the
  // per-XCD L2 instead of flushing it).  The exchange is per wavefront: each of
  // the four wavefronts owns a slice of the workgroup's tile (its rows and
  // columns of the LDS reduction above) and an arrival counter of its own.  A
  // wavefront waits until its own partial stores have been acknowledged (vmcnt
  // counts stores on gfx9), then counts itself in; the wavefront that arrives
  // last at a slice adds that slice's tiles in split order, so the sum is
  // reproducible.  No workgroup barrier: the wavefronts of a workgroup do not
  // wait for each other's trips to memory.
  if (!fin_wave) return;
  // The hardware order is: partial stores acknowledged (vmcnt(0)) -> counter increment -> partial loads
  // (issued after the increment has returned).  The compiler must keep that order too: relaxed atomics
  // to different addresses may legally be reordered, so the increment sits between two signal fences
  // (compiler-only barriers: no instruction, no cache writeback).
  __atomic_signal_fence(__ATOMIC_SEQ_CST);
  __builtin_amdgcn_s_waitcnt(0x0f70);              // vmcnt(0)
  __atomic_signal_fence(__ATOMIC_SEQ_CST);
  int* counter = a.counters + (int)blockIdx.x * W + wave;
  int old = 0;
  if (lane == 0) old = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  old = __builtin_amdgcn_readfirstlane(old);
  __atomic_signal_fence(__ATOMIC_SEQ_CST);
  if (old != a.splits - 1) return;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = 16 * mt + 4 * kq + ri;
    if (!fin_wave || m >= a.M) continue;
    float v[CW];
#pragma unroll
    for (int t = 0; t < CW; ++t) v[t] = 0.f;
    // four splits' tiles are requested together and then added in split order: one trip to memory
    // per four splits instead of one per split (a loop of load-then-add waits for every load in turn)
    for (int sp = 0; sp < a.splits; sp += 4) {
      float w[4][CW];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int spj = min(sp + j, a.splits - 1);   // past the end: a repeat that is not added
        load_partial<CW>(a.partial + ((size_t)spj * Mpad + m) * N + ncol + tc, w[j]);
      }
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (sp + j < a.splits) {
#pragma unroll
          for (int t = 0; t < CW; ++t) v[t] += w[j][t];
        }
    }
    store_out_row<DT, CW>(a.out + (size_t)m * N + ncol + tc, a.bias, ncol + tc, v);
  }
  if (lane == 0) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

struct StreamPlan { int nt, splits; };

template <int DT, int MT, int ZK>
static void launch_spf(const StreamArgs& a, int nt, hipStream_t st) {
  dim3 grid(a.N / 128 * (8 / nt), a.splits), block(256);
#define MQ_STREAM_LAUNCH(SPF, NT) \
  hipLaunchKernelGGL((w4a16_stream_kernel<DT, MT, ZK, SPF, NT>), grid, block, 0, st, a)
  if (a.gs % 128 != 0) {
    // 32 scale rows per K block: callers keep these launches to 32 rows (64 rows x 8 tiles spill)
    if constexpr (MT <= 2) MQ_STREAM_LAUNCH(1, 8);
  }
  else if (nt == 8) {
    if constexpr (MT <= 2) MQ_STREAM_LAUNCH(4, 8);    // 64 rows x 8 tiles do not fit the register file
  }
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

// Work split: tiles of 16 columns per workgroup (NT = 8, 4, 2, 1) and K ranges (splits) that separate
// workgroups sum through the workspace.  Chosen by a cost per workgroup, fitted to the measured times of
// every (NT, splits) pair on 18 layer shapes of five model families at M = 16 and 64 (within 1 % of the
// best pair on 30 of 35, 14 % at worst; the rule before it -- the grid nearest to one workgroup per CU --
// was up to 50 % off outside the Llama-3-8B shapes, mostly by overshooting the CU count a little, which
// costs a second round):
//   bytes a workgroup pulls into its CU: its share of the packed weights plus half of the activation
//   bytes of its K range (every workgroup of a slab reads them again, from the L2; narrowing the tile
//   group multiplies the workgroups without any exchange but not their activation reads),
//   times the rounds the grid needs on the chip; a K split never goes beyond one round,
//   plus, for a split, a fixed 45 KB (the dependent round trips of the exchange) and 2.5 x the partial
//   tiles the last workgroup of a slab adds up.
StreamPlan w4a16_stream_auto_plan(int M, int K, int N, int gs) {
  const int slabs = N / 128, G = K / 128, cus = device_cu_count();
  const int maxs = G / 8 > 0 ? (G / 8 < 32 ? G / 8 : 32) : 1;
  StreamPlan p = {8, 1};
  if (gs % 128 != 0) {
    // groups of 64 / 32: eight tiles per workgroup only; as many K ranges as stay within one round
    for (int s = 2; s <= maxs; ++s)
      if ((long)slabs * s <= cus) p.splits = s;
    return p;
  }
  const double Mp = M <= 16 ? 16 : (M <= 32 ? 32 : 64);
  double best = -1.0;
  // (64 rows x 8 tiles of accumulators do not fit the register file; one tile per workgroup reads the
  // activations of all of K per 16 columns: up to K = 8192)
  for (int nt = M > 32 ? 4 : 8; nt >= 1; nt >>= 1) {
    if (nt == 1 && K > 8192) continue;
    const long wg = (long)slabs * (8 / nt);
    for (int s = 1; s <= maxs; ++s) {
      const long W = wg * s;
      if (s > 1 && W > cus) break;
      const long rounds = (W + cus - 1) / cus;
      const double bw = (double)K * N / 2 / (double)W, bx = Mp * K * 2 / s;
      const double cost = (double)rounds * (bw + 0.5 * bx) + (s > 1 ? 45000.0 + 2.5 * s * nt * Mp * 64 : 0.0);
      if (best < 0 || cost < best) { best = cost; p.nt = nt; p.splits = s; }
    }
  }
  return p;
}

// The arrival counters own a fixed region at the start of the workspace, whatever the shape:
// one workspace serves layers of different widths, and the counters must stay zero between
// launches -- a width-dependent boundary would let one layer's partial tiles land on the
// counters of a wider layer.
static constexpr size_t STREAM_COUNTER_BYTES = (size_t)64 << 10;

size_t w4a16_stream_workspace_bytes(int M, int N) {
  const int Mpad = M <= 16 ? 16 : (M <= 32 ? 32 : 64);
  return STREAM_COUNTER_BYTES + (size_t)32 * Mpad * N * sizeof(float);
}

// exactly what the automatic plan of a launch of up to 64 rows uses (0: K is not split)
size_t w4a16_stream_plan_workspace_bytes(int M, int K, int N, int gs) {
  const StreamPlan plan = w4a16_stream_auto_plan(M, K, N, gs);
  const int G = K / 128;
  int splits = plan.splits > G ? G : plan.splits;
  if (splits > 32) splits = 32;
  while (splits > 1 && ((G + splits - 1) / splits) * (splits - 1) >= G) --splits;
  if (splits <= 1) return 0;
  const int Mpad = M <= 16 ? 16 : (M <= 32 ? 32 : 64);
  return STREAM_COUNTER_BYTES + (size_t)splits * Mpad * N * sizeof(float);
}

// split_k: bits 0..7 force the split factor, bits 8..15 the tiles per
// workgroup (1, 2, 4 or 8); 0 in a field = automatic.
int w4a16_stream_launch(void* out, const void* x, const int32_t* qweight, const void* scales,
                        const void* zeros, int zeros_kind, const void* bias, int M, int K, int N,
                        int group_size, int dtype, void* workspace, size_t workspace_bytes,
                        int split_k, hipStream_t st) {
  StreamArgs a = {};
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
  MQ_REQUIRE(group_size % 128 == 0 || M <= 32, "w4a16_gemm(stream): group sizes below 128 take at most 32 rows per launch, got %d", M);
  MQ_REQUIRE((size_t)M * K * 2 < ((size_t)1 << 31) && (size_t)(K / group_size) * N * 2 < ((size_t)1 << 31) &&
                 (size_t)K * group_size < ((size_t)1 << 32),
             "w4a16_gemm(stream): activations and scales must each stay below 2 GiB (M=%d K=%d N=%d)", M, K, N);
  a.gs_magic = (uint32_t)((((uint64_t)1 << 32) + group_size - 1) / group_size);
  if (force_nt) {
    MQ_REQUIRE(force_nt == 1 || force_nt == 2 || force_nt == 4 || force_nt == 8,
               "w4a16_gemm: tiles per workgroup must be 1, 2, 4 or 8, got %d", force_nt);
    MQ_REQUIRE(force_nt == 8 || group_size % 128 == 0,
               "w4a16_gemm: tile groups below 8 need group_size %% 128 == 0");
    plan.nt = (force_nt == 8 && M > 32) ? 4 : force_nt;
    if (!force_s) plan.splits = 1;
  }
  int splits = force_s ? force_s : plan.splits;
  if (splits > G) splits = G;
  if (splits > 32) splits = 32;
  // no empty splits: ceil(G / splits) * (splits - 1) < G
  while (splits > 1 && ((G + splits - 1) / splits) * (splits - 1) >= G) --splits;
  a.splits = splits;
  a.per = (G + splits - 1) / splits;
  a.qrows = K / group_size;
  a.partial = nullptr;
  a.counters = nullptr;
  if (splits > 1) {
    const int Mpad = M <= 16 ? 16 : (M <= 32 ? 32 : 64);
    const size_t cbytes = STREAM_COUNTER_BYTES;
    MQ_REQUIRE((size_t)(N / 16) * 4 * sizeof(int) <= cbytes, "w4a16_gemm(stream): N=%d needs more arrival counters than the workspace holds", N);
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

// Fused-MoE grouped GEMM for blocks of 16 or 32 slots (decode-sized token counts): one launch over
// (tile groups, blocks); K is never split, so there is no workspace.
template <int DT, int ZK>
static void launch_grouped_nt(const StreamArgs& a, int mt, int nt, int blocks, hipStream_t st) {
  dim3 grid(a.N / 128 * (8 / nt), 1, blocks), block(256);
#define MQ_GR_LAUNCH(MT, NT) hipLaunchKernelGGL((w4a16_stream_kernel<DT, MT, ZK, 4, NT, true>), grid, block, 0, st, a)
  if (mt == 1) {
    if (nt == 8) MQ_GR_LAUNCH(1, 8);
    else if (nt == 4) MQ_GR_LAUNCH(1, 4);
    else MQ_GR_LAUNCH(1, 2);
  } else {
    if (nt == 8) MQ_GR_LAUNCH(2, 8);
    else if (nt == 4) MQ_GR_LAUNCH(2, 4);
    else MQ_GR_LAUNCH(2, 2);
  }
#undef MQ_GR_LAUNCH
}

int w4a16_stream_grouped_launch(void* out, const void* x, const int32_t* qweight, const void* scales,
                                const void* zeros, int zeros_kind, const float* topk_weights,
                                const int32_t* sorted_ids, const int32_t* expert_ids, const int32_t* npp,
                                int numel, int topk, int block_size, int max_blocks, int E, int K, int N,
                                int group_size, int dtype, hipStream_t st) {
  MQ_REQUIRE(block_size == 16 || block_size == 32, "moe_w4a16(stream): blocks of 16 or 32 slots, got %d", block_size);
  const int mt = block_size / 16;
  MQ_REQUIRE(group_size % 128 == 0 && K % 128 == 0 && N % 128 == 0,
             "moe_w4a16(stream): K=%d, N=%d and group_size=%d must be multiples of 128", K, N, group_size);
  const int rows = numel / (topk > 0 ? topk : 1) + 1;
  MQ_REQUIRE((size_t)rows * K * 2 < ((size_t)1 << 31) && (size_t)(K / group_size) * N * 2 < ((size_t)1 << 31) &&
                 (size_t)K * group_size < ((size_t)1 << 32),
             "moe_w4a16(stream): activations and one expert's scales must each stay below 2 GiB (K=%d N=%d)", K, N);
  StreamArgs a = {};
  a.out = (uint16_t*)out;
  a.x = (const uint16_t*)x;
  a.qw = (const u4*)qweight;
  a.scales = (const uint16_t*)scales;
  a.zeros = zeros;
  a.bias = nullptr;
  a.M = (numel + topk - 1) / topk;                 // rows of x
  a.K = K; a.N = N; a.gs = group_size;
  a.gs_magic = (uint32_t)((((uint64_t)1 << 32) + group_size - 1) / group_size);
  a.splits = 1;
  a.per = K / 128;
  a.qrows = K / group_size;
  a.sorted_ids = sorted_ids; a.expert_ids = expert_ids; a.npp = npp; a.topk_weights = topk_weights;
  a.numel = numel; a.topk = topk; a.E = E;
  a.w_stride = (long)(K / 8) * N / 4;
  a.s_stride = (long)(K / group_size) * N;
  a.z_stride = zeros_kind == MI355Q_ZP_PACKED ? (long)(K / group_size) * (N / 8) : (long)(K / group_size) * N;
  // tiles per workgroup: all eight of a slab unless that leaves the chip short of workgroups
  const int slabs = N / 128, cus = device_cu_count();
  int nt = 8;
  while (nt > 2 && (long)slabs * (8 / nt) * max_blocks < 2L * cus) nt >>= 1;
#define MQ_GR_ZK(DT)                                                                          \
  do {                                                                                        \
    if (zeros_kind == MI355Q_ZP_NONE) launch_grouped_nt<DT, MI355Q_ZP_NONE>(a, mt, nt, max_blocks, st);    \
    else if (zeros_kind == MI355Q_ZP_PACKED) launch_grouped_nt<DT, MI355Q_ZP_PACKED>(a, mt, nt, max_blocks, st); \
    else launch_grouped_nt<DT, MI355Q_ZP_PRESCALED>(a, mt, nt, max_blocks, st);               \
  } while (0)
  if (dtype == MI355Q_F16) MQ_GR_ZK(MI355Q_F16);
  else MQ_GR_ZK(MI355Q_BF16);
#undef MQ_GR_ZK
  MQ_LAUNCH_CHECK("moe_w4a16(stream)");
  return 0;
}

}  // namespace mi355q
