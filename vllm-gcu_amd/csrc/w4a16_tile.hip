// W4A16 LDS-staged MFMA GEMM for large M (prefill-shaped) on gfx950.
//
// Workgroup tile 128 (M) x 256 (N), K step 128 (one slab K block), 4
// wavefronts side by side along N: wave w owns 64 columns (four 16-column
// tiles of one slab) for all 128 rows.  Because the slab layout already stores
// each lane's MFMA B operand contiguously, a wavefront dequantises its own
// columns straight into B operands in registers -- the exact integers (q - z),
// the group scale is applied to the fp32 partial sum of each K block -- and
// every operand is reused for all row tiles of the wavefront.  The activation
// tile is shared by the wavefronts through LDS (double buffered, rows padded by
// 32 B so the operand reads are bank-conflict free).  fp32 accumulate.  The
// fp16 128-row variant runs a hand-pipelined K loop (see PIPE below), the
// others a plain one.
#include "common.h"

namespace mi355q {

namespace {

constexpr int BN = 256, BK = 128;
// bytes per LDS row: 256 + 32 of padding.  Measured on MI355X, the MFMA operand
// read (lane = row + 16 * chunk, 16 B each) runs at the full LDS rate with a
// 288-byte pitch and at half of it with 272 or 264
constexpr int A_ROW = BK * 2 + 32;

struct TileArgs {
  uint16_t* out;
  const uint16_t* x;
  const u4* qw;
  const uint16_t* scales;       // group scales in the activation type, or
  const float* scales_f32;      // ... in fp32 (SF32 kernels; the other pointer is unused)
  const float* out_scale;       // optional device scalar multiplied into every output
  const float* row_scale;       // [M] per-row multiplier of the output (IOBF kernels: bf16 rows staged as fp16)
  const void* zeros;
  const uint16_t* bias;
  int M, K, N, gs;
  // grouped (MoE) mode: rows come from sorted_ids, weights from expert_ids
  const int* sorted_ids;      // [blocks * BM] flat (token, slot) ids, pad = numel
  const int* expert_ids;      // [blocks]
  const int* npp;             // device scalar: padded id count
  const float* topk_weights;  // [numel] or null
  int numel, topk, E;
  // split-K: blockIdx.z takes K blocks [z * kper, (z + 1) * kper) and writes an fp32 partial
  // tile to partial[z][M][N] (grouped: M = numel, rows indexed by slot id, routing weight not yet
  // applied); a second kernel adds the partials up
  int kper;                   // K blocks per split (G when there is no split)
  uint32_t gpk_magic;         // narrow kernel: ceil(2^32 / (gs / 128)), 0 when a group is one K block
  float* partial;             // null: write the output directly
  long w_stride, s_stride, z_stride;   // per-expert strides in elements of the respective arrays
};

// B operands are the exact integers (q - z) in the activation type; the group
// scale multiplies the fp32 partial sum of each 128-row K block instead of
// every weight, so the only rounding left is that of the fp32 accumulation.
// (a & mask) | orv in one v_and_or_b32: the kernels keep the mask in a scalar and the magic in a
// vector register (an opaque asm) -- as literals the compiler has to emit an and + or pair.
struct DqConst {
  uint32_t magic, mlo, mhi;
};
__device__ __forceinline__ DqConst dq_consts() {
  DqConst k = {0x64006400u, 0x000f000fu, 0x00f000f0u};
  asm volatile("" : "+v"(k.magic));
  asm volatile("" : "+s"(k.mlo));
  asm volatile("" : "+s"(k.mhi));
  return k;
}

template <int DT> struct TileMma;
template <> struct TileMma<MI355Q_F16> {
  typedef h8 vec;
  static __device__ __forceinline__ f4 run(vec a, vec b, f4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
  // one packed word -> 8 values (q - z); zz = {1024 + z, 64 + z}
  static __device__ __forceinline__ vec dequant(uint32_t w, h2 zz, const DqConst& k) {
    const h2 zlo = {zz.x, zz.x}, zhi = {zz.y, zz.y};
    const h2 sixteenth = {(_Float16)0.0625f, (_Float16)0.0625f};
    uint32_t w8 = w >> 8;
    h2 a0 = bitcast<h2>((w & k.mlo) | k.magic);       // 1024 + q
    h2 a1 = bitcast<h2>((w & k.mhi) | k.magic);       // 1024 + 16 q
    h2 a2 = bitcast<h2>((w8 & k.mlo) | k.magic);
    h2 a3 = bitcast<h2>((w8 & k.mhi) | k.magic);
    h2 r0 = a0 - zlo;
    h2 r1 = __builtin_elementwise_fma(a1, sixteenth, -zhi);
    h2 r2 = a2 - zlo;
    h2 r3 = __builtin_elementwise_fma(a3, sixteenth, -zhi);
    return (h8){r0.x, r0.y, r1.x, r1.y, r2.x, r2.y, r3.x, r3.y};
  }
};
template <> struct TileMma<MI355Q_BF16> {
  typedef b8 vec;
  static __device__ __forceinline__ f4 run(vec a, vec b, f4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
  // The fp16 patterns 1024 + q and 1024 + 16 q, minus 1024 + z respectively times 1 / 16 minus 64 + z, in one
  // mixed-precision fused multiply-add per weight (fp16 sources, exact fp32 result q - z), then one packed
  // conversion per pair: the small integer is exact in bf16 too.  Four instructions per pair.
  static __device__ __forceinline__ uint32_t pair(h2 a, float m, _Float16 z) {
    typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
    const bf2 r = {(__bf16)__builtin_fmaf((float)a.x, m, -(float)z), (__bf16)__builtin_fmaf((float)a.y, m, -(float)z)};
    return bitcast<uint32_t>(r);
  }
  static __device__ __forceinline__ vec dequant(uint32_t w, h2 zz, const DqConst& k) {
    float one = 1.0f, sixteenth = 0.0625f;
    asm volatile("" : "+s"(one));                     // (as a literal the multiplication folds away and the
    asm volatile("" : "+s"(sixteenth));               //  conversion becomes an instruction of its own)
    const uint32_t w8 = w >> 8;
    const u4 r = {pair(bitcast<h2>((w & k.mlo) | k.magic), one, zz.x), pair(bitcast<h2>((w & k.mhi) | k.magic), sixteenth, zz.y),
                  pair(bitcast<h2>((w8 & k.mlo) | k.magic), one, zz.x), pair(bitcast<h2>((w8 & k.mhi) | k.magic), sixteenth, zz.y)};
    return bitcast<vec>(r);
  }
};

// MT = row tiles of 16 per workgroup (block rows BM = 16 MT); GROUPED selects
// the MoE row gather.  WM = 1: four wavefronts, each all BM rows of its 64
// columns.  WM = 2: eight wavefronts, the upper four take the upper half of
// the rows (both halves dequantise the same weights, but two wavefronts per
// SIMD keep the matrix pipe fed while one of them waits or dequantises).
// GPB = quantisation groups per K block of 128: 1 for group sizes that are multiples of 128, 2 / 4 for
// groups of 64 / 32 (plain loop only: each group's steps accumulate into a partial tile of their own).
// IOBF (with DT = fp16; grouped: the multiplier belongs to the row the slot was gathered from): the activations are bf16 rows that a pass before this kernel scaled by a
// power of two each and stored as fp16 (exact: eight mantissa bits into eleven); scales, pre-scaled
// zero-points, bias and output are bf16, and the epilogue multiplies each row by its power of two.
template <int DT, int ZK, int MT, bool GROUPED, int WM, bool SF32 = false, int GPB = 1, bool IOBF = false>
__global__ void __launch_bounds__(256 * WM, WM == 1 ? 2 : 1)
w4a16_tile_kernel(TileArgs a) {
  typedef TileMma<DT> MM;
  typedef typename MM::vec vec;
  static_assert(!IOBF || (DT == MI355Q_F16 && MT == 4 && WM == 1), "bf16 in and out around the fp16 loop: 64-row tiles");
  typedef Elem<IOBF ? MI355Q_BF16 : DT> IO;       // the type of scales, pre-scaled zero-points, bias and output
  static_assert(MT % WM == 0, "row tiles split evenly over the wavefront rows");
  constexpr int BM = 16 * MT;
  constexpr int MTW = MT / WM;                    // row tiles per wavefront
  constexpr int NTHR = 256 * WM;
  constexpr int A_BUF = BM * A_ROW;
  extern __shared__ __align__(16) unsigned char lds[];
  __shared__ int tok[GROUPED ? BM : 1];
  __shared__ int live_s;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = (tid >> 6) & 3, wmh = tid >> 8;
  const int c = lane & 15, kq = lane >> 4;
  const int N = a.N, K = a.K, M = a.M;
  const int G = K >> 7;
  const int m0 = blockIdx.y * BM;
  const u4* qw = a.qw;
  const uint16_t* scales = a.scales;
  const float* scales32 = a.scales_f32;
  const char* zeros = (const char*)a.zeros;
  // row tiles of the block that hold at least one real slot (the pads of an expert's last block
  // are skipped by the matrix instructions); bit = row tile
  int live_tiles = (1 << MT) - 1;
  if (GROUPED) {
    if (m0 >= *a.npp) return;                       // block beyond the padded ids
    const long e = a.expert_ids[blockIdx.y];
    if (e < 0 || e >= a.E) {                        // not one of this rank's experts: zero rows, no weights read
      const int col0 = blockIdx.x * BN, ncols = min(BN, N - col0);
      if (a.partial) {
        // split K: the reduction sums every split's rows, so each split zeroes its own
        const int per_row = ncols >> 2;
        for (int i = tid; i < BM * per_row; i += NTHR) {
          const int r = i / per_row, piece = i - r * per_row;
          const int id = a.sorted_ids[m0 + r];
          if (id < a.numel)
            *(f4*)(a.partial + ((size_t)blockIdx.z * a.numel + id) * N + col0 + 4 * piece) = (f4){0.f, 0.f, 0.f, 0.f};
        }
      } else {
        zero_block_columns(a.out, a.sorted_ids + m0, BM, a.numel, N, col0, ncols, NTHR);
      }
      return;
    }
    qw += e * a.w_stride;
    if (SF32) scales32 += e * a.s_stride;
    else scales += e * a.s_stride;
    if (zeros) zeros += e * a.z_stride * (ZK == MI355Q_ZP_PACKED ? 4 : 2);
    if (tid == 0) live_s = 0;
    for (int r = tid; r < BM; r += NTHR) tok[r] = a.sorted_ids[m0 + r];
    __syncthreads();
    if (tid < BM) {
      const unsigned long long valid = __ballot(tok[tid] < a.numel);
      if (lane == 0) {
        int m = 0;
#pragma unroll
        for (int t = 0; t < 4; ++t) m |= ((valid >> (16 * t)) & 0xffffull) ? (1 << t) : 0;
        if (m) atomicOr(&live_s, m << (4 * (tid >> 6)));
      }
    }
    __syncthreads();
    live_tiles = live_s;
    if (live_tiles == 0) return;                    // pads only
  }
  auto tile_live = [&](int mt) { return !GROUPED || ((live_tiles >> (wmh * MTW + mt)) & 1); };
  // N may end in the middle of the 256-column tile: the two wavefronts of a
  // missing slab compute on the previous one and skip the epilogue
  const bool live = (blockIdx.x * 2 + (wave >> 1)) < (N >> 7);
  const int slab = live ? blockIdx.x * 2 + (wave >> 1) : (N >> 7) - 1;
  const int t0 = (wave & 1) * 4;
  const int ncol = 128 * slab + 8 * c + t0;          // first of this lane's 4 columns

  f4 acc[MTW][4];
#pragma unroll
  for (int mt = 0; mt < MTW; ++mt)
#pragma unroll
    for (int t = 0; t < 4; ++t) acc[mt][t] = (f4){0.f, 0.f, 0.f, 0.f};

  const DqConst dqk = dq_consts();

  // global -> register staging of the next activation tile: thread tid loads
  // MTW chunks of 16 B: row = pass * 16 WM + tid / 16, chunk = tid % 16
  const int arow = tid >> 4, achunk = tid & 15;
  // byte offsets from a.x (32-bit: the host checks that the activation matrix is below 4 GiB)
  uint32_t aofs[MTW];
#pragma unroll
  for (int p = 0; p < MTW; ++p) {
    int row;
    if (GROUPED) row = min(tok[p * 16 * WM + arow], a.numel - 1) / a.topk;   // pads read a valid row
    else row = min(m0 + p * 16 * WM + arow, M - 1);
    aofs[p] = ((uint32_t)row * (uint32_t)K + 8u * achunk) * 2u;
  }
  u4 areg[MTW];
  auto load_a = [&](int g) {
#pragma unroll
    for (int p = 0; p < MTW; ++p) areg[p] = *(const u4*)((const char*)a.x + (aofs[p] + 256u * (uint32_t)g));
  };
  auto store_a = [&](unsigned buf_off) {
    unsigned char* base = lds + buf_off;
#pragma unroll
    for (int p = 0; p < MTW; ++p) *(u4*)(base + (p * 16 * WM + arow) * A_ROW + achunk * 16) = areg[p];
  };

  const u4* wbase = qw + ((size_t)slab * G * 8 + t0) * 64 + lane;
  uint2 sreg;
  f4 sreg32;
  uint32_t zreg = 0x88888888u;
  uint2 zsreg = {0u, 0u};
  // groups 1 .. GPB - 1 of the K block (group sizes below 128)
  uint2 sregx[GPB > 1 ? GPB - 1 : 1];
  uint32_t zregx[GPB > 1 ? GPB - 1 : 1];
  uint2 zsregx[GPB > 1 ? GPB - 1 : 1];
  auto load_w = [&](u4 (&w)[4], int g) {
    const u4* p = wbase + (size_t)g * 512;
#pragma unroll
    for (int t = 0; t < 4; ++t) w[t] = p[t * 64];
  };
  auto load_sz = [&](int g) {
    const int qrow = (128 * g) / a.gs;
    if (SF32) sreg32 = *(const f4*)(scales32 + (size_t)qrow * N + ncol);
    else sreg = *(const uint2*)(scales + (size_t)qrow * N + ncol);
    if (ZK == MI355Q_ZP_PACKED) zreg = ((const uint32_t*)zeros)[(size_t)qrow * (N >> 3) + (ncol >> 3)] >> (4 * t0);
    if (ZK == MI355Q_ZP_PRESCALED) zsreg = *(const uint2*)((const uint16_t*)zeros + (size_t)qrow * N + ncol);
    if constexpr (GPB > 1) {
#pragma unroll
      for (int sg = 1; sg < GPB; ++sg) {
        const size_t r = (size_t)(qrow + sg);
        sregx[sg - 1] = *(const uint2*)(scales + r * N + ncol);
        if (ZK == MI355Q_ZP_PACKED) zregx[sg - 1] = ((const uint32_t*)zeros)[r * (N >> 3) + (ncol >> 3)] >> (4 * t0);
        if (ZK == MI355Q_ZP_PRESCALED) zsregx[sg - 1] = *(const uint2*)((const uint16_t*)zeros + r * N + ncol);
      }
    }
  };

  const int gb = (int)blockIdx.z * a.kper, ge = min(G, gb + a.kper);
  // The pipelined loop needs nearly the whole register file; it is used where it fits
  // (fp16, 128-row tiles), the plain loop elsewhere (bf16 with packed zero-points spills 30-56 registers
  // into the K loop there: gate_up at M = 2048 646 us against 560 us on the plain loop).
  constexpr bool PIPE = MTW == 4 && DT == MI355Q_F16 && ZK != MI355Q_ZP_PRESCALED && !SF32 && GPB == 1;
  // (a grouped block with at most a quarter of its row tiles holding real slots takes the plain loop,
  // which skips the others: the pipelined loop has no room for branches -- guarding its matrix
  // instructions cost 17 % on full blocks -- and beats the plain loop once two of four tiles are live;
  // Mixtral-8x7B layer, 512 tokens: 587-601 us without skipping, 571-572 with this rule, 576-579
  // when every partly filled block takes the plain loop)
  bool done = false;
  if constexpr (PIPE) if (!GROUPED || __builtin_popcount(live_tiles) > MT / 4) {
    done = true;
    // Software pipeline, written out because the compiler otherwise sinks every
    // load next to its use.  Activations: global loads at the top of the K block
    // before their use, stored into the other LDS buffer near its end.  Weights:
    // two register sets that swap roles every K block; a set is re-requested as
    // soon as its last word has been dequantised.  B operands of K step s + 1 are dequantised while the matrix
    // instructions of step s run, one column tile per matrix group; A operands
    // come from LDS two matrix groups ahead.  Each K block accumulates into its
    // own partial tile, scaled into the running sum as its rows finish.  The one
    // barrier per K block sits just before the first read of the other buffer:
    // all reads of the current buffer have been issued by then (and the barrier
    // waits for them), so two buffers are enough.
    // scales stay packed as loaded (two per register) and are widened where they are used
    uint2 sc, scp;
    auto scale_of = [&](uint2 sv, int t) {
      const uint32_t sw = (t < 2) ? sv.x : sv.y;
      return IO::to_f32((uint16_t)((t & 1) ? (sw >> 16) : (sw & 0xffffu)));
    };
    h2 zz[4];
    auto prep = [&]() {
      sc = sreg;
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        if (ZK == MI355Q_ZP_PRESCALED) {
          const uint32_t zw = (t < 2) ? zsreg.x : zsreg.y;
          // the loader pre-multiplied an integer zero-point by the scale
          // (z * s rounded to the activation type): recover the integer
          const float zf = __builtin_rintf(IO::to_f32((uint16_t)((t & 1) ? (zw >> 16) : (zw & 0xffffu))) / scale_of(sc, t));
          zz[t] = (h2){(_Float16)(1024.0f + zf), (_Float16)(64.0f + zf)};
        } else {
          // fp16 bit patterns directly: 1024 + z = 0x6400 | z, 64 + z = 0x5400 | z << 4
          const uint32_t z = (zreg >> (4 * t)) & 15u;
          zz[t] = bitcast<h2>(0x54006400u | z | (z << 20));
        }
      }
    };
    const unsigned aoff = (wmh * MTW * 16 + c) * A_ROW + kq * 16;
    auto lds_a = [&](unsigned buf_off, int mt, int st) {
      return bitcast<vec>(*(const u4*)(lds + buf_off + aoff + mt * 16 * A_ROW + st * 64));
    };

    u4 w0[4], w1[4];
    load_a(gb);
    load_w(w0, gb);
    load_sz(gb);
    store_a(0);
    prep();
    vec bv[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) bv[t] = MM::dequant(w0[t][0], zz[t], dqk);
    load_w(w1, min(gb + 1, ge - 1));
    load_sz(min(gb + 1, ge - 1));
    f4 part[MTW][4];
    __syncthreads();
    constexpr int NJ = 4 * MTW;                      // matrix groups (K step x row tile) per K block
    constexpr int TPG = 4 / MTW > 0 ? 4 / MTW : 1;   // column tiles dequantised per group
    static_assert(MTW == 1 || MTW == 2 || MTW == 4, "row tiles per wavefront");
      constexpr int PF = 2;                          // LDS prefetch distance in matrix groups
    vec avr[4];
#pragma unroll
    for (int j = 0; j < PF; ++j) avr[j] = lds_a(0, j % MTW, j / MTW);
    unsigned cur = 0, nxt = A_BUF;

    auto kblock = [&](int g, u4 (&wc)[4], u4 (&wn)[4]) {
      load_a(min(g + 1, ge - 1));
      __builtin_amdgcn_sched_barrier(0);
      vec bn[4];
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const int st = j / MTW, mt = j % MTW;
        if (j == (NJ >= 8 ? NJ - 4 : 0)) store_a(nxt);   // block g + 1, requested at the top
        if (j == NJ - PF) __syncthreads();
        {
          const int jj = j + PF;
          avr[jj % 4] = jj < NJ ? lds_a(cur, jj % MTW, jj / MTW) : lds_a(nxt, (jj - NJ) % MTW, (jj - NJ) / MTW);
        }
        if (st == 3 && mt == 0) {
          // operands of the next K block from here on; its words arrived during this one
          scp = sc;
          prep();
          load_sz(min(g + 2, ge - 1));
        }
#pragma unroll
        for (int t = mt * TPG; t < (mt + 1) * TPG; ++t)
          bn[t] = MM::dequant(st < 3 ? wc[t][st + 1] : wn[t][0], zz[t], dqk);
        if (st == 2 && mt == MTW - 1) load_w(wc, min(g + 2, ge - 1));   // last word of wc just went
#pragma unroll
        for (int t = 0; t < 4; ++t)
          part[mt][t] = MM::run(avr[j % 4], bv[t], st == 0 ? (f4){0.f, 0.f, 0.f, 0.f} : part[mt][t]);
        if (st == 3 && mt > 0) {
#pragma unroll
          for (int t = 0; t < 4; ++t) acc[mt - 1][t] += scale_of(scp, t) * part[mt - 1][t];
        }
        if (mt == MTW - 1) {
#pragma unroll
          for (int t = 0; t < 4; ++t) bv[t] = bn[t];
        }
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int t = 0; t < 4; ++t) acc[MTW - 1][t] += scale_of(scp, t) * part[MTW - 1][t];
      const unsigned o = cur;
      cur = nxt;
      nxt = o;
    };
    for (int g = gb;; g += 2) {
      kblock(g, w0, w1);
      if (g + 1 >= ge) break;
      kblock(g + 1, w1, w0);
      if (g + 2 >= ge) break;
    }
  }
  if (!done) {
    // Plain loop: operands of the whole K block dequantised up front, the next block's loads
    // pinned at the top, one partial tile per row tile.  Two wavefronts per SIMD cover each
    // other's dequantisation bursts.
    u4 wreg[4];
    load_a(gb);
    load_w(wreg, gb);
    load_sz(gb);
    store_a(0);
    __syncthreads();
    for (int g = gb; g < ge; ++g) {
      const unsigned buf = ((g - gb) & 1) * A_BUF;
      u4 wcur[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) wcur[t] = wreg[t];
      float sc[GPB][4];
      h2 zz[GPB][4];
#pragma unroll
      for (int sg = 0; sg < GPB; ++sg) {
        const uint2 sv = sg == 0 ? sreg : sregx[sg > 0 ? sg - 1 : 0], zsv = sg == 0 ? zsreg : zsregx[sg > 0 ? sg - 1 : 0];
        const uint32_t zv = sg == 0 ? zreg : zregx[sg > 0 ? sg - 1 : 0];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const uint32_t sw = (t < 2) ? sv.x : sv.y;
          sc[sg][t] = SF32 ? sreg32[t] : IO::to_f32((uint16_t)((t & 1) ? (sw >> 16) : (sw & 0xffffu)));
          float zf;
          if (ZK == MI355Q_ZP_PRESCALED) {
            const uint32_t zw = (t < 2) ? zsv.x : zsv.y;
            // the loader pre-multiplied an integer zero-point by the scale
            // (z * s rounded to the activation type): recover the integer
            zf = __builtin_rintf(IO::to_f32((uint16_t)((t & 1) ? (zw >> 16) : (zw & 0xffffu))) / sc[sg][t]);
          } else {
            zf = (float)((zv >> (4 * t)) & 15u);
          }
          zz[sg][t] = (h2){(_Float16)(1024.0f + zf), (_Float16)(64.0f + zf)};
        }
      }
      const int gn = min(g + 1, ge - 1);
      load_a(gn);
      load_w(wreg, gn);
      load_sz(gn);
      __builtin_amdgcn_sched_barrier(0);     // keep the prefetch at the top: a full K block to land

      // all 16 B operands of this K block (4 steps x 4 column tiles)
      vec bv[4][4];
#pragma unroll
      for (int s = 0; s < 4; ++s)
#pragma unroll
        for (int t = 0; t < 4; ++t) bv[s][t] = MM::dequant(wcur[t][s], zz[s * GPB / 4][t], dqk);

      const unsigned char* abase = lds + buf + (wmh * MTW * 16 + c) * A_ROW + kq * 16;
#pragma unroll
      for (int mt = 0; mt < MTW; ++mt) {
        if (!tile_live(mt)) continue;
#pragma unroll
        for (int sg = 0; sg < GPB; ++sg) {
          f4 part[4];
#pragma unroll
          for (int t = 0; t < 4; ++t) part[t] = (f4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int s = sg * (4 / GPB); s < (sg + 1) * (4 / GPB); ++s) {
            const vec av = bitcast<vec>(*(const u4*)(abase + mt * 16 * A_ROW + s * 64));
#pragma unroll
            for (int t = 0; t < 4; ++t) part[t] = MM::run(av, bv[s][t], part[t]);
          }
#pragma unroll
          for (int t = 0; t < 4; ++t) acc[mt][t] += sc[sg][t] * part[t];
        }
      }
      // the other buffer was last read one iteration ago: every wavefront has
      // passed the barrier below since, so it can be overwritten now
      store_a(A_BUF - buf);
      __syncthreads();
    }
  }

  // ---- epilogue: 4 adjacent columns per (row tile, i) ----
  if (!live) return;
  const float oscale = a.out_scale ? *a.out_scale : 1.0f;
  float bs[4] = {0.f, 0.f, 0.f, 0.f};
  if (a.bias) {
#pragma unroll
    for (int t = 0; t < 4; ++t) bs[t] = IO::to_f32(a.bias[ncol + t]);
  }
#pragma unroll
  for (int mt = 0; mt < MTW; ++mt)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      int m;
      float rw = oscale;
      bool ok;
      if (GROUPED) {
        m = tok[(wmh * MTW + mt) * 16 + 4 * kq + i];
        ok = m < a.numel;
        if (ok && a.topk_weights) rw *= a.topk_weights[m];
        if (IOBF && ok && !a.partial) rw *= a.row_scale[a.topk == 1 ? m : m / a.topk];
      } else {
        m = m0 + (wmh * MTW + mt) * 16 + 4 * kq + i;
        ok = m < M;
        if (IOBF && ok && !a.partial) rw *= a.row_scale[m];
      }
      if (a.partial) {
        if (ok) {
          float* pp = a.partial + ((size_t)blockIdx.z * M + m) * N + ncol;
          *(f4*)pp = (f4){acc[mt][0][i], acc[mt][1][i], acc[mt][2][i], acc[mt][3][i]};
        }
      } else if (ok) {
        uint2 o;
        o.x = (uint32_t)IO::from_f32(acc[mt][0][i] * rw + bs[0]) |
              ((uint32_t)IO::from_f32(acc[mt][1][i] * rw + bs[1]) << 16);
        o.y = (uint32_t)IO::from_f32(acc[mt][2][i] * rw + bs[2]) |
              ((uint32_t)IO::from_f32(acc[mt][3][i] * rw + bs[3]) << 16);
        *(uint2*)(a.out + (size_t)m * N + ncol) = o;
      }
    }
}

// out[m, n] = sum over splits of partial[s][m][n] (+ bias[n]), added in split order
// times row_weight[m] when given (the routing weights of a grouped launch)
template <int DT>
__global__ void __launch_bounds__(256)
w4a16_splitk_reduce_kernel(uint16_t* out, const float* partial, const uint16_t* bias, const float* row_weight,
                           long MN, int N, int splits) {
  const long i = ((long)blockIdx.x * 256 + threadIdx.x) * 4;
  if (i >= MN) return;
  f4 v = *(const f4*)(partial + i);
  // four splits requested together, added in split order (a loop of load-then-add would wait for a
  // trip to memory per split)
  int s = 1;
  for (; s + 3 < splits; s += 4) {
    const f4 p0 = *(const f4*)(partial + (size_t)s * MN + i), p1 = *(const f4*)(partial + (size_t)(s + 1) * MN + i);
    const f4 p2 = *(const f4*)(partial + (size_t)(s + 2) * MN + i), p3 = *(const f4*)(partial + (size_t)(s + 3) * MN + i);
    v += p0;
    v += p1;
    v += p2;
    v += p3;
  }
  for (; s < splits; ++s) v += *(const f4*)(partial + (size_t)s * MN + i);
  if (row_weight) v *= row_weight[i / N];
  if (bias) {
    const int n = (int)(i % N);
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] += Elem<DT>::to_f32(bias[n + e]);
  }
  uint2 o;
  o.x = (uint32_t)Elem<DT>::from_f32(v[0]) | ((uint32_t)Elem<DT>::from_f32(v[1]) << 16);
  o.y = (uint32_t)Elem<DT>::from_f32(v[2]) | ((uint32_t)Elem<DT>::from_f32(v[3]) << 16);
  *(uint2*)(out + i) = o;
}

// The same for a grouped launch: the rows are visited through the aligned id list, so a slot id that the
// alignment dropped (an expert outside [0, E), a row past the valid count) -- whose partial rows no
// split wrote -- is left alone, exactly as the unsplit launch leaves it.
template <int DT>
__global__ void __launch_bounds__(256)
w4a16_grouped_reduce_kernel(uint16_t* out, const float* partial, const float* row_weight,
                            const int32_t* sorted_ids, const int32_t* npp, int numel, int N, int splits,
                            const float* row_scale, int topk) {
  const int n4 = N >> 2;
  const long t = (long)blockIdx.x * 256 + threadIdx.x;
  const long p = t / n4;
  if (p >= *npp) return;
  const int id = sorted_ids[p];
  if (id >= numel || id < 0) return;
  const long MN = (long)numel * N;
  const long i = (long)id * N + (t - p * n4) * 4;
  f4 v = *(const f4*)(partial + i);
  int s = 1;
  for (; s + 3 < splits; s += 4) {
    const f4 p0 = *(const f4*)(partial + (size_t)s * MN + i), p1 = *(const f4*)(partial + (size_t)(s + 1) * MN + i);
    const f4 p2 = *(const f4*)(partial + (size_t)(s + 2) * MN + i), p3 = *(const f4*)(partial + (size_t)(s + 3) * MN + i);
    v += p0;
    v += p1;
    v += p2;
    v += p3;
  }
  for (; s < splits; ++s) v += *(const f4*)(partial + (size_t)s * MN + i);
  if (row_weight) v *= row_weight[id];
  if (row_scale) v *= row_scale[id / topk];          // bf16 rows staged as fp16: the gathered row's power of two
  uint2 o;
  o.x = (uint32_t)Elem<DT>::from_f32(v[0]) | ((uint32_t)Elem<DT>::from_f32(v[1]) << 16);
  o.y = (uint32_t)Elem<DT>::from_f32(v[2]) | ((uint32_t)Elem<DT>::from_f32(v[3]) << 16);
  *(uint2*)(out + i) = o;
}

template <int DT, int ZK, int MT, bool GROUPED, int WM, bool SF32>
hipError_t launch_wm(const TileArgs& a, int row_blocks, hipStream_t st) {
  constexpr int BM = 16 * MT;
  const int G = a.K >> 7;
  dim3 grid((a.N + BN - 1) / BN, row_blocks, (G + a.kper - 1) / a.kper), block(256 * WM);
  const size_t shmem = 2 * BM * A_ROW;             // up to 72 KiB: above the 64 KiB default
  static hipError_t attr = hipFuncSetAttribute((const void*)w4a16_tile_kernel<DT, ZK, MT, GROUPED, WM, SF32>,
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
  if (attr != hipSuccess) return attr;
  hipLaunchKernelGGL((w4a16_tile_kernel<DT, ZK, MT, GROUPED, WM, SF32>), grid, block, shmem, st, a);
  return hipSuccess;
}

// group sizes of 64 and 32 (two and four groups per K block): dense 64-row tiles, MoE blocks of 64 and 128 slots
template <int DT, int ZK, int MT, bool GROUPED, int GPB>
hipError_t launch_small_groups_one(const TileArgs& a, int row_blocks, hipStream_t st) {
  constexpr int WM = MT >= 8 ? 2 : 1;
  const int G = a.K >> 7;
  dim3 grid((a.N + BN - 1) / BN, row_blocks, (G + a.kper - 1) / a.kper), block(256 * WM);
  const size_t shmem = 2 * 16 * MT * A_ROW;
  static hipError_t attr = hipFuncSetAttribute((const void*)w4a16_tile_kernel<DT, ZK, MT, GROUPED, WM, false, GPB>,
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
  if (attr != hipSuccess) return attr;
  hipLaunchKernelGGL((w4a16_tile_kernel<DT, ZK, MT, GROUPED, WM, false, GPB>), grid, block, shmem, st, a);
  return hipSuccess;
}
template <int DT, int MT, bool GROUPED>
hipError_t launch_small_groups(const TileArgs& a, int zk, int gpb, int row_blocks, hipStream_t st) {
  if (gpb == 2) {
    if (zk == MI355Q_ZP_NONE) return launch_small_groups_one<DT, MI355Q_ZP_NONE, MT, GROUPED, 2>(a, row_blocks, st);
    if (zk == MI355Q_ZP_PACKED) return launch_small_groups_one<DT, MI355Q_ZP_PACKED, MT, GROUPED, 2>(a, row_blocks, st);
    return launch_small_groups_one<DT, MI355Q_ZP_PRESCALED, MT, GROUPED, 2>(a, row_blocks, st);
  }
  if (zk == MI355Q_ZP_NONE) return launch_small_groups_one<DT, MI355Q_ZP_NONE, MT, GROUPED, 4>(a, row_blocks, st);
  if (zk == MI355Q_ZP_PACKED) return launch_small_groups_one<DT, MI355Q_ZP_PACKED, MT, GROUPED, 4>(a, row_blocks, st);
  return launch_small_groups_one<DT, MI355Q_ZP_PRESCALED, MT, GROUPED, 4>(a, row_blocks, st);
}

template <int DT, int ZK, int MT, bool GROUPED, bool SF32 = false>
hipError_t launch_one(const TileArgs& a, int row_blocks, hipStream_t st) {
  // up to 64 rows: four wavefronts, each all rows of its 64 columns, two workgroups per CU;
  // 128-row tiles (MoE blocks of 128 only): eight wavefronts, 2 (M) x 4 (N)
  constexpr int WM = MT >= 8 ? 2 : 1;
  return launch_wm<DT, ZK, MT, GROUPED, WM, SF32>(a, row_blocks, st);
}

// ---- narrow column tiles for mid-sized M ---------------------------------------------------------
// Between the decode kernel's 32 rows and a few hundred rows the weights are read about once (a
// streaming problem) while a 256-column tile leaves a narrow layer with a handful of workgroups, which
// K then has to be split many ways to occupy the chip: at M = 128 on a 4096-column layer eight splits
// wrote and re-read 17 MB of fp32 partial tiles, more time than the GEMM itself.  Here a wavefront
// owns NTW = 1 or 2 of the 16-column tiles (64 or 128 columns per workgroup), so the columns supply
// the workgroups and K is split little or not at all; the 16 MT activation rows are still shared by the
// four wavefronts through LDS.  Plain loop (the compiler schedules it), several workgroups per CU.
template <int DT, int ZK, int MT, int NTW, int D>
__global__ void __launch_bounds__(256, 2)
w4a16_tile_narrow_kernel(TileArgs a) {
  typedef TileMma<DT> MM;
  typedef typename MM::vec vec;
  constexpr int BM = 16 * MT, A_BUF = BM * A_ROW;
  extern __shared__ __align__(16) unsigned char lds[];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int c = lane & 15, kq = lane >> 4;
  const int N = a.N, K = a.K, M = a.M;
  const int G = K >> 7;
  const int m0 = blockIdx.y * BM;
  // tile index inside the matrix: 8 tiles per 128-column slab; tile t of a slab holds its columns 8 c + t
  const int tile = ((int)blockIdx.x * 4 + wave) * NTW;
  const bool live = tile < (N >> 4);
  const int slab = live ? tile >> 3 : 0;
  const int t0 = live ? tile & 7 : 0;
  const int ncol = 128 * slab + 8 * c + t0;          // first of this lane's NTW adjacent columns

  f4 acc[MT][NTW];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int t = 0; t < NTW; ++t) acc[mt][t] = (f4){0.f, 0.f, 0.f, 0.f};
  const DqConst dqk = dq_consts();

  const int arow = tid >> 4, achunk = tid & 15;
  // Buffer loads: lane offset in a register, block offset in a scalar, so a load costs no vector
  // arithmetic, and a block index past the matrix reads zeros instead of faulting (the ring runs D
  // blocks ahead of the last one).
  typedef __amdgpu_buffer_rsrc_t rsrc_t;
  auto make_rsrc = [](const void* p, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)bytes, 0x00020000);
  };
  const int rows_q = K / a.gs;
  const rsrc_t xres = make_rsrc(a.x, (uint32_t)M * (uint32_t)K * 2u);
  const rsrc_t wres = make_rsrc(a.qw + (size_t)slab * G * 512, (uint32_t)G * 8192u);
  const rsrc_t sres = make_rsrc(a.scales, (uint32_t)rows_q * (uint32_t)N * 2u);
  const rsrc_t zres = make_rsrc(a.zeros, ZK == MI355Q_ZP_PACKED ? (uint32_t)rows_q * (uint32_t)(N >> 3) * 4u
                                                                 : (uint32_t)rows_q * (uint32_t)N * 2u);
  uint32_t aofs[MT];
#pragma unroll
  for (int p = 0; p < MT; ++p)
    aofs[p] = ((uint32_t)min(m0 + p * 16 + arow, M - 1) * (uint32_t)K + 8u * achunk) * 2u;
  const uint32_t wofs = (uint32_t)(t0 * 64 + lane) * 16u;
  // A K block is short here (a few hundred cycles), far shorter than a trip to memory: the loads of
  // D blocks are in flight at any time, each block's in its own slot of a register ring (the loop
  // is unrolled D times, so the slots are fixed registers).
  u4 ar[D][MT], wr[D][NTW];
  // scales (and float zero-points) of the aligned group of four tiles this wavefront's tiles lie in:
  // whole 8-byte loads (a 16-bit load only writes half a register, which ties it to the register's
  // previous load and serialises the ring)
  uint2 sr[D], zsr[D];
  uint32_t zr[D];
  const int tsel = 16 * (t0 & 3), ncol4 = ncol - (t0 & 3);
  auto pick = [&](uint2 v, int t) {
    const unsigned long long q = ((unsigned long long)v.y << 32) | v.x;
    return (uint16_t)(q >> (tsel + 16 * t));
  };
  const int gb = (int)blockIdx.z * a.kper, ge = min(G, gb + a.kper);
  auto issue = [&](int d, int g) {
#pragma unroll
    for (int p = 0; p < MT; ++p)
      ar[d][p] = bitcast<u4>(__builtin_amdgcn_raw_buffer_load_b128(xres, (int)aofs[p], g * 256, 0));
#pragma unroll
    for (int t = 0; t < NTW; ++t)
      wr[d][t] = bitcast<u4>(__builtin_amdgcn_raw_buffer_load_b128(wres, (int)wofs, g * 8192 + t * 1024, 0));
    const int qrow = a.gpk_magic ? (int)__umulhi((uint32_t)g, a.gpk_magic) : g;
    sr[d] = bitcast<uint2>(__builtin_amdgcn_raw_buffer_load_b64(sres, ncol4 * 2, qrow * N * 2, 0));
    if (ZK == MI355Q_ZP_PACKED)
      zr[d] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(zres, (ncol >> 3) * 4, qrow * (N >> 3) * 4, 0);
    if (ZK == MI355Q_ZP_PRESCALED)
      zsr[d] = bitcast<uint2>(__builtin_amdgcn_raw_buffer_load_b64(zres, ncol4 * 2, qrow * N * 2, 0));
  };
  auto store_a = [&](int d, unsigned buf_off) {
#pragma unroll
    for (int p = 0; p < MT; ++p) *(u4*)(lds + buf_off + (p * 16 + arow) * A_ROW + achunk * 16) = ar[d][p];
  };
#pragma unroll
  for (int d = 0; d < D; ++d) issue(d, gb + d);
  store_a(0, 0);
  __syncthreads();
  auto kblock = [&](int d, int g) {
    const unsigned buf = ((g - gb) & 1) * A_BUF;
    u4 wcur[NTW];
    float sc[NTW];
    h2 zz[NTW];
#pragma unroll
    for (int t = 0; t < NTW; ++t) {
      wcur[t] = wr[d][t];
      sc[t] = Elem<DT>::to_f32(pick(sr[d], t));
      float zf;
      if (ZK == MI355Q_ZP_PRESCALED) zf = __builtin_rintf(Elem<DT>::to_f32(pick(zsr[d], t)) / sc[t]);   // z * s -> z
      else if (ZK == MI355Q_ZP_PACKED) zf = (float)((zr[d] >> (4 * (t0 + t))) & 15u);
      else zf = 8.0f;
      zz[t] = (h2){(_Float16)(1024.0f + zf), (_Float16)(64.0f + zf)};
    }
    vec bv[4][NTW];
#pragma unroll
    for (int st = 0; st < 4; ++st)
#pragma unroll
      for (int t = 0; t < NTW; ++t) bv[st][t] = MM::dequant(wcur[t][st], zz[t], dqk);
    // the activations of block g went to LDS during block g - 1: the slot is free again
    issue(d, g + D);
    const unsigned char* abase = lds + buf + c * A_ROW + kq * 16;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      f4 part[NTW];
#pragma unroll
      for (int t = 0; t < NTW; ++t) part[t] = (f4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int st = 0; st < 4; ++st) {
        const vec av = bitcast<vec>(*(const u4*)(abase + mt * 16 * A_ROW + st * 64));
#pragma unroll
        for (int t = 0; t < NTW; ++t) part[t] = MM::run(av, bv[st][t], part[t]);
      }
#pragma unroll
      for (int t = 0; t < NTW; ++t) acc[mt][t] += sc[t] * part[t];
    }
    // block g + 1 into the other buffer (last read during block g - 1: every wavefront has passed
    // the barrier since)
    store_a((d + 1) % D, A_BUF - buf);
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);               // blocks stay apart: merged, their operands overflow the registers
  };
  // whole rounds of the ring without a branch inside (a branch between the blocks makes the
  // compiler wait for every load in flight at each of them), then the remaining blocks one by one
  int g0 = gb;
  for (; g0 + D <= ge; g0 += D) {
#pragma unroll
    for (int d = 0; d < D; ++d) kblock(d, g0 + d);
  }
#pragma unroll
  for (int d = 0; d < D - 1; ++d) {
    if (g0 + d < ge) kblock(d, g0 + d);
  }

  if (!live) return;
  float bs[NTW];
#pragma unroll
  for (int t = 0; t < NTW; ++t) bs[t] = a.bias ? Elem<DT>::to_f32(a.bias[ncol + t]) : 0.f;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = m0 + mt * 16 + 4 * kq + i;
      if (m >= M) continue;
      if (a.partial) {
        float* pp = a.partial + ((size_t)blockIdx.z * M + m) * N + ncol;
#pragma unroll
        for (int t = 0; t < NTW; ++t) pp[t] = acc[mt][t][i];
      } else {
        uint16_t* po = a.out + (size_t)m * N + ncol;
        if (NTW == 2) {
          *(uint32_t*)po = (uint32_t)Elem<DT>::from_f32(acc[mt][0][i] + bs[0]) |
                           ((uint32_t)Elem<DT>::from_f32(acc[mt][NTW - 1][i] + bs[NTW - 1]) << 16);
        } else {
#pragma unroll
          for (int t = 0; t < NTW; ++t) po[t] = Elem<DT>::from_f32(acc[mt][t][i] + bs[t]);
        }
      }
    }
}

// The one configuration that is launched: 32-row blocks, one tile per wavefront, two K blocks in
// flight.  Measured on the Llama-3-8B layers for 33..128 rows: rings of 4 and 8 blocks were no
// faster (the deeper rings spill: every slot is live across the whole unrolled loop), nor were
// 64-row blocks or two tiles per wavefront.
template <int DT, int ZK>
hipError_t launch_narrow_zk(const TileArgs& a, int row_blocks, hipStream_t st) {
  constexpr int MT = 2, NTW = 1, D = 2;
  const int G = a.K >> 7;
  dim3 grid((a.N / 16 + 4 * NTW - 1) / (4 * NTW), row_blocks, (G + a.kper - 1) / a.kper), block(256);
  const size_t shmem = 2 * 16 * MT * A_ROW;
  hipLaunchKernelGGL((w4a16_tile_narrow_kernel<DT, ZK, MT, NTW, D>), grid, block, shmem, st, a);
  return hipSuccess;
}
template <int DT>
hipError_t launch_narrow(const TileArgs& a, int zk, int row_blocks, hipStream_t st) {
  if (zk == MI355Q_ZP_NONE) return launch_narrow_zk<DT, MI355Q_ZP_NONE>(a, row_blocks, st);
  if (zk == MI355Q_ZP_PACKED) return launch_narrow_zk<DT, MI355Q_ZP_PACKED>(a, row_blocks, st);
  return launch_narrow_zk<DT, MI355Q_ZP_PRESCALED>(a, row_blocks, st);
}

template <int DT, int MT, bool GROUPED>
hipError_t launch_zk(const TileArgs& a, int zk, int row_blocks, hipStream_t st) {
  if constexpr (GROUPED) {
    // fp32 group scales: symmetric int4 experts only
    if (a.scales_f32) return launch_one<DT, MI355Q_ZP_NONE, MT, true, true>(a, row_blocks, st);
  }
  if (zk == MI355Q_ZP_NONE) return launch_one<DT, MI355Q_ZP_NONE, MT, GROUPED>(a, row_blocks, st);
  if (zk == MI355Q_ZP_PACKED) return launch_one<DT, MI355Q_ZP_PACKED, MT, GROUPED>(a, row_blocks, st);
  return launch_one<DT, MI355Q_ZP_PRESCALED, MT, GROUPED>(a, row_blocks, st);
}

template <int DT, bool GROUPED>
hipError_t launch_mt(const TileArgs& a, int zk, int mt, int row_blocks, hipStream_t st) {
  switch (mt) {
    case 1: return launch_zk<DT, 1, GROUPED>(a, zk, row_blocks, st);
    case 2: return launch_zk<DT, 2, GROUPED>(a, zk, row_blocks, st);
    case 4: return launch_zk<DT, 4, GROUPED>(a, zk, row_blocks, st);
    default: return launch_zk<DT, 8, GROUPED>(a, zk, row_blocks, st);
  }
}

// bf16 activations staged as fp16 rows: 64-row tiles on the pipelined fp16 loop, bf16 in and out
template <bool GROUPED>
hipError_t launch_iobf(const TileArgs& a, int zk, int row_blocks, hipStream_t st) {
  const int G = a.K >> 7;
  dim3 grid((a.N + BN - 1) / BN, row_blocks, (G + a.kper - 1) / a.kper), block(256);
  const size_t shmem = 2 * 64 * A_ROW;
  if (zk == MI355Q_ZP_NONE) {
    static hipError_t attr = hipFuncSetAttribute(
        (const void*)w4a16_tile_kernel<MI355Q_F16, MI355Q_ZP_NONE, 4, GROUPED, 1, false, 1, true>,
        hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
    if (attr != hipSuccess) return attr;
    hipLaunchKernelGGL((w4a16_tile_kernel<MI355Q_F16, MI355Q_ZP_NONE, 4, GROUPED, 1, false, 1, true>), grid, block, shmem, st, a);
  } else {
    static hipError_t attr = hipFuncSetAttribute(
        (const void*)w4a16_tile_kernel<MI355Q_F16, MI355Q_ZP_PACKED, 4, GROUPED, 1, false, 1, true>,
        hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
    if (attr != hipSuccess) return attr;
    hipLaunchKernelGGL((w4a16_tile_kernel<MI355Q_F16, MI355Q_ZP_PACKED, 4, GROUPED, 1, false, 1, true>), grid, block, shmem, st, a);
  }
  return hipSuccess;
}

// One workgroup per row of bf16 activations: the row's largest magnitude fixes a power of two 2^e that
// brings it into [2^14, 2^15); the row times 2^-e is stored as fp16 and 2^e as the row's output
// multiplier.  Exact for every element within 2^28 of the row's largest (eight mantissa bits fit in
// eleven, the scaling is a power of two); smaller ones lose at most 2^-40 of that largest magnitude in
// fp16's subnormal range.  A row that holds an infinity or a NaN is stored unscaled (they stay what
// they are; its finite elements beyond the fp16 range become infinities).
// HELD: the row stays in registers between the two passes (K up to 16384); else it is read twice.
// Workgroups past the rows (64 of them, when scale_max is given) each scan a 64th of the bf16 group
// scales for the largest magnitude, which the ring kernels turn into one power of two for all scales.
template <bool HELD>
__global__ void __launch_bounds__(256)
bf16_rows_to_f16_kernel(const uint16_t* __restrict__ x, uint16_t* __restrict__ x16, float* __restrict__ row_scale, int K,
                        int rows, const u4* __restrict__ scales, long scale_chunks, uint32_t* __restrict__ scale_max) {
  __shared__ uint32_t wmax[4];
  const int tid = threadIdx.x;
  if ((int)blockIdx.x >= rows) {
    const long per = (scale_chunks + 63) / 64, b = (long)blockIdx.x - rows;
    const long end = (b + 1) * per < scale_chunks ? (b + 1) * per : scale_chunks;
    uint32_t mx = 0;
    for (long i = b * per + tid; i < end; i += 256) {
      const u4 v = scales[i];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t lo = v[j] & 0x7fffu, hi = (v[j] >> 16) & 0x7fffu;
        mx = mx > lo ? mx : lo;
        mx = mx > hi ? mx : hi;
      }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const uint32_t other = (uint32_t)__shfl_xor((int)mx, o, 64);
      mx = mx > other ? mx : other;
    }
    if ((tid & 63) == 0) wmax[tid >> 6] = mx;
    __syncthreads();
    if (tid == 0) {
      mx = wmax[0];
      for (int w = 1; w < 4; ++w) mx = mx > wmax[w] ? mx : wmax[w];
      scale_max[b] = mx;
    }
    return;
  }
  const u4* row = (const u4*)(x + (size_t)blockIdx.x * K);
  u4* orow = (u4*)(x16 + (size_t)blockIdx.x * K);
  const int chunks = K >> 3;                        // 16-byte pieces of eight elements
  uint32_t mx = 0;
  u4 held[HELD ? 8 : 1];
  if (HELD) {
#pragma unroll
    for (int r = 0; r < 8; ++r) held[r] = tid + 256 * r < chunks ? row[tid + 256 * r] : (u4){0u, 0u, 0u, 0u};
#pragma unroll
    for (int r = 0; r < 8; ++r)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t lo = held[r][j] & 0x7fffu, hi = (held[r][j] >> 16) & 0x7fffu;
        mx = mx > lo ? mx : lo;
        mx = mx > hi ? mx : hi;
      }
  } else {
    for (int i = tid; i < chunks; i += 256) {
      const u4 v = row[i];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t lo = v[j] & 0x7fffu, hi = (v[j] >> 16) & 0x7fffu;
        mx = mx > lo ? mx : lo;
        mx = mx > hi ? mx : hi;
      }
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const uint32_t other = (uint32_t)__shfl_xor((int)mx, o, 64);
    mx = mx > other ? mx : other;
  }
  if ((tid & 63) == 0) wmax[tid >> 6] = mx;
  __syncthreads();
  mx = wmax[0];
#pragma unroll
  for (int w = 1; w < 4; ++w) mx = mx > wmax[w] ? mx : wmax[w];
  const int expo = (int)(mx >> 7);                  // biased exponent of the largest magnitude
  int e = 0;
  if (mx != 0 && expo != 255) {
    e = (expo > 0 ? expo : 1) - 127 - 14;
    if (e < -126) e = -126;
  }
  const float down = bitcast<float>((uint32_t)(127 - e) << 23);
  if (tid == 0) row_scale[blockIdx.x] = bitcast<float>((uint32_t)(127 + e) << 23);
  auto convert = [&](u4 v) {
    u4 o;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const _Float16 lo = (_Float16)(bitcast<float>(v[j] << 16) * down);
      const _Float16 hi = (_Float16)(bitcast<float>(v[j] & 0xffff0000u) * down);
      o[j] = (uint32_t)bitcast<uint16_t>(lo) | ((uint32_t)bitcast<uint16_t>(hi) << 16);
    }
    return o;
  };
  if (HELD) {
#pragma unroll
    for (int r = 0; r < 8; ++r)
      if (tid + 256 * r < chunks) orow[tid + 256 * r] = convert(held[r]);
  } else {
    for (int i = tid; i < chunks; i += 256) orow[i] = convert(row[i]);     // (second read of the row: from the cache)
  }
}

}  // namespace

// sum of the fp32 partial tiles of a dense split-K launch into the output (+ bias), in split order;
// row_weight (optional): a multiplier per output row, applied to the sum before the bias
static int splitk_reduce_rows_launch(void* out, const float* partial, const void* bias, int M, int N, int splits,
                                     int dtype, hipStream_t st, const float* row_weight) {
  const long MN = (long)M * N;
  const unsigned blocks = (unsigned)((MN / 4 + 255) / 256);
  if (dtype == MI355Q_F16)
    hipLaunchKernelGGL((w4a16_splitk_reduce_kernel<MI355Q_F16>), dim3(blocks), dim3(256), 0, st, (uint16_t*)out, partial,
                       (const uint16_t*)bias, row_weight, MN, N, splits);
  else
    hipLaunchKernelGGL((w4a16_splitk_reduce_kernel<MI355Q_BF16>), dim3(blocks), dim3(256), 0, st, (uint16_t*)out, partial,
                       (const uint16_t*)bias, row_weight, MN, N, splits);
  MQ_LAUNCH_CHECK("w4a16_gemm(split-K reduce)");
  return 0;
}
int w4a16_splitk_reduce_launch(void* out, const float* partial, const void* bias, int M, int N, int splits,
                               int dtype, hipStream_t st) {
  return splitk_reduce_rows_launch(out, partial, bias, M, N, splits, dtype, st, nullptr);
}

// split-K plan for grids that leave most of the chip idle: as many splits as
// bring the grid to about one workgroup per CU, at least 4 K blocks each, and
// partial tiles of at most TILE_SPLITK_BYTES in total
constexpr size_t TILE_SPLITK_BYTES = (size_t)64 << 20;
static int tile_rows_mt(int M, int N) {
  // 64-row tiles for every dense shape: four wavefronts on the pipelined loop, two workgroups
  // per CU -- measured equal or faster than 128-row tiles of eight wavefronts from M = 65 to
  // 8192 (M = 2048: qkv 134 -> 112 us, gate_up 461 -> 449 us), fp16 and bf16
  (void)M;
  (void)N;
  return 4;
}
static int tile_splits(int M, int K, int N) {
  const int mt = tile_rows_mt(M, N), G = K / 128;
  const long wgs = (long)((M + 16 * mt - 1) / (16 * mt)) * ((N + BN - 1) / BN);
  // 64-row tiles run two workgroups per CU
  const long target = (long)device_cu_count() * (mt == 4 ? 2 : 1);
  long s;
  if (wgs * 5 >= target * 2) {
    // 40 % of a round or more (a wide layer at about a hundred rows: N 28672, M 128: 47 -> 43 us
    // without the two-way split).  A workgroup alone on its CU runs a K block in about 60 %
    // of the time of two that share one, so between 1/2 and 0.7 of a round over a long K three
    // splits (two even rounds of a third of K) beat one uneven round: K 14336, N 4096,
    // M 1100..1280: 203 -> 167..175 us; above that, and for K 4096, no split count gained.
    if (mt != 4 || wgs * 10 > target * 7 || G < 64) return 1;
    s = 3;
  } else {
    // 128-row tiles: the nearest count; 64-row tiles must all be resident at once (a second
    // round of a few workgroups would double the time), so never above the target
    s = mt == 4 ? target / wgs : (target + wgs / 2) / wgs;
  }
  if (s > G / 4) s = G / 4;
  while (s > 1 && (size_t)s * M * N * sizeof(float) > TILE_SPLITK_BYTES) --s;
  return s < 1 ? 1 : (int)s;
}
// 33..128 rows on a layer of moderate K whose 256-column tiles would need K split many ways: the
// narrow kernel (32 rows x 64 columns per workgroup) with as few splits as bring the grid to about
// two workgroups per CU, four at most.  Returns the split count, 0 = use the wide tiles.
// (Llama-3-8B o / qkv, M = 64: 16.7 / 19.6 -> 13.9 / 16.7 us; M = 128: 22.1 / 23.4 -> 17.8 / 20.8 us;
// K = 14336 and N = 28672 measured equal or slower and stay on the wide tiles.)
static int tile_narrow_splits(int M, int K, int N) {
  if (M <= 32 || M > 128 || K > 8192 || N > 8192) return 0;
  const long wgs = (long)((M + 31) / 32) * (N / 64), target = 2L * device_cu_count();
  if (wgs >= target) return 1;
  long s = target / wgs;
  if (s > 4) s = 4;
  if (s > K / 128 / 4) s = K / 128 / 4;
  return s < 1 ? 1 : (int)s;
}
int w4a16_mid_splits(int M, int K, int N, int tw);
int w4a16_mid_launch(void* out, const void* x, const int32_t* qweight, const void* scales, const void* zeros,
                     int zeros_kind, const void* bias, int M, int K, int N, int group_size, int dtype,
                     void* workspace, size_t workspace_bytes, int splits, int tw, hipStream_t st);
int w4a16_mid_launch_staged(void* out, const void* x16, const int32_t* qweight, const void* scales, const void* zeros,
                            int zeros_kind, const void* bias, int M, int K, int N, int group_size,
                            const float* row_scale, const uint32_t* scale_max, int tw, hipStream_t st);

// Above 128 rows three kernels can take a dense fp16 layer: the 64-row tiles of this file, two workgroups
// per CU, or the 128-row workgroups with the LDS ring (w4a16_mid.hip), one per CU, 256 or 512 columns
// wide.  A full round of the 512-column workgroups covers twice the columns in about 1.7 times the time
// of the other two, so it wins wherever the rounds come out even, and loses where its coarser grid
// leaves a nearly empty last round or where K would have to be split to fill the chip.  All three are
// priced in microseconds per K block from what was measured, with weights cold in the caches, on 120
// (shape, M) points of ten Llama- and Qwen-shaped layers, M = 129..8192: full rounds 2.15 for a pair
// of 64-row tiles sharing a CU (1.0 for a last round that leaves each workgroup alone on its CU), 2.05
// and 3.55 for the ring workgroups, whose last round costs 1.25 respectively 1.8 when nearly empty and
// grows linearly with the share of the CUs it occupies; plus a reduction launch when K is split.
// Taking the cheapest by these prices is within 0.6 % of the best of the three on average over those
// points (11 % at worst) and 4.5 % faster than the 64-row tiles alone (always the best: 5.1 %).
static double tile_time_model(int M, int K, int N) {
  const long cus = device_cu_count(), G = K / 128;
  const int s = tile_splits(M, K, N);
  const long wgs = (long)((M + 63) / 64) * ((N + BN - 1) / BN) * s, kper = (G + s - 1) / s;
  const long full = wgs / (2 * cus), rest = wgs - full * 2 * cus;
  return (double)kper * (full * 2.15 + (rest == 0 ? 0.0 : rest <= cus ? 1.0 : 2.15)) + (s > 1 ? 6.0 : 0.0) + 5.0;
}
static double mid_time_model(int M, int K, int N, int tw) {
  const long cus = device_cu_count(), G = K / 128;
  const int s = w4a16_mid_splits(M, K, N, tw);
  const long wgs = (long)((M + 127) / 128) * ((N + 128 * tw - 1) / (128 * tw)) * s, kper = (G + s - 1) / s;
  const long full = wgs / cus, rest = wgs - full * cus;
  const double cf = tw == 4 ? 3.55 : 2.05, ca = tw == 4 ? 1.8 : 1.25;
  return (double)kper * (full * cf + (rest == 0 ? 0.0 : ca + (cf - ca) * (double)rest / (double)cus)) +
         (s > 1 ? 6.0 : 0.0) + 6.0;
}
// 0: the 64-row tiles; 2 / 4: the ring kernel with that many column tiles per wavefront
static int tile_ring_plan(int M, int K, int N) {
  if (M <= 128) return 0;
  double best = tile_time_model(M, K, N);
  int plan = 0;
  const double t2 = mid_time_model(M, K, N, 2);
  if (t2 < best) { best = t2; plan = 2; }
  if (w4a16_mid_splits(M, K, N, 4) == 1 && mid_time_model(M, K, N, 4) < best) plan = 4;
  return plan;
}
// 33..128 rows: the ring kernel with one 16-column tile per wavefront (workgroups of 128 columns), K
// split so that the grid stays within one workgroup per CU.  Returns the split count, 0 = not taken.
// It pays where a workgroup walks ten K blocks or more (the ring has to fill before the first
// matrix instruction): K 14336 x N 4096 at M = 64 / 128: 24.0 / 29.4 -> 19.6 / 29.2 us, 8192 x 8192:
// 24.9 / 36.7 -> 20.6 / 30.0 us, 4096 x 28672: 29.9 / 39.3 -> 26.6 / 38.4 us; with fewer blocks per
// workgroup (K 4096 on layers up to 6144 wide) the narrow tiles stay ahead, and up to 64 rows on a
// layer of 200 column tiles or more the 64-row tiles do (K 8192 x N 28672, M = 48: 41.9 against 46.2 us).
static int ring_small_splits(int M, int K, int N) {
  if (M <= 32 || M > 128) return 0;
  const long cus = device_cu_count(), ctiles = N / 128, G = K / 128;
  if (ctiles >= 200 && M <= 64) return 0;
  long s = cus / ctiles;
  if (s > G / 8) s = G / 8;
  while (s > 1 && (size_t)s * M * N * sizeof(float) > TILE_SPLITK_BYTES) --s;
  if (s < 1) s = 1;
  const long kper = (G + s - 1) / s;
  if (kper < 10) return 0;
  return (int)((G + kper - 1) / kper);
}

size_t w4a16_tile_workspace_bytes(int M, int K, int N) {
  // (the choice between the kernels also depends on the dtype and the group size, which this
  // function does not see: room for whichever plan is larger)
  const int narrow = tile_narrow_splits(M, K, N);
  const int s = narrow ? narrow : tile_splits(M, K, N);
  // (the 512-column ring workgroups are only taken where they need no split)
  int sr = tile_ring_plan(M, K, N) == 2 ? w4a16_mid_splits(M, K, N, 2) : 1;
  const int ss = ring_small_splits(M, K, N);
  if (ss > sr) sr = ss;
  const int m = s > sr ? s : sr;
  return m > 1 ? (size_t)m * M * N * sizeof(float) : 0;
}

// bf16 activations staged as fp16: where the staging area sits in the workspace (behind the split-K
// partial tiles), how many rows it holds at most, and from how many rows on it pays
constexpr size_t BF16_STAGE_OFFSET = TILE_SPLITK_BYTES;
constexpr size_t BF16_STAGE_SCALE_BYTES = (size_t)64 << 10;          // one multiplier per staged row
constexpr size_t BF16_STAGE_BYTES = (size_t)64 << 20;
constexpr int BF16_STAGE_MIN_M = 65;
// (measured, us, staged against the bf16 loop: K 4096 x N 28672 at M = 129 / 2048 / 8192: 68 / 477 / 1812
// against 85 / 578 / 2202; K 4096 x N 6144 at 256 / 512 / 2048: 34 / 49 / 119 against 35 / 55 / 136; K 4096 x
// N 4096 at 512 / 1024 / 4096: 38 / 53 / 151 against 39 / 58 / 170; K 14336 x N 4096 at 512 / 2048: 85 / 258
// against 91 / 299; 65..128 rows, K 4096 x N 28672 at M = 80 / 100 / 128: 49 / 51 / 51 against 60: the conversion
// pass costs 5-25 us, so the output has to have about two million elements)
static bool bf16_stage_pays(int M, int N) { return M >= BF16_STAGE_MIN_M && (long)M * N >= (7L << 18); }

size_t w4a16_bf16_stage_workspace_bytes(int M, int K) {
  if (M < BF16_STAGE_MIN_M) return 0;
  const size_t rows = (size_t)M * K * 2;
  return BF16_STAGE_OFFSET + BF16_STAGE_SCALE_BYTES + (rows < BF16_STAGE_BYTES ? rows : BF16_STAGE_BYTES);
}

static int tile_launch_dense(void* out, const void* x, const int32_t* qweight, const void* scales,
                             const void* zeros, int zeros_kind, const void* bias, int M, int K, int N,
                             int group_size, int dtype, void* workspace, size_t workspace_bytes,
                             const float* row_scale, hipStream_t st);

// bf16 activations through the fp16 kernels.  The rows are stored in the staging area of the workspace
// as fp16 times a power of two each (exact); the pipelined 64-row tile loop multiplies them with the
// exact integers q - z, the ring kernels with (q - z) s in fp16, as for fp16 activations; inputs taller
// than the area go in row chunks.  force_tw: -1 the kernels the fp16 path would take for the chunk
// (ring workgroups where their rounds are priced lower and K stays unsplit), 0 the 64-row tiles,
// 2 / 4 ring workgroups of 256 / 512 columns.  BF16_STAGE_NOT_TAKEN: group size, zero-point kind or
// workspace do not allow it, nothing was launched.
constexpr int BF16_STAGE_NOT_TAKEN = -12345;
int w4a16_bf16_staged_launch(void* out, const void* x, const int32_t* qweight, const void* scales, const void* zeros,
                             int zeros_kind, const void* bias, int M, int K, int N, int group_size, void* workspace,
                             size_t workspace_bytes, int force_tw, hipStream_t st) {
  if (group_size % 128 != 0 || zeros_kind == MI355Q_ZP_PRESCALED || M <= 64 || !workspace ||
      workspace_bytes <= BF16_STAGE_OFFSET + BF16_STAGE_SCALE_BYTES)
    return BF16_STAGE_NOT_TAKEN;
  // Rows per chunk for a staging area that starts `off` bytes into the workspace
  auto rows_per_chunk = [&](size_t off) -> long {
    const size_t room = workspace_bytes - off - BF16_STAGE_SCALE_BYTES;
    long rows_max = (long)(room / ((size_t)K * 2));
    // (the last 64 words of the multiplier area hold the scale maxima for the ring kernels)
    if (rows_max > (long)(BF16_STAGE_SCALE_BYTES / sizeof(float)) - 64) rows_max = BF16_STAGE_SCALE_BYTES / sizeof(float) - 64;
    rows_max &= ~63L;
    if (rows_max < 256 && rows_max < M) return 0;
    const long chunks = (M + rows_max - 1) / rows_max;
    return (((M + chunks - 1) / chunks) + 63) & ~63L;
  };
  // The area lies behind the split-K partial tiles -- or, where no chunk's launch splits K (tall
  // inputs: exactly those that would otherwise need many chunks), at the front of the workspace
  size_t off = 0;
  long per = rows_per_chunk(0);
  if (per > 0) {
    const int last = (int)(M % per ? M % per : per);
    if (tile_splits((int)(per < M ? per : M), K, N) != 1 || tile_splits(last, K, N) != 1) per = 0;
  }
  if (per == 0) {
    off = BF16_STAGE_OFFSET;
    per = rows_per_chunk(off);
    if (per == 0) return BF16_STAGE_NOT_TAKEN;
  }
  float* rs = (float*)((char*)workspace + off);
  uint32_t* smax = (uint32_t*)rs + BF16_STAGE_SCALE_BYTES / sizeof(float) - 64;
  uint16_t* x16 = (uint16_t*)((char*)workspace + off + BF16_STAGE_SCALE_BYTES);
  const long scale_chunks = (long)(K / group_size) * N / 8;
  bool scanned = false;
  for (long m0 = 0; m0 < M; m0 += per) {
    const int mc = (int)(M - m0 < per ? M - m0 : per);
    int tw = force_tw;
    if (tw < 0) {
      tw = tile_ring_plan(mc, K, N);
      if (tw == 2 && w4a16_mid_splits(mc, K, N, 2) != 1) tw = 0;
    }
    if (mc <= 64) tw = 0;                          // (a short last chunk: the ring kernels here are the 128-row ones)
    const bool scan = tw && !scanned;
    scanned |= scan;
    if (K <= 16384)
      hipLaunchKernelGGL(bf16_rows_to_f16_kernel<true>, dim3(mc + (scan ? 64 : 0)), dim3(256), 0, st,
                         (const uint16_t*)x + (size_t)m0 * K, x16, rs, K, mc, (const u4*)scales, scale_chunks, smax);
    else
      hipLaunchKernelGGL(bf16_rows_to_f16_kernel<false>, dim3(mc + (scan ? 64 : 0)), dim3(256), 0, st,
                         (const uint16_t*)x + (size_t)m0 * K, x16, rs, K, mc, (const u4*)scales, scale_chunks, smax);
    MQ_LAUNCH_CHECK("w4a16_gemm(bf16 rows to fp16)");
    int rc;
    if (tw)
      rc = w4a16_mid_launch_staged((uint16_t*)out + (size_t)m0 * N, x16, qweight, scales, zeros, zeros_kind, bias, mc, K, N,
                                   group_size, rs, smax, tw, st);
    else
      rc = tile_launch_dense((uint16_t*)out + (size_t)m0 * N, x16, qweight, scales, zeros, zeros_kind, bias, mc, K, N,
                             group_size, MI355Q_BF16, workspace, off, rs, st);
    if (rc) return rc;
  }
  return 0;
}

int w4a16_tile_launch(void* out, const void* x, const int32_t* qweight, const void* scales,
                      const void* zeros, int zeros_kind, const void* bias, int M, int K, int N,
                      int group_size, int dtype, void* workspace, size_t workspace_bytes, bool allow_ring,
                      hipStream_t st) {
  // groups of 64 and 32: two and four groups per K block, 64-row tiles with the plain loop only
  const bool small_groups = group_size == 64 || group_size == 32;
  MQ_REQUIRE(group_size % 128 == 0 || small_groups,
             "w4a16_gemm: the MFMA kernel needs a group size of 32, 64 or a multiple of 128, got %d", group_size);
  MQ_REQUIRE((size_t)M * K * 2 < ((size_t)1 << 32), "w4a16_gemm: activation matrix %d x %d is 4 GiB or more", M, K);
  if (allow_ring && dtype == MI355Q_F16 && !small_groups) {
    if (const int tw = tile_ring_plan(M, K, N))
      return w4a16_mid_launch(out, x, qweight, scales, zeros, zeros_kind, bias, M, K, N, group_size, dtype,
                              workspace, workspace_bytes, 0, tw, st);
    if (const int ss = ring_small_splits(M, K, N))
      return w4a16_mid_launch(out, x, qweight, scales, zeros, zeros_kind, bias, M, K, N, group_size, dtype, workspace,
                              workspace_bytes, ss, 1, st);
  }
  // bf16 with a workspace that has the staging area: the rows become fp16 times a power of two each
  // and take the fp16 loops (the bf16 loop has no room for the pipeline: it spills)
  if (allow_ring && dtype == MI355Q_BF16 && bf16_stage_pays(M, N)) {
    const int rc = w4a16_bf16_staged_launch(out, x, qweight, scales, zeros, zeros_kind, bias, M, K, N, group_size, workspace,
                                            workspace_bytes, -1, st);
    if (rc != BF16_STAGE_NOT_TAKEN) return rc;
  }
  return tile_launch_dense(out, x, qweight, scales, zeros, zeros_kind, bias, M, K, N, group_size, dtype, workspace,
                           workspace_bytes, nullptr, st);
}

// 64-row tiles (or the narrow tiles) for one dense problem; row_scale: bf16 rows staged as fp16 (x points
// at the staged rows, dtype stays bf16 for scales, bias and output)
static int tile_launch_dense(void* out, const void* x, const int32_t* qweight, const void* scales,
                             const void* zeros, int zeros_kind, const void* bias, int M, int K, int N,
                             int group_size, int dtype, void* workspace, size_t workspace_bytes,
                             const float* row_scale, hipStream_t st) {
  const bool small_groups = group_size == 64 || group_size == 32;
  TileArgs a = {};
  a.row_scale = row_scale;
  a.out = (uint16_t*)out;
  a.x = (const uint16_t*)x;
  a.qw = (const u4*)qweight;
  a.scales = (const uint16_t*)scales;
  a.zeros = zeros;
  a.bias = (const uint16_t*)bias;
  a.M = M; a.K = K; a.N = N; a.gs = group_size;
  int mt = tile_rows_mt(M, N);
  int ntw = 4;
  const int G = K / 128;
  int splits = tile_splits(M, K, N);
  const int narrow = (small_groups || row_scale) ? 0 : tile_narrow_splits(M, K, N);
  if (narrow) {
    mt = 2;
    ntw = 1;
    splits = narrow;
  }
  const int row_blocks = (M + 16 * mt - 1) / (16 * mt);
  if (splits > 1 && (!workspace || workspace_bytes < (size_t)splits * M * N * sizeof(float))) splits = 1;
  a.kper = (G + splits - 1) / splits;
  splits = (G + a.kper - 1) / a.kper;                // no empty splits
  a.partial = splits > 1 ? (float*)workspace : nullptr;
  hipError_t e;
  const uint32_t gpk = (uint32_t)group_size / 128u;
  a.gpk_magic = gpk > 1 ? (uint32_t)((((uint64_t)1 << 32) + gpk - 1) / gpk) : 0u;
  if (row_scale)
    e = launch_iobf<false>(a, zeros_kind, row_blocks, st);
  else if (small_groups)
    e = (dtype == MI355Q_F16) ? launch_small_groups<MI355Q_F16, 4, false>(a, zeros_kind, 128 / group_size, row_blocks, st)
                              : launch_small_groups<MI355Q_BF16, 4, false>(a, zeros_kind, 128 / group_size, row_blocks, st);
  else if (ntw < 4)
    e = (dtype == MI355Q_F16) ? launch_narrow<MI355Q_F16>(a, zeros_kind, row_blocks, st)
                              : launch_narrow<MI355Q_BF16>(a, zeros_kind, row_blocks, st);
  else
    e = (dtype == MI355Q_F16) ? launch_mt<MI355Q_F16, false>(a, zeros_kind, mt, row_blocks, st)
                              : launch_mt<MI355Q_BF16, false>(a, zeros_kind, mt, row_blocks, st);
  MQ_REQUIRE(e == hipSuccess, "w4a16_gemm(tile): cannot reserve LDS: %s", hipGetErrorString(e));
  MQ_LAUNCH_CHECK("w4a16_gemm(tile)");
  if (splits > 1) return splitk_reduce_rows_launch(out, (const float*)workspace, bias, M, N, splits, dtype, st, row_scale);
  return 0;
}

int w4a16_stream_grouped_launch(void* out, const void* x, const int32_t* qweight, const void* scales,
                                const void* zeros, int zeros_kind, const float* topk_weights,
                                const int32_t* sorted_ids, const int32_t* expert_ids, const int32_t* npp,
                                int numel, int topk, int block_size, int max_blocks, int E, int K, int N,
                                int group_size, int dtype, hipStream_t st);

// Split-K plan of a grouped launch.  The host does not know how many blocks the alignment filled, so
// the grid is estimated as every slot in a full block plus half a block of pads per expert.  A long K
// with a narrow N (the second expert GEMM of a gated MLP) leaves the chip part empty and makes its few
// workgroups very long; K is split until about two and a half workgroups per resident slot exist,
// keeping at least 16 K blocks per split (Mixtral-8x7B layer, 512 tokens, second GEMM: 4 splits
// measured best of 1..7; every further split adds 17 MB of partial tiles).
static int grouped_splits(int numel, int block_size, int max_blocks, int E, int K, int N) {
  if (block_size != 64) return 1;                  // the 64-row pipelined kernel only
  const int G = K / 128;
  long blocks = (numel + block_size - 1) / block_size + (E + 1) / 2;
  if (blocks > max_blocks) blocks = max_blocks;
  const long wgs = blocks * ((N + BN - 1) / BN), slots = 2L * device_cu_count();
  if (wgs >= 2 * slots || G < 32) return 1;
  long s = (5 * slots / 2 + wgs - 1) / wgs;
  if (s > G / 16) s = G / 16;
  while (s > 1 && (size_t)s * numel * N * sizeof(float) > TILE_SPLITK_BYTES * 2) --s;
  return s < 1 ? 1 : (int)s;
}
// bf16 activations of a grouped launch staged as fp16 rows (blocks of 64 slots, outputs of two million
// elements or more): the area follows the partial tiles of the launch's split-K plan
static bool grouped_stage_pays(int numel, int block_size, int N) {
  return block_size == 64 && (long)numel * N >= (1L << 21);
}
static size_t grouped_partial_bytes(int splits, int numel, int N) {
  return splits > 1 ? (((size_t)splits * numel * N * sizeof(float)) + 255) & ~(size_t)255 : 0;
}
size_t w4a16_grouped_workspace_bytes(int numel, int block_size, int max_blocks, int E, int K, int N) {
  const int s = grouped_splits(numel, block_size, max_blocks, E, K, N);
  size_t need = s > 1 ? (size_t)s * numel * N * sizeof(float) : 0;
  // (neither the dtype nor topk is known here: room for bf16 rows of one slot each)
  // (asked for while everything stays within 128 MiB; a larger workspace is used when it is there)
  const size_t staged = grouped_partial_bytes(s, numel, N) + BF16_STAGE_SCALE_BYTES + (size_t)numel * K * 2;
  if (grouped_stage_pays(numel, block_size, N) && staged <= 2 * BF16_STAGE_BYTES) need = staged;
  return need;
}

int w4a16_grouped_launch(void* out, const void* x, const int32_t* qweight, const void* scales,
                         const float* scales_f32, const float* out_scale,
                         const void* zeros, int zeros_kind, const float* topk_weights,
                         const int32_t* sorted_ids, const int32_t* expert_ids, const int32_t* npp,
                         int numel, int topk, int block_size, int max_blocks, int E, int K, int N,
                         int group_size, int dtype, void* workspace, size_t workspace_bytes, hipStream_t st) {
  // groups of 64 and 32: the plain loop of the MFMA kernel at every block size
  const bool small_groups = group_size == 64 || group_size == 32;
  MQ_REQUIRE(group_size % 128 == 0 || (small_groups && !scales_f32 && !out_scale),
             "moe_w4a16: group_size=%d must be 32, 64 or a multiple of 128 (a multiple of 128 with fp32 scales)", group_size);
  MQ_REQUIRE((size_t)(numel / (topk > 0 ? topk : 1)) * K * 2 < ((size_t)1 << 32),
             "moe_w4a16: activation matrix of %d rows x %d is 4 GiB or more", numel / (topk > 0 ? topk : 1), K);
  MQ_REQUIRE(block_size == 16 || block_size == 32 || block_size == 64 || block_size == 128,
             "moe_w4a16: block_size=%d must be 16, 32, 64 or 128", block_size);
  // blocks of 16 or 32 slots (decode-sized token counts): the layer is bound by the experts' weights,
  // which the streaming kernel reads faster than the MFMA tile kernel with one or two row tiles
  // (the grouped streaming kernel takes groups that are multiples of 128 only)
  if (block_size <= 32 && !scales_f32 && !out_scale && !small_groups)
    return w4a16_stream_grouped_launch(out, x, qweight, scales, zeros, zeros_kind, topk_weights, sorted_ids,
                                       expert_ids, npp, numel, topk, block_size, max_blocks, E, K, N, group_size,
                                       dtype, st);
  TileArgs a = {};
  a.out = (uint16_t*)out;
  a.x = (const uint16_t*)x;
  a.qw = (const u4*)qweight;
  a.scales = (const uint16_t*)scales;
  a.scales_f32 = scales_f32;
  a.out_scale = out_scale;
  MQ_REQUIRE(!scales_f32 || (zeros_kind == MI355Q_ZP_NONE && !zeros),
             "moe_w4a16: fp32 group scales go with symmetric weights only");
  a.zeros = zeros;
  a.M = numel; a.K = K; a.N = N; a.gs = group_size;
  a.sorted_ids = sorted_ids; a.expert_ids = expert_ids; a.npp = npp; a.topk_weights = topk_weights;
  a.numel = numel; a.topk = topk; a.E = E;
  const int G = K / 128;
  int splits = (scales_f32 || out_scale) ? 1 : grouped_splits(numel, block_size, max_blocks, E, K, N);
  if (splits > 1 && (!workspace || workspace_bytes < (size_t)splits * numel * N * sizeof(float))) splits = 1;
  a.kper = (G + splits - 1) / splits;
  splits = (G + a.kper - 1) / a.kper;              // no empty splits
  a.partial = splits > 1 ? (float*)workspace : nullptr;
  // bf16 at prefill token counts: the rows staged as fp16 times a power of two each take the pipelined
  // fp16 loop (see w4a16_bf16_staged_launch); the multiplier of a slot is that of the row it was gathered from
  bool staged = false;
  if (dtype == MI355Q_BF16 && !small_groups && !scales_f32 && !out_scale && zeros_kind != MI355Q_ZP_PRESCALED &&
      grouped_stage_pays(numel, block_size, N) && workspace && topk > 0) {
    const size_t poff = grouped_partial_bytes(splits, numel, N);
    const int rows = numel / topk;
    if (rows > 0 && rows <= (int)(BF16_STAGE_SCALE_BYTES / sizeof(float)) &&
        poff + BF16_STAGE_SCALE_BYTES + (size_t)rows * K * 2 <= workspace_bytes) {
      float* rs = (float*)((char*)workspace + poff);
      uint16_t* x16 = (uint16_t*)((char*)workspace + poff + BF16_STAGE_SCALE_BYTES);
      if (K <= 16384)
        hipLaunchKernelGGL(bf16_rows_to_f16_kernel<true>, dim3(rows), dim3(256), 0, st, (const uint16_t*)x, x16, rs, K, rows,
                           (const u4*)nullptr, 0L, (uint32_t*)nullptr);
      else
        hipLaunchKernelGGL(bf16_rows_to_f16_kernel<false>, dim3(rows), dim3(256), 0, st, (const uint16_t*)x, x16, rs, K, rows,
                           (const u4*)nullptr, 0L, (uint32_t*)nullptr);
      MQ_LAUNCH_CHECK("moe_w4a16(bf16 rows to fp16)");
      a.x = x16;
      a.row_scale = rs;
      staged = true;
    }
  }
  a.w_stride = (long)(K / 8) * N / 4;              // u4 elements per expert
  a.s_stride = (long)(K / group_size) * N;
  a.z_stride = zeros_kind == MI355Q_ZP_PACKED ? (long)(K / group_size) * (N / 8) : (long)(K / group_size) * N;
  hipError_t e;
  if (staged) {
    e = launch_iobf<true>(a, zeros_kind, max_blocks, st);
  } else if (small_groups) {
    const int gpb = 128 / group_size;
    if (block_size == 16)
      e = (dtype == MI355Q_F16) ? launch_small_groups<MI355Q_F16, 1, true>(a, zeros_kind, gpb, max_blocks, st)
                                : launch_small_groups<MI355Q_BF16, 1, true>(a, zeros_kind, gpb, max_blocks, st);
    else if (block_size == 32)
      e = (dtype == MI355Q_F16) ? launch_small_groups<MI355Q_F16, 2, true>(a, zeros_kind, gpb, max_blocks, st)
                                : launch_small_groups<MI355Q_BF16, 2, true>(a, zeros_kind, gpb, max_blocks, st);
    else if (block_size == 64)
      e = (dtype == MI355Q_F16) ? launch_small_groups<MI355Q_F16, 4, true>(a, zeros_kind, gpb, max_blocks, st)
                                : launch_small_groups<MI355Q_BF16, 4, true>(a, zeros_kind, gpb, max_blocks, st);
    else
      e = (dtype == MI355Q_F16) ? launch_small_groups<MI355Q_F16, 8, true>(a, zeros_kind, gpb, max_blocks, st)
                                : launch_small_groups<MI355Q_BF16, 8, true>(a, zeros_kind, gpb, max_blocks, st);
  } else {
    e = (dtype == MI355Q_F16) ? launch_mt<MI355Q_F16, true>(a, zeros_kind, block_size / 16, max_blocks, st)
                              : launch_mt<MI355Q_BF16, true>(a, zeros_kind, block_size / 16, max_blocks, st);
  }
  MQ_REQUIRE(e == hipSuccess, "moe_w4a16: cannot reserve LDS: %s", hipGetErrorString(e));
  MQ_LAUNCH_CHECK("moe_w4a16");
  if (splits > 1) {
    // the reduction walks the aligned id list (at most max_blocks * block_size positions, cut at *npp on
    // the device): rows of ids that the alignment dropped have no partial tiles and are not touched
    const long threads = (long)max_blocks * block_size * (N / 4);
    const unsigned blocks = (unsigned)((threads + 255) / 256);
    if (dtype == MI355Q_F16)
      hipLaunchKernelGGL((w4a16_grouped_reduce_kernel<MI355Q_F16>), dim3(blocks), dim3(256), 0, st, (uint16_t*)out,
                         (const float*)workspace, topk_weights, sorted_ids, npp, numel, N, splits, (const float*)nullptr, 1);
    else
      hipLaunchKernelGGL((w4a16_grouped_reduce_kernel<MI355Q_BF16>), dim3(blocks), dim3(256), 0, st, (uint16_t*)out,
                         (const float*)workspace, topk_weights, sorted_ids, npp, numel, N, splits, a.row_scale, topk);
    MQ_LAUNCH_CHECK("moe_w4a16(split-K reduce)");
  }
  return 0;
}

}  // namespace mi355q
