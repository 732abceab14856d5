// fp8-e4m3 block-scaled GEMM for more than 64 rows on the 128-deep fp8 MFMA of gfx950
// (v_mfma_f32_16x16x128_f8f6f4, twice the rate of the 32-deep one), with the 128 x 128 block
// scales applied to the fp32 partial sum of every K block.
//
//   out[m, n] = sum_kb x_scale[m, kb] * w_scale[n / 128, kb] * sum_{k in block kb} x[m, k] * w[n, k]
//
// Same machinery as the int8 GEMM next door: a workgroup of eight wavefronts
// (4 x 2, each 64 rows of x by 64 rows of w) owns a 256 x 128 output tile; K
// advances in LDS tiles of 128 bytes per row, which is exactly one scale block
// and one MFMA deep; tiles go from global memory straight into LDS (16 B per
// lane, no staging registers; 16-byte-chunk XOR swizzle, or chunk-major for
// kslab weights) in three stages; operand reads are hand-written and
// hand-waited for.  A K block's MFMA starts from zero and its result joins the
// running sum multiplied by the block's scale.  128 columns are exactly one
// scale block, so the weight scale of a tile and K block is a single number;
// it and the activation scales of the K block (one per row) travel with the
// tiles through LDS (4-byte direct-to-LDS copies).  Two wavefronts per SIMD
// leave each 256 registers: 64 running sums, two sets of x operands, one set
// of w operands that is re-read tile by tile behind the MFMAs (see `step`).
//
// PC variant (per-token x per-channel scales, cutlass_scaled_mm on fp8 operands): the scales live
// outside the K sum, so every MFMA accumulates straight into the running sum, no scales travel
// through LDS, and the epilogue multiplies by x_scale[m] (or one value) and w_scale[n] (or one value).
//
// OP16 variant (unquantised fp16 / bf16 experts at prefill token counts, grouped launches only): the
// same tiles of 128 bytes per row hold 64 elements of 16 bits; a lane's two 16-byte chunks are the
// operands of two 32-deep 16-bit MFMAs (chunk kq: elements 8 kq .. 8 kq + 7 of the first 32, chunk
// 4 + kq: of the second 32), which take as long as the one 128-deep fp8 MFMA.  No scales anywhere.
// The host passes K and the row strides in bytes.
#include "common.h"

namespace mi355q {
int kcontig_fp8_pc_launch(void* out, const void* a, const void* w, const float* a_scale, int scale_per_row,
                          const float* w_scale, int scale_per_col, const void* bias, int M, int K, int N,
                          int out_dtype, int w_layout, hipStream_t st);
namespace {

constexpr int FTM = 256, FTN = 128, FTKB = 128;
constexpr int F8_THREADS = 512;

struct F8Args {
  void* out;                // [M, N] f16 / bf16, row stride ldo elements
  const uint8_t* x;         // [M, K] fp8, row stride ldx bytes
  const uint8_t* w;         // [N, K] fp8 row-major (row stride ldw) or in the kslab order
  const float* x_scale;     // [M, K / 128]; PC: [M] or one value
  const float* w_scale;     // [N / 128, K / 128]; PC: [N] or one value
  int xs_mul, ws_mul;       // PC: index multipliers of x_scale / w_scale (1 = per token / per channel, 0 = one value)
  const float* xs_t;        // dense launches: block scales of the activations, K block major, xs_t[kb * xs_ld + m];
  long xs_ld;               // null: x_scale as given (a row's K blocks side by side)
  const void* bias;         // [N] in the output dtype or null
  int M, N, K;
  long ldx, ldw, ldo;
  int w_kslab;              // 1: kslab order of 1-byte elements; 2: of 2-byte elements (OP16; K blocks of 256 bytes)
  int n_panels_swizzle;
  int ksplits;              // > 1: every output tile is worked on by `ksplits` workgroups, each a range of K blocks,
  float* partial;           //      which leave their fp32 sums in partial[split][M][N]; the epilogue is a second launch
  // grouped (MoE) launches: a row tile is one align block of 256 slot ids of one expert
  const int32_t* sorted_ids;   // [blocks * 256] flat (token, slot) ids, pad = numel
  const int32_t* expert_ids;   // [blocks]
  const int32_t* npp;          // device scalar: padded id count
  const float* topk_weights;   // [numel] or null
  int numel, topk, E, max_blocks;
  int block_rows;              // slot ids per align block: 256, or 128 (the upper half of every row tile is empty:
                               // its wavefronts only copy, as in a dense launch of up to 128 rows)
  long w_stride, ws_stride;    // per expert: bytes of weights, floats of weight scales
};

__device__ __forceinline__ void dma16(const void* gptr, void* lds_wave_base) {
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)gptr,
                                   (__attribute__((address_space(3))) void*)lds_wave_base, 16, 0, 0);
}
// 64 x 4 B: lane l lands at base + 4 l
__device__ __forceinline__ void dma4(const void* gptr, void* lds_wave_base) {
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)gptr,
                                   (__attribute__((address_space(3))) void*)lds_wave_base, 4, 0, 0);
}

typedef int i8v __attribute__((ext_vector_type(8)));

// GROUPED: the fused-MoE grouped GEMM at prefill token counts.  Row tile b is align block b (256 slot
// ids of expert expert_ids[b]): x rows and their scales are gathered through the ids (row id / topk),
// weights and weight scales are the expert's, output row id gets the result (times its routing weight).
// Blocks past num_tokens_post_pad do not exist (the tile count is read on the device); a block of an
// expert outside [0, E) writes zeros.  No K ranges, no bias.
template <int DT, bool PC, bool GROUPED = false, bool OP16 = false>
__global__ void __launch_bounds__(F8_THREADS, 1)
fp8_block_gemm_kernel(F8Args a) {
  static_assert(!GROUPED || !PC || OP16, "the grouped form exists for block scales and for 16-bit operands");
  static_assert(!OP16 || (PC && GROUPED), "16-bit operands: grouped launches, no scales");
  constexpr int WN = 2, NI = 4, NJ = 4;                 // 4 x 2 wavefronts of 64 x 64
  constexpr int X_BYTES = FTM * FTKB, W_BYTES = FTN * FTKB, XS_BYTES = FTM * 4;
  constexpr int WS_BYTES = 256;                         // the tile's weight scale of a K block, 64 copies
  constexpr int STAGE_BYTES = X_BYTES + W_BYTES + XS_BYTES + WS_BYTES;
  constexpr int XCOPIES = FTM / 8 / 8, WCOPIES = FTN / 8 / 8;       // 1 KiB copies per wavefront
  extern __shared__ __align__(16) unsigned char lds[];
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l16 = lane & 15, kq = lane >> 4;
  const int wm = wave / WN, wn = wave % WN;
  const int M = a.M, N = a.N, K = a.K, KB = K >> 7;

  int mtiles = (M + FTM - 1) / FTM;
  if (GROUPED) {
    const int blocks = (*a.npp + a.block_rows - 1) / a.block_rows;
    mtiles = __builtin_amdgcn_readfirstlane(blocks < a.max_blocks ? blocks : a.max_blocks);
  }
  const int ntiles_n = N / FTN;
  const int ksplits = (!GROUPED && a.ksplits > 1) ? a.ksplits : 1;
  const int total_tiles = mtiles * ntiles_n * ksplits;   // (split K: tile ids count (output tile, K range) pairs)
  if (GROUPED && (int)blockIdx.x >= total_tiles) return;  // (the grid is sized for the largest block count the ids can fill)
  auto tile_origin = [&](int tile, int& m0, int& n0) {
    int tm, tn;
    if (GROUPED) {
      // block-major: neighbouring workgroups share a block's activation rows
      tm = tile / ntiles_n;
      tn = tile - tm * ntiles_n;
    } else if (ksplits > 1) {
      const int t = tile / ksplits;
      tm = t % mtiles;
      tn = t / mtiles;
    } else if (a.n_panels_swizzle) {
      // XCD x takes the weight panels tn = x, x + 8, ...; it sweeps them for a chunk of 8 row tiles
      // (2048 rows of x: what its L2 can keep warm next to a panel) before the next chunk
      const int x = tile & 7, j = tile >> 3;
      const int P = ntiles_n >> 3, full = (mtiles >> 3) << 3;           // panels per XCD, row tiles in whole chunks
      int tj;
      if (j < full * P) {
        const int c = j / (8 * P), r = j - c * 8 * P;
        tj = r >> 3;
        tm = c * 8 + (r & 7);
      } else {
        const int rem = mtiles - full, r = j - full * P;
        tj = r / rem;
        tm = full + r % rem;
      }
      tn = tj * 8 + x;
    } else {
      tm = tile % mtiles;
      tn = tile / mtiles;
    }
    m0 = tm * FTM;
    n0 = tn * FTN;
  };

  f4 acc[NI][NJ];

  // global -> LDS: lane = 8 * row + slot, slot p of row r receives chunk p ^ (r & 7); kslab weights
  // chunk-major (lane = 8 * position + row, position p of an odd 8-row group holding chunk p ^ 1)
  const int crow = lane >> 3, cchunk = (lane & 7) ^ (crow & 7);
  uint32_t xo[XCOPIES], wo[WCOPIES], xso = 0;
  int wsbase = 0;
  const uint8_t *xtile, *wtile;
  const float* xsbase = a.x_scale;
  const long xs_kstride = (!GROUPED && a.xs_t) ? a.xs_ld : 1;       // floats between the K blocks of a row's scale
  auto set_copy_tile = [&](int tile) {
    int m0, n0;
    tile_origin(tile, m0, n0);
    long ebytes = 0;
    int escales = 0;
    if (GROUPED) {
      const int* ids = a.sorted_ids + (m0 / FTM) * a.block_rows;
#pragma unroll
      for (int p = 0; p < XCOPIES; ++p) {
        // (blocks of 128: the upper half of the tile copies the lower half's rows once more; nobody multiplies them)
        const int id = ids[((wave + 8 * p) * 8 + crow) & (a.block_rows - 1)];
        xo[p] = (uint32_t)(max(0, min(id, a.numel - 1)) / a.topk) * (uint32_t)a.ldx + (uint32_t)(16 * cchunk);   // pads read a valid row
      }
      int e = a.expert_ids[m0 / FTM];
      e = __builtin_amdgcn_readfirstlane((e < 0 || e >= a.E) ? 0 : e);     // (a foreign expert's block is computed and zeroed)
      ebytes = (long)e * a.w_stride;
      escales = e * (int)a.ws_stride;
    } else {
#pragma unroll
      for (int p = 0; p < XCOPIES; ++p) {
        const int r = (wave + 8 * p) * 8 + crow;
        xo[p] = (uint32_t)((min(m0 + r, M - 1) - m0) * a.ldx + 16 * cchunk);
      }
    }
#pragma unroll
    for (int p = 0; p < WCOPIES; ++p) {
      if (OP16 && a.w_kslab) {
        // 2-byte elements: a K block of the kslab order is 256 bytes per row = two of this kernel's K
        // tiles; chunk c of K tile h is vector c & 3 of lane quarter 2 h + (c >> 2)
        const uint32_t n = (uint32_t)(n0 + (wave + 8 * p) * 8 + (lane & 7));
        const uint32_t c = (uint32_t)((lane >> 3) ^ (wave & 1));
        wo[p] = ((n >> 6) * (uint32_t)(K >> 8) * 4u + ((n & 63u) >> 4)) * 4096u + (c & 3u) * 1024u +
                ((c >> 2) * 16u + (n & 15u)) * 16u;
      } else if (a.w_kslab) {
        const uint32_t n = (uint32_t)(n0 + (wave + 8 * p) * 8 + (lane & 7));
        const uint32_t c = (uint32_t)((lane >> 3) ^ (wave & 1));
        wo[p] = ((n >> 6) * (uint32_t)(K >> 7) * 4u + ((n & 63u) >> 4)) * 2048u + (c & 1u) * 1024u +
                ((c >> 1) * 16u + (n & 15u)) * 16u;
      } else {
        const int r = (wave + 8 * p) * 8 + crow;
        wo[p] = (uint32_t)(r * a.ldw + 16 * cchunk);
      }
    }
    // activation scales: wavefronts 0..3 copy 64 rows each (index in floats)
    // (split K: the tile's range starts kb0 K blocks into every row; 64 kslab rows interleave their K blocks)
    const int kb0 = ksplits > 1 ? (tile % ksplits) * (KB / ksplits) : 0;
    if (!GROUPED && a.xs_t) {
      // K block major: the 64 scales of a copy lie side by side (4 cache lines instead of 64)
      xso = (uint32_t)min(m0 + 64 * (wave & 3) + lane, M - 1);
      xsbase = a.xs_t + (long)kb0 * a.xs_ld;
    } else if (GROUPED) {
      const int id = a.sorted_ids[(m0 / FTM) * a.block_rows + ((64 * (wave & 3) + lane) & (a.block_rows - 1))];
      xso = (uint32_t)(max(0, min(id, a.numel - 1)) / a.topk) * (uint32_t)KB;
      xsbase = a.x_scale;
    } else {
      xso = (uint32_t)min(m0 + 64 * (wave & 3) + lane, M - 1) * (uint32_t)KB + (uint32_t)kb0;
      xsbase = a.x_scale;
    }
    wsbase = escales + (n0 >> 7) * KB + kb0;       // wavefront 4 copies the tile's weight scale
    xtile = GROUPED ? a.x : a.x + (long)m0 * a.ldx + (long)kb0 * FTKB;
    wtile = a.w + ebytes + (a.w_kslab ? (long)kb0 * FTKB * 64 : (long)n0 * a.ldw + (long)kb0 * FTKB);
  };
  constexpr int NSLOT = XCOPIES + WCOPIES + 1;
  auto copy_slot = [&](int s, int stage, int kt) {
    unsigned char* xs = lds + stage * STAGE_BYTES;
    if (s < XCOPIES) {
      dma16(xtile + (long)kt * FTKB + xo[s], xs + (wave + 8 * s) * 1024);
    } else if (s < XCOPIES + WCOPIES) {
      const int p = s - XCOPIES;
      const long koff = (OP16 && a.w_kslab) ? (long)(kt >> 1) * 16384 + (kt & 1) * 512
                                            : (a.w_kslab ? (long)kt * FTKB * 64 : (long)kt * FTKB);
      dma16(wtile + koff + wo[p < WCOPIES ? p : 0], xs + X_BYTES + (wave + 8 * p) * 1024);
    } else if (PC) {
      // no scales inside the K sum
    } else if (wave < 4) {
      dma4(xsbase + xso + (long)kt * xs_kstride, xs + X_BYTES + W_BYTES + wave * 256);
    } else if (wave == 4) {
      dma4(a.w_scale + wsbase + kt, xs + X_BYTES + W_BYTES + XS_BYTES);
    }
  };

  // operand reads (assembly, waited for by hand: see the int8 kernel).  Lane (l16, kq) takes the
  // 16-byte chunks kq and 4 + kq of row l16 of a 16-row tile: together the 32 bytes of K it feeds
  // to the 128-deep MFMA.  Which 32 of the 128 a lane holds does not matter as long as both
  // operands hold the same ones.
  const uint32_t lds_base = (uint32_t)(size_t)(__attribute__((address_space(3))) unsigned char*)lds;
  uint32_t lo[2], wlo[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    lo[h] = lds_base + (uint32_t)(l16 * FTKB + (((4 * h + kq) ^ (l16 & 7)) * 16));
    wlo[h] = a.w_kslab ? lds_base + (uint32_t)((l16 >> 3) * 1024 + (((4 * h + kq) ^ (l16 >> 3)) * 128) + (l16 & 7) * 16)
                       : lo[h];
  }
  const uint32_t xwave = wm * (16 * NJ) * FTKB, wwave = X_BYTES + wn * (16 * NI) * FTKB;
  const uint32_t xsaddr = lds_base + X_BYTES + W_BYTES + (uint32_t)(wm * 64 + l16) * 4u;
  // The operands of one K block: two 16-byte halves per 16-row tile.  The x tiles and the
  // activation scales of this lane's four row tiles (rows wm * 64 + 16 j + l16) have two register
  // sets that swap roles every K block.  The w tiles of rows 0..2 have one: the MFMAs walk the w
  // tiles in order, so tile i is re-read for the next K block as soon as its four MFMAs are under
  // way; only the last w tile, in use until the end of the K block, has two sets.  (Two full sets
  // would need 128 registers of the 256 a wavefront has at two wavefronts per SIMD.)
  struct XOps { i4 bx[2][NJ]; float xs[NJ]; float ws; };
  typedef i4 WTile[2];
  auto read_x = [&](XOps& f, int h, int j, uint32_t stage_off) {
    const uint32_t xb = lo[h] + stage_off + xwave;
#pragma unroll
    for (int jj = 0; jj < NJ; ++jj)
      if (jj == j) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(f.bx[h][jj]) : "v"(xb), "n"(jj * 16 * FTKB));
  };
  auto read_w = [&](WTile& t, int i, uint32_t stage_off) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const uint32_t wb = wlo[h] + stage_off + wwave;
#pragma unroll
      for (int ii = 0; ii < NI; ++ii)
        if (ii == i) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(t[h]) : "v"(wb), "n"(ii * 16 * FTKB));
    }
  };
  auto read_xs = [&](XOps& f, uint32_t stage_off) {
    if (PC) return;
    const uint32_t ad = xsaddr + stage_off;
#pragma unroll
    for (int j = 0; j < NJ; ++j)
      asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(f.xs[j]) : "v"(ad), "n"(j * 64));
    asm volatile("ds_read_b32 %0, %1" : "=v"(f.ws) : "v"(lds_base + (uint32_t)(X_BYTES + W_BYTES + XS_BYTES) + stage_off));
  };
  WTile w012[3];
  auto lds_wait = [&](XOps& f, WTile& w3) {
    // every register the reads of a step write, exactly once each
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(f.bx[0][0]), "+v"(f.bx[0][1]), "+v"(f.bx[0][2]), "+v"(f.bx[0][3]), "+v"(f.bx[1][0]),
                   "+v"(f.bx[1][1]), "+v"(f.bx[1][2]), "+v"(f.bx[1][3]), "+v"(w012[0][0]), "+v"(w012[0][1]),
                   "+v"(w012[1][0]), "+v"(w012[1][1]), "+v"(w012[2][0]), "+v"(w012[2][1]), "+v"(w3[0]),
                   "+v"(w3[1]), "+v"(f.xs[0]), "+v"(f.xs[1]), "+v"(f.xs[2]), "+v"(f.xs[3]), "+v"(f.ws));
  };

  // One K block: one 128-deep MFMA per (w tile i, x tile j), started from zero; its result joins
  // the running sum with the block's scale two MFMAs later, when the matrix pipe has delivered it.
  // Between the MFMAs: the operand and scale reads of the next K block (a w tile one MFMA after
  // the last one that used it) and the copy slots of the K block three ahead.
  auto step = [&](const XOps& cur, XOps& nxt, const WTile& w3cur, WTile& w3nxt, uint32_t rso, int cstage, int kt) {
    float sc[NJ];
#pragma unroll
    for (int j = 0; j < NJ; ++j) sc[j] = cur.xs[j] * cur.ws;
    f4 ring[4];
    const bool odd_slots = wave < 4;
    int n = 0;
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const i4 a0 = i < 3 ? w012[i < 3 ? i : 0][0] : w3cur[0], a1 = i < 3 ? w012[i < 3 ? i : 0][1] : w3cur[1];
        const i8v av = __builtin_shufflevector(a0, a1, 0, 1, 2, 3, 4, 5, 6, 7);
        const i8v bv = __builtin_shufflevector(cur.bx[0][j], cur.bx[1][j], 0, 1, 2, 3, 4, 5, 6, 7);
        if constexpr (OP16) {
          if constexpr (DT == MI355Q_F16) {
            acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(bitcast<h8>(a0), bitcast<h8>(cur.bx[0][j]), acc[i][j], 0, 0, 0);
            acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(bitcast<h8>(a1), bitcast<h8>(cur.bx[1][j]), acc[i][j], 0, 0, 0);
          } else {
            acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(bitcast<b8>(a0), bitcast<b8>(cur.bx[0][j]), acc[i][j], 0, 0, 0);
            acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(bitcast<b8>(a1), bitcast<b8>(cur.bx[1][j]), acc[i][j], 0, 0, 0);
          }
        } else if (PC) acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(av, bv, acc[i][j], 0, 0, 0, 0, 0, 0);
        else ring[n & 3] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(av, bv, (f4){0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
        if (!PC && n >= 2) {
          const int pn = n - 2;
          acc[pn / NJ][pn % NJ] += sc[pn % NJ] * ring[pn & 3];
          // (pinned here: left alone, the compiler gives every MFMA a result tile of its own and sinks all
          // sixty-four multiply-adds behind the last MFMA, where the matrix pipe waits for them)
          asm volatile("" : "+v"(acc[pn / NJ][pn % NJ]));
        }
        __builtin_amdgcn_sched_barrier(0);
        if (n == 0) read_w(w3nxt, 3, rso);
        if (n == 4) read_w(w012[0], 0, rso);
        if (n == 8) read_w(w012[1], 1, rso);
        if (n == 12) read_w(w012[2], 2, rso);
        // x tiles: one read after each of MFMAs 1 2 3, 5 6 7, 9 10; the scales after 13
        if ((n & 3) != 0 && n < 11) {
          const int r = n - 1 - (n >> 2);             // 0..7
          read_x(nxt, r >> 2, r & 3, rso);
        }
        if (n == 13) read_xs(nxt, rso);
        // copy slot k after MFMA 2 k + 1 in wavefronts 0..3, after MFMA 2 k + 2 in wavefronts 4..7: the
        // address unit takes one copy (1 KiB) at a time, and eight in the same cycle queue up
        if (n >= 1 && n <= 2 * NSLOT && ((n & 1) != 0) == odd_slots) copy_slot((n - 1) >> 1, cstage, kt);
        __builtin_amdgcn_sched_barrier(0);
        ++n;
      }
    if (!PC) {
#pragma unroll
      for (int pn = NI * NJ - 2; pn < NI * NJ; ++pn) acc[pn / NJ][pn % NJ] += sc[pn % NJ] * ring[pn & 3];
    }
  };
  static_assert(NI == 4 && NJ == 4 && NSLOT <= 8, "the read and copy schedule is written for 16 MFMAs per K block");

  // Stream of K blocks across this workgroup's output tiles, three LDS stages (element g in stage
  // g % 3).  Step g multiplies element g from registers, reads element g + 1 from LDS into the
  // other register set, and issues the copy of element g + 3 into g's stage (every wavefront
  // finished reading g before the barrier that opened the step).  The step ends when this
  // wavefront's copies of element g + 2 have landed -- those of g + 3 stay in flight -- and a
  // barrier makes that true for everybody's.
  const int nt = KB / ksplits;                     // K blocks per (output tile, K range)
  // (kept in a register: read through the dispatch packet it is fetched again in every iteration)
  const int gdim = __builtin_amdgcn_readfirstlane((int)gridDim.x);
  int tile = blockIdx.x;
  int copy_tile = tile;
  set_copy_tile(tile);
  // element (T + d) of the stream seen from K block T of `tile`: its K block, after moving the copy
  // offsets to its output tile; past the last output tile a harmless re-read that nobody consumes
  auto ahead_kt = [&](int T, int d) {
    int kt = T + d, ahead = 0;
    while (kt >= nt) { kt -= nt; ++ahead; }
    const int want = tile + ahead * gdim;
    if (want >= total_tiles) return nt - 1;
    if (want != copy_tile) { set_copy_tile(want); copy_tile = want; }
    return kt;
  };
  auto wait_all_but_last_step = [&]() {
    // copies per step and wavefront: 4 x + 2 w, and one of scales in wavefronts 0..4
    if (!PC && wave <= 4) __builtin_amdgcn_s_waitcnt(0x0f77);  // vmcnt(7)
    else __builtin_amdgcn_s_waitcnt(0x0f76);                   // vmcnt(6)
  };
#pragma unroll
  for (int d = 0; d < 3; ++d) {
    const int kt = ahead_kt(0, d);
#pragma unroll
    for (int s = 0; s < NSLOT; ++s) copy_slot(s, d, kt);
  }
  wait_all_but_last_step();                        // elements 0 and 1 landed
  __builtin_amdgcn_s_barrier();
  XOps o0 = {}, o1 = {};
  WTile w3a, w3b;
#pragma unroll
  for (int r = 0; r < 8; ++r) read_x(o0, r >> 2, r & 3, 0);
#pragma unroll
  for (int i = 0; i < 3; ++i) read_w(w012[i], i, 0);
  read_w(w3a, 3, 0);
  read_xs(o0, 0);
  lds_wait(o0, w3a);
  __builtin_amdgcn_s_barrier();                    // nobody still reads element 0 when step 0 overwrites its stage
  int st = 0;                                      // stage of the current element
  // One row tile in all (M <= 256) and none of its rows in this wavefront's share: the wavefront only
  // copies.  It keeps the workgroup's barriers and its own copy slots, and leaves the matrix pipe and
  // the LDS read port of its SIMD to the wavefront that has rows (65 .. 128 rows: half the wavefronts).
  if (GROUPED ? wm * (16 * NJ) >= a.block_rows : (mtiles == 1 && wm * (16 * NJ) >= M)) {
    for (; tile < total_tiles; tile += gdim) {
      for (int T = 0; T < nt; ++T) {
        const int kt = ahead_kt(T, 3);
#pragma unroll
        for (int s = 0; s < NSLOT; ++s) copy_slot(s, st, kt);
        wait_all_but_last_step();
        __builtin_amdgcn_s_barrier();
        st = st == 2 ? 0 : st + 1;
      }
    }
    __builtin_amdgcn_s_waitcnt(0x0f70);            // vmcnt(0)
    return;
  }
  for (; tile < total_tiles; tile += gdim) {
    int m0, n0;
    tile_origin(tile, m0, n0);
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
      for (int j = 0; j < NJ; ++j) acc[i][j] = (f4){0.f, 0.f, 0.f, 0.f};
    // two K blocks per iteration so that the register sets swap roles without copies
    for (int T = 0; T < nt; T += 2) {
      {
        const int kt = ahead_kt(T, 3);
        const int nst = st == 2 ? 0 : st + 1;
        step(o0, o1, w3a, w3b, (uint32_t)(nst * STAGE_BYTES), st, kt);
        lds_wait(o1, w3b);
        wait_all_but_last_step();
        __builtin_amdgcn_s_barrier();
        st = nst;
      }
      if (T + 1 < nt) {
        const int kt = ahead_kt(T + 1, 3);
        const int nst = st == 2 ? 0 : st + 1;
        step(o1, o0, w3b, w3a, (uint32_t)(nst * STAGE_BYTES), st, kt);
        lds_wait(o0, w3a);
        wait_all_but_last_step();
        __builtin_amdgcn_s_barrier();
        st = nst;
      } else {
        // odd number of K blocks: the next element sits in the other set, move it where the next tile expects it
        o0 = o1;
        w3a[0] = w3b[0];
        w3a[1] = w3b[1];
      }
    }

    // ---- epilogue: lane holds, per (w tile i, x tile j), output row m = .. + l16 and columns
    // n = .. + 4 kq + {0..3}
    if (ksplits > 1) {
      // split K: the fp32 sums of this K range, nothing else; bias (and the scales that live outside the
      // K sum) are the second launch's
      float* const part = a.partial + (long)(tile % ksplits) * M * N;
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const int m = m0 + wm * (16 * NJ) + j * 16 + l16;
        if (m >= M) continue;
#pragma unroll
        for (int i = 0; i < NI; ++i) *(f4*)(part + (long)m * N + n0 + wn * (16 * NI) + i * 16 + 4 * kq) = acc[i][j];
      }
      __builtin_amdgcn_s_waitcnt(0x0f70);          // vmcnt(0), as below
      continue;
    }
    if (GROUPED) {
      const int e = a.expert_ids[m0 / FTM];
      const bool foreign = e < 0 || e >= a.E;
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const int id = a.sorted_ids[(m0 / FTM) * a.block_rows + wm * (16 * NJ) + j * 16 + l16];
        if (id >= a.numel || id < 0) continue;
        const float rw = foreign ? 0.0f : (a.topk_weights ? a.topk_weights[id] : 1.0f);
#pragma unroll
        for (int i = 0; i < NI; ++i) {
          const int n = n0 + wn * (16 * NI) + i * 16 + 4 * kq;
          float v[4];
#pragma unroll
          for (int c = 0; c < 4; ++c) v[c] = foreign ? 0.0f : acc[i][j][c] * rw;
          u2 o;
          o.x = (uint32_t)Elem<DT>::from_f32(v[0]) | ((uint32_t)Elem<DT>::from_f32(v[1]) << 16);
          o.y = (uint32_t)Elem<DT>::from_f32(v[2]) | ((uint32_t)Elem<DT>::from_f32(v[3]) << 16);
          *(u2*)((uint16_t*)a.out + (long)id * a.ldo + n) = o;
        }
      }
      __builtin_amdgcn_s_waitcnt(0x0f70);          // vmcnt(0), as below
      continue;
    }
    float bia[NI][4];
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int n = n0 + wn * (16 * NI) + i * 16 + 4 * kq;
#pragma unroll
      for (int e = 0; e < 4; ++e) bia[i][e] = a.bias ? Elem<DT>::to_f32(((const uint16_t*)a.bias)[n + e]) : 0.0f;
    }
    float wsc[NI][4];
    if (PC) {
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        const int n = n0 + wn * (16 * NI) + i * 16 + 4 * kq;
#pragma unroll
        for (int e = 0; e < 4; ++e) wsc[i][e] = a.w_scale[(n + e) * a.ws_mul];
      }
    }
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const int m = m0 + wm * (16 * NJ) + j * 16 + l16;
      if (m >= M) continue;
      const float xsc = PC ? a.x_scale[(long)m * a.xs_mul] : 1.0f;
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        const int n = n0 + wn * (16 * NI) + i * 16 + 4 * kq;
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = plus_bias(PC ? scaled_sum(acc[i][j][e], xsc, wsc[i][e]) : acc[i][j][e], bia[i][e]);
        u2 o;
        o.x = (uint32_t)Elem<DT>::from_f32(v[0]) | ((uint32_t)Elem<DT>::from_f32(v[1]) << 16);
        o.y = (uint32_t)Elem<DT>::from_f32(v[2]) | ((uint32_t)Elem<DT>::from_f32(v[3]) << 16);
        *(u2*)((uint16_t*)a.out + (long)m * a.ldo + n) = o;
      }
    }
    // the stores above count in vmcnt too and need not finish in order with the copies: start the
    // next tile's counting from zero
    __builtin_amdgcn_s_waitcnt(0x0f70);            // vmcnt(0)
  }
  // no copy may still be writing LDS when the workgroup retires
  __builtin_amdgcn_s_waitcnt(0x0f70);              // vmcnt(0)
}

// Second launch of a split: the ranges' sums added in range order (run-to-run identical), then the epilogue.
template <int DT, bool PC>
__global__ void __launch_bounds__(256)
fp8_splitk_epilogue_kernel(F8Args a) {
  const long q = (long)blockIdx.x * 256 + threadIdx.x;     // 4 adjacent columns of one row
  const int nq = a.N / 4;
  if (q >= (long)a.M * nq) return;
  const int m = (int)(q / nq), n = (int)(q % nq) * 4;
  f4 acc = {0.f, 0.f, 0.f, 0.f};
  for (int s = 0; s < a.ksplits; ++s) acc += *(const f4*)(a.partial + ((long)s * a.M + m) * a.N + n);
  const float xsc = PC ? a.x_scale[(long)m * a.xs_mul] : 1.0f;
  float v[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const float b = a.bias ? Elem<DT>::to_f32(((const uint16_t*)a.bias)[n + e]) : 0.0f;
    v[e] = plus_bias(PC ? scaled_sum(acc[e], xsc, a.w_scale[(n + e) * a.ws_mul]) : acc[e], b);
  }
  u2 o;
  o.x = (uint32_t)Elem<DT>::from_f32(v[0]) | ((uint32_t)Elem<DT>::from_f32(v[1]) << 16);
  o.y = (uint32_t)Elem<DT>::from_f32(v[2]) | ((uint32_t)Elem<DT>::from_f32(v[3]) << 16);
  *(u2*)((uint16_t*)a.out + (long)m * a.ldo + n) = o;
}

// Activation block scales [rows, KB] -> K block major [KB, ld] for the tile kernel's copies: a workgroup's 256
// scales of a K block then lie side by side instead of one per cache line (every column tile of a row tile reads
// them again).
__global__ void __launch_bounds__(256)
fp8_scales_kmajor_kernel(const float* xs, float* out, int rows, int KB, long ld) {
  __shared__ float t[32][33];
  const int p0 = blockIdx.x * 32, k0 = blockIdx.y * 32;
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;       // 32 x 8
  for (int r = ty; r < 32; r += 8) {
    const int p = p0 + r, kb = k0 + tx;
    float v = 0.0f;
    if (p < rows && kb < KB) v = xs[(long)p * KB + kb];
    t[r][tx] = v;
  }
  __syncthreads();
  for (int r = ty; r < 32; r += 8) {
    const int kb = k0 + r, p = p0 + tx;
    if (p < rows && kb < KB) out[(long)kb * ld + p] = t[tx][r];
  }
}

int fp8_scales_kmajor_launch(const float* xs, float* out, int rows, int KB, long ld, hipStream_t st) {
  hipLaunchKernelGGL(fp8_scales_kmajor_kernel, dim3((unsigned)((rows + 31) / 32), (unsigned)((KB + 31) / 32)), dim3(256), 0, st,
                     xs, out, rows, KB, ld);
  MQ_LAUNCH_CHECK("fp8 gemm (scales, K block major)");
  return 0;
}

constexpr size_t F8_SPLITK_BYTES = (size_t)64 << 20;
constexpr size_t F8_WS_OFFSET = (size_t)1 << 20;     // the first MiB of a workspace belongs to the W4A16 arrival counters

// K ranges for a shape: as many as put about one 256 x 128 tile on every CU, each at least eight K
// blocks long, a divisor of the K block count, partial sums within 64 MiB.  1: no split.
int fp8_ksplits(int M, int N, int K) {
  const long cus = device_cu_count(), tiles = (long)((M + FTM - 1) / FTM) * (N / FTN);
  const int nt = K / FTKB;
  if (N % FTN != 0 || tiles < 1 || tiles * 2 > cus) return 1;
  long s = cus / tiles;
  if (s > 8) s = 8;
  if (s > nt / 8) s = nt / 8;
  while (s > 1 && (nt % s != 0 || (size_t)s * M * N * sizeof(float) > F8_SPLITK_BYTES)) --s;
  return s < 1 ? 1 : (int)s;
}

template <int DT, bool PC>
int launch_f8(const F8Args& a, hipStream_t st);

template <int DT, bool PC>
int launch_f8_splitk(const F8Args& a, int splits, void* workspace, hipStream_t st) {
  F8Args b = a;
  b.ksplits = splits;
  b.partial = (float*)((char*)workspace + F8_WS_OFFSET);
  if (int rc = launch_f8<DT, PC>(b, st)) return rc;
  const long quads = (long)a.M * (a.N / 4);
  hipLaunchKernelGGL((fp8_splitk_epilogue_kernel<DT, PC>), dim3((unsigned)((quads + 255) / 256)), dim3(256), 0, st, b);
  MQ_LAUNCH_CHECK("fp8 gemm (split-K epilogue)");
  return 0;
}

// Rows from which the tile kernel with K ranges side by side is ahead of the weight-streaming kernel,
// whose time grows with the rows (in steps at 17 and 33: its row tiles) while the split tile kernel's
// hardly does (measured, us at 16 / 24 / 32 / 40 / 64 rows, streaming against split: K 28672 N 8192
// 43/53/60/72/92 against 53/52/53/53/54; K 16384 N 7168 24/31/31/39/53 against 34/32/32/32/34; K 14336
// N 4096 17/21/25/32/45 against 20/21/21/21/23; K 7168 N 4096 9/12/14/18/25 against 16/16/17/17/18;
// K 8192 N 8192 14/18/19/23/30 against 23/23/22/23/24; K 8192 N 10240, three ranges, 23/29/33/42/55 against
// 31/31/31/32/33; K 4096 N 4096 7/9/10/13/16 against 15/15/15/16/17).
int fp8_split_min_rows(int N, int K, int splits) {
  (void)N;
  if (splits < 3) return 64;
  if (K >= 12288) return 24;
  if (K >= 7168) return 32;
  return 64;
}

// with a workspace that holds the plan's partial sums: K ranges side by side; else the plain launch
// bytes of the K block major copy of the activation scales (rows padded to whole 64-byte lines)
size_t fp8_scales_kmajor_bytes(long rows, int K) { return (size_t)((rows + 15) / 16 * 16) * (K / FTKB) * sizeof(float); }

template <int DT, bool PC>
int launch_f8_auto(F8Args& a, void* workspace, size_t workspace_bytes, hipStream_t st) {
  a.ksplits = 1;
  a.partial = nullptr;
  a.xs_t = nullptr;
  a.xs_ld = 0;
  const int splits = fp8_ksplits(a.M, a.N, a.K);
  const bool split = splits > 1 && workspace && workspace_bytes >= F8_WS_OFFSET + (size_t)splits * a.M * a.N * sizeof(float);
  // (it pays where many column tiles read a row tile's scales again: measured, us, K 8192 x N 28672 at M = 128 / 256 /
  // 2048: 75 / 97 / 549 -> 67 / 86 / 529; K 16384 x N 7168 at 2048 / 8192: 289 / 1063 -> 277 / 997; layers of fewer
  // tiles gain nothing and pay for the extra launch)
  const long ntiles = a.N / FTN, tiles = (long)((a.M + FTM - 1) / FTM) * ntiles;
  if (!PC && workspace && (ntiles >= 128 || tiles >= 384)) {
    // block scales: with room behind the partial sums, the activation scales are re-ordered K block major first
    const size_t off = F8_WS_OFFSET + (split ? (size_t)splits * a.M * a.N * sizeof(float) : 0);
    if (workspace_bytes >= off + fp8_scales_kmajor_bytes(a.M, a.K)) {
      float* xt = (float*)((char*)workspace + off);
      const long ld = (a.M + 15) / 16 * 16;
      if (int rc = fp8_scales_kmajor_launch(a.x_scale, xt, a.M, a.K / FTKB, ld, st)) return rc;
      a.xs_t = xt;
      a.xs_ld = ld;
    }
  }
  if (split) return launch_f8_splitk<DT, PC>(a, splits, workspace, st);
  return launch_f8<DT, PC>(a, st);
}

template <int DT, bool PC>
int launch_f8(const F8Args& a, hipStream_t st) {
  const int mtiles = (a.M + FTM - 1) / FTM, ntiles = a.N / FTN;
  F8Args b = a;
  const int ks = a.ksplits > 1 ? a.ksplits : 1;
  b.n_panels_swizzle = (ntiles % 8 == 0 && ks == 1) ? 1 : 0;
  const size_t shmem = 3 * (size_t)(FTM * FTKB + FTN * FTKB + FTM * 4 + 256);
  static hipError_t attr = hipFuncSetAttribute((const void*)fp8_block_gemm_kernel<DT, PC>,
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
  MQ_REQUIRE(attr == hipSuccess, "fp8 gemm: cannot reserve %zu bytes of LDS: %s", shmem, hipGetErrorString(attr));
  int grid = mtiles * ntiles * ks, cus = device_cu_count() / 8 * 8;
  if (cus >= 8 && grid > cus) grid = cus;
  hipLaunchKernelGGL((fp8_block_gemm_kernel<DT, PC>), dim3(grid), dim3(F8_THREADS), shmem, st, b);
  MQ_LAUNCH_CHECK("fp8 gemm");
  return 0;
}

template <int DT, bool OP16 = false>
int launch_f8_grouped(const F8Args& a, hipStream_t st) {
  const size_t shmem = 3 * (size_t)(FTM * FTKB + FTN * FTKB + FTM * 4 + 256);
  static hipError_t attr = hipFuncSetAttribute((const void*)fp8_block_gemm_kernel<DT, OP16, true, OP16>,
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
  MQ_REQUIRE(attr == hipSuccess, "moe_gemm(MFMA tiles): cannot reserve %zu bytes of LDS: %s", shmem, hipGetErrorString(attr));
  long grid = (long)a.max_blocks * (a.N / FTN);
  const long cus = device_cu_count();
  if (grid > cus) grid = cus;
  hipLaunchKernelGGL((fp8_block_gemm_kernel<DT, OP16, true, OP16>), dim3((unsigned)grid), dim3(F8_THREADS), shmem, st, a);
  MQ_LAUNCH_CHECK("moe_gemm(MFMA tiles)");
  return 0;
}

}  // namespace

// The fused-MoE grouped GEMM with 128 x 128 block scales on align blocks of 256 or 128 slot ids: the MFMA
// tile kernel above with its rows gathered through the ids (prefill token counts; smaller blocks take the
// weight-streaming kernel).  Arguments as mi355q_moe_gemm's; checked by the caller.
int fp8_block_grouped_launch(void* out, const void* a, const void* w, const float* a_scale, const float* w_scale,
                             const float* topk_weights, const int32_t* sorted_ids, const int32_t* expert_ids,
                             const int32_t* npp, int numel, int topk, int block_size, int max_blocks, int E, int K, int N,
                             int out_dtype, int w_kslab, hipStream_t st) {
  MQ_REQUIRE(N % 128 == 0 && K % 128 == 0, "moe_gemm(fp8 tiles): N=%d and K=%d must be multiples of 128", N, K);
  MQ_REQUIRE(block_size == 256 || block_size == 128, "moe_gemm(fp8 tiles): block_size=%d must be 128 or 256", block_size);
  MQ_REQUIRE(out_dtype == MI355Q_F16 || out_dtype == MI355Q_BF16, "moe_gemm(fp8 tiles): output dtype %d", out_dtype);
  MQ_REQUIRE(((size_t)numel / topk + 1) * K < ((size_t)1 << 32) && (size_t)N * K < ((size_t)1 << 32),
             "moe_gemm(fp8 tiles): activations and one expert's weights must each stay below 4 GiB");
  F8Args g = {};
  g.out = out; g.x = (const uint8_t*)a; g.w = (const uint8_t*)w; g.x_scale = a_scale; g.w_scale = w_scale;
  g.M = numel; g.N = N; g.K = K; g.ldx = K; g.ldw = K; g.ldo = N;
  g.w_kslab = w_kslab;
  g.ksplits = 1;
  g.sorted_ids = sorted_ids; g.expert_ids = expert_ids; g.npp = npp; g.topk_weights = topk_weights;
  g.numel = numel; g.topk = topk; g.E = E; g.max_blocks = max_blocks;
  g.block_rows = block_size;
  g.w_stride = (long)N * K;
  g.ws_stride = (long)(N / 128) * (K / 128);
  return out_dtype == MI355Q_F16 ? launch_f8_grouped<MI355Q_F16>(g, st) : launch_f8_grouped<MI355Q_BF16>(g, st);
}

// The same for unquantised fp16 / bf16 experts ([E, N, K] row-major, or the kslab order of 2-byte elements):
// out[id] = x[id / topk] . w[e]^T (times the routing weight), fp32 sums.
int half_grouped_tile_launch(void* out, const void* a, const void* w, const float* topk_weights,
                             const int32_t* sorted_ids, const int32_t* expert_ids, const int32_t* npp, int numel, int topk,
                             int block_size, int max_blocks, int E, int K, int N, int dtype, int w_kslab, hipStream_t st) {
  MQ_REQUIRE(N % 128 == 0 && K % 128 == 0, "moe_gemm(16-bit tiles): N=%d and K=%d must be multiples of 128", N, K);
  MQ_REQUIRE(block_size == 256 || block_size == 128, "moe_gemm(16-bit tiles): block_size=%d must be 128 or 256", block_size);
  MQ_REQUIRE(dtype == MI355Q_F16 || dtype == MI355Q_BF16, "moe_gemm(16-bit tiles): dtype %d", dtype);
  MQ_REQUIRE(((size_t)numel / topk + 1) * K * 2 < ((size_t)1 << 32) && (size_t)N * K * 2 < ((size_t)1 << 32),
             "moe_gemm(16-bit tiles): activations and one expert's weights must each stay below 4 GiB");
  F8Args g = {};
  g.out = out; g.x = (const uint8_t*)a; g.w = (const uint8_t*)w;
  g.M = numel; g.N = N; g.K = 2 * K; g.ldx = 2L * K; g.ldw = 2L * K; g.ldo = N;     // K and operand strides in bytes
  g.w_kslab = w_kslab ? 2 : 0;
  g.ksplits = 1;
  g.sorted_ids = sorted_ids; g.expert_ids = expert_ids; g.npp = npp; g.topk_weights = topk_weights;
  g.numel = numel; g.topk = topk; g.E = E; g.max_blocks = max_blocks;
  g.block_rows = block_size;
  g.w_stride = 2L * N * K;
  return dtype == MI355Q_F16 ? launch_f8_grouped<MI355Q_F16, true>(g, st) : launch_f8_grouped<MI355Q_BF16, true>(g, st);
}

}  // namespace mi355q

using namespace mi355q;

extern "C" size_t mi355q_fp8_gemm_workspace_bytes(int M, int N, int K) {
  if (M <= 0 || N <= 0 || K <= 0 || K % 128 != 0) return 0;
  const int s = fp8_ksplits(M, N, K);
  return s > 1 && M > fp8_split_min_rows(N, K, s) ? F8_WS_OFFSET + (size_t)s * M * N * sizeof(float) : 0;
}

extern "C" int mi355q_fp8_block_gemm(void* out, const void* x, const void* w, const float* x_scale,
                                     const float* w_scale, const void* bias, int M, int N, int K, long ldx,
                                     long ldw, long ldo, int out_dtype, void* stream) {
  return mi355q_fp8_block_gemm_ws(out, x, w, x_scale, w_scale, bias, M, N, K, ldx, ldw, ldo, out_dtype, nullptr, 0, stream);
}

extern "C" int mi355q_fp8_block_gemm_ws(void* out, const void* x, const void* w, const float* x_scale,
                                        const float* w_scale, const void* bias, int M, int N, int K, long ldx,
                                        long ldw, long ldo, int out_dtype, void* workspace, size_t workspace_bytes,
                                        void* stream) {
  MQ_REQUIRE(M >= 0 && N > 0 && K > 0, "fp8_block_gemm: bad shape M=%d N=%d K=%d", M, N, K);
  if (M == 0) return 0;
  MQ_REQUIRE(out && x && w && x_scale && w_scale, "fp8_block_gemm: null pointer");
  MQ_REQUIRE(K % 128 == 0 && N % 128 == 0, "fp8_block_gemm: K=%d and N=%d must be multiples of 128", K, N);
  const bool kslab = ldw == 0;
  MQ_REQUIRE(ldx % 16 == 0 && ldx >= K && (kslab || (ldw % 16 == 0 && ldw >= K)),
             "fp8_block_gemm: operand row strides (%ld, %ld) must be >= K and multiples of 16", ldx, ldw);
  MQ_REQUIRE((size_t)N * K < ((size_t)1 << 32) && (size_t)M * (K / 128) < ((size_t)1 << 32) &&
                 (size_t)256 * (size_t)ldx < ((size_t)1 << 32) && (size_t)128 * (size_t)(kslab ? K : ldw) < ((size_t)1 << 32),
             "fp8_block_gemm: operands too large for 32-bit tile offsets (M=%d N=%d K=%d)", M, N, K);
  MQ_REQUIRE(ldo >= N && ldo % 4 == 0, "fp8_block_gemm: output row stride %ld must be >= N and a multiple of 4", ldo);
  MQ_REQUIRE(out_dtype == MI355Q_F16 || out_dtype == MI355Q_BF16, "fp8_block_gemm: bad out dtype %d", out_dtype);
  F8Args a;
  a.out = out; a.x = (const uint8_t*)x; a.w = (const uint8_t*)w; a.x_scale = x_scale; a.w_scale = w_scale;
  a.bias = bias; a.M = M; a.N = N; a.K = K; a.ldx = ldx; a.ldw = ldw; a.ldo = ldo;
  a.w_kslab = kslab ? 1 : 0;
  a.n_panels_swizzle = 0;
  a.xs_mul = a.ws_mul = 0;
  if (out_dtype == MI355Q_F16) return launch_f8_auto<MI355Q_F16, false>(a, workspace, workspace_bytes, as_stream(stream));
  return launch_f8_auto<MI355Q_BF16, false>(a, workspace, workspace_bytes, as_stream(stream));
}

// fp8 x fp8 with per-token (or one) activation scale and per-channel (or one) weight scale, fp32
// accumulation over the whole of K:  out[m, n] = (sum_k x[m, k] w[n, k]) * x_scale[m] * w_scale[n] (+ bias[n])
extern "C" int mi355q_fp8_scaled_gemm(void* out, const void* x, const void* w, const float* x_scale,
                                      int x_scale_per_row, const float* w_scale, int w_scale_per_col,
                                      const void* bias, int M, int N, int K, long ldx, long ldw, long ldo,
                                      int out_dtype, void* stream) {
  return mi355q_fp8_scaled_gemm_ws(out, x, w, x_scale, x_scale_per_row, w_scale, w_scale_per_col, bias, M, N, K, ldx, ldw,
                                   ldo, out_dtype, nullptr, 0, stream);
}

extern "C" int mi355q_fp8_scaled_gemm_ws(void* out, const void* x, const void* w, const float* x_scale,
                                         int x_scale_per_row, const float* w_scale, int w_scale_per_col,
                                         const void* bias, int M, int N, int K, long ldx, long ldw, long ldo,
                                         int out_dtype, void* workspace, size_t workspace_bytes, void* stream) {
  MQ_REQUIRE(M >= 0 && N > 0 && K > 0, "fp8_scaled_gemm: bad shape M=%d N=%d K=%d", M, N, K);
  if (M == 0) return 0;
  MQ_REQUIRE(out && x && w && x_scale && w_scale, "fp8_scaled_gemm: null pointer");
  MQ_REQUIRE(K % 128 == 0 && N % 4 == 0, "fp8_scaled_gemm: K=%d must be a multiple of 128 and N=%d of 4", K, N);
  MQ_REQUIRE(out_dtype == MI355Q_F16 || out_dtype == MI355Q_BF16, "fp8_scaled_gemm: bad out dtype %d", out_dtype);
  const bool kslab = ldw == 0;
  MQ_REQUIRE(!kslab || N % 64 == 0, "fp8_scaled_gemm: weights in the kslab order need N=%d %% 64 == 0", N);
  MQ_REQUIRE(ldx >= K && (kslab || ldw >= K) && ldo >= N,
             "fp8_scaled_gemm: row strides (%ld, %ld, %ld) must cover K=%d / N=%d", ldx, ldw, ldo, K, N);
  // the MFMA tile kernel from 65 rows on when its 256 x 128 tiles fill a good part of the chip; below
  // (and for shapes it does not take) the weight-streaming kernel, which wants dense operands
  const long tiles = (long)((M + FTM - 1) / FTM) * (N / FTN);
  const bool tile_ok = N % 128 == 0 && ldx % 16 == 0 && (kslab || ldw % 16 == 0) && ldo % 4 == 0 &&
                       (size_t)N * K < ((size_t)1 << 32) && (size_t)256 * (size_t)ldx < ((size_t)1 << 32) &&
                       (size_t)128 * (size_t)(kslab ? K : ldw) < ((size_t)1 << 32);
  const bool stream_ok = ldx == K && (kslab || ldw == K) && ldo == N && (size_t)N * K * 2 < ((size_t)1 << 32) &&
                         (size_t)M * K * 2 < ((size_t)1 << 32);
  // (from 33 rows on layers of 128 tiles or more: the wavefronts without rows only copy there)
  // (and, with a workspace, wherever the split plan asks for one: K ranges side by side fill the chip)
  const size_t split_bytes = mi355q_fp8_gemm_workspace_bytes(M, N, K);
  const bool split_ok = tile_ok && workspace && split_bytes > 0 && workspace_bytes >= split_bytes;
  if (tile_ok && ((M > 64 && tiles >= 64) || (M > 32 && tiles >= 128) || split_ok || !stream_ok)) {
    F8Args a;
    a.out = out; a.x = (const uint8_t*)x; a.w = (const uint8_t*)w; a.x_scale = x_scale; a.w_scale = w_scale;
    a.bias = bias; a.M = M; a.N = N; a.K = K; a.ldx = ldx; a.ldw = ldw; a.ldo = ldo;
    a.w_kslab = kslab ? 1 : 0;
    a.n_panels_swizzle = 0;
    a.xs_mul = x_scale_per_row ? 1 : 0;
    a.ws_mul = w_scale_per_col ? 1 : 0;
    if (out_dtype == MI355Q_F16) return launch_f8_auto<MI355Q_F16, true>(a, workspace, workspace_bytes, as_stream(stream));
    return launch_f8_auto<MI355Q_BF16, true>(a, workspace, workspace_bytes, as_stream(stream));
  }
  MQ_REQUIRE(stream_ok, "fp8_scaled_gemm: M=%d N=%d K=%d with row strides (%ld, %ld, %ld) fits neither kernel "
             "(dense operands, or N %% 128 == 0 with strides that are multiples of 16)", M, N, K, ldx, ldw, ldo);
  // the streaming kernel covers 64 rows (128 on narrow layers) per pass over the weights
  return kcontig_fp8_pc_launch(out, x, w, x_scale, x_scale_per_row, w_scale, w_scale_per_col, bias, M, K, N, out_dtype,
                               kslab ? 1 : 0, as_stream(stream));
}
