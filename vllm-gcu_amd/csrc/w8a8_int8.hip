// W8A8 int8 GEMM on the gfx950 int8 MFMA (v_mfma_i32_16x16x64_i8) with the
// per-token x per-channel scales (and bias) fused into the epilogue, plus the
// per-token / static int8 activation quantisers that feed it.
//
// GEMM: out[M, N] = (xq[M, K] . wq[N, K]^T in int32) * x_scale[m] * w_scale[n].
// Both operands are K-contiguous (that is what the MFMA lanes consume: 16
// consecutive k per lane).  A workgroup of eight wavefronts owns a 256 x TN
// output tile, TN = 256 (2 x 4 wavefronts of 128 x 64) or 224 (4 x 2 wavefronts
// of 64 x 112; 28672 = 128 x 224, so the Llama-3-70B MLP shape makes exactly
// four full rounds of 256 workgroups).  K advances in LDS tiles of 128 bytes
// per row: a whole 128-byte line per row and request, which halves the L2
// request count of a 64-byte tile (the L2 was the busiest unit).  Tiles go
// from global memory straight into LDS (global_load ... lds, 16 B per lane, no
// staging registers) with a 16-byte-chunk XOR swizzle that keeps the 128-bit
// operand reads bank-conflict free.  Two LDS stages and two register sets of
// operands: while half a tile (k = 64) is multiplied, the next half's operands
// are read from LDS, and the copy of the tile after next is in flight.  The
// weights take the A operand slot so that each lane ends up with 4 consecutive
// output columns (one 8-byte store).
#include "common.h"

namespace mi355q {
namespace {

constexpr int TM = 256, TKB = 128;                // tile rows of x, bytes of K per LDS tile row
constexpr int GEMM_THREADS = 512;

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
  long ldacc;               // row stride of acc_out (elements)
  int x_scale_per_row, w_scale_per_col, bias_f32;
  int n_panels_swizzle;     // non-zero: XCD-aware tile order
  int w_kslab;              // w is in the kslab order (see include/mi355q.h) instead of row-major
  int wide_stores;          // N, ldo and the output address allow 16-byte stores of 8 adjacent 16-bit outputs
  int ksplits;              // > 1: every output tile is worked on by `ksplits` workgroups, each a K range of its own,
  int32_t* partial;         //      which leave their int32 sums in partial[split][M][N]; the epilogue is a second launch
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

// WM x WN wavefronts, each NJ x NI MFMA tiles of 16 x 16 (rows of x by rows of w)
// GROUPED: the fused-MoE grouped GEMM at prefill token counts.  Row tile b is align block b (256 slot
// ids of expert expert_ids[b]): x rows are gathered through the ids (row id / topk), weights and
// weight scales are the expert's, output row id gets the result times x_scale of its row, the
// expert's w_scale and its routing weight.  Blocks past num_tokens_post_pad do not exist (the tile
// count is read on the device); a block of an expert outside [0, E) writes zeros.  No K ranges, no bias.
template <int DT, int WM, int WN, int NI, int NJ, bool GROUPED = false>
__global__ void __launch_bounds__(GEMM_THREADS, 1)
w8a8_int8_gemm_kernel(I8Args a) {
  static_assert(WM * WN == 8 && WM * NJ * 16 == TM, "eight wavefronts cover 256 rows of x");
  constexpr int TN = WN * NI * 16;
  constexpr int X_BYTES = TM * TKB, W_BYTES = TN * TKB, STAGE_BYTES = X_BYTES + W_BYTES;
  // LDS stages: three where they fit (the 128-column tile: 3 x 48 KiB), else two
  constexpr int STAGES = 3 * STAGE_BYTES <= 160 * 1024 ? 3 : 2;
  constexpr int XCOPIES = TM / 8 / 8;                   // 1 KiB copies (8 rows) per wavefront, x tile
  constexpr int WGROUPS = TN / 8;                       // 8-row groups of the w tile
  constexpr int WCOPIES = (WGROUPS + 7) / 8;
  extern __shared__ __align__(16) unsigned char lds[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l16 = lane & 15, kq = lane >> 4;
  const int wm = wave / WN, wn = wave % WN;
  const int M = a.M, N = a.N, K = a.K;

  // Persistent workgroups: workgroup w takes output tiles w, w + grid, ...
  // Tile coordinates: with the swizzle, the tiles whose id is congruent mod 8
  // (they run on one XCD, the grid being a multiple of 8) sweep all row tiles
  // of the same weight panels.
  int mtiles = (M + TM - 1) / TM;
  if (GROUPED) {
    const int blocks = (*a.npp + a.block_rows - 1) / a.block_rows;
    mtiles = __builtin_amdgcn_readfirstlane(blocks < a.max_blocks ? blocks : a.max_blocks);
  }
  const int ntiles_n = (N + TN - 1) / TN;
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
    m0 = tm * TM;
    n0 = tn * TN;
  };

  i4 acc[NI][NJ];    // [n tile][m tile]: weights are the MFMA "A" operand

  // global -> LDS.  One copy moves 8 tile rows of 128 bytes: lane = 8 * row +
  // slot, and slot p of row r receives the row's 16-byte chunk p ^ (r & 7), so
  // that the operand reads below (16 rows x 4 chunks per instruction) spread
  // over all banks.  8 consecutive lanes fetch one whole 128-byte line.
  // Wavefront v copies row groups v, v + 8, ...; rows past the matrix edge
  // re-read the last row (their results are never stored).
  const int crow = lane >> 3, cchunk = (lane & 7) ^ (crow & 7);
  uint32_t xo[XCOPIES], wo[WCOPIES];
  const int8_t *xtile, *wtile;
  auto set_copy_tile = [&](int tile) {         // the output tile whose operands the copies fetch
    int m0, n0;
    tile_origin(tile, m0, n0);
    long ebytes = 0;
    if (GROUPED) {
      const int* ids = a.sorted_ids + (m0 / TM) * a.block_rows;
#pragma unroll
      for (int p = 0; p < XCOPIES; ++p) {
        // (blocks of 128: the upper half of the tile copies the lower half's rows once more; nobody multiplies them)
        const int id = ids[((wave + 8 * p) * 8 + crow) & (a.block_rows - 1)];
        xo[p] = (uint32_t)(max(0, min(id, a.numel - 1)) / a.topk) * (uint32_t)a.ldx + (uint32_t)(16 * cchunk);   // pads read a valid row
      }
      int e = a.expert_ids[m0 / TM];
      e = __builtin_amdgcn_readfirstlane((e < 0 || e >= a.E) ? 0 : e);     // (a foreign expert's block is computed and zeroed)
      ebytes = (long)e * a.w_stride;
    } else {
#pragma unroll
      for (int p = 0; p < XCOPIES; ++p) {
        const int r = (wave + 8 * p) * 8 + crow;
        xo[p] = (uint32_t)((min(m0 + r, M - 1) - m0) * a.ldx + 16 * cchunk);
      }
    }
#pragma unroll
    for (int p = 0; p < WCOPIES; ++p) {
      const int r = (wave + 8 * p) * 8 + crow;
      if (a.w_kslab) {
        // kslab: [N/64][K/128][4 tiles of 16 rows][2 vectors][64 lanes = 16 rows x 4 segments][16 B].
        // One chunk of 8 consecutive rows is 128 contiguous bytes there, so lane = 8 * position +
        // row: 8 consecutive lanes again fetch one whole line, and LDS holds the group chunk-major,
        // position p of an odd group holding chunk p ^ 1 (see the operand reads).
        const uint32_t n = (uint32_t)min(n0 + (wave + 8 * p) * 8 + (lane & 7), N - 1);
        const uint32_t c = (uint32_t)((lane >> 3) ^ (wave & 1));
        wo[p] = ((n >> 6) * (uint32_t)(K >> 7) * 4u + ((n & 63u) >> 4)) * 2048u + (c & 1u) * 1024u +
                ((c >> 1) * 16u + (n & 15u)) * 16u;
      } else {
        wo[p] = (uint32_t)((min(n0 + r, N - 1) - n0) * a.ldw + 16 * cchunk);
      }
    }
    // (split K: the tile's K range starts kbeg bytes into every row; 64 kslab rows interleave their K tiles)
    const long kbeg = ksplits > 1 ? (long)(tile % ksplits) * (K / ksplits) : 0;
    xtile = GROUPED ? a.x : a.x + (long)m0 * a.ldx + kbeg;
    wtile = a.w + ebytes + (a.w_kslab ? kbeg * 64 : (long)n0 * a.ldw + kbeg);
  };
  // copy slot s of this wavefront: slots 0 .. XCOPIES-1 are its x row groups,
  // the rest its w row groups (the last one only exists for some wavefronts)
  constexpr int NSLOT = XCOPIES + WCOPIES;
  auto copy_slot = [&](int s, int stage, int k0) {
    unsigned char* xs = lds + stage * STAGE_BYTES;
    if (s < XCOPIES) {
      dma16(xtile + k0 + xo[s], xs + (wave + 8 * s) * 1024);
    } else {
      const int p = s - XCOPIES;
      // a K tile of 128 bytes per row is 8 KiB further on in the kslab order
      if (wave + 8 * p < WGROUPS)
        dma16(wtile + (a.w_kslab ? (long)k0 * 64 : (long)k0) + wo[p < WCOPIES ? p : 0], xs + X_BYTES + (wave + 8 * p) * 1024);
    }
  };
  auto issue = [&](int stage, int k0) {
#pragma unroll
    for (int s = 0; s < NSLOT; ++s) copy_slot(s, stage, k0);
  };

  // Operand reads: lane (l16, kq) of half h takes chunk 4 h + kq of row l16 of
  // each 16-row MFMA tile.  They are written in assembly and waited for by
  // hand: with a direct-to-LDS copy in flight the compiler turns every wait it
  // inserts itself into "wait for everything", which would serialise the
  // reads of the next operands with the MFMAs of the current ones; reads it
  // cannot see need no wait of its own.  lds_wait ties the registers to the
  // wait so that their first use cannot move above it.
  const uint32_t lds_base = (uint32_t)(size_t)(__attribute__((address_space(3))) unsigned char*)lds;
  uint32_t lo[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) lo[h] = lds_base + (uint32_t)(l16 * TKB + (((4 * h + kq) ^ (l16 & 7)) * 16));
  // kslab weights lie chunk-major in LDS: 8-row group, then chunk position (chunk ^ 1 in odd
  // groups, so that the two groups of a 16-row tile fall on different banks), then row
  uint32_t wlo[2];
#pragma unroll
  for (int h = 0; h < 2; ++h)
    wlo[h] = a.w_kslab ? lds_base + (uint32_t)((l16 >> 3) * 1024 + (((4 * h + kq) ^ (l16 >> 3)) * 128) + (l16 & 7) * 16)
                       : lo[h];
  const uint32_t xwave = wm * (16 * NJ) * TKB, wwave = X_BYTES + wn * (16 * NI) * TKB;
  struct Frag { i4 bx[NJ]; i4 aw[NI]; };
  // read r of an operand set: r < NJ is x tile r, the rest are w tiles
  auto read_one = [&](Frag& f, int r, uint32_t xb, uint32_t wb) {
#pragma unroll
    for (int j = 0; j < NJ; ++j)
      if (r == j) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(f.bx[j]) : "v"(xb), "n"(j * 16 * TKB));
#pragma unroll
    for (int i = 0; i < NI; ++i)
      if (r == NJ + i) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(f.aw[i]) : "v"(wb), "n"(i * 16 * TKB));
  };
  auto read_frag = [&](Frag& f, int stage, int h) {
    const uint32_t xb = lo[h] + (uint32_t)(stage * STAGE_BYTES) + xwave;
    const uint32_t wb = wlo[h] + (uint32_t)(stage * STAGE_BYTES) + wwave;
#pragma unroll
    for (int r = 0; r < NJ + NI; ++r) read_one(f, r, xb, wb);
  };
  auto lds_wait = [&](Frag& f) {
    // "s_waitcnt lgkmcnt(0)" with every operand register as an in/out operand
    // (each register exactly once: a duplicate would come back as a stale copy)
    static_assert((NJ == 8 && NI == 4) || (NJ == 4 && NI == 7) || (NJ == 4 && NI == 4), "operand lists are written out");
    if constexpr (NJ == 4 && NI == 4) {
      asm volatile("s_waitcnt lgkmcnt(0)"
                   : "+v"(f.bx[0]), "+v"(f.bx[1]), "+v"(f.bx[2]), "+v"(f.bx[3]), "+v"(f.aw[0]), "+v"(f.aw[1]),
                     "+v"(f.aw[2]), "+v"(f.aw[3]));
    } else if constexpr (NJ == 8) {
      asm volatile("s_waitcnt lgkmcnt(0)"
                   : "+v"(f.bx[0]), "+v"(f.bx[1]), "+v"(f.bx[2]), "+v"(f.bx[3]), "+v"(f.bx[4]), "+v"(f.bx[5]),
                     "+v"(f.bx[6]), "+v"(f.bx[7]), "+v"(f.aw[0]), "+v"(f.aw[1]), "+v"(f.aw[2]), "+v"(f.aw[3]));
    } else {
      asm volatile("s_waitcnt lgkmcnt(0)"
                   : "+v"(f.bx[0]), "+v"(f.bx[1]), "+v"(f.bx[2]), "+v"(f.bx[3]), "+v"(f.aw[0]), "+v"(f.aw[1]),
                     "+v"(f.aw[2]), "+v"(f.aw[3]), "+v"(f.aw[4]), "+v"(f.aw[5]), "+v"(f.aw[6]));
    }
  };
  // One half: the MFMAs of `cur`, and between them (a) the LDS reads of the
  // next operand set `nxt`, one after each of the first MFMAs, and (b) copy
  // slots SB .. SE-1 of a later tile, the first after MFMA C0 and then one
  // every CE MFMAs.  Everything a wavefront has to issue besides MFMAs is
  // spread out like this on purpose: the eight wavefronts run in lockstep
  // behind the workgroup barrier, so a phase of reads or copies of its own
  // would idle the matrix pipes of the whole CU (a burst of copies also blocks
  // every wavefront in the address unit, 64 B/clk per CU).
  constexpr int RE = 2;                             // one LDS read every RE MFMAs (1 and 3 were measured: slower)
  auto half = [&](const Frag& cur, Frag& nxt, int rstage, int rh, int SB, int SE, int C0, int CE,
                  int cstage, int k0) {
    const uint32_t xb = lo[rh] + (uint32_t)(rstage * STAGE_BYTES) + xwave;
    const uint32_t wb = wlo[rh] + (uint32_t)(rstage * STAGE_BYTES) + wwave;
    int n = 0;
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(cur.aw[i], cur.bx[j], acc[i][j], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        if (n % RE == 0 && n / RE < NJ + NI) read_one(nxt, n / RE, xb, wb);
        if (n >= C0 && (n - C0) % CE == 0 && SB + (n - C0) / CE < SE) copy_slot(SB + (n - C0) / CE, cstage, k0);
        __builtin_amdgcn_sched_barrier(0);
        ++n;
      }
  };
  constexpr int NM = NI * NJ;
  // copy slots: the first after MFMA C0, then one every CE MFMAs (closer together in the narrow tile)
  constexpr int CP0 = NM >= 24 ? 3 : 1, CPE = NM >= 24 ? 3 : 2;
  static_assert(NM > CP0 + CPE * (NSLOT - 1) && NM >= RE * (NJ + NI), "not enough MFMAs to spread the copies and reads");

  // The K tiles of all the output tiles of this workgroup form one stream;
  // stream element g lives in LDS stage g % STAGES.  Half 0 of element g multiplies
  // (g, 0) while it reads (g, 1); half 1 multiplies (g, 1) while it reads
  // (g + 1, 0) and issues the copy of element g + STAGES into g's stage.  The
  // barrier between the halves means: everybody's copies of element g + 1 have
  // landed, and everybody has finished reading element g.  With two stages that
  // is a wait for every copy of this wavefront; with three the copies of
  // element g + 2, issued one element ago, stay in flight (the wait leaves the
  // last NSLOT: every wavefront issues exactly NSLOT copies per element there).
  // The stream runs across output tiles, so the first K tiles of the next
  // output tile arrive while the epilogue of this one runs; past the last
  // output tile the copies re-read its last K tile into a stage nobody reads.
  static_assert(STAGES == 2 || (WCOPIES * 8 == WGROUPS && NSLOT == 6), "the three-stage wait counts six copies per wavefront and element");
  const int nt = K / TKB / ksplits;                // K tiles per (output tile, K range)
  // (kept in a register: read through the dispatch packet it is fetched again in every iteration)
  const int gdim = __builtin_amdgcn_readfirstlane((int)gridDim.x);
  int tile = blockIdx.x;
  int copy_tile = tile;
  set_copy_tile(tile);
  // K tile of the element d ahead of K tile T of `tile`, after moving the copy offsets to its
  // output tile; past the last output tile a harmless re-read that is never consumed
  auto ahead_k0 = [&](int T, int d) {
    int kt = T + d, ahead = 0;
    while (kt >= nt) { kt -= nt; ++ahead; }
    const int want = tile + ahead * gdim;
    if (want >= total_tiles) return (nt - 1) * TKB;
    if (want != copy_tile) { set_copy_tile(want); copy_tile = want; }
    return kt * TKB;
  };
  auto wait_landed = [&]() {
    if constexpr (STAGES == 3) __builtin_amdgcn_s_waitcnt(0x0f76);   // vmcnt(6): all but the newest element
    else __builtin_amdgcn_s_waitcnt(0x0f70);                          // vmcnt(0)
  };
#pragma unroll
  for (int d = 0; d < STAGES; ++d) issue(d, ahead_k0(0, d));
  if constexpr (STAGES == 3) __builtin_amdgcn_s_waitcnt(0x0f7c);     // vmcnt(12): element 0 landed
  else __builtin_amdgcn_s_waitcnt(0x0f70);
  __builtin_amdgcn_s_barrier();
  int st = 0;                                      // stage of the current K tile
  // One row tile in all (M <= 256) and none of its rows in this wavefront's share: the wavefront only
  // copies.  It keeps the workgroup's barriers and its own copy slots, and leaves the matrix pipe and
  // the LDS read port of its SIMD to the wavefront that has rows (65 .. 128 rows: half the wavefronts).
  if (GROUPED ? wm * (16 * NJ) >= a.block_rows : (mtiles == 1 && wm * (16 * NJ) >= M)) {
    for (; tile < total_tiles; tile += gdim) {
      for (int T = 0; T < nt; ++T) {
        wait_landed();
        __builtin_amdgcn_s_barrier();
        issue(st, ahead_k0(T, STAGES));
        st = st + 1 == STAGES ? 0 : st + 1;
      }
    }
    __builtin_amdgcn_s_waitcnt(0x0f70);            // vmcnt(0)
    return;
  }
  Frag f0, f1;
  read_frag(f0, 0, 0);
  lds_wait(f0);
  for (; tile < total_tiles; tile += gdim) {
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
      for (int j = 0; j < NJ; ++j) acc[i][j] = (i4){0, 0, 0, 0};
    for (int T = 0; T < nt; ++T) {
      const int nst = st + 1 == STAGES ? 0 : st + 1;
      half(f0, f1, st, 1, 0, 0, 0, 1, st, 0);
      lds_wait(f1);
      wait_landed();                               // my copies of the next element landed
      __builtin_amdgcn_s_barrier();                // bare barrier: the waits are explicit, no fence needed
      const int k0 = ahead_k0(T, STAGES);
      half(f1, f0, nst, 0, 0, NSLOT, CP0, CPE, st, k0);
      lds_wait(f0);
      st = nst;
    }

    // ---- epilogue: lane holds, per (n tile i, m tile j), output row
    // m = .. + l16 and columns n = .. + 4 kq + {0..3}.  Every scale and bias
    // value the lane needs is loaded before the first store: the compiler must
    // assume the output may alias them, so loads placed between the stores
    // would each wait out a full memory round trip.
    int m0, n0;
    tile_origin(tile, m0, n0);
    if (ksplits > 1) {
      // split K: the int32 sums of this K range, nothing else; scales and bias are the second launch's
      int32_t* const part = a.partial + (long)(tile % ksplits) * M * N;
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const int m = m0 + wm * (16 * NJ) + j * 16 + l16;
        if (m >= M) continue;
#pragma unroll
        for (int i = 0; i < NI; ++i) {
          const int n = n0 + wn * (16 * NI) + i * 16 + 4 * kq;
          if (n < N) *(i4*)(part + (long)m * N + n) = acc[i][j];
        }
      }
      if constexpr (STAGES == 3) __builtin_amdgcn_s_waitcnt(0x0f70);
      read_frag(f0, st, 0);
      lds_wait(f0);
      continue;
    }
    if (GROUPED) {
      const int e = a.expert_ids[m0 / TM];
      const bool foreign = e < 0 || e >= a.E;
      const float* wsp = a.w_scale + (long)(foreign ? 0 : e) * a.ws_stride;
      float wsg[NI][4];
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        const int n = min(n0 + wn * (16 * NI) + i * 16 + 4 * kq, N - 4);
#pragma unroll
        for (int c = 0; c < 4; ++c) wsg[i][c] = wsp[n + c];
      }
      int idj[NJ];
      float xsg[NJ], rwg[NJ];
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const int id = a.sorted_ids[(m0 / TM) * a.block_rows + wm * (16 * NJ) + j * 16 + l16];
        const bool live = id >= 0 && id < a.numel;
        idj[j] = live ? id : -1;
        xsg[j] = a.x_scale[a.x_scale_per_row ? (live ? id / a.topk : 0) : 0];
        rwg[j] = foreign ? 0.0f : ((live && a.topk_weights) ? a.topk_weights[id] : 1.0f);
      }
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        if (idj[j] < 0) continue;
#pragma unroll
        for (int i = 0; i < NI; ++i) {
          const int n = n0 + wn * (16 * NI) + i * 16 + 4 * kq;
          if (n >= N) continue;
          float v[4];
#pragma unroll
          for (int c = 0; c < 4; ++c) v[c] = foreign ? 0.0f : scaled_sum((float)acc[i][j][c], xsg[j], wsg[i][c]) * rwg[j];
          store4<DT>(a.out, (long)idj[j] * a.ldo + n, v);
        }
      }
      if constexpr (STAGES == 3) __builtin_amdgcn_s_waitcnt(0x0f70);
      read_frag(f0, st, 0);
      lds_wait(f0);
      continue;
    }
    float xsc[NJ];
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const int m = min(m0 + wm * (16 * NJ) + j * 16 + l16, M - 1);
      xsc[j] = a.x_scale ? a.x_scale[a.x_scale_per_row ? m : 0] : 1.0f;
    }
    float wsc[NI][4], bia[NI][4];
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int n = min(n0 + wn * (16 * NI) + i * 16 + 4 * kq, N - 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        wsc[i][e] = a.w_scale ? a.w_scale[a.w_scale_per_col ? n + e : 0] : 1.0f;
        bia[i][e] = a.bias ? load_bias<DT>(a.bias, a.bias_f32, n + e) : 0.0f;
      }
    }
    // 16-bit outputs leave in 16-byte pieces where the layout allows: the lanes of a row that hold
    // columns 4 kq .. 4 kq + 3 of two neighbouring column tiles trade halves (v_permlane16_swap:
    // lanes 16..31 of the first register with lanes 0..15 of the second, likewise 48..63 with
    // 32..47), after which lane kq holds 8 adjacent columns of tile i + (kq & 1) -- a store
    // instruction then writes 64 contiguous bytes per row instead of 32
    const bool wide = DT != MI355Q_F32 && a.wide_stores;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const int m = m0 + wm * (16 * NJ) + j * 16 + l16;
      if (m >= M) continue;
      auto scaled = [&](int i, float* v) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          v[e] = scaled_sum((float)acc[i][j][e], xsc[j], wsc[i][e]);
          if (a.bias) v[e] = plus_bias(v[e], bia[i][e]);
        }
      };
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        const int n = n0 + wn * (16 * NI) + i * 16 + 4 * kq;
        if (a.acc_out && n < N) *(i4*)(a.acc_out + (long)m * a.ldacc + n) = acc[i][j];
        if (DT != MI355Q_F32 && wide && (i & 1) == 0 && i + 1 < NI) {
          typedef Elem<DT == MI355Q_F32 ? MI355Q_F16 : DT> E;
          float v0[4], v1[4];
          scaled(i, v0);
          scaled(i + 1, v1);
          uint32_t p[2][2];
          p[0][0] = (uint32_t)E::from_f32(v0[0]) | ((uint32_t)E::from_f32(v0[1]) << 16);
          p[0][1] = (uint32_t)E::from_f32(v0[2]) | ((uint32_t)E::from_f32(v0[3]) << 16);
          p[1][0] = (uint32_t)E::from_f32(v1[0]) | ((uint32_t)E::from_f32(v1[1]) << 16);
          p[1][1] = (uint32_t)E::from_f32(v1[2]) | ((uint32_t)E::from_f32(v1[3]) << 16);
          const auto lo2 = __builtin_amdgcn_permlane16_swap(p[0][0], p[1][0], false, false);
          const auto hi2 = __builtin_amdgcn_permlane16_swap(p[0][1], p[1][1], false, false);
          const int nw = n0 + wn * (16 * NI) + (i + (kq & 1)) * 16 + 8 * (kq >> 1);
          if (nw < N) *(u4*)((uint16_t*)a.out + (long)m * a.ldo + nw) = (u4){lo2[0], hi2[0], lo2[1], hi2[1]};
        } else if (!(DT != MI355Q_F32 && wide && (i & 1) == 1)) {
          if (n >= N) continue;                     // N is a multiple of 4
          float v[4];
          scaled(i, v);
          store4<DT>(a.out, (long)m * a.ldo + n, v);
        }
      }
    }
    // The operands of the next output tile's first half are read again here
    // rather than kept from the last half above: that frees their registers
    // for the epilogue (the copy has landed: it was waited for at the last
    // barrier of the K loop).
    if constexpr (STAGES == 3) __builtin_amdgcn_s_waitcnt(0x0f70);   // the stores counted too: start again from zero
    read_frag(f0, st, 0);
    lds_wait(f0);
  }
  // no copy may still be writing LDS when the workgroup retires
  __builtin_amdgcn_s_waitcnt(0x0f70);              // vmcnt(0)
}

// ---- activation quantisers -------------------------------------------------
template <int DT>
__device__ __forceinline__ float ld_act(const void* p, long i) {
  if (DT == MI355Q_F32) return ((const float*)p)[i];
  return Elem<DT == MI355Q_F32 ? MI355Q_F16 : DT>::to_f32(((const uint16_t*)p)[i]);
}

template <int DT>
__device__ __forceinline__ float ld_half(uint16_t raw) {
  return Elem<DT == MI355Q_F32 ? MI355Q_F16 : DT>::to_f32(raw);
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
  // 16-bit inputs with K % 8 == 0: 16-byte loads, 8-byte stores (8 elements per lane and step)
  const bool vec8 = DT != MI355Q_F32 && (K & 7) == 0;
  const uint16_t* xr = (const uint16_t*)x + (long)row * K;
  if (vec8) {
    for (int c = threadIdx.x; c < (K >> 3); c += 256) {
      const u4 v = *(const u4*)(xr + 8 * c);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        mx = fmaxf(mx, fabsf(ld_half<DT>((uint16_t)(v[i] & 0xffffu))));
        mx = fmaxf(mx, fabsf(ld_half<DT>((uint16_t)(v[i] >> 16))));
      }
    }
  } else {
    for (int k = threadIdx.x; k < K; k += 256) mx = fmaxf(mx, fabsf(ld_act<DT>(x, (long)row * K + k)));
  }
  mx = wave_max(mx);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = mx;
  __syncthreads();
  mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  if (threadIdx.x == 0) scales[row] = mx / 127.0f;
  const float inv = 127.0f / mx;                // inf for an all-zero row
  if (vec8) {
    for (int c = threadIdx.x; c < (K >> 3); c += 256) {
      const u4 v = *(const u4*)(xr + 8 * c);    // the row was just read: an L2 hit
      uint32_t q[2] = {0u, 0u};
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const uint32_t w = v[e >> 1];
        float y = ld_half<DT>((uint16_t)((e & 1) ? (w >> 16) : (w & 0xffffu))) * inv;
        if (y != y) y = 0.f;                    // 0 * inf
        q[e >> 2] |= ((uint32_t)(uint8_t)sat_rne_s8(y)) << (8 * (e & 3));
      }
      *(u2*)(out + (long)row * K + 8 * c) = (u2){q[0], q[1]};
    }
    return;
  }
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

// silu(x[:, :d]) * x[:, d:] rounded to the input dtype, then quantised like
// static_int8_quant (reciprocal of the scale rounded to the input dtype)
template <int DT>
__global__ void __launch_bounds__(256)
silu_mul_static_int8_quant_kernel(int8_t* out, const uint16_t* x, const float* scale, int per_channel, long total, int d) {
  long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const long r = i / d;
  const int c = (int)(i - r * d);
  float inv = 1.0f / scale[per_channel ? c : 0];
  inv = Elem<DT>::to_f32(Elem<DT>::from_f32(inv));
  const float l = Elem<DT>::to_f32(x[r * 2 * d + c]), g = Elem<DT>::to_f32(x[r * 2 * d + d + c]);
  const float act = Elem<DT>::to_f32(Elem<DT>::from_f32(l * (1.0f / (1.0f + expf(-l))) * g));
  out[i] = sat_rne_s8(act * inv);
}

// static per-expert, per-input-channel quantisation of the rows a fused-MoE GEMM is about to read:
// out[t, :] = sat_s8(rne(x[t / topk, :] * rec[e, :])) for every (token, slot) id t listed in
// sorted_ids, e being the expert of its align block; the product is taken in fp32.  One workgroup
// per sorted position; ids of blocks whose expert lies outside [0, E) get zero rows.
template <int DT>
__global__ void __launch_bounds__(256)
moe_expert_int8_quant_kernel(int8_t* out, const uint16_t* x, const uint16_t* rec, const int* sorted_ids,
                             const int* expert_ids, const int* npp, int block_size, int numel, int topk, int E, int K) {
  const int p = blockIdx.x;
  if (p >= *npp) return;
  const long t = sorted_ids[p];
  if (t >= numel) return;                                      // pad
  const int e = expert_ids[p / block_size];
  const bool local = e >= 0 && e < E;
  const uint16_t* xr = x + (t / topk) * (long)K;
  const uint16_t* rr = rec + (long)(local ? e : 0) * K;
  for (int c = threadIdx.x; c < (K >> 3); c += 256) {
    const u4 xv = *(const u4*)(xr + 8 * c), rv = *(const u4*)(rr + 8 * c);
    uint32_t q[2] = {0u, 0u};
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t xw = xv[i >> 1], rw = rv[i >> 1];
      const float y = ld_half<DT>((uint16_t)((i & 1) ? (xw >> 16) : (xw & 0xffffu))) *
                      ld_half<DT>((uint16_t)((i & 1) ? (rw >> 16) : (rw & 0xffffu)));
      q[i >> 2] |= ((uint32_t)(uint8_t)(local ? sat_rne_s8(y) : (int8_t)0)) << (8 * (i & 3));
    }
    *(u2*)(out + t * (long)K + 8 * c) = (u2){q[0], q[1]};
  }
}

template <int DT, int WM, int WN, int NI, int NJ>
int launch_tile(const I8Args& a, hipStream_t st) {
  constexpr int TN = WN * NI * 16;
  const int mtiles = (a.M + TM - 1) / TM, ntiles = (a.N + TN - 1) / TN;
  I8Args b = a;
  const int ks = a.ksplits > 1 ? a.ksplits : 1;
  b.n_panels_swizzle = (ntiles % 8 == 0 && ks == 1) ? 1 : 0;
  const size_t stage = (size_t)(TM + TN) * TKB;
  const size_t shmem = (3 * stage <= 160 * 1024 ? 3 : 2) * stage;   // 144 KiB (three stages), 120 or 128 KiB (two)
  static hipError_t attr = hipFuncSetAttribute((const void*)w8a8_int8_gemm_kernel<DT, WM, WN, NI, NJ>,
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
  MQ_REQUIRE(attr == hipSuccess, "w8a8_int8_gemm: cannot reserve %zu bytes of LDS: %s", shmem,
             hipGetErrorString(attr));
  // one workgroup per CU (a multiple of 8, so tile id mod 8 stays the XCD)
  int grid = mtiles * ntiles * ks, cus = device_cu_count() / 8 * 8;
  if (cus >= 8 && grid > cus) grid = cus;
  hipLaunchKernelGGL((w8a8_int8_gemm_kernel<DT, WM, WN, NI, NJ>), dim3(grid), dim3(GEMM_THREADS), shmem, st, b);
  MQ_LAUNCH_CHECK("w8a8_int8_gemm");
  return 0;
}

// Columns [n0, n1) of the problem as a launch of its own (n0 a multiple of 128): the operand, scale,
// bias and output pointers move to the first column, the row strides stay.
template <int DT, int WM, int WN, int NI, int NJ>
int launch_columns(const I8Args& a, int n0, int n1, hipStream_t st) {
  I8Args b = a;
  b.N = n1 - n0;
  b.w = a.w + (size_t)n0 * (size_t)(a.w_kslab ? a.K : a.ldw);       // 64 kslab columns are K * 64 bytes too
  if (a.w_scale && a.w_scale_per_col) b.w_scale = a.w_scale + n0;
  if (a.bias) b.bias = (const char*)a.bias + (size_t)n0 * ((a.bias_f32 || DT == MI355Q_F32) ? 4 : 2);
  b.out = (char*)a.out + (size_t)n0 * (DT == MI355Q_F32 ? 4 : 2);
  if (a.acc_out) b.acc_out = a.acc_out + n0;
  return launch_tile<DT, WM, WN, NI, NJ>(b, st);
}

// ---- split K -----------------------------------------------------------------------------------
// A layer with few output tiles (N 4096 .. 10240 at a few hundred rows) leaves most CUs without a
// tile while the others walk a long K.  The sums are integers, so K can be cut into ranges whose
// int32 sums add up exactly: the result is bit for bit that of the unsplit launch.  Second launch:
// sum of the ranges, then the epilogue of the GEMM kernel in its order of operations.
template <int DT>
__global__ void __launch_bounds__(256)
w8a8_splitk_epilogue_kernel(I8Args a) {
  const long q = (long)blockIdx.x * 256 + threadIdx.x;     // 4 adjacent columns of one row
  const int nq = a.N / 4;
  if (q >= (long)a.M * nq) return;
  const int m = (int)(q / nq), n = (int)(q % nq) * 4;
  i4 acc = {0, 0, 0, 0};
  for (int s = 0; s < a.ksplits; ++s) acc += *(const i4*)(a.partial + ((long)s * a.M + m) * a.N + n);
  if (a.acc_out) *(i4*)(a.acc_out + (long)m * a.ldacc + n) = acc;
  const float xsc = a.x_scale ? a.x_scale[a.x_scale_per_row ? m : 0] : 1.0f;
  float v[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const float wsc = a.w_scale ? a.w_scale[a.w_scale_per_col ? n + e : 0] : 1.0f;
    v[e] = scaled_sum((float)acc[e], xsc, wsc);
    if (a.bias) v[e] = plus_bias(v[e], load_bias<DT>(a.bias, a.bias_f32, n + e));
  }
  store4<DT>(a.out, (long)m * a.ldo + n, v);
}

constexpr size_t I8_SPLITK_BYTES = (size_t)64 << 20;
constexpr size_t I8_WS_OFFSET = (size_t)1 << 20;     // the first MiB of a workspace belongs to the W4A16 arrival counters

// K ranges for a shape: as many as put about one 256 x 128 tile on every CU, each at least eight K
// tiles long, a divisor of the K tile count, partial sums within 64 MiB.  1: no split.
int int8_ksplits(int M, int N, int K) {
  const long cus = device_cu_count(), tiles = (long)((M + TM - 1) / TM) * ((N + 127) / 128);
  const int nt = K / TKB;
  if (N % 4 != 0 || tiles * 2 > cus) return 1;
  long s = cus / tiles;
  if (s > 8) s = 8;
  if (s > nt / 8) s = nt / 8;
  while (s > 1 && (nt % s != 0 || (size_t)s * M * N * sizeof(int32_t) > I8_SPLITK_BYTES)) --s;
  return s < 1 ? 1 : (int)s;
}

// The same for several row tiles on a layer of few columns (a few thousand rows on N 4096: 128 tiles of
// 256 x 256, half a round): K ranges of 256 x 256 tiles, which move a third fewer bytes per multiply-add
// than the 256 x 128 tiles that would fill the round unsplit (us, K 14336 x N 4096 at M = 1536 / 2048: 146 / 145 ->
// 110 / 122; K 18944 x N 3584: 186 / 187 -> 130 / 137; K 28672 x N 8192 at M = 768 / 1024: 309 / 320 -> 219 / 247;
// K 8192 x N 8192 at M = 512 / 768: 63 / 94 -> 53 / 83).  0: not this case.
int int8_ksplits_wide(int M, int N, int K) {
  const long cus = device_cu_count(), mtiles = (M + TM - 1) / TM;
  const long t256 = mtiles * ((N + 255) / 256), t128 = mtiles * ((N + 127) / 128);
  const int nt = K / TKB;
  if (N % 4 != 0 || mtiles < 2 || t128 * 2 <= cus || t256 * 2 > cus) return 0;
  long s = cus / t256;
  if (s > nt / 32) s = nt / 32;                      // (ranges of 4096 bytes of K or more: K = 4096 stays unsplit, 49 against 61 us)
  if (s > 8) s = 8;
  if (s > nt / 8) s = nt / 8;
  while (s > 1 && (nt % s != 0 || (size_t)s * M * N * sizeof(int32_t) > I8_SPLITK_BYTES)) --s;
  return s < 2 ? 0 : (int)s;
}

template <int DT>
int launch_gemm_splitk(const I8Args& a, int splits, void* workspace, hipStream_t st, bool wide = false) {
  I8Args b = a;
  b.ksplits = splits;
  b.partial = (int32_t*)((char*)workspace + I8_WS_OFFSET);
  if (int rc = wide ? launch_tile<DT, 2, 4, 4, 8>(b, st) : launch_tile<DT, 4, 2, 4, 4>(b, st)) return rc;
  const long quads = (long)a.M * (a.N / 4);
  hipLaunchKernelGGL((w8a8_splitk_epilogue_kernel<DT>), dim3((unsigned)((quads + 255) / 256)), dim3(256), 0, st, b);
  MQ_LAUNCH_CHECK("w8a8_int8_gemm(split-K epilogue)");
  return 0;
}

// Tile width.  One workgroup per CU works through the output tiles in rounds; a last round that is
// only part full idles the rest of the chip for a whole tile time.  Measured per round of 256 CUs on
// K = 8192 (256 rows x TN columns per CU): TN = 256: 101 us, 224: 98.8 us, 128: 55 us -- the widest
// tile is the cheapest per column.  So: as many FULL rounds of 256-wide tiles as the columns give, and
// the remaining columns as a second launch with the width that wastes least (M 2048, N 28672: three
// rounds of 256 and one of 128 instead of four of 224: 395 -> 387 us; under the profiler the two
// launches last 315-337 us and 65-70 us, i.e. a round costs a little more when three follow each other
// than the single-round figures above say).  A single width is kept where it is as good.
template <int DT>
int launch_gemm(const I8Args& a, hipStream_t st) {
  const long cus = device_cu_count(), mtiles = (a.M + TM - 1) / TM;
  auto rounds = [&](long cols, long w) { return (mtiles * ((cols + w - 1) / w) + cus - 1) / cus; };
  const double c256 = 1.0, c224 = 0.978, c128 = 0.545;            // cost of one round, relative
  const long t256 = mtiles * ((a.N + 255) / 256), t224 = mtiles * ((a.N + 223) / 224);
  // a single row of tiles that leaves most CUs idle: tiles half as wide (the launch is bound by
  // the weight stream, which then comes in over twice as many CUs)
  const long t128 = mtiles * ((a.N + 127) / 128);
  const long r224 = rounds(a.N, 224), r256 = rounds(a.N, 256);
  if (mtiles == 1 && (t224 < r224 * 224 ? t224 : t256) * 3 <= cus * 2 && t128 > t224) return launch_tile<DT, 4, 2, 4, 4>(a, st);
  double best = r224 * c224 < r256 * c256 ? r224 * c224 : r256 * c256;
  int split = 0, tail_w = 0;
  const long full = t256 / cus;                       // whole rounds of 256-wide tiles
  if (full >= 1 && cus % mtiles == 0) {
    const long ncols = full * (cus / mtiles) * 256;   // columns they cover
    if (ncols < a.N) {
      const long rest = a.N - ncols;
      const double tails[3] = {rounds(rest, 128) * c128, rounds(rest, 224) * c224, rounds(rest, 256) * c256};
      const int widths[3] = {128, 224, 256};
      for (int i = 0; i < 3; ++i)
        if (full * c256 + tails[i] < best - 0.05) {   // (a second launch has to pay for itself)
          best = full * c256 + tails[i];
          split = (int)ncols;
          tail_w = widths[i];
        }
    }
  }
  if (split) {
    if (int rc = launch_columns<DT, 2, 4, 4, 8>(a, 0, split, st)) return rc;
    if (tail_w == 128) return launch_columns<DT, 4, 2, 4, 4>(a, split, a.N, st);
    if (tail_w == 224) return launch_columns<DT, 4, 2, 7, 4>(a, split, a.N, st);
    return launch_columns<DT, 2, 4, 4, 8>(a, split, a.N, st);
  }
  if (r224 * c224 < r256 * c256) return launch_tile<DT, 4, 2, 7, 4>(a, st);
  return launch_tile<DT, 2, 4, 4, 8>(a, st);
}

template <int DT>
int launch_tile_grouped(const I8Args& a, hipStream_t st) {
  const size_t shmem = 3 * (size_t)(TM + 128) * TKB;
  static hipError_t attr = hipFuncSetAttribute((const void*)w8a8_int8_gemm_kernel<DT, 4, 2, 4, 4, true>,
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
  MQ_REQUIRE(attr == hipSuccess, "moe_gemm(int8 tiles): cannot reserve %zu bytes of LDS: %s", shmem, hipGetErrorString(attr));
  long grid = (long)a.max_blocks * ((a.N + 127) / 128);
  const long cus = device_cu_count();
  if (grid > cus) grid = cus;
  hipLaunchKernelGGL((w8a8_int8_gemm_kernel<DT, 4, 2, 4, 4, true>), dim3((unsigned)grid), dim3(GEMM_THREADS), shmem, st, a);
  MQ_LAUNCH_CHECK("moe_gemm(int8 tiles)");
  return 0;
}

}  // namespace

// The fused-MoE grouped GEMM on int8 experts (per-token x per-channel scales) on align blocks of 256 or 128 slot
// ids: the MFMA tile kernel above with its rows gathered through the ids (prefill token counts; smaller
// blocks take the weight-streaming kernel).  Arguments as mi355q_moe_gemm's; checked by the caller.
int int8_grouped_launch(void* out, const void* a, const void* w, const float* a_scale, int a_scale_per_row,
                        const float* w_scale, const float* topk_weights, const int32_t* sorted_ids,
                        const int32_t* expert_ids, const int32_t* npp, int numel, int topk, int block_size, int max_blocks,
                        int E, int K, int N, int out_dtype, int w_kslab, hipStream_t st) {
  MQ_REQUIRE(block_size == 256 || block_size == 128, "moe_gemm(int8 tiles): block_size=%d must be 128 or 256", block_size);
  MQ_REQUIRE(N % 4 == 0 && K % 128 == 0 && (!w_kslab || N % 64 == 0), "moe_gemm(int8 tiles): bad shape N=%d K=%d", N, K);
  MQ_REQUIRE(out_dtype == MI355Q_F16 || out_dtype == MI355Q_BF16, "moe_gemm(int8 tiles): output dtype %d", out_dtype);
  MQ_REQUIRE(a_scale && w_scale, "moe_gemm(int8 tiles): scales missing");
  MQ_REQUIRE(((size_t)numel / topk + 1) * K < ((size_t)1 << 32) && (size_t)N * K < ((size_t)1 << 32),
             "moe_gemm(int8 tiles): activations and one expert's weights must each stay below 4 GiB");
  I8Args g = {};
  g.out = out; g.x = (const int8_t*)a; g.w = (const int8_t*)w; g.x_scale = a_scale; g.w_scale = w_scale;
  g.M = numel; g.N = N; g.K = K; g.ldx = K; g.ldw = K; g.ldo = N;
  g.x_scale_per_row = a_scale_per_row; g.w_scale_per_col = 1;
  g.w_kslab = w_kslab;
  g.ksplits = 1;
  g.sorted_ids = sorted_ids; g.expert_ids = expert_ids; g.npp = npp; g.topk_weights = topk_weights;
  g.numel = numel; g.topk = topk; g.E = E; g.max_blocks = max_blocks;
  g.block_rows = block_size;
  g.w_stride = (long)N * K;
  g.ws_stride = N;
  return out_dtype == MI355Q_F16 ? launch_tile_grouped<MI355Q_F16>(g, st) : launch_tile_grouped<MI355Q_BF16>(g, st);
}

}  // namespace mi355q

using namespace mi355q;

extern "C" size_t mi355q_w8a8_int8_workspace_bytes(int M, int N, int K) {
  if (M <= 0 || N <= 0 || K <= 0 || K % 128 != 0) return 0;
  int s = int8_ksplits(M, N, K);
  if (s <= 1) s = int8_ksplits_wide(M, N, K);
  return s > 1 ? I8_WS_OFFSET + (size_t)s * M * N * sizeof(int32_t) : 0;
}

extern "C" int mi355q_w8a8_int8_gemm(void* out, int32_t* acc_out, const int8_t* x, const int8_t* w,
                                     const float* x_scale, int x_scale_per_row, const float* w_scale,
                                     int w_scale_per_col, const void* bias, int bias_f32, int M, int N,
                                     int K, long ldx, long ldw, long ldo, int out_dtype, void* stream) {
  return mi355q_w8a8_int8_gemm_ws(out, acc_out, x, w, x_scale, x_scale_per_row, w_scale, w_scale_per_col, bias, bias_f32,
                                  M, N, K, ldx, ldw, ldo, out_dtype, nullptr, 0, stream);
}

extern "C" int mi355q_w8a8_int8_gemm_ws(void* out, int32_t* acc_out, const int8_t* x, const int8_t* w,
                                        const float* x_scale, int x_scale_per_row, const float* w_scale,
                                        int w_scale_per_col, const void* bias, int bias_f32, int M, int N,
                                        int K, long ldx, long ldw, long ldo, int out_dtype, void* workspace,
                                        size_t workspace_bytes, void* stream) {
  MQ_REQUIRE(M >= 0 && N > 0 && K > 0, "w8a8_int8_gemm: bad shape M=%d N=%d K=%d", M, N, K);
  if (M == 0) return 0;
  MQ_REQUIRE(out && x && w, "w8a8_int8_gemm: null pointer");
  MQ_REQUIRE(K % 128 == 0, "w8a8_int8_gemm: K=%d must be a multiple of 128", K);
  MQ_REQUIRE(N % 4 == 0, "w8a8_int8_gemm: N=%d must be a multiple of 4", N);
  const bool kslab = ldw == 0;
  MQ_REQUIRE(ldx % 16 == 0 && ldx >= K && (kslab || (ldw % 16 == 0 && ldw >= K)),
             "w8a8_int8_gemm: operand row strides (%ld, %ld) must be >= K and multiples of 16", ldx, ldw);
  MQ_REQUIRE(!kslab || (N % 64 == 0 && (size_t)N * K < ((size_t)1 << 32)),
             "w8a8_int8_gemm: kslab weights need N=%d %% 64 == 0 and fewer than 4 Gi elements", N);
  MQ_REQUIRE(ldo >= N && ldo % 4 == 0, "w8a8_int8_gemm: output row stride %ld must be >= N and a multiple of 4", ldo);
  MQ_REQUIRE(out_dtype >= MI355Q_F16 && out_dtype <= MI355Q_F32, "w8a8_int8_gemm: bad out dtype %d", out_dtype);
  I8Args a;
  a.out = out; a.acc_out = acc_out; a.x = x; a.w = w; a.x_scale = x_scale; a.w_scale = w_scale;
  a.bias = bias; a.M = M; a.N = N; a.K = K; a.ldx = ldx; a.ldw = ldw; a.ldo = ldo; a.ldacc = N;
  a.x_scale_per_row = x_scale_per_row; a.w_scale_per_col = w_scale_per_col; a.bias_f32 = bias_f32;
  a.n_panels_swizzle = 0;
  a.w_kslab = kslab ? 1 : 0;
  a.wide_stores = (N % 8 == 0 && ldo % 8 == 0 && ((size_t)out & 15) == 0) ? 1 : 0;
  a.ksplits = 1;
  a.partial = nullptr;
  int splits = int8_ksplits(M, N, K);
  const bool wide = splits <= 1;
  if (wide) splits = int8_ksplits_wide(M, N, K);
  if (splits > 1 && workspace && workspace_bytes >= I8_WS_OFFSET + (size_t)splits * M * N * sizeof(int32_t)) {
    if (out_dtype == MI355Q_F16) return launch_gemm_splitk<MI355Q_F16>(a, splits, workspace, as_stream(stream), wide);
    if (out_dtype == MI355Q_BF16) return launch_gemm_splitk<MI355Q_BF16>(a, splits, workspace, as_stream(stream), wide);
    return launch_gemm_splitk<MI355Q_F32>(a, splits, workspace, as_stream(stream), wide);
  }
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

extern "C" int mi355q_moe_expert_int8_quant(int8_t* out, const void* x, const void* scale_rec,
                                            const int32_t* sorted_token_ids, const int32_t* expert_ids,
                                            const int32_t* num_tokens_post_pad, int max_sorted, int block_size,
                                            int numel, int topk, int E, int K, int dtype, void* stream) {
  MQ_REQUIRE(numel >= 0 && topk > 0 && E > 0 && K > 0 && K % 8 == 0 && block_size > 0 && max_sorted >= 0,
             "moe_expert_int8_quant: bad shape numel=%d topk=%d E=%d K=%d block=%d (K %% 8 == 0)", numel, topk, E, K,
             block_size);
  if (numel == 0 || max_sorted == 0) return 0;
  MQ_REQUIRE(out && x && scale_rec && sorted_token_ids && expert_ids && num_tokens_post_pad,
             "moe_expert_int8_quant: null pointer");
  MQ_REQUIRE(dtype == MI355Q_F16 || dtype == MI355Q_BF16, "moe_expert_int8_quant: dtype %d must be f16 or bf16", dtype);
  hipStream_t st = as_stream(stream);
  if (dtype == MI355Q_F16)
    hipLaunchKernelGGL((moe_expert_int8_quant_kernel<MI355Q_F16>), dim3(max_sorted), dim3(256), 0, st, out,
                       (const uint16_t*)x, (const uint16_t*)scale_rec, sorted_token_ids, expert_ids,
                       num_tokens_post_pad, block_size, numel, topk, E, K);
  else
    hipLaunchKernelGGL((moe_expert_int8_quant_kernel<MI355Q_BF16>), dim3(max_sorted), dim3(256), 0, st, out,
                       (const uint16_t*)x, (const uint16_t*)scale_rec, sorted_token_ids, expert_ids,
                       num_tokens_post_pad, block_size, numel, topk, E, K);
  MQ_LAUNCH_CHECK("moe_expert_int8_quant");
  return 0;
}

extern "C" int mi355q_silu_mul_static_int8_quant(int8_t* out, const void* x, const float* scale, int per_channel,
                                                 long rows, int d, int dtype, void* stream) {
  MQ_REQUIRE(rows >= 0 && d > 0, "silu_mul_static_int8_quant: bad shape rows=%ld d=%d", rows, d);
  if (rows == 0) return 0;
  MQ_REQUIRE(out && scale && x, "silu_mul_static_int8_quant: null pointer");
  MQ_REQUIRE(dtype == MI355Q_F16 || dtype == MI355Q_BF16, "silu_mul_static_int8_quant: dtype %d must be f16 or bf16", dtype);
  const long total = rows * d;
  const unsigned blocks = (unsigned)((total + 255) / 256);
  hipStream_t st = as_stream(stream);
  if (dtype == MI355Q_F16)
    hipLaunchKernelGGL((silu_mul_static_int8_quant_kernel<MI355Q_F16>), dim3(blocks), dim3(256), 0, st, out,
                       (const uint16_t*)x, scale, per_channel, total, d);
  else
    hipLaunchKernelGGL((silu_mul_static_int8_quant_kernel<MI355Q_BF16>), dim3(blocks), dim3(256), 0, st, out,
                       (const uint16_t*)x, scale, per_channel, total, d);
  MQ_LAUNCH_CHECK("silu_mul_static_int8_quant");
  return 0;
}
