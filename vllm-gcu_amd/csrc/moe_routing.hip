// MoE routing and token -> expert alignment on gfx950.
//
//  * topk_softmax        one wavefront per token: softmax over experts in
//                        fp32, then k rounds of a wavefront arg-max
//                        (value descending, index ascending on ties).
//  * grouped_topk        the same selection restricted to the best expert
//                        groups (group score = max, or sum of the top two
//                        biased scores when a correction bias is given).
//  * moe_align_block_size  stable counting sort of flat (token, slot) ids by
//                        expert with every expert's run padded to a multiple
//                        of the block size.  One workgroup; each wavefront
//                        owns a contiguous segment of ids, ranks inside a
//                        64-id tile come from ballots over the bits of the
//                        expert id (wavefront-level scan), segment bases from
//                        an LDS scan over wavefronts.
#include "common.h"

namespace mi355q {
namespace {

constexpr int MAX_E = 1024;          // experts per token row handled by the routing kernels
// EPL (template parameter below) = experts per lane: 1, 4 or 16 for up to 64, 256 or 1024 experts

template <int DT>
__device__ __forceinline__ float ld_logit(const void* p, long i) {
  if (DT == MI355Q_F32) return ((const float*)p)[i];
  return Elem<DT == MI355Q_F32 ? MI355Q_F16 : DT>::to_f32(((const uint16_t*)p)[i]);
}

// arg-max over the wavefront: larger value wins, lower index on ties; the result is the same in every lane
__device__ __forceinline__ void wave_argmax(float& v, int& idx) {
  const float m = wave_max(v);
  int cand = (v == m) ? idx : 0x7fffffff;
  MQ_DPP_REDUCE(cand, 0x7fffffff, op_imin);
  v = m;
  idx = cand;
}

// scores of one row, expert e = lane + 64 j in s[j]; -inf beyond E
template <int DT, int EPL>
__device__ __forceinline__ void row_scores(const void* gating, long row, int E, int lane, int sigmoid,
                                           float* s) {
  float mx = -INFINITY;
#pragma unroll
  for (int j = 0; j < EPL; ++j) {
    const int e = lane + 64 * j;
    s[j] = e < E ? ld_logit<DT>(gating, row * E + e) : -INFINITY;
    mx = fmaxf(mx, s[j]);
  }
  if (sigmoid) {
#pragma unroll
    for (int j = 0; j < EPL; ++j)
      if (lane + 64 * j < E) s[j] = 1.0f / (1.0f + expf(-s[j]));
    return;
  }
  mx = wave_max(mx);
  float sum = 0.f;
#pragma unroll
  for (int j = 0; j < EPL; ++j) {
    const int e = lane + 64 * j;
    s[j] = e < E ? expf(s[j] - mx) : 0.f;
    sum += s[j];
  }
  sum = wave_sum(sum);
#pragma unroll
  for (int j = 0; j < EPL; ++j) s[j] = (lane + 64 * j < E) ? s[j] / sum : -INFINITY;
}

// k rounds of arg-max over sel[]; weights are read from w[] at the winner
template <int EPL>
__device__ __forceinline__ void select_topk(float* sel, const float* w, int lane, int k, float* out_w,
                                            int* out_i, long base, bool renorm) {
  float total = 0.f;
  float mine_w = 0.f;
  int mine_i = 0;
  for (int r = 0; r < k; ++r) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
#pragma unroll
    for (int j = 0; j < EPL; ++j) {
      const int e = lane + 64 * j;
      if (sel[j] > bv) { bv = sel[j]; bi = e; }   // ascending e within a lane: first max wins
    }
    wave_argmax(bv, bi);
    // the owner retires the winner; its (unbiased) weight is read from its lane (bi is uniform)
    float cw = 0.f;
#pragma unroll
    for (int j = 0; j < EPL; ++j) {
      if (j == (bi >> 6)) cw = w[j];
      if (lane + 64 * j == bi) sel[j] = -INFINITY;
    }
    const float wv = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(cw), bi & 63));
    total += wv;
    if (lane == r) { mine_w = wv; mine_i = bi; }
  }
  if (lane < k) {
    out_w[base + lane] = renorm ? mine_w / total : mine_w;
    out_i[base + lane] = mine_i;
  }
}

template <int DT, int EPL>
__global__ void __launch_bounds__(256)
topk_softmax_kernel(float* topk_w, int* topk_i, int* tok_exp, const void* gating, int M, int E, int k,
                    int renorm) {
  const int lane = threadIdx.x & 63;
  const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= M) return;
  float s[EPL], w[EPL];
  row_scores<DT, EPL>(gating, row, E, lane, 0, s);
#pragma unroll
  for (int j = 0; j < EPL; ++j) w[j] = s[j];
  select_topk<EPL>(s, w, lane, k, topk_w, topk_i, row * k, renorm != 0);
  if (tok_exp && lane < k) tok_exp[row * k + lane] = lane * M + (int)row;
}

template <int DT, int EPL>
__global__ void __launch_bounds__(256)
grouped_topk_kernel(float* topk_w, int* topk_i, const void* gating, const float* bias, int M, int E, int k,
                    int ngroup, int topk_group, int renorm, int sigmoid) {
  __shared__ float sh[4][64 * EPL];
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const long row = (long)blockIdx.x * 4 + wv;
  if (row >= M) return;
  float s[EPL], sel[EPL];
  row_scores<DT, EPL>(gating, row, E, lane, sigmoid, s);
#pragma unroll
  for (int j = 0; j < EPL; ++j) {
    const int e = lane + 64 * j;
    sel[j] = s[j];
    if (bias && e < E) sel[j] = s[j] + bias[e];
    if (e < E) sh[wv][e] = sel[j];
  }
  __builtin_amdgcn_wave_barrier();
  // lane g scores group g: max, or the sum of its two largest biased scores
  const int per = E / ngroup;
  float gs = -INFINITY;
  for (int g0 = 0; g0 < ngroup; g0 += 64) {     // ngroup <= 64 in practice: one pass
    const int g = g0 + lane;
    if (g < ngroup) {
      float m1 = -INFINITY, m2 = -INFINITY;
      for (int i = 0; i < per; ++i) {
        float v = sh[wv][g * per + i];
        if (v > m1) { m2 = m1; m1 = v; } else if (v > m2) { m2 = v; }
      }
      gs = bias ? m1 + m2 : m1;
    }
  }
  // keep the topk_group best groups (ties to the lower group)
  unsigned long long keep = 0ull;
  for (int r = 0; r < topk_group; ++r) {
    float bv = gs;
    int bi = lane < ngroup ? lane : 0x7fffffff;
    if (lane >= ngroup) bv = -INFINITY;
    wave_argmax(bv, bi);
    keep |= 1ull << bi;
    if (lane == bi) gs = -INFINITY;
  }
#pragma unroll
  for (int j = 0; j < EPL; ++j) {
    const int e = lane + 64 * j;
    if (e >= E || !((keep >> (e / per)) & 1ull)) sel[j] = -INFINITY;
  }
  select_topk<EPL>(sel, s, lane, k, topk_w, topk_i, row * k, renorm != 0);
}

// ---- align ------------------------------------------------------------------
constexpr int ALIGN_WAVES = 16;

template <typename IdT>
__global__ void __launch_bounds__(ALIGN_WAVES * 64)
moe_align_kernel(const IdT* __restrict__ topk_ids, int numel, int top, const int* valid_rows, int E, int B,
                 const int* expert_map, int* __restrict__ sorted_ids, int cap, int* __restrict__ expert_ids,
                 int nblocks_cap, int* __restrict__ npp) {
  extern __shared__ int sm[];
  int* cnt = sm;                                 // [ALIGN_WAVES][E] per-wavefront counts -> bases
  int* estart = sm + ALIGN_WAVES * E;            // [E + 1] padded start of each expert
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int nvalid = valid_rows ? min(numel, max(0, *valid_rows) * top) : numel;

  for (int i = tid; i < ALIGN_WAVES * E; i += blockDim.x) cnt[i] = 0;
  for (int i = tid; i < cap; i += blockDim.x) sorted_ids[i] = numel;     // pads / unused tail
  __syncthreads();

  // each wavefront owns a contiguous, 64-aligned segment of the ids
  const int tiles = (nvalid + 63) / 64;
  const int tiles_per = (tiles + ALIGN_WAVES - 1) / ALIGN_WAVES;
  const int seg_b = min(nvalid, wv * tiles_per * 64), seg_e = min(nvalid, (wv + 1) * tiles_per * 64);
  for (int i = seg_b + lane; i < seg_e; i += 64) {
    const int e = (int)topk_ids[i];
    if (e >= 0 && e < E) atomicAdd(&cnt[wv * E + e], 1);
  }
  __syncthreads();
  // per expert: exclusive scan over wavefronts, total -> padded size
  for (int e = tid; e < E; e += blockDim.x) {
    int run = 0;
    for (int w = 0; w < ALIGN_WAVES; ++w) {
      int c = cnt[w * E + e];
      cnt[w * E + e] = run;
      run += c;
    }
    estart[e + 1] = (run + B - 1) / B * B;       // padded count, scanned below
  }
  __syncthreads();
  // exclusive scan of the padded counts by the first wavefront: each lane sums a run of
  // consecutive experts, the lane totals are scanned with shuffles
  if (wv == 0) {
    const int per = (E + 63) / 64;
    const int e0 = min(E, lane * per), e1 = min(E, e0 + per);
    int sum = 0;
    for (int e = e0; e < e1; ++e) sum += estart[e + 1];
    int incl = sum;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int up = __shfl_up(incl, o);
      if (lane >= o) incl += up;
    }
    int run = incl - sum;                          // exclusive prefix of this lane's run
    const int total = __shfl(incl, 63);
    // estart[e] must not be overwritten before the lane that reads estart[e + 1] = old count
    // of expert e has consumed it: every lane first reads its own run, then all write
    // a lane's run is at most 16 experts: the launch caps E at what 64 KiB of LDS hold (below 1024)
    int vals[16];
#pragma unroll
    for (int k = 0; k < 16; ++k) vals[k] = (e0 + k < e1) ? estart[e0 + k + 1] : 0;
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int k = 0; k < 16; ++k)
      if (e0 + k < e1) {
        estart[e0 + k] = run;
        run += vals[k];
      }
    if (lane == 63) estart[E] = total;
    if (lane == 0) *npp = total;
  }
  __syncthreads();
  // block -> expert table (unused blocks get expert 0)
  for (int b = tid; b < nblocks_cap; b += blockDim.x) expert_ids[b] = 0;
  __syncthreads();
  for (int e = tid; e < E; e += blockDim.x) {
    const int me = expert_map ? expert_map[e] : e;
    for (int b = estart[e] / B; b < estart[e + 1] / B; ++b) expert_ids[b] = me;
  }
  // stable scatter: tile by tile, rank inside the tile from ballots
  const int ebits = E > 1 ? 32 - __builtin_clz((unsigned)(E - 1)) : 0;
  for (int t0 = seg_b; t0 < seg_e; t0 += 64) {
    const int i = t0 + lane;
    int e = -1;
    if (i < seg_e) {
      e = (int)topk_ids[i];
      if (e < 0 || e >= E) e = -1;
    }
    // lanes of the tile that hold the same expert: the ballots of the id's bits, each taken as it is or
    // inverted according to the lane's own bit, intersected (no loop over the distinct experts of the tile)
    unsigned long long same = __ballot(e >= 0);
    for (int b = 0; b < ebits; ++b) {
      const bool bit = (e >> b) & 1;
      const unsigned long long set = __ballot(bit);
      same &= bit ? set : ~set;
    }
    int slot = 0, rank = 0;
    if (e >= 0) {
      rank = __popcll(same & ((1ull << lane) - 1ull));
      slot = estart[e] + cnt[wv * E + e] + rank;   // read before the lowest lane of the set bumps the count
    }
    __builtin_amdgcn_wave_barrier();
    if (e >= 0) {
      sorted_ids[slot] = i;
      if (rank == 0) cnt[wv * E + e] += __popcll(same);
    }
    __builtin_amdgcn_wave_barrier();
  }
}

}  // namespace
}  // namespace mi355q

using namespace mi355q;

extern "C" int mi355q_topk_softmax(float* topk_weights, int32_t* topk_ids, int32_t* token_expert_indices,
                                   const void* gating, int M, int E, int topk, int renormalize, int dtype,
                                   void* stream) {
  MQ_REQUIRE(M >= 0 && E > 0 && topk > 0, "topk_softmax: bad shape M=%d E=%d topk=%d", M, E, topk);
  if (M == 0) return 0;
  MQ_REQUIRE(topk_weights && topk_ids && gating, "topk_softmax: null pointer");
  MQ_REQUIRE(E <= MAX_E && topk <= 64 && topk <= E, "topk_softmax: E=%d (max %d) / topk=%d (max 64) unsupported", E, MAX_E, topk);
  dim3 grid((M + 3) / 4), block(256);
  hipStream_t st = as_stream(stream);
  MQ_REQUIRE(dtype == MI355Q_F32 || dtype == MI355Q_F16 || dtype == MI355Q_BF16, "topk_softmax: bad dtype %d", dtype);
#define MQ_TOPK_LAUNCH(DT, EPL) \
  hipLaunchKernelGGL((topk_softmax_kernel<DT, EPL>), grid, block, 0, st, topk_weights, topk_ids, token_expert_indices, gating, M, E, topk, renormalize)
#define MQ_TOPK_EPL(DT) \
  do { if (E <= 64) MQ_TOPK_LAUNCH(DT, 1); else if (E <= 256) MQ_TOPK_LAUNCH(DT, 4); else MQ_TOPK_LAUNCH(DT, 16); } while (0)
  if (dtype == MI355Q_F32) MQ_TOPK_EPL(MI355Q_F32);
  else if (dtype == MI355Q_F16) MQ_TOPK_EPL(MI355Q_F16);
  else MQ_TOPK_EPL(MI355Q_BF16);
#undef MQ_TOPK_EPL
#undef MQ_TOPK_LAUNCH
  MQ_LAUNCH_CHECK("topk_softmax");
  return 0;
}

extern "C" int mi355q_grouped_topk(float* topk_weights, int32_t* topk_ids, const void* gating,
                                   const float* bias, int M, int E, int topk, int renormalize,
                                   int num_expert_group, int topk_group, int scoring_sigmoid, int dtype,
                                   void* stream) {
  MQ_REQUIRE(M >= 0 && E > 0 && topk > 0, "grouped_topk: bad shape M=%d E=%d topk=%d", M, E, topk);
  if (M == 0) return 0;
  MQ_REQUIRE(topk_weights && topk_ids && gating, "grouped_topk: null pointer");
  MQ_REQUIRE(E <= MAX_E && topk <= 64, "grouped_topk: E=%d (max %d) / topk=%d (max 64) unsupported", E, MAX_E, topk);
  MQ_REQUIRE(num_expert_group > 0 && num_expert_group <= 64 && E % num_expert_group == 0,
             "grouped_topk: num_expert_group=%d must divide E=%d and be <= 64", num_expert_group, E);
  MQ_REQUIRE(topk_group > 0 && topk_group <= num_expert_group, "grouped_topk: topk_group=%d out of range", topk_group);
  MQ_REQUIRE(topk <= topk_group * (E / num_expert_group), "grouped_topk: topk=%d exceeds the experts of %d groups", topk, topk_group);
  MQ_REQUIRE(!bias || E / num_expert_group >= 2, "grouped_topk: a correction bias needs at least 2 experts per group");
  dim3 grid((M + 3) / 4), block(256);
  hipStream_t st = as_stream(stream);
  MQ_REQUIRE(dtype == MI355Q_F32 || dtype == MI355Q_F16 || dtype == MI355Q_BF16, "grouped_topk: bad dtype %d", dtype);
#define MQ_GTOPK_LAUNCH(DT, EPL) \
  hipLaunchKernelGGL((grouped_topk_kernel<DT, EPL>), grid, block, 0, st, topk_weights, topk_ids, gating, bias, M, E, topk, num_expert_group, topk_group, renormalize, scoring_sigmoid)
#define MQ_GTOPK_EPL(DT) \
  do { if (E <= 64) MQ_GTOPK_LAUNCH(DT, 1); else if (E <= 256) MQ_GTOPK_LAUNCH(DT, 4); else MQ_GTOPK_LAUNCH(DT, 16); } while (0)
  if (dtype == MI355Q_F32) MQ_GTOPK_EPL(MI355Q_F32);
  else if (dtype == MI355Q_F16) MQ_GTOPK_EPL(MI355Q_F16);
  else MQ_GTOPK_EPL(MI355Q_BF16);
#undef MQ_GTOPK_EPL
#undef MQ_GTOPK_LAUNCH
  MQ_LAUNCH_CHECK("grouped_topk");
  return 0;
}

extern "C" int mi355q_moe_align_block_size(const void* topk_ids, int ids_are_int64, int numel, int topk,
                                           const int32_t* valid_rows, int num_experts, int block_size,
                                           const int32_t* expert_map, int32_t* sorted_token_ids,
                                           int32_t* expert_ids, int32_t* num_tokens_post_pad, void* stream) {
  MQ_REQUIRE(numel >= 0 && num_experts > 0 && block_size > 0 && topk > 0,
             "moe_align_block_size: bad arguments numel=%d E=%d block=%d topk=%d", numel, num_experts, block_size, topk);
  MQ_REQUIRE(sorted_token_ids && expert_ids && num_tokens_post_pad && (topk_ids || numel == 0),
             "moe_align_block_size: null pointer");
  const size_t shmem = ((size_t)ALIGN_WAVES * num_experts + num_experts + 1) * sizeof(int);
  MQ_REQUIRE(shmem <= 64 * 1024 && num_experts <= 1024, "moe_align_block_size: num_experts=%d too large", num_experts);
  const int cap = numel + num_experts * (block_size - 1);
  const int nblocks = cap / block_size;
  hipStream_t st = as_stream(stream);
  if (ids_are_int64)
    hipLaunchKernelGGL((moe_align_kernel<long>), dim3(1), dim3(ALIGN_WAVES * 64), shmem, st, (const long*)topk_ids, numel, topk, valid_rows, num_experts, block_size, expert_map, sorted_token_ids, cap, expert_ids, nblocks, num_tokens_post_pad);
  else
    hipLaunchKernelGGL((moe_align_kernel<int>), dim3(1), dim3(ALIGN_WAVES * 64), shmem, st, (const int*)topk_ids, numel, topk, valid_rows, num_experts, block_size, expert_map, sorted_token_ids, cap, expert_ids, nblocks, num_tokens_post_pad);
  MQ_LAUNCH_CHECK("moe_align_block_size");
  return 0;
}
