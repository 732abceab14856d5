// Skinny GEMMs whose weights are K-contiguous ([N, K] per expert): fp8-e4m3
// with 128x128 block scales, int8 with per-token x per-channel scales, plain
// fp16/bf16, and int8 weights with 16-bit activations (W8A16).  Used for the
// fused-MoE grouped GEMM ("non-gather": rows are picked through
// sorted_token_ids, weights through expert_ids) and for dense small-M calls.
//
// Weight layouts.  Row-major [N, K] (the checkpoint's) works, but a wavefront
// load instruction then touches 16 rows and uses half of each 128-byte line
// (measured: 4.4 TB/s on the DeepSeek-style fp8 layer).  The "kslab" layout
// stores every 64-column x 128-k block of a wavefront in the order its lanes
// consume it -- [N/64][K/128][4 tiles][vector][64 lanes][16 B] -- so that each
// load instruction reads one contiguous KiB and a wavefront walks one
// contiguous stream (5.9 TB/s on the same layer); mi355q_kslab_repack converts.
//
// These shapes are bound by the HBM stream of the weights.  A workgroup (4
// wavefronts) owns up to 64 rows and 256 columns; a wavefront owns 64 columns
// (four 16-row MFMA "A" tiles of weights) and every row tile of activations,
// so each weight byte is loaded once per workgroup and both operands go from
// global memory straight into MFMA registers: lane (r = l % 16, q = l / 16)
// holds the 32 consecutive k of row r that start at 128 kb + 32 q.  The next K
// block is prefetched while the current one is multiplied.  Block scales are
// applied to the fp32 partial sum of each 128-wide K block; the int8 mode
// keeps exact int32 accumulators to the end.
#include "common.h"

namespace mi355q {
namespace {

enum { KC_FP8_BLOCK = 0, KC_INT8 = 1, KC_F16 = 2, KC_BF16 = 3, KC_W8A16_F16 = 4, KC_W8A16_BF16 = 5,
       KC_W8A16G_F16 = 6, KC_W8A16G_BF16 = 7,     // G: group-wise scales [E, K/g, N], g = 64 or 128
       KC_FP8_PC = 8 };                           // fp8 with per-token x per-channel (or per-tensor) scales

struct KcArgs {
  void* out;                   // [rows_out, N] f16/bf16
  const void* a;               // activations [Ma, K]
  const void* w;               // weights [E, N, K]
  const float* a_scale;        // fp8 block: [Ma, K/128]; int8 / fp8 per token: [Ma] (one value with sc_row = 0)
  const void* w_scale;         // fp8 block: f32 [E, ceil(N/128), K/128]; int8 / fp8 per channel: f32 [E, N] (one value
                               // with sc_col = 0); W8A16: act dtype [E, N] or [E, K/g, N]
  int sc_row, sc_col;          // int8 / fp8 per token x per channel: index multipliers of a_scale / w_scale (1, or 0 = per tensor)
  const void* bias;            // [N] in out dtype, dense mode only
  int M, N, K;
  int kslab;                   // weights are in the kslab layout (N % 64 == 0)
  int wgroup;                  // W8A16 group-wise modes: 64 or 128
  int wide_stores;             // N % 8 == 0 and a 16-byte aligned output below 4 GiB: 16-byte stores of 8 adjacent outputs
  // grouped mode
  const int* sorted_ids;
  const int* expert_ids;
  const int* npp;
  const float* topk_weights;
  int numel, topk, block_size, E;
  long w_stride, ws_stride;    // per-expert strides (elements)
};

template <int MODE> struct Kc;
template <> struct Kc<KC_FP8_BLOCK> {
  static constexpr int ABYTES = 1, WBYTES = 1;
  typedef f4 acc_t;
};
template <> struct Kc<KC_INT8> {
  static constexpr int ABYTES = 1, WBYTES = 1;
  typedef i4 acc_t;
};
template <> struct Kc<KC_FP8_PC> {
  static constexpr int ABYTES = 1, WBYTES = 1;
  typedef f4 acc_t;
};
template <> struct Kc<KC_F16> {
  static constexpr int ABYTES = 2, WBYTES = 2;
  typedef f4 acc_t;
};
template <> struct Kc<KC_BF16> {
  static constexpr int ABYTES = 2, WBYTES = 2;
  typedef f4 acc_t;
};
template <> struct Kc<KC_W8A16_F16> {
  static constexpr int ABYTES = 2, WBYTES = 1;
  typedef f4 acc_t;
};
template <> struct Kc<KC_W8A16_BF16> {
  static constexpr int ABYTES = 2, WBYTES = 1;
  typedef f4 acc_t;
};
template <> struct Kc<KC_W8A16G_F16> : Kc<KC_W8A16_F16> {};
template <> struct Kc<KC_W8A16G_BF16> : Kc<KC_W8A16_BF16> {};

// 16 signed bytes -> 16 halves / bfloat16 (exact)
__device__ __forceinline__ void s8x16_to_f16(const u4& v, u4& lo, u4& hi) {
  uint32_t o[8];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int w = (int)v[i];
    _Float16 h0 = (_Float16)(float)(int8_t)(w & 0xff), h1 = (_Float16)(float)(int8_t)((w >> 8) & 0xff);
    _Float16 h2 = (_Float16)(float)(int8_t)((w >> 16) & 0xff), h3 = (_Float16)(float)(int8_t)((w >> 24) & 0xff);
    o[2 * i] = (uint32_t)bitcast<uint16_t>(h0) | ((uint32_t)bitcast<uint16_t>(h1) << 16);
    o[2 * i + 1] = (uint32_t)bitcast<uint16_t>(h2) | ((uint32_t)bitcast<uint16_t>(h3) << 16);
  }
  lo = (u4){o[0], o[1], o[2], o[3]};
  hi = (u4){o[4], o[5], o[6], o[7]};
}
__device__ __forceinline__ void s8x16_to_bf16(const u4& v, u4& lo, u4& hi) {
  uint32_t o[8];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int w = (int)v[i];
    uint32_t b0 = bitcast<uint32_t>((float)(int8_t)(w & 0xff)) >> 16, b1 = bitcast<uint32_t>((float)(int8_t)((w >> 8) & 0xff)) >> 16;
    uint32_t b2 = bitcast<uint32_t>((float)(int8_t)((w >> 16) & 0xff)) >> 16, b3 = bitcast<uint32_t>((float)(int8_t)((w >> 24) & 0xff)) >> 16;
    o[2 * i] = b0 | (b1 << 16);
    o[2 * i + 1] = b2 | (b3 << 16);
  }
  lo = (u4){o[0], o[1], o[2], o[3]};
  hi = (u4){o[4], o[5], o[6], o[7]};
}

// KS (dense launches of few row blocks): the four wavefronts of a workgroup share one group of 64
// columns and take its K blocks round-robin, partial sums meet in LDS.  With one or two row blocks
// there are only a few hundred wavefronts of 64 columns each; that leaves most of the chip idle
// and every wavefront with the whole of K as one dependent chain of loads.
// NI (KS only): 16-column tiles per workgroup, 4, 2 or 1 -- a layer of a few thousand columns has only 64
// to 128 groups of 64 columns, a quarter to half of the CUs; with 32 or 16 columns per workgroup every
// CU streams a share of the weights (and reads the activations once more per workgroup).
template <int MODE, int ODT, int MT, bool GROUPED, bool KS = false, int NI = 4>
__global__ void __launch_bounds__(256, 1)
kcontig_gemm_kernel(KcArgs a) {
  static_assert(NI == 4 || (KS && (NI == 1 || NI == 2)), "narrow column groups exist for the K-split form only");
  typedef Kc<MODE> T;
  typedef typename T::acc_t acc_t;
  constexpr int BM = 16 * MT;
  constexpr bool W8H = MODE == KC_W8A16_F16 || MODE == KC_W8A16G_F16;     // int8 weights, f16 activations
  constexpr bool W8B = MODE == KC_W8A16_BF16 || MODE == KC_W8A16G_BF16;   // ... bf16 activations
  constexpr bool GW = MODE == KC_W8A16G_F16 || MODE == KC_W8A16G_BF16;    // group-wise weight scales
  constexpr int AV = T::ABYTES * 2;               // 16-byte vectors per lane per K block (activations)
  constexpr int WV = T::WBYTES * 2;               // ... weights
  // (the wavefront index is made visibly uniform: K-block offsets that depend on it are scalar operands of
  // the buffer loads, and a value the compiler cannot prove uniform costs a loop around every load)
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r16 = lane & 15, q = lane >> 4;
  const int N = a.N, K = a.K;
  const int KB = K >> 7;
  const int m0 = blockIdx.y * BM;
  long expert = 0;
  // slot ids of this lane's rows (row r16 of each row tile): one load per lane, in flight together with
  // the expert id and the block count -- a chain of dependent loads in front of the weight stream costs
  // one loaded memory latency each, per workgroup
  int tok[MT];
#pragma unroll
  for (int j = 0; j < MT; ++j) tok[j] = 0;
  if (GROUPED) {
    const int npp = *a.npp;
    expert = a.expert_ids[m0 / a.block_size];
#pragma unroll
    for (int j = 0; j < MT; ++j) tok[j] = a.sorted_ids[m0 + 16 * j + r16];   // (the array is padded to whole blocks)
    if (m0 >= npp) return;
    if (expert < 0 || expert >= a.E) {             // not one of this rank's experts: zero rows, no weights read
      const int col0 = blockIdx.x * 256;
      zero_block_columns((uint16_t*)a.out, a.sorted_ids + m0, BM, a.numel, N, col0, min(256, N - col0), 256);
      return;
    }
  }
  const int n0 = KS ? blockIdx.x * (16 * NI) : blockIdx.x * 256 + wave * 64;
  if (n0 >= N) return;
  // Operands are addressed through buffer descriptors: a 32-bit lane offset plus a scalar K-block offset
  // per load (no 64-bit address arithmetic in the loop; the host checks that one expert's weights, the
  // activations and their scales each stay below 4 GiB).
  const rsrc_t wres = make_rsrc((const char*)a.w + expert * a.w_stride * T::WBYTES, (uint32_t)((size_t)N * K * T::WBYTES));
  const uint32_t kstride = a.kslab ? 4 * 2048 * T::WBYTES : 128 * T::WBYTES;   // bytes between K blocks
  const uint32_t vstride = a.kslab ? 1024 : 16;                                 // ... between the 16-byte vectors of a lane
  uint32_t woff[NI];
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    if (a.kslab) {
      // (tile (n0 >> 4) + i of the layer: group of 64 columns, tile within the group)
      woff[i] = (uint32_t)((((size_t)(n0 >> 6) * KB) * 4 + ((n0 >> 4) & 3) + i) * (2048 * T::WBYTES) + lane * 16);
    } else {
      const int n = min(n0 + 16 * i + r16, N - 1);
      woff[i] = (uint32_t)(((size_t)n * K + 32 * q) * T::WBYTES);
    }
  }
  const int arows = GROUPED ? (a.numel + a.topk - 1) / a.topk : a.M;          // rows of the activation matrix
  const rsrc_t xres = make_rsrc(a.a, (uint32_t)((size_t)arows * K * T::ABYTES));
  const rsrc_t asres = make_rsrc(a.a_scale, MODE == KC_FP8_BLOCK ? (uint32_t)((size_t)arows * KB * 4) : 0u);
  uint32_t aoff[MT];
  int arow[MT];

  acc_t acc[NI][MT];
#pragma unroll
  for (int i = 0; i < NI; ++i)
#pragma unroll
    for (int j = 0; j < MT; ++j) acc[i][j] = (acc_t){0, 0, 0, 0};

  struct Blk {
    u4 w[NI][WV];
    u4 x[MT][AV];
    float as[MODE == KC_FP8_BLOCK ? MT : 1];
    float ws;
    uint2 gs[GW ? NI : 1][2];   // group-wise scales of this lane's 4 columns per row tile, per 64-wide half
  };
  const uint16_t* ws16 = (const uint16_t*)a.w_scale + expert * a.ws_stride;
  const int gper = GW ? 128 / a.wgroup : 1;        // scale groups per K block
  const float* wsf = (const float*)a.w_scale + expert * a.ws_stride;
  const rsrc_t wsres = make_rsrc(wsf, MODE == KC_FP8_BLOCK ? (uint32_t)((size_t)((N + 127) >> 7) * KB * 4) : 0u);
  const int wsrow = (n0 >> 7) * KB;
  auto load_w = [&](Blk& b, int kb) {
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
      for (int v = 0; v < WV; ++v)     // streamed once: non-temporal
        b.w[i][v] = bitcast<u4>(__builtin_amdgcn_raw_buffer_load_b128(wres, (int)woff[i], (int)(kb * kstride + v * vstride), 2));
    // one block scale per wavefront and K block: a scalar offset, no lane address
    if (MODE == KC_FP8_BLOCK) b.ws = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(wsres, 0, (wsrow + kb) * 4, 0));
    if (GW) {
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        const int n = min(n0 + 16 * i + 4 * q, N - 4);
#pragma unroll
        for (int h = 0; h < 2; ++h)
          b.gs[i][h] = *(const uint2*)(ws16 + (size_t)(kb * gper + min(h, gper - 1)) * N + n);
      }
    }
  };
  auto load_x = [&](Blk& b, int kb) {
#pragma unroll
    for (int j = 0; j < MT; ++j)
#pragma unroll
      for (int v = 0; v < AV; ++v)
        b.x[j][v] = bitcast<u4>(__builtin_amdgcn_raw_buffer_load_b128(xres, (int)(aoff[j] + 16 * v), kb * 128 * T::ABYTES, 0));
    if (MODE == KC_FP8_BLOCK) {
#pragma unroll
      for (int j = 0; j < MT; ++j)
        b.as[j] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(asres, arow[j] * KB * 4, kb * 4, 0));
    }
  };
  auto load_blk = [&](Blk& b, int kb) {
    load_w(b, kb);
    load_x(b, kb);
  };

  auto compute_blk = [&](const Blk& b, int kb) {
    if (MODE == KC_FP8_BLOCK) {
#pragma unroll
      for (int i = 0; i < NI; ++i)
#pragma unroll
        for (int j = 0; j < MT; ++j) {
          f4 part = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int v = 0; v < 2; ++v) {
            const u4 wv = b.w[i][v], xv = b.x[j][v];
            long w0 = (long)((unsigned long)wv[0] | ((unsigned long)wv[1] << 32));
            long w1 = (long)((unsigned long)wv[2] | ((unsigned long)wv[3] << 32));
            long x0 = (long)((unsigned long)xv[0] | ((unsigned long)xv[1] << 32));
            long x1 = (long)((unsigned long)xv[2] | ((unsigned long)xv[3] << 32));
            part = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(w0, x0, part, 0, 0, 0);
            part = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(w1, x1, part, 0, 0, 0);
          }
          const float sc = b.as[j] * b.ws;
          acc[i][j] = bitcast<acc_t>(bitcast<f4>(acc[i][j]) + sc * part);
        }
    } else if (MODE == KC_FP8_PC) {
      // scales live outside the K sum: the products of all K blocks go into one fp32 accumulator
#pragma unroll
      for (int i = 0; i < NI; ++i)
#pragma unroll
        for (int j = 0; j < MT; ++j) {
          f4 sum = bitcast<f4>(acc[i][j]);
#pragma unroll
          for (int v = 0; v < 2; ++v) {
            const u4 wv = b.w[i][v], xv = b.x[j][v];
            long w0 = (long)((unsigned long)wv[0] | ((unsigned long)wv[1] << 32));
            long w1 = (long)((unsigned long)wv[2] | ((unsigned long)wv[3] << 32));
            long x0 = (long)((unsigned long)xv[0] | ((unsigned long)xv[1] << 32));
            long x1 = (long)((unsigned long)xv[2] | ((unsigned long)xv[3] << 32));
            sum = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(w0, x0, sum, 0, 0, 0);
            sum = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(w1, x1, sum, 0, 0, 0);
          }
          acc[i][j] = bitcast<acc_t>(sum);
        }
    } else if (MODE == KC_INT8) {
#pragma unroll
      for (int i = 0; i < NI; ++i)
#pragma unroll
        for (int j = 0; j < MT; ++j)
#pragma unroll
          for (int v = 0; v < 2; ++v)
            acc[i][j] = bitcast<acc_t>(__builtin_amdgcn_mfma_i32_16x16x64_i8(
                bitcast<i4>(b.w[i][v]), bitcast<i4>(b.x[j][v]), bitcast<i4>(acc[i][j]), 0, 0, 0));
    } else {
      // 16-bit activations; weights 16-bit, or int8 converted on the fly
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        u4 wv[4];
        if (MODE == KC_F16 || MODE == KC_BF16) {
#pragma unroll
          for (int v = 0; v < 4; ++v) wv[v] = b.w[i][v % WV];
        } else if (W8H) {
          s8x16_to_f16(b.w[i][0], wv[0], wv[1]);
          s8x16_to_f16(b.w[i][WV - 1], wv[2], wv[3]);
        } else {
          s8x16_to_bf16(b.w[i][0], wv[0], wv[1]);
          s8x16_to_bf16(b.w[i][WV - 1], wv[2], wv[3]);
        }
#pragma unroll
        for (int j = 0; j < MT; ++j) {
          auto mma = [&](const u4& wop, int v, f4 c) {
            if (MODE == KC_F16 || W8H)
              return __builtin_amdgcn_mfma_f32_16x16x32_f16(bitcast<h8>(wop), bitcast<h8>(b.x[j][v % AV]), c, 0, 0, 0);
            return __builtin_amdgcn_mfma_f32_16x16x32_bf16(bitcast<b8>(wop), bitcast<b8>(b.x[j][v % AV]), c, 0, 0, 0);
          };
          if (!GW) {
            f4 sum = bitcast<f4>(acc[i][j]);
#pragma unroll
            for (int v = 0; v < 4; ++v) sum = mma(wv[v], v, sum);
            acc[i][j] = bitcast<acc_t>(sum);
          } else {
            // A lane holds 32 consecutive k (32 q ..), so a 64-wide scale group is a pair of
            // lane quarters, not a pair of steps: with two groups per K block each one is
            // multiplied on its own with the other quarters' weights zeroed.
#pragma unroll
            for (int h = 0; h < 2; ++h) {
              if (h >= gper) break;
              const bool mine = gper == 1 || (q >> 1) == h;
              f4 sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
              for (int v = 0; v < 4; ++v) sum = mma(mine ? wv[v] : (u4){0u, 0u, 0u, 0u}, v, sum);
              const uint2 sv = b.gs[i][h];
              f4 t = bitcast<f4>(acc[i][j]);
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                const uint32_t sw = e < 2 ? sv.x : sv.y;
                const uint16_t raw = (uint16_t)((e & 1) ? (sw >> 16) : (sw & 0xffffu));
                t[e] += sum[e] * (W8H ? Elem<MI355Q_F16>::to_f32(raw) : Elem<MI355Q_BF16>::to_f32(raw));
              }
              acc[i][j] = bitcast<acc_t>(t);
            }
          }
        }
      }
    }
    (void)kb;
  };

  {
    constexpr int kstep = KS ? 4 : 1;
    const int kfirst = KS ? wave : 0;
    Blk b0, b1;
    // the first weights are requested before the slot ids are looked at: they depend on the expert only
    // (unconditional where K is not split over the wavefronts: behind a branch the wait for the ids
    // below would have to cover both paths, i.e. wait for these requests too)
    if (!KS || kfirst < KB) load_w(b0, kfirst);
    __builtin_amdgcn_sched_barrier(0);               // (keeps the requests above in front of the wait for the ids)
#pragma unroll
    for (int j = 0; j < MT; ++j) {
      int row;
      if (GROUPED) row = min(tok[j], a.numel - 1) / a.topk;
      else row = min(m0 + 16 * j + r16, a.M - 1);
      arow[j] = row;
      aoff[j] = (uint32_t)(((size_t)row * K + 32 * q) * T::ABYTES);
    }
    if (!KS || kfirst < KB) {
      const int klast = kfirst + (KB - 1 - kfirst) / kstep * kstep;   // this wavefront's last block
      load_x(b0, kfirst);
      int kb = kfirst;
      while (true) {
        load_blk(b1, min(kb + kstep, klast));
        __builtin_amdgcn_sched_barrier(0);
        compute_blk(b0, kb);
        __builtin_amdgcn_sched_barrier(0);
        kb += kstep;
        if (kb >= KB) break;
        load_blk(b0, min(kb + kstep, klast));
        __builtin_amdgcn_sched_barrier(0);
        compute_blk(b1, kb);
        __builtin_amdgcn_sched_barrier(0);
        kb += kstep;
        if (kb >= KB) break;
      }
    }
  }

  acc_t fin[MT];
  // KS: wavefront w sums the four partial sums of column tile w (in wavefront order) and stores
  // it; two row tiles at a time go through LDS
  constexpr int RJ = MT < 2 ? MT : 2;
  __shared__ uint32_t red[KS ? 4 : 1][KS ? 4 * NI * RJ : 1][64];
  if (KS) {
#pragma unroll
    for (int jc = 0; jc < MT; jc += RJ) {
      if (jc) __syncthreads();
#pragma unroll
      for (int i = 0; i < NI; ++i)
#pragma unroll
        for (int j = 0; j < RJ; ++j)
#pragma unroll
          for (int e = 0; e < 4; ++e)
            red[KS ? wave : 0][KS ? (i * RJ + j) * 4 + e : 0][lane] = bitcast<u4>(acc[i][jc + j])[e];
      __syncthreads();
#pragma unroll
      for (int j = 0; j < RJ; ++j) {
        if (NI < 4 && wave >= NI) break;             // (fewer column tiles than wavefronts: the others only contributed)
        u4 t;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int slot = (wave * RJ + j) * 4 + e;
          if (MODE == KC_INT8) {
            int v = (int)red[0][KS ? slot : 0][lane];
#pragma unroll
            for (int w = 1; w < 4; ++w) v += (int)red[KS ? w : 0][KS ? slot : 0][lane];
            t[e] = (uint32_t)v;
          } else {
            float v = bitcast<float>(red[0][KS ? slot : 0][lane]);
#pragma unroll
            for (int w = 1; w < 4; ++w) v += bitcast<float>(red[KS ? w : 0][KS ? slot : 0][lane]);
            t[e] = bitcast<uint32_t>(v);
          }
        }
        fin[jc + j] = bitcast<acc_t>(t);
      }
    }
  }

  // ---- epilogue: lane holds row (l % 16) of each row tile and columns
  // n0 + 16 i + 4 q + {0..3}
  if (KS && NI < 4 && wave >= NI) return;
  const bool wide = !KS && a.wide_stores;
  const rsrc_t ores = make_rsrc(a.out, (uint32_t)((size_t)(GROUPED ? a.numel : a.M) * N * 2));
#pragma unroll
  for (int j = 0; j < MT; ++j) {
    int m;
    bool ok;
    float rw = 1.0f;
    if (GROUPED) {
      m = tok[j];
      ok = m < a.numel;
      if (ok && a.topk_weights) rw = a.topk_weights[m];
    } else {
      m = m0 + 16 * j + r16;
      ok = m < a.M;
    }
    if (!ok) continue;
    float xs = 1.0f;
    if ((MODE == KC_INT8 || MODE == KC_FP8_PC) && a.a_scale) xs = a.a_scale[arow[j] * a.sc_row];
    uint32_t held[2] = {0u, 0u};                   // packed outputs of the even column tile of a pair
#pragma unroll
    for (int i = 0; i < (KS ? 1 : 4); ++i) {
      const int n = n0 + 16 * (KS ? wave : i) + 4 * q;
      if (!wide && n >= N) continue;
      float v[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        if (wide && n >= N) { v[e] = 0.f; continue; }
        if (MODE == KC_INT8) {
          const float ws = ((const float*)a.w_scale)[expert * a.ws_stride + (n + e) * a.sc_col];
          v[e] = scaled_sum((float)bitcast<i4>(KS ? fin[j] : acc[i][j])[e], xs, ws);
        } else if (MODE == KC_FP8_PC) {
          const float ws = ((const float*)a.w_scale)[expert * a.ws_stride + (n + e) * a.sc_col];
          v[e] = scaled_sum(bitcast<f4>(KS ? fin[j] : acc[i][j])[e], xs, ws);
        } else if ((W8H || W8B) && !GW) {
          const uint16_t raw = ((const uint16_t*)a.w_scale)[expert * a.ws_stride + n + e];
          const float ws = W8H ? Elem<MI355Q_F16>::to_f32(raw) : Elem<MI355Q_BF16>::to_f32(raw);
          v[e] = bitcast<f4>(KS ? fin[j] : acc[i][j])[e] * ws;
        } else {
          v[e] = bitcast<f4>(KS ? fin[j] : acc[i][j])[e];
        }
        v[e] *= rw;
        if (!GROUPED && a.bias) v[e] = plus_bias(v[e], Elem<ODT>::to_f32(((const uint16_t*)a.bias)[n + e]));
      }
      u2 o;
      o.x = (uint32_t)Elem<ODT>::from_f32(v[0]) | ((uint32_t)Elem<ODT>::from_f32(v[1]) << 16);
      o.y = (uint32_t)Elem<ODT>::from_f32(v[2]) | ((uint32_t)Elem<ODT>::from_f32(v[3]) << 16);
      if (!wide) {
        *(u2*)((uint16_t*)a.out + (size_t)m * N + n) = o;
      } else if ((i & 1) == 0) {
        held[0] = o.x;
        held[1] = o.y;
      } else {
        // the lanes of a row that hold columns 4 q .. 4 q + 3 of two neighbouring column tiles trade
        // halves (v_permlane16_swap: lanes 16..31 of the first register with lanes 0..15 of the second,
        // likewise 48..63 with 32..47): lane q then holds 8 adjacent columns of tile i - 1 + (q & 1) and
        // a store instruction writes 64 contiguous bytes per row instead of 32
        const auto lo2 = __builtin_amdgcn_permlane16_swap(held[0], o.x, false, false);
        const auto hi2 = __builtin_amdgcn_permlane16_swap(held[1], o.y, false, false);
        const int nw = n0 + 16 * (i - 1 + (q & 1)) + 8 * (q >> 1);
        // written through (sc0 sc1): the scattered output rows leave the L2 as they are produced instead of
        // being evicted later in between the weight reads (1-2 % on the DeepSeek-style layer)
        if (nw < N)
          __builtin_amdgcn_raw_buffer_store_b128(
              bitcast<__attribute__((__vector_size__(4 * sizeof(unsigned int)))) unsigned int>((u4){lo2[0], hi2[0], lo2[1], hi2[1]}),
              ores, (int)(((size_t)m * N + nw) * 2), 0, 17);
      }
    }
  }
}

// row-major [batch, N, K] -> kslab: one 16-byte chunk per thread
__global__ void __launch_bounds__(256)
kslab_repack_kernel(const u4* src, u4* dst, long chunks, int N, int K, int wb) {
  const long c = (long)blockIdx.x * 256 + threadIdx.x;
  if (c >= chunks) return;
  const int wv = 2 * wb, KB = K >> 7;
  const long per_mat = (long)N * K * wb / 16;
  const long e = c / per_mat;
  long r = c - e * per_mat;
  const int lane = (int)(r & 63); r >>= 6;
  const int v = (int)(r % wv); r /= wv;
  const int i = (int)(r & 3); r >>= 2;
  const int kb = (int)(r % KB);
  const long ng = r / KB;
  const long n = ng * 64 + i * 16 + (lane & 15);
  const long byte = ((long)kb * 128 + 32 * (lane >> 4)) * wb + 16 * v;
  dst[c] = src[e * per_mat + (n * K * wb + byte) / 16];
}

template <int MODE, int ODT, bool GROUPED>
void launch_mt(const KcArgs& a, int mt, int row_blocks, hipStream_t st) {
  if constexpr (!GROUPED && !(MODE == KC_FP8_BLOCK || MODE == KC_FP8_PC || MODE == KC_INT8)) {
    // 16-bit activations have no 64-row form with K split inside the workgroup (registers), and 64-row
    // blocks of 256 columns are few on all but the widest layers at a few hundred rows (N 4096 at
    // M = 64: 16 workgroups, 79 us): 32-row blocks with the split instead, while they are too few
    // (K 4096, W8A16, us: N 4096 at M = 64 / 128 / 512: 79 / 78 / 80 -> 14 / 16 / 53; N 14336 at 64 / 128: 81 / 80 -> 31 / 57;
    // at 512 rows, 448 workgroups of 64 x 256, the 64-row blocks are ahead again: 156 against 169)
    if (mt == 4 && (long)((a.N + 255) / 256) * row_blocks * 2 < 3L * device_cu_count()) {
      mt = 2;
      row_blocks = (a.M + 31) / 32;
    }
  }
  dim3 grid((a.N + 255) / 256, row_blocks), block(256);
  if constexpr (!GROUPED) {
    // too few workgroups to fill the chip: split K inside the workgroup
    // (64-row launches only for one-byte weights x one-byte activations: the others run out of registers)
    if ((mt <= 2 || MODE == KC_FP8_BLOCK || MODE == KC_FP8_PC || MODE == KC_INT8) &&
        (a.N + 255) / 256 * row_blocks < 2 * device_cu_count()) {
      // a layer of few columns: 32 or 16 columns per workgroup, so that about every CU has one (up to
      // 64 rows with 8-bit weights and activations, up to 32 rows otherwise)
      constexpr bool BYTES = MODE == KC_FP8_BLOCK || MODE == KC_FP8_PC || MODE == KC_INT8;
      {
        const long cus = device_cu_count(), groups = (long)((a.N + 63) / 64) * row_blocks;
        if (mt <= (BYTES ? 4 : 2) && groups * 4 < cus * 3) {
          const bool one = groups * 8 < cus * 3;       // even 32-column workgroups would leave a quarter of the CUs idle
          dim3 gn(one ? (a.N + 15) / 16 : (a.N + 31) / 32, row_blocks);
          if (mt == 1 && one) hipLaunchKernelGGL((kcontig_gemm_kernel<MODE, ODT, 1, false, true, 1>), gn, block, 0, st, a);
          else if (mt == 1) hipLaunchKernelGGL((kcontig_gemm_kernel<MODE, ODT, 1, false, true, 2>), gn, block, 0, st, a);
          else if (mt == 2 && one) hipLaunchKernelGGL((kcontig_gemm_kernel<MODE, ODT, 2, false, true, 1>), gn, block, 0, st, a);
          else if (mt == 2) hipLaunchKernelGGL((kcontig_gemm_kernel<MODE, ODT, 2, false, true, 2>), gn, block, 0, st, a);
          else if constexpr (BYTES) {
            if (one) hipLaunchKernelGGL((kcontig_gemm_kernel<MODE, ODT, 4, false, true, 1>), gn, block, 0, st, a);
            else hipLaunchKernelGGL((kcontig_gemm_kernel<MODE, ODT, 4, false, true, 2>), gn, block, 0, st, a);
          }
          return;
        }
      }
      dim3 gks((a.N + 63) / 64, row_blocks);
      if (mt == 1) hipLaunchKernelGGL((kcontig_gemm_kernel<MODE, ODT, 1, false, true>), gks, block, 0, st, a);
      else if (mt == 2) hipLaunchKernelGGL((kcontig_gemm_kernel<MODE, ODT, 2, false, true>), gks, block, 0, st, a);
      else if constexpr (MODE == KC_FP8_BLOCK || MODE == KC_FP8_PC || MODE == KC_INT8) {
        if (mt == 4) hipLaunchKernelGGL((kcontig_gemm_kernel<MODE, ODT, 4, false, true>), gks, block, 0, st, a);
        else if constexpr (MODE == KC_FP8_BLOCK || MODE == KC_FP8_PC)
          hipLaunchKernelGGL((kcontig_gemm_kernel<MODE, ODT, 8, false, true>), gks, block, 0, st, a);
      }
      return;
    }
  }
  switch (mt) {
    case 1: hipLaunchKernelGGL((kcontig_gemm_kernel<MODE, ODT, 1, GROUPED>), grid, block, 0, st, a); break;
    case 2: hipLaunchKernelGGL((kcontig_gemm_kernel<MODE, ODT, 2, GROUPED>), grid, block, 0, st, a); break;
    default: hipLaunchKernelGGL((kcontig_gemm_kernel<MODE, ODT, 4, GROUPED>), grid, block, 0, st, a); break;
  }
}

template <bool GROUPED>
int launch_mode(const KcArgs& a, int mode, int odt, int mt, int row_blocks, hipStream_t st) {
#define KC_CASE(M_, O_) \
  if (mode == M_ && odt == O_) { launch_mt<M_, O_, GROUPED>(a, mt, row_blocks, st); return 0; }
  KC_CASE(KC_FP8_BLOCK, MI355Q_BF16)
  KC_CASE(KC_FP8_BLOCK, MI355Q_F16)
  KC_CASE(KC_FP8_PC, MI355Q_BF16)
  KC_CASE(KC_FP8_PC, MI355Q_F16)
  KC_CASE(KC_INT8, MI355Q_F16)
  KC_CASE(KC_INT8, MI355Q_BF16)
  KC_CASE(KC_F16, MI355Q_F16)
  KC_CASE(KC_BF16, MI355Q_BF16)
  KC_CASE(KC_W8A16_F16, MI355Q_F16)
  KC_CASE(KC_W8A16_BF16, MI355Q_BF16)
  KC_CASE(KC_W8A16G_F16, MI355Q_F16)
  KC_CASE(KC_W8A16G_BF16, MI355Q_BF16)
#undef KC_CASE
  set_error("kcontig_gemm: unsupported mode %d with output dtype %d", mode, odt);
  return 1;
}

int pick_mt(int rows) { return rows <= 16 ? 1 : (rows <= 32 ? 2 : 4); }

}  // namespace

int w4a16_grouped_launch(void* out, const void* x, const int32_t* qweight, const void* scales,
                         const float* scales_f32, const float* out_scale,
                         const void* zeros, int zeros_kind, const float* topk_weights,
                         const int32_t* sorted_ids, const int32_t* expert_ids, const int32_t* npp,
                         int numel, int topk, int block_size, int max_blocks, int E, int K, int N,
                         int group_size, int dtype, void* workspace, size_t workspace_bytes, hipStream_t st);
size_t w4a16_grouped_workspace_bytes(int numel, int block_size, int max_blocks, int E, int K, int N);
int int8_grouped_launch(void* out, const void* a, const void* w, const float* a_scale, int a_scale_per_row,
                        const float* w_scale, const float* topk_weights, const int32_t* sorted_ids,
                        const int32_t* expert_ids, const int32_t* npp, int numel, int topk, int block_size, int max_blocks,
                        int E, int K, int N, int out_dtype, int w_kslab, hipStream_t st);
int fp8_block_grouped_launch(void* out, const void* a, const void* w, const float* a_scale, const float* w_scale,
                             const float* topk_weights, const int32_t* sorted_ids, const int32_t* expert_ids,
                             const int32_t* npp, int numel, int topk, int block_size, int max_blocks, int E, int K, int N,
                             int out_dtype, int w_kslab, hipStream_t st);

int half_grouped_tile_launch(void* out, const void* a, const void* w, const float* topk_weights,
                             const int32_t* sorted_ids, const int32_t* expert_ids, const int32_t* npp, int numel, int topk,
                             int block_size, int max_blocks, int E, int K, int N, int dtype, int w_kslab, hipStream_t st);

// fp8 x fp8 with scales outside the K sum (per token or one value; per output channel or one value), M <= 128:
// the weight-streaming kernel.  Arguments are checked by the caller (mi355q_fp8_scaled_gemm).
int kcontig_fp8_pc_launch(void* out, const void* a, const void* w, const float* a_scale, int scale_per_row,
                          const float* w_scale, int scale_per_col, const void* bias, int M, int K, int N,
                          int out_dtype, int w_layout, hipStream_t st) {
  KcArgs g = {};
  g.out = out; g.a = a; g.w = w; g.a_scale = a_scale; g.w_scale = w_scale; g.bias = bias;
  g.M = M; g.N = N; g.K = K; g.kslab = w_layout;
  g.sc_row = scale_per_row ? 1 : 0;
  g.sc_col = scale_per_col ? 1 : 0;
  g.wide_stores = (N % 8 == 0 && ((size_t)out & 15) == 0 && (size_t)M * N * 2 < ((size_t)1 << 32)) ? 1 : 0;
  g.numel = M; g.topk = 1; g.block_size = 64;
  int mt = pick_mt(M < 64 ? M : 64);
  if (M > 64 && M <= 128 && (N + 255) / 256 < 2 * device_cu_count()) mt = 8;   // one 128-row block: weights streamed once
  const int row_blocks = (M + 16 * mt - 1) / (16 * mt);
  int rc = launch_mode<false>(g, KC_FP8_PC, out_dtype, mt, row_blocks, st);
  if (rc) return rc;
  MQ_LAUNCH_CHECK("fp8_scaled_gemm");
  return 0;
}

}  // namespace mi355q

using namespace mi355q;

extern "C" size_t mi355q_moe_gemm_workspace_bytes(int quant_mode, int numel, int block_size, int max_blocks, int E,
                                                  int K, int N) {
  if (quant_mode != 0 || numel <= 0 || K <= 0 || N <= 0 || K % 128 || N % 128) return 0;
  return w4a16_grouped_workspace_bytes(numel, block_size, max_blocks, E, K, N);
}

// quant_mode of the MoE / dense entry points
//   0 = W4A16 (slab-layout int4), 1 = fp8 block-scaled, 2 = int8 per-token x per-channel,
//   3 = unquantised 16-bit, 4 = W8A16 (int8 weights, per-channel scale in the activation dtype)
extern "C" int mi355q_moe_gemm(void* out, const void* a, const void* w, const float* a_scale,
                               const void* w_scale, const void* w_zeros, int zeros_kind, int quant_mode,
                               int group_size, const float* topk_weights, const int32_t* sorted_token_ids,
                               const int32_t* expert_ids, const int32_t* num_tokens_post_pad, int numel,
                               int topk, int block_size, int max_blocks, int E, int K, int N, int act_dtype,
                               int out_dtype, int w_layout, void* workspace, size_t workspace_bytes,
                               void* stream) {
  MQ_REQUIRE(numel >= 0 && topk > 0 && E > 0 && K > 0 && N > 0, "moe_gemm: bad shape");
  if (numel == 0 || max_blocks == 0) return 0;
  MQ_REQUIRE(out && a && w && sorted_token_ids && expert_ids && num_tokens_post_pad, "moe_gemm: null pointer");
  MQ_REQUIRE(block_size >= 16 && block_size % 16 == 0, "moe_gemm: block_size=%d must be a multiple of 16", block_size);
  MQ_REQUIRE(K % 128 == 0, "moe_gemm: K=%d must be a multiple of 128", K);
  hipStream_t st = as_stream(stream);
  if (quant_mode == 0) {
    MQ_REQUIRE(N % 128 == 0, "moe_gemm(w4a16): N=%d must be a multiple of 128", N);
    MQ_REQUIRE(w_scale, "moe_gemm(w4a16): scales missing");
    MQ_REQUIRE(out_dtype == act_dtype, "moe_gemm(w4a16): output dtype must equal the activation dtype");
    return w4a16_grouped_launch(out, a, (const int32_t*)w, w_scale, nullptr, nullptr, w_zeros, zeros_kind,
                                topk_weights, sorted_token_ids, expert_ids, num_tokens_post_pad, numel, topk,
                                block_size, max_blocks, E, K, N, group_size <= 0 ? K : group_size, act_dtype,
                                workspace, workspace_bytes, st);
  }
  if (quant_mode == 5) {
    MQ_REQUIRE(N % 128 == 0, "moe_gemm(w4, fp32 scales): N=%d must be a multiple of 128", N);
    MQ_REQUIRE(w_scale, "moe_gemm(w4, fp32 scales): scales missing");
    MQ_REQUIRE(out_dtype == act_dtype, "moe_gemm(w4, fp32 scales): output dtype must equal the activation dtype");
    MQ_REQUIRE(!w_zeros && zeros_kind == MI355Q_ZP_NONE, "moe_gemm(w4, fp32 scales): symmetric weights only");
    return w4a16_grouped_launch(out, a, (const int32_t*)w, nullptr, (const float*)w_scale, a_scale, nullptr,
                                MI355Q_ZP_NONE, topk_weights, sorted_token_ids, expert_ids, num_tokens_post_pad,
                                numel, topk, block_size, max_blocks, E, K, N, group_size <= 0 ? K : group_size,
                                act_dtype, nullptr, 0, st);
  }
  MQ_REQUIRE(N % 4 == 0, "moe_gemm: N=%d must be a multiple of 4", N);
  MQ_REQUIRE(w_layout == 0 || (w_layout == 1 && N % 64 == 0), "moe_gemm: weight layout %d needs N=%d %% 64 == 0", w_layout, N);
  MQ_REQUIRE((size_t)N * K * 2 < ((size_t)1 << 32) && ((size_t)numel / topk + 1) * K * 2 < ((size_t)1 << 32),
             "moe_gemm: one expert's weights and the activations must each stay below 4 GiB (N=%d K=%d, %d slots)", N, K, numel);
  KcArgs g = {};
  g.out = out; g.a = a; g.w = w; g.a_scale = a_scale; g.w_scale = w_scale; g.bias = nullptr;
  g.M = numel; g.N = N; g.K = K; g.kslab = w_layout;
  g.sc_row = g.sc_col = 1;
  g.wide_stores = (N % 8 == 0 && ((size_t)out & 15) == 0 && (size_t)numel * N * 2 < ((size_t)1 << 32)) ? 1 : 0;
  g.sorted_ids = sorted_token_ids; g.expert_ids = expert_ids; g.npp = num_tokens_post_pad;
  g.topk_weights = topk_weights; g.numel = numel; g.topk = topk; g.block_size = block_size; g.E = E;
  g.w_stride = (long)N * K;
  int mode;
  if (quant_mode == 1) {
    MQ_REQUIRE(a_scale && w_scale, "moe_gemm(fp8): scales missing");
    MQ_REQUIRE(group_size == 128, "moe_gemm(fp8): only 128x128 block scales are supported, got %d", group_size);
    // blocks of 256 slots (prefill token counts): the MFMA tile kernel with gathered rows
    // (blocks of 128 -- also a block size of the weight-streaming kernel -- from 40 rows per expert on average)
    if ((block_size == 256 || (block_size == 128 && (long)numel >= 40L * E)) && N % 128 == 0)
      return fp8_block_grouped_launch(out, a, w, a_scale, (const float*)w_scale, topk_weights, sorted_token_ids, expert_ids,
                                      num_tokens_post_pad, numel, topk, block_size, max_blocks, E, K, N, out_dtype,
                                      w_layout, st);
    mode = KC_FP8_BLOCK;
    g.ws_stride = (long)((N + 127) / 128) * (K / 128);
  } else if (quant_mode == 2) {
    MQ_REQUIRE(w_scale, "moe_gemm(int8): weight scales missing");
    // blocks of 256 slots (prefill token counts): the MFMA tile kernel with gathered rows
    if ((block_size == 256 || (block_size == 128 && (long)numel >= 40L * E)) && a_scale)
      return int8_grouped_launch(out, a, w, a_scale, 1, (const float*)w_scale, topk_weights, sorted_token_ids, expert_ids,
                                 num_tokens_post_pad, numel, topk, block_size, max_blocks, E, K, N, out_dtype,
                                 w_layout, st);
    mode = KC_INT8;
    g.ws_stride = N;
  } else if (quant_mode == 3) {
    // blocks of 256 / 128 slots (prefill token counts): the MFMA tile kernel with gathered rows
    if ((block_size == 256 || (block_size == 128 && (long)numel >= 40L * E)) && N % 128 == 0 && out_dtype == act_dtype)
      return half_grouped_tile_launch(out, a, w, topk_weights, sorted_token_ids, expert_ids, num_tokens_post_pad, numel,
                                      topk, block_size, max_blocks, E, K, N, act_dtype, w_layout, st);
    mode = act_dtype == MI355Q_F16 ? KC_F16 : KC_BF16;
  } else if (quant_mode == 4) {
    MQ_REQUIRE(w_scale, "moe_gemm(w8a16): weight scales missing");
    if (group_size <= 0 || group_size == K) {
      mode = act_dtype == MI355Q_F16 ? KC_W8A16_F16 : KC_W8A16_BF16;
      g.ws_stride = N;
    } else {
      MQ_REQUIRE(group_size == 64 || group_size == 128, "moe_gemm(w8a16): group size %d must be 64, 128 or per channel", group_size);
      mode = act_dtype == MI355Q_F16 ? KC_W8A16G_F16 : KC_W8A16G_BF16;
      g.wgroup = group_size;
      g.ws_stride = (long)(K / group_size) * N;
    }
  } else {
    MQ_REQUIRE(false, "moe_gemm: unknown quant_mode %d", quant_mode);
  }
  // row tiles per workgroup: the align block, capped at 64 rows
  const int rows_per_wg = block_size >= 64 ? 64 : block_size;
  MQ_REQUIRE(block_size % rows_per_wg == 0 && (rows_per_wg == 16 || rows_per_wg == 32 || rows_per_wg == 64),
             "moe_gemm: block_size=%d unsupported", block_size);
  const int row_blocks = max_blocks * (block_size / rows_per_wg);
  int rc = launch_mode<true>(g, mode, out_dtype, pick_mt(rows_per_wg), row_blocks, st);
  if (rc) return rc;
  MQ_LAUNCH_CHECK("moe_gemm");
  return 0;
}

extern "C" int mi355q_kcontig_gemm(void* out, const void* a, const void* w, const float* a_scale,
                                   const void* w_scale, const void* bias, int quant_mode, int group_size,
                                   int M, int K, int N, int act_dtype, int out_dtype, int w_layout, void* stream) {
  MQ_REQUIRE(M >= 0 && K > 0 && N > 0, "kcontig_gemm: bad shape M=%d K=%d N=%d", M, K, N);
  if (M == 0) return 0;
  MQ_REQUIRE(out && a && w, "kcontig_gemm: null pointer");
  MQ_REQUIRE(K % 128 == 0 && N % 4 == 0, "kcontig_gemm: K=%d must be a multiple of 128 and N=%d of 4", K, N);
  MQ_REQUIRE(w_layout == 0 || (w_layout == 1 && N % 64 == 0), "kcontig_gemm: weight layout %d needs N=%d %% 64 == 0", w_layout, N);
  MQ_REQUIRE((size_t)N * K * 2 < ((size_t)1 << 32) && (size_t)M * K * 2 < ((size_t)1 << 32),
             "kcontig_gemm: the weights and the activations must each stay below 4 GiB (M=%d N=%d K=%d)", M, N, K);
  KcArgs g = {};
  g.out = out; g.a = a; g.w = w; g.a_scale = a_scale; g.w_scale = w_scale; g.bias = bias;
  g.M = M; g.N = N; g.K = K; g.kslab = w_layout;
  g.sc_row = g.sc_col = 1;
  g.wide_stores = (N % 8 == 0 && ((size_t)out & 15) == 0 && (size_t)M * N * 2 < ((size_t)1 << 32)) ? 1 : 0;
  g.numel = M; g.topk = 1; g.block_size = 64;
  int mode;
  if (quant_mode == 1) {
    MQ_REQUIRE(a_scale && w_scale, "kcontig_gemm(fp8): scales missing");
    MQ_REQUIRE(group_size == 128, "kcontig_gemm(fp8): only 128x128 block scales are supported, got %d", group_size);
    mode = KC_FP8_BLOCK;
  } else if (quant_mode == 2) {
    MQ_REQUIRE(w_scale, "kcontig_gemm(int8): weight scales missing");
    mode = KC_INT8;
  } else if (quant_mode == 3) {
    mode = act_dtype == MI355Q_F16 ? KC_F16 : KC_BF16;
  } else if (quant_mode == 4) {
    MQ_REQUIRE(w_scale, "kcontig_gemm(w8a16): weight scales missing");
    if (group_size <= 0 || group_size == K) {
      mode = act_dtype == MI355Q_F16 ? KC_W8A16_F16 : KC_W8A16_BF16;
    } else {
      MQ_REQUIRE(group_size == 64 || group_size == 128, "kcontig_gemm(w8a16): group size %d must be 64, 128 or per channel", group_size);
      mode = act_dtype == MI355Q_F16 ? KC_W8A16G_F16 : KC_W8A16G_BF16;
      g.wgroup = group_size;
    }
  } else {
    MQ_REQUIRE(false, "kcontig_gemm: unknown quant_mode %d", quant_mode);
  }
  int mt = pick_mt(M < 64 ? M : 64);
  // 65..128 rows of fp8: one 128-row block, so that the weights are streamed once (the launch then
  // always splits K inside the workgroup, see launch_mt; K 8192, N 28672: 87..119 us against 139 us.
  // The int8 variant of it spills and is slower than the MFMA tile kernel.)
  if (mode == KC_FP8_BLOCK && M > 64 && M <= 128 &&
      (N + 255) / 256 < 2 * device_cu_count())
    mt = 8;
  const int row_blocks = (M + 16 * mt - 1) / (16 * mt);
  int rc = launch_mode<false>(g, mode, out_dtype, mt, row_blocks, as_stream(stream));
  if (rc) return rc;
  MQ_LAUNCH_CHECK("kcontig_gemm");
  return 0;
}

extern "C" int mi355q_kslab_repack(const void* src, void* dst, int batch, int N, int K, int elem_bytes,
                                   void* stream) {
  MQ_REQUIRE(batch > 0 && N > 0 && K > 0, "kslab_repack: bad shape batch=%d N=%d K=%d", batch, N, K);
  MQ_REQUIRE(src && dst && src != dst, "kslab_repack: needs distinct source and destination");
  MQ_REQUIRE(N % 64 == 0 && K % 128 == 0, "kslab_repack: N=%d must be a multiple of 64 and K=%d of 128", N, K);
  MQ_REQUIRE(elem_bytes == 1 || elem_bytes == 2, "kslab_repack: element size %d must be 1 or 2", elem_bytes);
  const long chunks = (long)batch * N * K * elem_bytes / 16;
  hipLaunchKernelGGL(kslab_repack_kernel, dim3((unsigned)((chunks + 255) / 256)), dim3(256), 0, as_stream(stream),
                     (const u4*)src, (u4*)dst, chunks, N, K, elem_bytes);
  MQ_LAUNCH_CHECK("kslab_repack");
  return 0;
}
