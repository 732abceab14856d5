// fp8-e4m3 block-scaled GEMM for prefill-sized M on the gfx950 fp8 MFMA
// (v_mfma_f32_16x16x32_fp8_fp8), with the 128 x 128 block scales applied to
// the fp32 partial sum of every K block.
//
//   out[m, n] = sum_kb x_scale[m, kb] * w_scale[n / 128, kb] * sum_{k in block kb} x[m, k] * w[n, k]
//
// Same machinery as the int8 GEMM next door: a workgroup of eight wavefronts
// (4 x 2, each 64 rows of x by 64 rows of w) owns a 256 x 128 output tile; K
// advances in LDS tiles of 128 bytes per row, which is exactly one scale block;
// tiles go from global memory straight into LDS (16 B per lane, no staging
// registers; 16-byte-chunk XOR swizzle, or chunk-major for kslab weights) in
// two stages; operand reads are hand-written and hand-waited for.  The tile is
// 128 columns wide because each K block needs its own set of partial
// accumulators next to the running sum (2 x 64 registers per lane); 128 columns
// are also exactly one scale block, so the weight scale of a tile and K block
// is a single number.  The activation scales of a K block (one per row) travel
// with the x tile through LDS (4-byte direct-to-LDS copies).
#include "common.h"

namespace mi355q {
namespace {

constexpr int FTM = 256, FTN = 128, FTKB = 128;
constexpr int F8_THREADS = 512;

struct F8Args {
  void* out;                // [M, N] f16 / bf16, row stride ldo elements
  const uint8_t* x;         // [M, K] fp8, row stride ldx bytes
  const uint8_t* w;         // [N, K] fp8 row-major (row stride ldw) or in the kslab order
  const float* x_scale;     // [M, K / 128]
  const float* w_scale;     // [N / 128, K / 128]
  const void* bias;         // [N] in the output dtype or null
  int M, N, K;
  long ldx, ldw, ldo;
  int w_kslab;
  int n_panels_swizzle;
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

__device__ __forceinline__ long lo64(i4 v) { return (long)((unsigned long)(uint32_t)v[0] | ((unsigned long)(uint32_t)v[1] << 32)); }
__device__ __forceinline__ long hi64(i4 v) { return (long)((unsigned long)(uint32_t)v[2] | ((unsigned long)(uint32_t)v[3] << 32)); }

template <int DT>
__global__ void __launch_bounds__(F8_THREADS, 1)
fp8_block_gemm_kernel(F8Args a) {
  constexpr int WN = 2, NI = 4, NJ = 4;                 // 4 x 2 wavefronts of 64 x 64
  constexpr int X_BYTES = FTM * FTKB, W_BYTES = FTN * FTKB, XS_BYTES = FTM * 4;
  constexpr int STAGE_BYTES = X_BYTES + W_BYTES + XS_BYTES;
  constexpr int XCOPIES = FTM / 8 / 8, WCOPIES = FTN / 8 / 8;       // 1 KiB copies per wavefront
  extern __shared__ __align__(16) unsigned char lds[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l16 = lane & 15, kq = lane >> 4;
  const int wm = wave / WN, wn = wave % WN;
  const int M = a.M, N = a.N, K = a.K, KB = K >> 7;

  const int mtiles = (M + FTM - 1) / FTM;
  const int ntiles_n = N / FTN;
  const int total_tiles = mtiles * ntiles_n;
  auto tile_origin = [&](int tile, int& m0, int& n0) {
    int tm, tn;
    if (a.n_panels_swizzle) {
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

  f4 acc[NI][NJ], part[NI][NJ];

  // global -> LDS: lane = 8 * row + slot, slot p of row r receives chunk p ^ (r & 7); kslab weights
  // chunk-major (lane = 8 * position + row, position p of an odd 8-row group holding chunk p ^ 1)
  const int crow = lane >> 3, cchunk = (lane & 7) ^ (crow & 7);
  uint32_t xo[XCOPIES], wo[WCOPIES], xso = 0;
  const uint8_t *xtile, *wtile;
  auto set_copy_tile = [&](int tile) {
    int m0, n0;
    tile_origin(tile, m0, n0);
#pragma unroll
    for (int p = 0; p < XCOPIES; ++p) {
      const int r = (wave + 8 * p) * 8 + crow;
      xo[p] = (uint32_t)((min(m0 + r, M - 1) - m0) * a.ldx + 16 * cchunk);
    }
#pragma unroll
    for (int p = 0; p < WCOPIES; ++p) {
      if (a.w_kslab) {
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
    xso = (uint32_t)min(m0 + 64 * (wave & 3) + lane, M - 1) * (uint32_t)KB;
    xtile = a.x + (long)m0 * a.ldx;
    wtile = a.w_kslab ? a.w : a.w + (long)n0 * a.ldw;
  };
  constexpr int NSLOT = XCOPIES + WCOPIES + 1;
  auto copy_slot = [&](int s, int stage, int kt) {
    unsigned char* xs = lds + stage * STAGE_BYTES;
    if (s < XCOPIES) {
      dma16(xtile + (long)kt * FTKB + xo[s], xs + (wave + 8 * s) * 1024);
    } else if (s < XCOPIES + WCOPIES) {
      const int p = s - XCOPIES;
      dma16(wtile + (a.w_kslab ? (long)kt * FTKB * 64 : (long)kt * FTKB) + wo[p < WCOPIES ? p : 0],
            xs + X_BYTES + (wave + 8 * p) * 1024);
    } else if (wave < 4) {
      dma4(a.x_scale + xso + kt, xs + X_BYTES + W_BYTES + wave * 256);
    }
  };
  auto issue = [&](int stage, int kt) {
#pragma unroll
    for (int s = 0; s < NSLOT; ++s) copy_slot(s, stage, kt);
  };

  // operand reads (assembly, waited for by hand: see the int8 kernel)
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
  struct Frag { i4 bx[NJ]; i4 aw[NI]; };
  auto read_one = [&](Frag& f, int r, uint32_t xb, uint32_t wb) {
#pragma unroll
    for (int j = 0; j < NJ; ++j)
      if (r == j) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(f.bx[j]) : "v"(xb), "n"(j * 16 * FTKB));
#pragma unroll
    for (int i = 0; i < NI; ++i)
      if (r == NJ + i) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(f.aw[i]) : "v"(wb), "n"(i * 16 * FTKB));
  };
  auto read_frag = [&](Frag& f, int stage, int h) {
    const uint32_t xb = lo[h] + (uint32_t)(stage * STAGE_BYTES) + xwave;
    const uint32_t wb = wlo[h] + (uint32_t)(stage * STAGE_BYTES) + wwave;
#pragma unroll
    for (int r = 0; r < NJ + NI; ++r) read_one(f, r, xb, wb);
  };
  auto lds_wait = [&](Frag& f) {
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(f.bx[0]), "+v"(f.bx[1]), "+v"(f.bx[2]), "+v"(f.bx[3]), "+v"(f.aw[0]), "+v"(f.aw[1]),
                   "+v"(f.aw[2]), "+v"(f.aw[3]));
  };
  // the activation scales of this lane's four row tiles (rows wm * 64 + 16 j + l16) for one K block
  float xsv[NJ];
  auto read_xs = [&](int stage) {
    const uint32_t ad = xsaddr + (uint32_t)(stage * STAGE_BYTES);
#pragma unroll
    for (int j = 0; j < NJ; ++j)
      asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(xsv[j]) : "v"(ad), "n"(j * 64));
  };
  auto xs_wait = [&]() {
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(xsv[0]), "+v"(xsv[1]), "+v"(xsv[2]), "+v"(xsv[3]));
  };

  // One half of a K block: 2 MFMAs (k = 32 each) per (w tile i, x tile j).  Between them: the
  // LDS reads of the next operand set, one per pair for the first eight pairs, and copy slots
  // SB .. SE-1 of a later K block, one after every other pair.  The second half adds the block's
  // partial sums to the running sums with the block's scale.
  float sc[NJ];
  auto half = [&](const Frag& cur, Frag& nxt, int rstage, int rh, bool second, int SB, int SE, int cstage, int kt) {
    const uint32_t xb = lo[rh] + (uint32_t)(rstage * STAGE_BYTES) + xwave;
    const uint32_t wb = wlo[rh] + (uint32_t)(rstage * STAGE_BYTES) + wwave;
    int n = 0;
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        f4 c = second ? part[i][j] : (f4){0.f, 0.f, 0.f, 0.f};
        c = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(lo64(cur.aw[i]), lo64(cur.bx[j]), c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(hi64(cur.aw[i]), hi64(cur.bx[j]), c, 0, 0, 0);
        part[i][j] = c;
        // the block's partial sum joins the running sum one pair later, when the MFMA has delivered it
        if (second && n > 0) {
          const int pi = (n - 1) / NJ, pj = (n - 1) % NJ;
          acc[pi][pj] += sc[pj] * part[pi][pj];
        }
        __builtin_amdgcn_sched_barrier(0);
        if (n < NJ + NI) read_one(nxt, n, xb, wb);
        if ((n & 1) && SB + (n >> 1) < SE) copy_slot(SB + (n >> 1), cstage, kt);
        __builtin_amdgcn_sched_barrier(0);
        ++n;
      }
    if (second) acc[NI - 1][NJ - 1] += sc[NJ - 1] * part[NI - 1][NJ - 1];
  };
  static_assert(NI * NJ >= NJ + NI && NI * NJ / 2 >= NSLOT, "not enough MFMA pairs to spread the copies and reads");

  // Stream of K blocks across this workgroup's output tiles, two LDS stages
  // (element g in stage g % 2): half 0 of element g multiplies (g, 0) while it
  // reads (g, 1) and the block's activation scales; half 1 multiplies (g, 1),
  // reads (g + 1, 0) and issues the copy of element g + 2 into g's stage.
  const int nt = KB;
  // (kept in a register: read through the dispatch packet it is fetched again in every iteration)
  const int gdim = __builtin_amdgcn_readfirstlane((int)gridDim.x);
  int tile = blockIdx.x;
  set_copy_tile(tile);
  issue(0, 0);
  issue(1, min(1, nt - 1));
  int copy_tile = tile;
  if (nt == 1 && tile + gdim < total_tiles) {
    copy_tile = tile + gdim;
    set_copy_tile(copy_tile);
    issue(1, 0);
  }
  __builtin_amdgcn_s_waitcnt(0x0f70);              // vmcnt(0)
  __builtin_amdgcn_s_barrier();
  Frag f0, f1;
  read_frag(f0, 0, 0);
  lds_wait(f0);
  int g = 0;
  for (; tile < total_tiles; tile += gdim) {
    int m0, n0;
    tile_origin(tile, m0, n0);
    const float* wsp = a.w_scale + (long)(n0 >> 7) * KB;
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
      for (int j = 0; j < NJ; ++j) acc[i][j] = (f4){0.f, 0.f, 0.f, 0.f};
    for (int T = 0; T < nt; ++T, ++g) {
      const int st = g & 1;
      const float wsv = wsp[T];
      read_xs(st);
      half(f0, f1, st, 1, false, 0, 0, st, 0);
      lds_wait(f1);
      xs_wait();
#pragma unroll
      for (int j = 0; j < NJ; ++j) sc[j] = xsv[j] * wsv;
      __builtin_amdgcn_s_waitcnt(0x0f70);          // vmcnt(0): my copies of element g + 1 landed
      __builtin_amdgcn_s_barrier();
      int kt = T + 2, ahead = 0;
      while (kt >= nt) { kt -= nt; ++ahead; }
      const int want = tile + ahead * gdim;
      if (want >= total_tiles) kt = nt - 1;        // past the end: harmless re-read, never consumed
      else if (want != copy_tile) { set_copy_tile(want); copy_tile = want; }
      half(f1, f0, st ^ 1, 0, true, 0, NSLOT, st, kt);
      lds_wait(f0);
    }

    // ---- epilogue: lane holds, per (w tile i, x tile j), output row m = .. + l16 and columns
    // n = .. + 4 kq + {0..3}
    float bia[NI][4];
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int n = n0 + wn * (16 * NI) + i * 16 + 4 * kq;
#pragma unroll
      for (int e = 0; e < 4; ++e) bia[i][e] = a.bias ? Elem<DT>::to_f32(((const uint16_t*)a.bias)[n + e]) : 0.0f;
    }
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const int m = m0 + wm * (16 * NJ) + j * 16 + l16;
      if (m >= M) continue;
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        const int n = n0 + wn * (16 * NI) + i * 16 + 4 * kq;
        u2 o;
        o.x = (uint32_t)Elem<DT>::from_f32(acc[i][j][0] + bia[i][0]) | ((uint32_t)Elem<DT>::from_f32(acc[i][j][1] + bia[i][1]) << 16);
        o.y = (uint32_t)Elem<DT>::from_f32(acc[i][j][2] + bia[i][2]) | ((uint32_t)Elem<DT>::from_f32(acc[i][j][3] + bia[i][3]) << 16);
        *(u2*)((uint16_t*)a.out + (long)m * a.ldo + n) = o;
      }
    }
    read_frag(f0, g & 1, 0);
    lds_wait(f0);
  }
  // no copy may still be writing LDS when the workgroup retires
  __builtin_amdgcn_s_waitcnt(0x0f70);              // vmcnt(0)
}

template <int DT>
int launch_f8(const F8Args& a, hipStream_t st) {
  const int mtiles = (a.M + FTM - 1) / FTM, ntiles = a.N / FTN;
  F8Args b = a;
  b.n_panels_swizzle = (ntiles % 8 == 0) ? 1 : 0;
  const size_t shmem = 2 * (size_t)(FTM * FTKB + FTN * FTKB + FTM * 4);
  static hipError_t attr = hipFuncSetAttribute((const void*)fp8_block_gemm_kernel<DT>,
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
  MQ_REQUIRE(attr == hipSuccess, "fp8_block_gemm: cannot reserve %zu bytes of LDS: %s", shmem, hipGetErrorString(attr));
  int grid = mtiles * ntiles, cus = device_cu_count() / 8 * 8;
  if (cus >= 8 && grid > cus) grid = cus;
  hipLaunchKernelGGL((fp8_block_gemm_kernel<DT>), dim3(grid), dim3(F8_THREADS), shmem, st, b);
  MQ_LAUNCH_CHECK("fp8_block_gemm");
  return 0;
}

}  // namespace
}  // namespace mi355q

using namespace mi355q;

extern "C" int mi355q_fp8_block_gemm(void* out, const void* x, const void* w, const float* x_scale,
                                     const float* w_scale, const void* bias, int M, int N, int K, long ldx,
                                     long ldw, long ldo, int out_dtype, void* stream) {
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
  if (out_dtype == MI355Q_F16) return launch_f8<MI355Q_F16>(a, as_stream(stream));
  return launch_f8<MI355Q_BF16>(a, as_stream(stream));
}
