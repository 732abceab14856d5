// W4A16 MFMA GEMM in which every operand reaches the CU through a ring of LDS stages (fp16).
//
// One workgroup per CU owns all rows of a block (16 MT, up to 128) of 512, 256 or 128 columns and walks K
// (or its share of K) in blocks of 128.  Everything a K block needs -- the activation rows, the packed
// weights, the group scales and zero-points -- is copied from global memory straight into a ring of LDS
// stages (global_load_lds, 16 B per lane, no staging registers) several K blocks ahead; the ring is the
// latency cover that a second workgroup per CU provides in the 64-row tile kernel.  Each of the eight
// wavefronts (two per SIMD: one wavefront alone issues an instruction every five or six clocks, too
// few for the matrix pipe) owns all row tiles of TW = 4, 2 or 1 of the 16-column tiles: no weight is
// dequantised twice.  B operands are scaled, (q - z) * s rounded to fp16 -- the dequantised weight the
// operator is defined on -- so the matrix instructions accumulate in place.
//
// Three uses: above 128 rows (TW = 2 or 4, workgroups of 256 or 512 columns, row blocks in blockIdx.y)
// where a round model prices it below the 64-row tiles, and from 33 to 128 rows (TW = 1, workgroups of
// 128 columns: twice the workgroups, so K needs half the splits) where a workgroup walks ten K blocks
// or more.  With TW = 4 an activation operand read from LDS feeds four matrix instructions instead of
// two -- the LDS reads per matrix instruction fall from 0.75 to 0.5 and the copies per column from a
// 128-row block of activations per 256 columns to one per 512 -- at the price of a ring of two stages
// instead of three and of registers: the 128 accumulators of the 8 x 4 tiles leave room for a ring of
// four activation operands and one set of packed weights, read twice per K block.
//
// The copies are issued from inline assembly, so the compiler does not know of them: it schedules and
// waits for the LDS reads itself (lgkmcnt), and the waits for the copies (vmcnt) are written by hand.
// No load that the compiler can see is in flight while a copy is (prologue and epilogue drain first).
#include "common.h"

namespace mi355q {

int w4a16_splitk_reduce_launch(void* out, const float* partial, const void* bias, int M, int N, int splits,
                               int dtype, hipStream_t st);

namespace {

struct MidArgs {
  uint16_t* out;
  const uint16_t* x;
  const u4* qw;
  const uint16_t* scales;
  const void* zeros;
  const uint16_t* bias;
  int M, K, N;
  int kper;                   // K blocks per split (blockIdx.z)
  uint32_t gpk, gpk_magic;    // K blocks per group and ceil(2^32 / gpk)
  float* partial;             // split K: fp32 tiles [split][M][N]; null: write the output
  // IOBF kernels (bf16 rows staged as fp16 times a power of two each; scales, bias and output bf16):
  const float* row_scale;     // [M] the power of two each staged row has to be multiplied back by
  const uint32_t* scale_max;  // [64] largest scale magnitude (bf16 bits) of 64 slices of the scales array
};

// TW: 16-column tiles per wavefront -- 2: a workgroup of 256 columns; 4: of 512 columns (128 rows only);
// 1: of 128 columns (one slab), for launches of up to 128 rows, where 256-column workgroups are too few
// to fill the chip without splitting K
template <int MT, int TW>
struct MidCfg {
  static constexpr int BM = 16 * MT;
  static constexpr int BNW = 128 * TW;                // columns per workgroup
  static constexpr int A_BYTES = BM * 256;            // 128 halves per row
  static constexpr int W_OFF = A_BYTES;               // 8 wavefronts x TW column tiles x 1 KiB
  static constexpr int SZ_OFF = A_BYTES + 8192 * TW;  // 8 wavefronts x (256 B of scales + 256 B of zero-points)
  static constexpr int STAGE = A_BYTES + 8192 * TW + 4096;
  static constexpr int D = (160 * 1024 - 1024) / STAGE < 6 ? (160 * 1024 - 1024) / STAGE : 6;   // stages in the ring
  static constexpr int XC = MT >= 2 ? MT / 2 : 1;     // activation copies (4 rows each) per wavefront and stage
};

// 64 lanes x 16 B from saddr + voff into LDS at lds_addr + 16 * lane
__device__ __forceinline__ void dma16(uint32_t voff, const void* sbase, uint32_t lds_addr) {
  // (uniform by construction; inside a divergent region the compiler may otherwise keep it in a vector register)
  lds_addr = __builtin_amdgcn_readfirstlane(lds_addr);
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               :
               : "v"(voff), "s"(sbase), "s"(lds_addr)
               : "memory");
}

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}

struct MidDq {
  uint32_t magic, mlo, mhi;
};

// Pair p (0..3) of one packed word -> two of the 8 weights of an MFMA K step, (q - z) * s in fp16,
// as the 32-bit word p of the B operand.  zlo = 1024 + z, zhi = 64 + z (PRESCALED: 1024 and 64, and
// zs = z * s is subtracted after the scaling).  Three or four instructions: the K loop deals them out
// between the matrix instructions instead of dequantising an operand in one burst.
template <int ZK>
__device__ __forceinline__ uint32_t mid_dequant_pair(uint32_t w, int p, _Float16 zlo1, _Float16 zhi1, _Float16 s1,
                                                     _Float16 zs1, const MidDq& k) {
  const h2 zlo = {zlo1, zlo1}, zhi = {zhi1, zhi1}, ss = {s1, s1}, zs = {zs1, zs1};
  const h2 sixteenth = {(_Float16)0.0625f, (_Float16)0.0625f};
  const uint32_t ws = (p & 2) ? w >> 8 : w;
  h2 r;
  if (p & 1) {
    const h2 a = bitcast<h2>((ws & k.mhi) | k.magic);  // 1024 + 16 q
    r = __builtin_elementwise_fma(a, sixteenth, -zhi);
  } else {
    const h2 a = bitcast<h2>((ws & k.mlo) | k.magic);  // 1024 + q
    r = a - zlo;
  }
  if (ZK == MI355Q_ZP_PRESCALED) r = __builtin_elementwise_fma(r, ss, -zs);
  else r *= ss;
  return bitcast<uint32_t>(r);
}

// IOBF: the activations are bf16 rows that a pass before this kernel stored as fp16 times a power of
// two each; the scales are bf16 and become fp16 here, times one power of two for the whole array that
// brings the largest of them into [2^10, 2^11) -- (q - z) s stays below fp16's largest number and a
// scale 2^24 below the largest one still keeps all its bits; the epilogue undoes both powers of two
// exactly (one ldexp per output) and rounds to bf16.
template <int ZK, int MT, int TW, bool IOBF = false>
__global__ void __launch_bounds__(512, 1)
w4a16_mid_kernel(MidArgs a) {
  static_assert(!IOBF || ZK != MI355Q_ZP_PRESCALED, "pre-scaled zero-points stay with the bf16 kernel");
  typedef MidCfg<MT, TW> C;
  constexpr int D = C::D, STAGE = C::STAGE, XC = C::XC;
  constexpr bool HASZ = ZK != MI355Q_ZP_NONE;
  constexpr int NSLOT = XC + TW + 1;                  // copy slots per wavefront and stage (the last: scales + zeros)
  constexpr int NC = XC + TW + 1 + (HASZ ? 1 : 0);    // copy instructions per wavefront and stage
  static_assert((D - 1) * NC <= 63, "vmcnt is a 6-bit counter");
  extern __shared__ __align__(16) unsigned char lds[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c = lane & 15, kq = lane >> 4;
  const int N = a.N, K = a.K, M = a.M, G = K >> 7;
  const int m0 = blockIdx.y * C::BM;
  // N may end in the middle of a 256-column tile: the wavefronts of the missing slab work on the
  // previous one and their columns are never stored
  const int wslab = TW == 4 ? wave >> 1 : TW == 2 ? wave >> 2 : 0;   // slab of the workgroup this wavefront works on
  const bool live = (blockIdx.x * TW + wslab) < (N >> 7);
  const int slab = live ? blockIdx.x * TW + wslab : (N >> 7) - 1;
  const int t0 = TW == 4 ? (wave & 1) * 4 : TW == 2 ? (wave & 3) * 2 : wave;   // first of this wavefront's TW tiles of the slab
  const int gb = (int)blockIdx.z * a.kper, ge = min(G, gb + a.kper);
  const uint32_t lds_base =
      __builtin_amdgcn_readfirstlane((uint32_t)(size_t)(__attribute__((address_space(3))) unsigned char*)lds);
  int sshift = 0;                                     // IOBF: scales are multiplied by 2^sshift
  if (IOBF) {
    uint32_t mx = a.scale_max[lane];
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const uint32_t other = (uint32_t)__shfl_xor((int)mx, o, 64);
      mx = mx > other ? mx : other;
    }
    const int expo = (int)(mx >> 7);
    if (mx != 0 && expo != 255) sshift = 10 - ((expo > 0 ? expo : 1) - 127);
    sshift = __builtin_amdgcn_readfirstlane(sshift);
  }

  // ---- copies.  Activations: one copy moves 4 rows of 256 B; lane = 16 * row + position, and position p
  // of row r receives the row's 16-byte chunk p ^ (r & 15), which keeps the MFMA operand reads (16 rows x
  // one chunk index per quarter wavefront) on 16 different bank groups.  Wavefront v copies row groups
  // v, v + 8, ...; rows past M re-read the last row (their results are never stored).
  uint32_t xo[XC];
#pragma unroll
  for (int p = 0; p < XC; ++p) {
    const int r = 4 * (wave + 8 * p) + (lane >> 4);
    const int row = min(m0 + r, M - 1);
    xo[p] = ((uint32_t)row * (uint32_t)K + 8u * (uint32_t)((lane & 15) ^ (r & 15))) * 2u;
  }
  const uint32_t lane16 = (uint32_t)lane * 16u;
  const uint32_t zlane = ZK == MI355Q_ZP_PACKED ? (uint32_t)(lane & 3) * 16u : lane16;
  const char* const xg = (const char*)a.x;
  const char* const wg = (const char*)a.qw + ((size_t)slab * G * 8 + t0) * 1024;
  const char* const sg = (const char*)a.scales + 256 * slab;
  const char* const zg = (const char*)a.zeros + (ZK == MI355Q_ZP_PACKED ? 64 : 256) * slab;
  const uint32_t zrow = ZK == MI355Q_ZP_PACKED ? (uint32_t)N / 2u : (uint32_t)N * 2u;
  // The workgroups of one split start together and stay roughly in step, and K block g of every
  // activation row lies a multiple of 8 KiB (Llama shapes) from that of the next: all of them would ask
  // the same few L2 channels for the same bytes at the same time.  Each column tile therefore walks its K
  // range from a different starting block (and wraps round): iteration i is K block gb + (rot + i) % nk.
  const int nk = ge - gb;
  const int rot = (int)(blockIdx.x % (unsigned)nk);
  auto copy_slot = [&](int s, int slot, int i) {
    const uint32_t sb = lds_base + (uint32_t)(slot * STAGE);
    int gq = rot + min(i, nk - 1);                    // past the end: a re-read into a stage nobody reads
    gq = gb + (gq >= nk ? gq - nk : gq);
    if (s < XC) {
      dma16(xo[s < XC ? s : 0], xg + (size_t)gq * 256, sb + (uint32_t)((wave + 8 * s) * 1024));
    } else if (s < XC + TW) {
      const int t = s - XC;
      dma16(lane16, wg + (size_t)gq * 8192 + t * 1024, sb + (uint32_t)(C::W_OFF + wave * 1024 * TW + t * 1024));
    } else {
      const uint32_t qrow = a.gpk_magic ? (uint32_t)(((uint64_t)(uint32_t)gq * a.gpk_magic) >> 32) : (uint32_t)gq;
      if (lane < 16) {
        dma16(lane16, sg + (size_t)qrow * N * 2, sb + (uint32_t)(C::SZ_OFF + wave * 512));
        if (HASZ) dma16(zlane, zg + (size_t)qrow * zrow, sb + (uint32_t)(C::SZ_OFF + wave * 512 + 256));
      }
    }
  };

  // ---- LDS reads (plain loads: the compiler places the waits)
  const uint32_t a_lane = (uint32_t)(c * 256);
  uint32_t a_pos[4];
#pragma unroll
  for (int st = 0; st < 4; ++st) a_pos[st] = a_lane + (uint32_t)(((4 * st + kq) ^ c) * 16);
  auto read_a = [&](int slot, int mt, int st) {
    return bitcast<h8>(*(const u4*)(lds + slot * STAGE + a_pos[st] + mt * 4096));
  };
  auto read_w = [&](u4 (&w)[TW], int slot) {
#pragma unroll
    for (int t = 0; t < TW; ++t) w[t] = *(const u4*)(lds + slot * STAGE + C::W_OFF + wave * 1024 * TW + t * 1024 + lane * 16);
  };
  struct Sz { uint2 s; uint2 zs; uint32_t z; };
  auto read_sz = [&](Sz& q, int slot) {
    const unsigned char* p = lds + slot * STAGE + C::SZ_OFF + wave * 512;
    // (one tile per wavefront: t0 may be odd, the 32-bit read starts at the even column below it)
    const int te = t0 & ~1;
    if (TW == 4) q.s = *(const uint2*)(p + (8 * c + t0) * 2);
    else q.s.x = *(const uint32_t*)(p + (8 * c + te) * 2) >> (16 * (t0 & 1));
    if (ZK == MI355Q_ZP_PACKED) q.z = *(const uint32_t*)(p + 256 + c * 4) >> (4 * t0);
    if (ZK == MI355Q_ZP_PRESCALED) {
      if (TW == 4) q.zs = *(const uint2*)(p + 256 + (8 * c + t0) * 2);
      else q.zs.x = *(const uint32_t*)(p + 256 + (8 * c + te) * 2) >> (16 * (t0 & 1));
    }
  };
  // per column tile: scale, 1024 + z, 64 + z, z * s
  _Float16 sc[TW], zlo[TW], zhi[TW], zsc[TW];
  auto prep = [&](const Sz& q) {
#pragma unroll
    for (int t = 0; t < TW; ++t) {
      const uint32_t sw = t < 2 ? q.s.x : q.s.y;
      if (IOBF) sc[t] = (_Float16)__builtin_ldexpf(bitcast<float>((t & 1) ? (sw & 0xffff0000u) : (sw << 16)), sshift);
      else sc[t] = bitcast<_Float16>((uint16_t)((t & 1) ? (sw >> 16) : (sw & 0xffffu)));
      if (ZK == MI355Q_ZP_PRESCALED) {
        const uint32_t zw = t < 2 ? q.zs.x : q.zs.y;
        zsc[t] = bitcast<_Float16>((uint16_t)((t & 1) ? (zw >> 16) : (zw & 0xffffu)));
        zlo[t] = (_Float16)1024.0f;
        zhi[t] = (_Float16)64.0f;
      } else {
        // fp16 bit patterns directly: 1024 + z = 0x6400 | z, 64 + z = 0x5400 | z << 4
        const uint32_t z = ZK == MI355Q_ZP_PACKED ? (q.z >> (4 * t)) & 15u : 8u;
        zlo[t] = bitcast<_Float16>((uint16_t)(0x6400u | z));
        zhi[t] = bitcast<_Float16>((uint16_t)(0x5400u | (z << 4)));
        zsc[t] = (_Float16)0.0f;
      }
    }
  };
  MidDq dqk = {0x64006400u, 0x000f000fu, 0x00f000f0u};
  asm volatile("" : "+v"(dqk.magic));
  asm volatile("" : "+s"(dqk.mlo));
  asm volatile("" : "+s"(dqk.mhi));

  f4 acc[MT][TW];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int t = 0; t < TW; ++t) acc[mt][t] = (f4){0.f, 0.f, 0.f, 0.f};

  // ---- prologue: the whole ring is requested, the first stage awaited
#pragma unroll
  for (int d = 0; d < D; ++d)
#pragma unroll
    for (int s = 0; s < NSLOT; ++s) copy_slot(s, d, d);
  wait_vmcnt<(D - 1) * NC>();
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  // A operands travel through a small ring of registers: group j (K step j / MT, row tile j % MT) uses
  // entry j % R and requests the operand of group j + PF.  A whole K step ahead where the registers
  // allow (R = 2 MT entries); with four column tiles per wavefront the 128 accumulator registers leave
  // room for a ring of four, three groups (twelve matrix instructions) ahead -- and for one set of
  // packed weights instead of two, re-read when its last word has been dequantised.
  constexpr int PF = TW == 4 ? 3 : MT, R = TW == 4 ? 4 : 2 * MT;
  constexpr bool WDB = TW != 4;                        // two sets of packed weights that swap roles per K block
  static_assert((4 * MT) % R == 0, "the ring index of a group is the same in every K block");
  u4 w0[TW], w1[WDB ? TW : 1];
  Sz sz;
  h8 av[R];
  u4 bv[2][TW];
  read_w(w0, 0);
  read_sz(sz, 0);
#pragma unroll
  for (int j = 0; j < PF; ++j) av[j % R] = read_a(0, j % MT, j / MT);
  prep(sz);
#pragma unroll
  for (int t = 0; t < TW; ++t)
#pragma unroll
    for (int p = 0; p < 4; ++p) bv[0][t][p] = mid_dequant_pair<ZK>(w0[t][0], p, zlo[t], zhi[t], sc[t], zsc[t], dqk);

  constexpr int NP = 4 * TW;                          // operand words dequantised per K step, dealt out over the MT groups
  constexpr int JX = 4 * MT - PF;                     // first group whose request goes to the next stage
  constexpr int CPG = (NSLOT + PF - 1) / PF;          // copy slots issued per group from there on
  int slot = 0;
  // One K block: four K steps of MT groups of TW matrix instructions, with the group's other work dealt
  // out behind them (a matrix instruction occupies its pipe for four issue slots).  While step st
  // multiplies, the B operands of step st + 1 are dequantised.  In step 2 the wavefront's own copies of
  // the next stage are awaited and its scales (and, with two weight sets, packed weights) read.  Before
  // group JX every LDS read of this stage has been issued and awaited: after the barrier there the stage
  // is refilled with K block i + D while the first A operands of block i + 1 are requested.
  auto kblock = [&](int i, u4 (&wc)[TW], u4 (&wn)[TW]) __attribute__((always_inline)) {
    const int nslot = slot + 1 == D ? 0 : slot + 1;
#pragma unroll
    for (int st = 0; st < 4; ++st) {
      const int cur = st & 1, nxt = cur ^ 1;
      if (st == 2) {
        wait_vmcnt<(D - 2) * NC>();
        if (WDB) read_w(wn, nslot);
        read_sz(sz, nslot);
      }
      if (st == 3) {
        if (!WDB) read_w(wn, nslot);                  // (its own copies: no barrier needed; wc and wn are one array)
        prep(sz);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const int j = st * MT + mt, jn = j + PF;
        if (j == JX) {
          asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
          __builtin_amdgcn_s_barrier();
          asm volatile("" ::: "memory");
          __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int t = 0; t < TW; ++t) {
          acc[mt][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av[j % R], bitcast<h8>(bv[cur][t]), acc[mt][t], 0, 0, 0);
          __builtin_amdgcn_sched_barrier(0);
          if (t == 0) {
            av[jn % R] = jn < 4 * MT ? read_a(slot, jn % MT, jn / MT) : read_a(nslot, (jn - 4 * MT) % MT, (jn - 4 * MT) / MT);
            if (j >= JX) {
#pragma unroll
              for (int sl = (j - JX) * CPG; sl < (j - JX + 1) * CPG && sl < NSLOT; ++sl) copy_slot(sl, slot, i + D);
            }
          }
          // the operand words of this group (word q belongs to group q * MT / NP), dealt out over its TW slices
          int k = 0;
#pragma unroll
          for (int q = 0; q < NP; ++q) {
            if (q * MT / NP != mt) continue;
            if (k++ % TW != (TW == 1 ? 0 : (t + 1) % TW)) continue;
            const int tt = q >> 2, p = q & 3;
            bv[nxt][tt][p] = mid_dequant_pair<ZK>(st < 3 ? wc[tt][st + 1] : wn[tt][0], p, zlo[tt], zhi[tt], sc[tt], zsc[tt], dqk);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
    slot = nslot;
  };
  for (int i = 0;; i += 2) {
    if (WDB) kblock(i, w0, (u4(&)[TW])w1);
    else kblock(i, w0, w0);
    if (i + 1 >= nk) break;
    if (WDB) kblock(i + 1, (u4(&)[TW])w1, w0);
    else kblock(i + 1, w0, w0);
    if (i + 2 >= nk) break;
  }
  // no copy may still be writing LDS when the workgroup retires, and none may be in flight next to the
  // loads below
  wait_vmcnt<0>();

  // ---- epilogue through LDS (the ring is free now): a lane holds TW adjacent columns of 4 rows per row
  // tile, which as stores would touch a few bytes in every 32; written to an fp32 tile in LDS and read
  // back row by row, every store instruction writes whole rows of the workgroup's columns.  (512 columns:
  // the tile goes through in two halves of 64 rows.)
  constexpr int EP = C::BNW * 4 + 16;                  // bytes per tile row in LDS
  constexpr int HALVES = TW == 4 ? 2 : 1, MTH = MT / HALVES;
  static_assert(16 * MTH * EP <= D * STAGE, "the output tile fits in the ring");
  // 4 columns per lane: a wavefront instruction covers part of a row, one row or two rows
  constexpr int LPR = C::BNW / 4;                      // lanes per row
  constexpr int RPI = LPR >= 64 ? 1 : 64 / LPR, IPR = LPR >= 64 ? LPR / 64 : 1;   // rows per instruction, instructions per row
  typedef Elem<IOBF ? MI355Q_BF16 : MI355Q_F16> IO;
  f4 bs[IPR];
#pragma unroll
  for (int q = 0; q < IPR; ++q) {
    bs[q] = (f4){0.f, 0.f, 0.f, 0.f};
    const int col = blockIdx.x * C::BNW + 4 * (lane % LPR) + 256 * q;
    if (a.bias && !a.partial && col < N) {
      const uint2 bw = *(const uint2*)(a.bias + col);
      bs[q] = (f4){IO::to_f32((uint16_t)(bw.x & 0xffffu)), IO::to_f32((uint16_t)(bw.x >> 16)),
                   IO::to_f32((uint16_t)(bw.y & 0xffffu)), IO::to_f32((uint16_t)(bw.y >> 16))};
    }
  }
#pragma unroll
  for (int h = 0; h < HALVES; ++h) {
    __syncthreads();                                   // every wavefront has left the K loop (or the half before)
    {
      unsigned char* base = lds + (128 * wslab + 8 * c + t0) * 4;
#pragma unroll
      for (int mh = 0; mh < MTH; ++mh)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int mt = h * MTH + mh;
          unsigned char* q = base + (mh * 16 + 4 * kq + i) * EP;
          if (TW == 4) *(f4*)q = (f4){acc[mt][0][i], acc[mt][1 % TW][i], acc[mt][2 % TW][i], acc[mt][3 % TW][i]};
          else if (TW == 2) *(f2*)q = (f2){acc[mt][0][i], acc[mt][TW - 1][i]};
          else *(float*)q = acc[mt][0][i];
        }
    }
    __syncthreads();
#pragma unroll
    for (int p = 0; p < 2 * MTH / RPI; ++p) {
      const int r = RPI * (wave + 8 * p) + (LPR >= 64 ? 0 : lane / LPR), m = m0 + h * 16 * MTH + r;
      if (m >= M) break;
      // IOBF: the row's power of two and the scales' in one exponent
      int back = 0;
      if (IOBF) back = (int)((bitcast<uint32_t>(a.row_scale[m]) >> 23) & 255u) - 127 - sshift;
#pragma unroll
      for (int q = 0; q < IPR; ++q) {
        const int col = blockIdx.x * C::BNW + 4 * (lane % LPR) + 256 * q;
        if (col >= N) continue;
        f4 v = *(const f4*)(lds + r * EP + (lane % LPR) * 16 + 1024 * q);
        if (IOBF) {
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = __builtin_ldexpf(v[e], back);
        }
        if (a.partial) {
          *(f4*)(a.partial + ((size_t)blockIdx.z * M + m) * N + col) = v;
        } else {
          uint2 o;
          o.x = (uint32_t)IO::from_f32(v[0] + bs[q][0]) | ((uint32_t)IO::from_f32(v[1] + bs[q][1]) << 16);
          o.y = (uint32_t)IO::from_f32(v[2] + bs[q][2]) | ((uint32_t)IO::from_f32(v[3] + bs[q][3]) << 16);
          *(uint2*)(a.out + (size_t)m * N + col) = o;
        }
      }
    }
  }
}

template <int ZK, int MT, int TW>
int launch_mid(const MidArgs& a, int row_blocks, int splits, hipStream_t st) {
  typedef MidCfg<MT, TW> C;
  const size_t shmem = (size_t)C::D * C::STAGE;
  static hipError_t attr = hipFuncSetAttribute((const void*)w4a16_mid_kernel<ZK, MT, TW>,
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
  MQ_REQUIRE(attr == hipSuccess, "w4a16_gemm(mid): cannot reserve %zu bytes of LDS: %s", shmem, hipGetErrorString(attr));
  dim3 grid((a.N + C::BNW - 1) / C::BNW, row_blocks, splits);
  hipLaunchKernelGGL((w4a16_mid_kernel<ZK, MT, TW>), grid, dim3(512), shmem, st, a);
  MQ_LAUNCH_CHECK("w4a16_gemm(mid)");
  return 0;
}

// bf16 rows staged as fp16: 128-row workgroups of 256 or 512 columns, no K split
template <int ZK, int TW>
int launch_mid_iobf(const MidArgs& a, int row_blocks, hipStream_t st) {
  typedef MidCfg<8, TW> C;
  const size_t shmem = (size_t)C::D * C::STAGE;
  static hipError_t attr = hipFuncSetAttribute((const void*)w4a16_mid_kernel<ZK, 8, TW, true>,
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
  MQ_REQUIRE(attr == hipSuccess, "w4a16_gemm(mid): cannot reserve %zu bytes of LDS: %s", shmem, hipGetErrorString(attr));
  dim3 grid((a.N + C::BNW - 1) / C::BNW, row_blocks, 1);
  hipLaunchKernelGGL((w4a16_mid_kernel<ZK, 8, TW, true>), grid, dim3(512), shmem, st, a);
  MQ_LAUNCH_CHECK("w4a16_gemm(mid, bf16 staged)");
  return 0;
}

template <int ZK>
int launch_mid_mt(const MidArgs& a, int mt, int tw, int row_blocks, int splits, hipStream_t st) {
  if (tw == 4) return launch_mid<ZK, 8, 4>(a, row_blocks, splits, st);
  if (tw == 1) {
    if (mt <= 2) return launch_mid<ZK, 2, 1>(a, row_blocks, splits, st);
    if (mt <= 4) return launch_mid<ZK, 4, 1>(a, row_blocks, splits, st);
    return launch_mid<ZK, 8, 1>(a, row_blocks, splits, st);
  }
  if (mt <= 2) return launch_mid<ZK, 2, 2>(a, row_blocks, splits, st);
  if (mt <= 4) return launch_mid<ZK, 4, 2>(a, row_blocks, splits, st);
  return launch_mid<ZK, 8, 2>(a, row_blocks, splits, st);
}

}  // namespace

// Row tiles of 16 per workgroup for M rows: the smallest of 2, 4, 8 that holds them all, 8 beyond.
static int mid_rows_mt(int M) { return M <= 32 ? 2 : M <= 64 ? 4 : 8; }

// K splits: as many as still fit the chip in one round (one workgroup per CU), each at least four K
// blocks long and the partial tiles within 64 MiB.
int w4a16_mid_splits(int M, int K, int N, int tw) {
  const int mt = mid_rows_mt(M), G = K / 128, bn = 128 * tw;
  const long wgs = (long)((M + 16 * mt - 1) / (16 * mt)) * ((N + bn - 1) / bn);
  const long cus = device_cu_count();
  long s = cus / wgs;
  if (s > G / 4) s = G / 4;
  while (s > 1 && (size_t)s * M * N * sizeof(float) > ((size_t)64 << 20)) --s;
  if (s < 1) s = 1;
  const int kper = (int)((G + s - 1) / s);
  return (G + kper - 1) / kper;
}

size_t w4a16_mid_workspace_bytes(int M, int K, int N) {
  const int s = w4a16_mid_splits(M, K, N, 2);
  return s > 1 ? (size_t)s * M * N * sizeof(float) : 0;
}

// fp16 activations, group sizes that are multiples of 128.  `splits` 0: the plan above.
int w4a16_mid_launch(void* out, const void* x, const int32_t* qweight, const void* scales, const void* zeros,
                     int zeros_kind, const void* bias, int M, int K, int N, int group_size, int dtype,
                     void* workspace, size_t workspace_bytes, int splits, int tw, hipStream_t st) {
  MQ_REQUIRE(dtype == MI355Q_F16 && group_size % 128 == 0,
             "w4a16_gemm(mid): fp16 and group sizes that are multiples of 128 only (dtype %d, group %d)", dtype, group_size);
  MQ_REQUIRE((size_t)M * K * 2 < ((size_t)1 << 32), "w4a16_gemm: activation matrix %d x %d is 4 GiB or more", M, K);
  const int G = K / 128;
  if (tw != 1 && tw != 4) tw = 2;
  if (splits <= 0) splits = w4a16_mid_splits(M, K, N, tw);
  if (splits > G) splits = G;
  if (splits > 1 && (!workspace || workspace_bytes < (size_t)splits * M * N * sizeof(float))) splits = 1;
  MidArgs a = {};
  a.out = (uint16_t*)out;
  a.x = (const uint16_t*)x;
  a.qw = (const u4*)qweight;
  a.scales = (const uint16_t*)scales;
  a.zeros = zeros;
  a.bias = (const uint16_t*)bias;
  a.M = M; a.K = K; a.N = N;
  a.kper = (G + splits - 1) / splits;
  splits = (G + a.kper - 1) / a.kper;                  // no empty splits
  a.gpk = (uint32_t)group_size / 128u;
  a.gpk_magic = a.gpk > 1 ? (uint32_t)((((uint64_t)1 << 32) + a.gpk - 1) / a.gpk) : 0u;
  a.partial = splits > 1 ? (float*)workspace : nullptr;
  const int mt = mid_rows_mt(M);
  const int row_blocks = (M + 16 * mt - 1) / (16 * mt);
  int rc;
  if (zeros_kind == MI355Q_ZP_NONE) rc = launch_mid_mt<MI355Q_ZP_NONE>(a, mt, tw, row_blocks, splits, st);
  else if (zeros_kind == MI355Q_ZP_PACKED) rc = launch_mid_mt<MI355Q_ZP_PACKED>(a, mt, tw, row_blocks, splits, st);
  else rc = launch_mid_mt<MI355Q_ZP_PRESCALED>(a, mt, tw, row_blocks, splits, st);
  if (rc) return rc;
  if (splits > 1) return w4a16_splitk_reduce_launch(out, (const float*)workspace, bias, M, N, splits, dtype, st);
  return 0;
}

// The same kernels on bf16 rows that the caller staged as fp16 (x16, one power of two per row in
// row_scale); scales, bias and output are bf16, scale_max holds the largest scale magnitude of 64 slices
// of the scales array.  128-row workgroups of 256 (tw 2) or 512 (tw 4) columns, K unsplit.
int w4a16_mid_launch_staged(void* out, const void* x16, const int32_t* qweight, const void* scales, const void* zeros,
                            int zeros_kind, const void* bias, int M, int K, int N, int group_size,
                            const float* row_scale, const uint32_t* scale_max, int tw, hipStream_t st) {
  MQ_REQUIRE(group_size % 128 == 0 && zeros_kind != MI355Q_ZP_PRESCALED && row_scale && scale_max && M > 64,
             "w4a16_gemm(mid, bf16 staged): group %d, zero-point kind %d, M %d not covered", group_size, zeros_kind, M);
  MidArgs a = {};
  a.out = (uint16_t*)out;
  a.x = (const uint16_t*)x16;
  a.qw = (const u4*)qweight;
  a.scales = (const uint16_t*)scales;
  a.zeros = zeros;
  a.bias = (const uint16_t*)bias;
  a.M = M; a.K = K; a.N = N;
  a.kper = K / 128;
  a.gpk = (uint32_t)group_size / 128u;
  a.gpk_magic = a.gpk > 1 ? (uint32_t)((((uint64_t)1 << 32) + a.gpk - 1) / a.gpk) : 0u;
  a.row_scale = row_scale;
  a.scale_max = scale_max;
  const int row_blocks = (M + 127) / 128;
  if (zeros_kind == MI355Q_ZP_NONE)
    return tw == 4 ? launch_mid_iobf<MI355Q_ZP_NONE, 4>(a, row_blocks, st) : launch_mid_iobf<MI355Q_ZP_NONE, 2>(a, row_blocks, st);
  return tw == 4 ? launch_mid_iobf<MI355Q_ZP_PACKED, 4>(a, row_blocks, st) : launch_mid_iobf<MI355Q_ZP_PACKED, 2>(a, row_blocks, st);
}

}  // namespace mi355q
