// Shared helpers for the gfx950 kernels: error reporting, vector types,
// small device utilities.  Everything here is internal to the library.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/mi355q.h"

namespace mi355q {

// ---- host-side error plumbing ---------------------------------------------
void set_error(const char* fmt, ...);

#define MQ_REQUIRE(cond, ...)                 \
  do {                                        \
    if (!(cond)) {                            \
      ::mi355q::set_error(__VA_ARGS__);       \
      return 1;                               \
    }                                         \
  } while (0)

#define MQ_LAUNCH_CHECK(what)                                              \
  do {                                                                     \
    hipError_t e__ = hipGetLastError();                                    \
    if (e__ != hipSuccess) {                                               \
      ::mi355q::set_error("%s: launch failed: %s", what,                   \
                          hipGetErrorString(e__));                         \
      return 2;                                                            \
    }                                                                      \
  } while (0)

// ---- vector types ----------------------------------------------------------
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef __bf16 b8 __attribute__((ext_vector_type(8)));
typedef short s8v __attribute__((ext_vector_type(8)));
typedef float f2 __attribute__((ext_vector_type(2)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f16v __attribute__((ext_vector_type(16)));
typedef int i4 __attribute__((ext_vector_type(4)));
typedef int i16v __attribute__((ext_vector_type(16)));
typedef uint32_t u2 __attribute__((ext_vector_type(2)));
typedef uint32_t u4 __attribute__((ext_vector_type(4)));

template <typename T, typename U>
__device__ __forceinline__ T bitcast(const U& u) {
  static_assert(sizeof(T) == sizeof(U), "bitcast size");
  return __builtin_bit_cast(T, u);
}

// bf16 -> f32 is a shift; f32 -> bf16 is the hardware conversion of gfx950 (v_cvt_pk_bf16_f32:
// round to nearest even, NaN stays NaN), one instruction where the bit manipulation took six
__device__ __forceinline__ float bf16_to_f32(uint16_t v) {
  return bitcast<float>((uint32_t)v << 16);
}
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
  return bitcast<uint16_t>((__bf16)f);
}

// Epilogue of the scaled integer / fp8 GEMMs, (sum * x_scale) * w_scale (+ bias), with every operation
// rounded on its own: left to the compiler's contraction rules the multiply-add pairs fuse in some
// kernels (and in some paths of one kernel) and not in others, and kernels that must agree bit for bit
// -- the tile kernels, the weight-streaming kernels, the split-K epilogue -- would differ in the last place.
__device__ __forceinline__ float scaled_sum(float sum, float x_scale, float w_scale) {
#pragma clang fp contract(off)
  const float t = sum * x_scale;
  return t * w_scale;
}
__device__ __forceinline__ float plus_bias(float v, float bias) {
#pragma clang fp contract(off)
  return v + bias;
}

template <int DT> struct Elem;            // activation element traits
template <> struct Elem<MI355Q_F16> {
  typedef _Float16 type;
  static __device__ __forceinline__ float to_f32(uint16_t raw) {
    return (float)bitcast<_Float16>(raw);
  }
  static __device__ __forceinline__ uint16_t from_f32(float f) {
    return bitcast<uint16_t>((_Float16)f);
  }
};
template <> struct Elem<MI355Q_BF16> {
  typedef __bf16 type;
  static __device__ __forceinline__ float to_f32(uint16_t raw) { return bf16_to_f32(raw); }
  static __device__ __forceinline__ uint16_t from_f32(float f) { return f32_to_bf16(f); }
};

// Kernels whose accumulators alone fill 128+ registers call this once: an
// inline-asm AGPR operand makes the compiler keep MFMA accumulators in the
// accumulation half of the register file (AGPR-form MFMA) instead of using it
// only as a spill area for VGPR-form MFMAs.
__device__ __forceinline__ void use_agpr_accumulators() {
  int t = 0;
  asm volatile("" : "+a"(t));
}

// Buffer loads: an offset at or past the descriptor's size reads as zero
// without touching memory, which makes "no such K block" a branch-free case
// (callers add 2^31 to the lane offset; every buffer here is below 2 GiB).
typedef __amdgpu_buffer_rsrc_t rsrc_t;
__device__ __forceinline__ rsrc_t make_rsrc(const void* p, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ u4 buf_load16(rsrc_t r, uint32_t off) {
  return bitcast<u4>(__builtin_amdgcn_raw_buffer_load_b128(r, (int)off, 0, 0));
}
// streamed once: non-temporal
__device__ __forceinline__ u4 buf_load16_nt(rsrc_t r, uint32_t off) {
  return bitcast<u4>(__builtin_amdgcn_raw_buffer_load_b128(r, (int)off, 0, 2));
}
// Wavefront reductions on the data-parallel-primitive path (lane shifts inside the vector ALU, no trip
// through the LDS crossbar).  Every lane of the wavefront must be active.
// Whole wavefront: an inclusive scan within each row of 16 lanes (shifts by 1, 2, 4, 8; lanes a shift
// does not reach keep the identity), then lane 15 of rows 0 and 2 joins rows 1 and 3, lane 31 joins
// rows 2 and 3, and lane 63 holds the result, which is read back as a scalar.
#define MQ_DPP_REDUCE(v, ident, OP)                                                                     \
  do {                                                                                                  \
    v = OP(v, __builtin_amdgcn_update_dpp(ident, v, 0x111, 0xf, 0xf, false)); /* row_shr:1 */           \
    v = OP(v, __builtin_amdgcn_update_dpp(ident, v, 0x112, 0xf, 0xf, false)); /* row_shr:2 */           \
    v = OP(v, __builtin_amdgcn_update_dpp(ident, v, 0x114, 0xf, 0xf, false)); /* row_shr:4 */           \
    v = OP(v, __builtin_amdgcn_update_dpp(ident, v, 0x118, 0xf, 0xf, false)); /* row_shr:8 */           \
    v = OP(v, __builtin_amdgcn_update_dpp(ident, v, 0x142, 0xa, 0xf, false)); /* row_bcast:15 */        \
    v = OP(v, __builtin_amdgcn_update_dpp(ident, v, 0x143, 0xc, 0xf, false)); /* row_bcast:31 */        \
    v = __builtin_amdgcn_readlane(v, 63);                                                               \
  } while (0)
__device__ __forceinline__ int op_fmax_bits(int a, int b) { return __float_as_int(fmaxf(__int_as_float(a), __int_as_float(b))); }
__device__ __forceinline__ int op_fadd_bits(int a, int b) { return __float_as_int(__int_as_float(a) + __int_as_float(b)); }
__device__ __forceinline__ int op_imin(int a, int b) { return a < b ? a : b; }
__device__ __forceinline__ float wave_max(float x) {
  int v = __float_as_int(x);
  MQ_DPP_REDUCE(v, (int)0xff800000, op_fmax_bits);   // identity: -inf
  return __int_as_float(v);
}
__device__ __forceinline__ float wave_sum(float x) {
  int v = __float_as_int(x);
  MQ_DPP_REDUCE(v, 0, op_fadd_bits);
  return __int_as_float(v);
}
// max over aligned groups of `lanes` lanes (a power of two, 2 .. 64), the result in every lane of the
// group: swaps inside quads, mirrors of the half row and of the row of 16 lanes, LDS shuffles only
// for what crosses rows
__device__ __forceinline__ float lane_group_max(float x, int lanes) {
  int v = __float_as_int(x);
  if (lanes >= 2) v = op_fmax_bits(v, __builtin_amdgcn_update_dpp(v, v, 0xB1, 0xf, 0xf, false));    // quad_perm [1,0,3,2]
  if (lanes >= 4) v = op_fmax_bits(v, __builtin_amdgcn_update_dpp(v, v, 0x4E, 0xf, 0xf, false));    // quad_perm [2,3,0,1]
  if (lanes >= 8) v = op_fmax_bits(v, __builtin_amdgcn_update_dpp(v, v, 0x141, 0xf, 0xf, false));   // row_half_mirror
  if (lanes >= 16) v = op_fmax_bits(v, __builtin_amdgcn_update_dpp(v, v, 0x140, 0xf, 0xf, false));  // row_mirror
  float m = __int_as_float(v);
  for (int o = 16; o < lanes; o <<= 1) m = fmaxf(m, __shfl_xor(m, o));
  return m;
}

// Fused-MoE grouped GEMMs: a block whose expert id lies outside [0, E) -- a non-local expert under an
// expert map, -1 in the reference (vllm_gcu/kernels/fused_moe.py:70-71, 106-107) -- contributes
// nothing.  Its workgroups read no weights and zero the columns [col0, col0 + ncols) (ncols % 4 == 0)
// of every valid slot row of the block; `ids` are the block's `rows` slot ids, pads >= numel.
__device__ __forceinline__ void zero_block_columns(uint16_t* out, const int* ids, int rows, int numel, int N,
                                                   int col0, int ncols, int nthreads) {
  const int per_row = ncols >> 2;
  for (int i = threadIdx.x; i < rows * per_row; i += nthreads) {
    const int r = i / per_row, piece = i - r * per_row;
    const int id = ids[r];
    if (id < numel) *(uint2*)(out + (size_t)id * N + col0 + 4 * piece) = make_uint2(0u, 0u);
  }
}

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

int device_cu_count();

}  // namespace mi355q
