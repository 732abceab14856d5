// W4A16 GEMM entry points: argument checks and the choice between the
// streaming (small M) and the LDS-staged MFMA (large M) kernels.
#include "common.h"

#include <mutex>

namespace mi355q {
int w4a16_stream_launch(void* out, const void* x, const int32_t* qweight, const void* scales,
                        const void* zeros, int zeros_kind, const void* bias, int M, int K, int N,
                        int group_size, int dtype, void* workspace, size_t workspace_bytes,
                        int split_k, hipStream_t st);
size_t w4a16_stream_workspace_bytes(int M, int N);
size_t w4a16_stream_plan_workspace_bytes(int M, int K, int N, int gs);
int w4a16_tile_launch(void* out, const void* x, const int32_t* qweight, const void* scales,
                      const void* zeros, int zeros_kind, const void* bias, int M, int K, int N,
                      int group_size, int dtype, void* workspace, size_t workspace_bytes, bool allow_ring,
                      hipStream_t st);
size_t w4a16_tile_workspace_bytes(int M, int K, int N);
size_t w4a16_bf16_stage_workspace_bytes(int M, int K);
int w4a16_bf16_staged_launch(void* out, const void* x, const int32_t* qweight, const void* scales, const void* zeros,
                             int zeros_kind, const void* bias, int M, int K, int N, int group_size, void* workspace,
                             size_t workspace_bytes, int force_tw, hipStream_t st);
int w4a16_mid_launch(void* out, const void* x, const int32_t* qweight, const void* scales, const void* zeros,
                     int zeros_kind, const void* bias, int M, int K, int N, int group_size, int dtype,
                     void* workspace, size_t workspace_bytes, int splits, int tw, hipStream_t st);
}  // namespace mi355q

using namespace mi355q;

static constexpr size_t TILE_WS_OFFSET = (size_t)1 << 20;

// streaming kernel up to 32 rows; 33..64 rows: the MFMA kernel where its pipelined loop exists
// (fp16, integer zero-points; measured equal or up to 22 % faster there), else streaming again.
// Groups of 64 and 32: the streaming kernel takes 32 rows per launch, so from 65 rows on the MFMA
// kernel's plain loop with two or four groups per K block takes over.
static int auto_family(int M, int group_size, int zeros_kind, int dtype) {
  if (group_size % 128 != 0) return ((group_size == 64 || group_size == 32) && M > 64) ? 2 : 1;
  const bool piped = dtype == MI355Q_F16 && zeros_kind != MI355Q_ZP_PRESCALED;
  return (M <= 32 || (M <= 64 && !piped)) ? 1 : 2;
}

extern "C" size_t mi355q_w4a16_workspace_bytes(int M, int K, int N) {
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  const size_t s = w4a16_stream_workspace_bytes(M > 64 ? 64 : M, N);
  // the split-K partials of the MFMA kernel live behind the first MiB, which
  // holds the streaming kernel's arrival counters (they must stay zero)
  const size_t t = M > 32 ? w4a16_tile_workspace_bytes(M, K, N) : 0;
  size_t tt = t ? t + TILE_WS_OFFSET : 0;
  // (this function does not see the dtype: room for the area that bf16 activations are staged in as
  // fp16 rows, behind the split-K partials -- a smaller workspace only means the bf16 loop runs instead)
  const size_t stage = w4a16_bf16_stage_workspace_bytes(M, K);
  if (stage && stage + TILE_WS_OFFSET > tt) tt = stage + TILE_WS_OFFSET;
  return s > tt ? s : tt;
}

namespace mi355q {
struct StreamPlan { int nt, splits; };
StreamPlan w4a16_stream_auto_plan(int M, int K, int N, int gs);
}  // namespace mi355q

// the work split the streaming (decode) kernel takes for a shape: tiles of 16 columns per workgroup and
// K splits across workgroups (what a caller sizes the workspace for, and what a profile was taken on)
extern "C" int mi355q_w4a16_stream_plan(int M, int K, int N, int group_size, int* tiles_per_workgroup,
                                        int* k_splits) {
  MQ_REQUIRE(M > 0 && K > 0 && N > 0 && K % 128 == 0 && N % 128 == 0, "w4a16_stream_plan: bad shape M=%d K=%d N=%d", M, K, N);
  MQ_REQUIRE(tiles_per_workgroup && k_splits, "w4a16_stream_plan: null pointer");
  const int gs = group_size <= 0 ? K : group_size;
  const StreamPlan p = w4a16_stream_auto_plan(M > 64 ? 64 : M, K, N, gs);
  const int G = K / 128;
  int splits = p.splits > G ? G : p.splits;
  if (splits > 32) splits = 32;
  while (splits > 1 && ((G + splits - 1) / splits) * (splits - 1) >= G) --splits;
  *tiles_per_workgroup = p.nt;
  *k_splits = splits;
  return 0;
}

extern "C" int mi355q_w4a16_gemm_ex(void* out, const void* x, const int32_t* qweight,
                                    const void* scales, const void* zeros, int zeros_kind,
                                    const void* bias, int M, int K, int N, int group_size,
                                    int dtype, void* workspace, size_t workspace_bytes,
                                    int split_k, int family, void* stream) {
  MQ_REQUIRE(M >= 0 && K > 0 && N > 0, "w4a16_gemm: bad shape M=%d K=%d N=%d", M, K, N);
  if (M == 0) return 0;
  MQ_REQUIRE(out && x && qweight && scales, "w4a16_gemm: null pointer");
  MQ_REQUIRE(K % 128 == 0 && N % 128 == 0,
             "w4a16_gemm: K=%d and N=%d must be multiples of 128 (slab layout)", K, N);
  MQ_REQUIRE(dtype == MI355Q_F16 || dtype == MI355Q_BF16, "w4a16_gemm: dtype %d not supported", dtype);
  if (group_size <= 0) group_size = K;
  MQ_REQUIRE(group_size % 32 == 0 && K % group_size == 0,
             "w4a16_gemm: group_size=%d must be a multiple of 32 dividing K=%d", group_size, K);
  MQ_REQUIRE(group_size % 128 == 0 || 128 % group_size == 0,
             "w4a16_gemm: group_size=%d must divide or be a multiple of 128", group_size);
  MQ_REQUIRE(zeros_kind >= MI355Q_ZP_NONE && zeros_kind <= MI355Q_ZP_PRESCALED,
             "w4a16_gemm: unknown zeros_kind %d", zeros_kind);
  MQ_REQUIRE(zeros_kind == MI355Q_ZP_NONE || zeros, "w4a16_gemm: zeros pointer missing");
  MQ_REQUIRE(family >= 0 && family <= 3, "w4a16_gemm: unknown kernel family %d", family);
  const int caller_family = family;       // 0: the library chooses, also between the two MFMA kernels
  if (family == 0) family = auto_family(M, group_size, zeros_kind, dtype);
  MQ_REQUIRE(family != 2 || group_size % 128 == 0 || group_size == 64 || group_size == 32,
             "w4a16_gemm: the MFMA kernel needs a group size of 32, 64 or a multiple of 128, got %d", group_size);
  if (family == 1) {
    // the streaming kernel covers 64 rows per launch (32 with group sizes
    // below 128, whose four scale rows per K block leave no registers for
    // more); taller inputs go through it in row chunks
    const size_t esz = 2;
    const int chunk = group_size % 128 == 0 ? 64 : 32;
    for (int m0 = 0; m0 < M; m0 += chunk) {
      const int mc = M - m0 < chunk ? M - m0 : chunk;
      int rc = w4a16_stream_launch((char*)out + (size_t)m0 * N * esz, (const char*)x + (size_t)m0 * K * esz,
                                   qweight, scales, zeros, zeros_kind, bias, mc, K, N, group_size, dtype,
                                   workspace, workspace_bytes, split_k, as_stream(stream));
      if (rc) return rc;
    }
    return 0;
  }
  const bool ws_ok = workspace && workspace_bytes > TILE_WS_OFFSET;
  if (family == 3 && dtype == MI355Q_BF16) {
    // bf16 rows staged as fp16 in the workspace, ring workgroups of 256 (or, bits 8..15 = 4, 512) columns
    const int rc = w4a16_bf16_staged_launch(out, x, qweight, scales, zeros, zeros_kind, bias, M, K, N, group_size,
                                            ws_ok ? (char*)workspace + TILE_WS_OFFSET : nullptr,
                                            ws_ok ? workspace_bytes - TILE_WS_OFFSET : 0,
                                            ((split_k >> 8) & 0xff) == 4 ? 4 : 2, as_stream(stream));
    MQ_REQUIRE(rc != -12345,
               "w4a16_gemm: the ring kernels are fp16 kernels; bf16 rows reach them through a workspace of "
               "mi355q_w4a16_workspace_bytes() bytes, above 64 rows, with group sizes that are multiples of 128 and "
               "zero-points that are not pre-scaled (M %d, group %d, zero-point kind %d, %zu bytes of workspace)",
               M, group_size, zeros_kind, workspace_bytes);
    return rc;
  }
  if (family == 3)
    return w4a16_mid_launch(out, x, qweight, scales, zeros, zeros_kind, bias, M, K, N, group_size, dtype,
                            ws_ok ? (char*)workspace + TILE_WS_OFFSET : nullptr,
                            ws_ok ? workspace_bytes - TILE_WS_OFFSET : 0, split_k & 0xff, (split_k >> 8) & 0xff, as_stream(stream));
  return w4a16_tile_launch(out, x, qweight, scales, zeros, zeros_kind, bias, M, K, N, group_size, dtype,
                           ws_ok ? (char*)workspace + TILE_WS_OFFSET : nullptr,
                           ws_ok ? workspace_bytes - TILE_WS_OFFSET : 0, caller_family == 0, as_stream(stream));
}

extern "C" int mi355q_w4a16_gemm(void* out, const void* x, const int32_t* qweight, const void* scales,
                                 const void* zeros, int zeros_kind, const void* bias, int M, int K,
                                 int N, int group_size, int dtype, void* workspace,
                                 size_t workspace_bytes, void* stream) {
  return mi355q_w4a16_gemm_ex(out, x, qweight, scales, zeros, zeros_kind, bias, M, K, N, group_size,
                              dtype, workspace, workspace_bytes, 0, 0, stream);
}

// ---- the same GEMM for callers that cannot allocate ----------------------------------------------
// Split-K partial tiles and arrival counters live in a fixed array in device memory instead of a
// caller's workspace.  Every GPU holds its own copy of the array (at its own address) from the
// moment the library is loaded there until the process ends; every call on a GPU shares it.
static constexpr size_t NOALLOC_SCRATCH_BYTES = (size_t)32 << 20;
static __device__ __align__(256) unsigned char scratch[NOALLOC_SCRATCH_BYTES];

namespace {
__global__ void __launch_bounds__(256) noalloc_clear_kernel(uint32_t* p, int words) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < words) p[i] = 0u;
}

// device address of `scratch` on the current device, looked up once per device
int noalloc_scratch_ptr(void** out) {
  static std::mutex mu;
  static void* ptrs[64];
  int dev = 0;
  MQ_REQUIRE(hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < 64, "w4a16_gemm_noalloc: no current device");
  std::lock_guard<std::mutex> lk(mu);
  if (!ptrs[dev]) {
    void* p = nullptr;
    hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    MQ_REQUIRE(e == hipSuccess && p, "w4a16_gemm_noalloc: cannot resolve the scratch array on device %d: %s", dev,
               hipGetErrorString(e));
    ptrs[dev] = p;
  }
  *out = ptrs[dev];
  return 0;
}
}  // namespace

extern "C" size_t mi355q_w4a16_noalloc_scratch_bytes(void) { return NOALLOC_SCRATCH_BYTES; }

extern "C" int mi355q_w4a16_gemm_noalloc(void* out, const void* x, const int32_t* qweight, const void* scales,
                                         const void* zeros, int zeros_kind, const void* bias, int M, int K,
                                         int N, int group_size, int dtype, void* stream) {
  MQ_REQUIRE(M >= 0 && K > 0 && N > 0, "w4a16_gemm_noalloc: bad shape M=%d K=%d N=%d", M, K, N);
  if (M == 0) return 0;
  // every argument check of the GEMM happens before the first launch (the clear below)
  MQ_REQUIRE(out && x && qweight && scales, "w4a16_gemm_noalloc: null pointer");
  MQ_REQUIRE(dtype == MI355Q_F16 || dtype == MI355Q_BF16, "w4a16_gemm_noalloc: dtype %d not supported", dtype);
  MQ_REQUIRE(K % 128 == 0 && N % 128 == 0,
             "w4a16_gemm_noalloc: K=%d and N=%d must be multiples of 128 (slab layout)", K, N);
  const int gs = group_size <= 0 ? K : group_size;
  MQ_REQUIRE(gs % 32 == 0 && K % gs == 0 && (gs % 128 == 0 || 128 % gs == 0),
             "w4a16_gemm_noalloc: group_size=%d must be a multiple of 32 dividing K=%d and dividing or a multiple of 128",
             gs, K);
  // what the plan of this shape needs, exactly -- the same plan mi355q_w4a16_gemm takes when its
  // workspace is large enough, so both entry points give bit-identical results
  const int family = auto_family(M, gs, zeros_kind, dtype);
  size_t need;
  bool counters = false;
  if (family == 1) {
    const int chunk = gs % 128 == 0 ? 64 : 32;
    need = w4a16_stream_plan_workspace_bytes(M < chunk ? M : chunk, K, N, gs);
    if (M > chunk && M % chunk) {
      const size_t tail = w4a16_stream_plan_workspace_bytes(M % chunk, K, N, gs);
      need = tail > need ? tail : need;
    }
    counters = need > 0;
  } else {
    const size_t t = w4a16_tile_workspace_bytes(M, K, N);
    need = t ? t + TILE_WS_OFFSET : 0;
  }
  MQ_REQUIRE(need <= NOALLOC_SCRATCH_BYTES,
             "w4a16_gemm_noalloc: M=%d K=%d N=%d splits K through %zu bytes of scratch, the fixed array holds %zu; "
             "use mi355q_w4a16_gemm with a workspace",
             M, K, N, need, NOALLOC_SCRATCH_BYTES);
  void* ws = nullptr;
  if (int rc = noalloc_scratch_ptr(&ws)) return rc;
  if (counters) {
    // the arrival counters must start at zero whatever an earlier call left behind (a fill kernel, not
    // a memset: callers may be capturing a graph)
    const int words = N / 16 * 4;                  // one counter per wavefront of every possible workgroup
    hipLaunchKernelGGL(noalloc_clear_kernel, dim3((words + 255) / 256), dim3(256), 0, as_stream(stream),
                       (uint32_t*)ws, words);
    MQ_LAUNCH_CHECK("w4a16_gemm_noalloc(clear)");
  }
  return mi355q_w4a16_gemm_ex(out, x, qweight, scales, zeros, zeros_kind, bias, M, K, N, group_size, dtype, ws,
                              NOALLOC_SCRATCH_BYTES, 0, 0, stream);
}
