// Host launchers of the tiled MFMA GEMMs (int8 -> int32, int8 / e4m3 with fused dequantizing
// epilogue, grouped mixture-of-experts variant).
#include "gemm_launch.hpp"
#include <mutex>

thread_local char g_fmsmo_last_error[256] = {0};

int fmsmo_check_launch() {
  hipError_t e = hipGetLastError();
  if (e == hipSuccess) return FMSMO_OK;
  snprintf(g_fmsmo_last_error, sizeof(g_fmsmo_last_error), "%s", hipGetErrorString(e));
  return FMSMO_ERR_LAUNCH;
}

unsigned long long*& fmsmo_clock_probe() {
  static thread_local unsigned long long* probe = nullptr;
  return probe;
}
extern "C" int fmsmo_debug_clock_probe(uint64_t* dev6) {
  if (((uintptr_t)dev6) & 7) return FMSMO_ERR_ALIGN;
  fmsmo_clock_probe() = (unsigned long long*)dev6;
  return FMSMO_OK;
}

extern "C" int fmsmo_abi_version(void) { return FMSMO_ABI_VERSION; }
extern "C" const char* fmsmo_last_error(void) { return g_fmsmo_last_error; }
extern "C" const char* fmsmo_status_str(int s) {
  switch (s) {
    case FMSMO_OK: return "ok";
    case FMSMO_ERR_NULL: return "a required pointer is NULL";
    case FMSMO_ERR_SHAPE: return "bad shape or leading dimension";
    case FMSMO_ERR_ALIGN: return "pointer, K or leading dimension not 16-byte aligned";
    case FMSMO_ERR_UNSUPPORTED: return "unsupported enum value or size";
    case FMSMO_ERR_LAUNCH: return "kernel launch failed";
    case FMSMO_ERR_SCRATCH: return "shape needs more scratch than the library's static buffer holds";
    default: return "unknown status";
  }
}


extern "C" int fmsmo_gemm_i8_i32_ws(const int8_t* a, int64_t lda, const int8_t* b, int64_t ldb,
                                    int32_t* c, int64_t ldc, int64_t M, int64_t N, int64_t K,
                                    void* workspace, int64_t workspace_bytes, fmsmo_stream_t stream) {
  int rc = check_gemm(a, lda, b, ldb, c, ldc, M, N, K);
  if (rc) return rc;
  if (M == 0) return FMSMO_OK;
  // a few tokens: the weight-streaming decode kernels, storing their int32 sums
  if ((M <= 16 && K % 128 == 0) || fmsmo_gemv_batch_ok(M, K))
    return fmsmo_gemv_dispatch(FMSMO_OP_I8, a, lda, b, ldb, nullptr, 1, nullptr, 1, nullptr, FMSMO_F32,
                               EPI_RAW_I32, c, FMSMO_F32, ldc, M, N, K, (hipStream_t)stream);
  GemmArgs g{};
  g.a = (const uint8_t*)a; g.b = (const uint8_t*)b; g.lda = lda; g.ldb = ldb;
  g.M = (int)M; g.N = (int)N; g.K = (int)K;
  // few output tiles and a long reduction: K slices into the workspace, added in a fixed order
  const SplitPlan plan = plan_split_k(M, N, K, workspace ? workspace_bytes : 0);
  if (plan.splits > 1 && workspace && workspace_bytes >= plan.ws_bytes && aligned16(workspace) &&
      plan.splits * M * lda < (1ll << 31))
    return launch_split_k_i32(plan, g, workspace, c, ldc, (hipStream_t)stream);
  EpiStoreI32 epi{c, ldc};
  launch_any<MMA_I8>(g, epi, (hipStream_t)stream);
  return fmsmo_check_launch();
}

extern "C" int fmsmo_gemm_i8_i32(const int8_t* a, int64_t lda, const int8_t* b, int64_t ldb,
                                 int32_t* c, int64_t ldc, int64_t M, int64_t N, int64_t K,
                                 fmsmo_stream_t stream) {
  return fmsmo_gemm_i8_i32_ws(a, lda, b, ldb, c, ldc, M, N, K, nullptr, 0, stream);
}

static int gemm_i8_dq_impl(const int8_t* a, int64_t lda, const int8_t* b, int64_t ldb,
                           const float* a_scale, int64_t a_scale_n, const float* w_scale,
                           int64_t w_scale_n, const void* bias, int bias_dtype, int epilogue,
                           void* y, int y_dtype, int64_t ldy, int64_t M, int64_t N, int64_t K,
                           void* workspace, int64_t workspace_bytes, fmsmo_stream_t stream) {
  int rc = check_gemm(a, lda, b, ldb, y, ldy, M, N, K);
  if (rc) return rc;
  rc = check_dq(a_scale, a_scale_n, w_scale, w_scale_n, bias, bias_dtype, y_dtype, M, N);
  if (rc) return rc;
  if (epilogue < FMSMO_EPI_REF_F16 || epilogue > FMSMO_EPI_F32_MULADD) return FMSMO_ERR_UNSUPPORTED;
  if (M == 0) return FMSMO_OK;
  if ((M <= 16 && K % 128 == 0) || fmsmo_gemv_batch_ok(M, K))
    return fmsmo_gemv_dispatch(FMSMO_OP_I8, a, lda, b, ldb, a_scale, a_scale_n, w_scale, w_scale_n,
                               bias, bias_dtype, epilogue, y, y_dtype, ldy, M, N, K,
                               (hipStream_t)stream);
  GemmArgs g{};
  g.a = (const uint8_t*)a; g.b = (const uint8_t*)b; g.lda = lda; g.ldb = ldb;
  g.M = (int)M; g.N = (int)N; g.K = (int)K;
  const int as = a_scale_n == 1 ? 0 : 1, ws = w_scale_n == 1 ? 0 : 1;
  const SplitPlan plan = plan_split_k(M, N, K, workspace ? workspace_bytes : 0);
  if (plan.splits > 1 && workspace && workspace_bytes >= plan.ws_bytes && aligned16(workspace) &&
      plan.splits * M * lda < (1ll << 31)) {
    if (epilogue == FMSMO_EPI_REF_F16)
      return launch_split_k<MMA_I8, true, int>(plan, g, workspace, a_scale, as, w_scale, ws, bias,
                                               bias_dtype, y, y_dtype, ldy, (hipStream_t)stream);
    return launch_split_k<MMA_I8, false, int>(plan, g, workspace, a_scale, as, w_scale, ws, bias,
                                              bias_dtype, y, y_dtype, ldy, (hipStream_t)stream,
                                              epilogue == FMSMO_EPI_F32_MULADD);
  }
  if (epilogue == FMSMO_EPI_REF_F16)
    return launch_dq<MMA_I8, true, int, false>(g, a_scale, as, w_scale, ws, bias, bias_dtype, y,
                                               y_dtype, ldy, (hipStream_t)stream);
  return launch_dq<MMA_I8, false, int, false>(g, a_scale, as, w_scale, ws, bias, bias_dtype, y,
                                              y_dtype, ldy, (hipStream_t)stream, true,
                                              epilogue == FMSMO_EPI_F32_MULADD);
}

extern "C" int fmsmo_gemm_i8_dq(const int8_t* a, int64_t lda, const int8_t* b, int64_t ldb,
                                const float* a_scale, int64_t a_scale_n, const float* w_scale,
                                int64_t w_scale_n, const void* bias, int bias_dtype, int epilogue,
                                void* y, int y_dtype, int64_t ldy, int64_t M, int64_t N,
                                int64_t K, fmsmo_stream_t stream) {
  return gemm_i8_dq_impl(a, lda, b, ldb, a_scale, a_scale_n, w_scale, w_scale_n, bias, bias_dtype,
                         epilogue, y, y_dtype, ldy, M, N, K, nullptr, 0, stream);
}

extern "C" int fmsmo_gemm_i8_dq_ws(const int8_t* a, int64_t lda, const int8_t* b, int64_t ldb,
                                   const float* a_scale, int64_t a_scale_n, const float* w_scale,
                                   int64_t w_scale_n, const void* bias, int bias_dtype,
                                   int epilogue, void* y, int y_dtype, int64_t ldy, int64_t M,
                                   int64_t N, int64_t K, void* workspace, int64_t workspace_bytes,
                                   fmsmo_stream_t stream) {
  return gemm_i8_dq_impl(a, lda, b, ldb, a_scale, a_scale_n, w_scale, w_scale_n, bias, bias_dtype,
                         epilogue, y, y_dtype, ldy, M, N, K, workspace, workspace_bytes, stream);
}

// ------------------------------------------------------------- entry point that allocates nothing
// Split-K partial sums in device memory that belongs to the library's code object instead of a
// caller's workspace.  `scratch` is a host-side stand-in for the array: its device address is
// looked up once per device (each GPU that loads the library holds its own copy) and only that
// address is handed to kernels.
static __device__ __align__(256) unsigned char scratch[FMSMO_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
void* g_scratch_ptr[kMaxDevices] = {nullptr};

int static_scratch(void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e == hipSuccess && (dev < 0 || dev >= kMaxDevices)) e = hipErrorInvalidDevice;
  if (e == hipSuccess) {
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (!g_scratch_ptr[dev]) {
      void* p = nullptr;
      e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));  // address on the CURRENT device
      if (e == hipSuccess && !p) e = hipErrorInvalidSymbol;
      if (e == hipSuccess) g_scratch_ptr[dev] = p;
    }
    if (e == hipSuccess) *out = g_scratch_ptr[dev];
  }
  if (e != hipSuccess) {
    snprintf(g_fmsmo_last_error, sizeof(g_fmsmo_last_error), "static scratch lookup: %s",
             hipGetErrorString(e));
    return FMSMO_ERR_LAUNCH;
  }
  return FMSMO_OK;
}
}  // namespace

extern "C" int fmsmo_gemm_i8_dq_noalloc(const int8_t* a, int64_t lda, const int8_t* b, int64_t ldb,
                                        const float* a_scale, int64_t a_scale_n,
                                        const float* w_scale, int64_t w_scale_n, const void* bias,
                                        int bias_dtype, int epilogue, void* y, int y_dtype,
                                        int64_t ldy, int64_t M, int64_t N, int64_t K,
                                        fmsmo_stream_t stream) {
  // arguments first: a rejected call touches nothing, not even the scratch lookup
  int rc0 = check_gemm(a, lda, b, ldb, y, ldy, M, N, K);
  if (rc0) return rc0;
  rc0 = check_dq(a_scale, a_scale_n, w_scale, w_scale_n, bias, bias_dtype, y_dtype, M, N);
  if (rc0) return rc0;
  if (epilogue < FMSMO_EPI_REF_F16 || epilogue > FMSMO_EPI_F32_MULADD) return FMSMO_ERR_UNSUPPORTED;
  if (M == 0) return FMSMO_OK;
  // the weight-streaming decode kernels use no scratch
  const bool decode = (M <= 16 && K % 128 == 0) || fmsmo_gemv_batch_ok(M, K);
  // (the plan that fits the scratch, if one does: else the preferred plan's size is reported)
  int64_t need = decode ? 0 : plan_split_k(M, N, K, (int64_t)FMSMO_STATIC_SCRATCH_BYTES).ws_bytes;
  if (need > (int64_t)FMSMO_STATIC_SCRATCH_BYTES) {
    snprintf(g_fmsmo_last_error, sizeof(g_fmsmo_last_error),
             "split-K partial sums of %lld x %lld x %lld need %lld bytes, the static scratch holds %lld",
             (long long)M, (long long)N, (long long)K, (long long)need,
             (long long)FMSMO_STATIC_SCRATCH_BYTES);
    return FMSMO_ERR_SCRATCH;
  }
  void* ws = nullptr;
  if (need > 0) {
    int rc = static_scratch(&ws);
    if (rc) return rc;
  }
  // every slice's kernel stores its whole M x N block of partial sums before the reduction reads
  // it, so nothing in the scratch has to start at zero
  return gemm_i8_dq_impl(a, lda, b, ldb, a_scale, a_scale_n, w_scale, w_scale_n, bias, bias_dtype,
                         epilogue, y, y_dtype, ldy, M, N, K, ws, need, stream);
}

extern "C" int64_t fmsmo_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K) {
  return plan_split_k(M, N, K).ws_bytes;
}

extern "C" int64_t fmsmo_gemm_tail_columns(int64_t M, int64_t N, int64_t K) {
  if (M <= 0 || N <= 0 || K <= 0 || M > 0x7fffffff || N > 0x7fffffff || K > 0x7fffffff) return 0;
  if ((M <= 16 && K % 128 == 0) || fmsmo_gemv_batch_ok(M, K)) return 0;
  return tail_split_columns((int)M, (int)N, (int)K);
}

extern "C" int fmsmo_gemm_plan(int64_t M, int64_t N, int64_t K, int with_workspace, int* kernel,
                               int* tile_m, int* tile_n, int* splits) {
  if (!kernel || !tile_m || !tile_n || !splits) return FMSMO_ERR_NULL;
  if (M <= 0 || N <= 0 || K <= 0 || M > 0x7fffffff || N > 0x7fffffff || K > 0x7fffffff)
    return FMSMO_ERR_SHAPE;
  if (K % 16) return FMSMO_ERR_ALIGN;
  *tile_m = *tile_n = 0;
  *splits = 1;
  if ((M <= 16 && K % 128 == 0) || fmsmo_gemv_batch_ok(M, K)) {
    *kernel = FMSMO_PLAN_DECODE;
    return FMSMO_OK;
  }
  if (use_tall_tiles(M, N, K)) {  // one pass of 128 x 64 tiles, with or without a workspace
    *kernel = FMSMO_PLAN_TILE_LDS_DMA;
    *tile_m = TileTallK::BM;
    *tile_n = TileTallK::BN;
    return FMSMO_OK;
  }
  const SplitPlan plan = with_workspace == 2 ? plan_split_k(M, N, K, (int64_t)FMSMO_STATIC_SCRATCH_BYTES)
                                             : plan_split_k(M, N, K);
  if (with_workspace == 2 && plan.ws_bytes > (int64_t)FMSMO_STATIC_SCRATCH_BYTES)
    return FMSMO_ERR_SCRATCH;  // what the noalloc entry point returns for this shape
  if (with_workspace && plan.splits > 1) {
    *kernel = plan.rs ? FMSMO_PLAN_TILE_REGISTER_STAGED : FMSMO_PLAN_TILE_LDS_DMA;
    *tile_m = plan.rs ? 256 : TileMid::BM;
    *tile_n = plan.rs ? 128 : plan.tall ? TileTallK::BN : TileMid::BN;
    *splits = plan.splits;
    return FMSMO_OK;
  }
  if (K % 64) {
    *kernel = FMSMO_PLAN_GENERIC;
    return FMSMO_OK;
  }
  const bool rs = K % 128 == 0 && use_register_staged(MMA_I8);
  const int bm[5] = {256, 128, 128, 256, 256}, bn[5] = {256, 256, 128, 192, 128};
  const int t = pick_tile((int)M, (int)N, rs);
  *kernel = (rs && (t == 0 || t >= 3)) ? FMSMO_PLAN_TILE_REGISTER_STAGED : FMSMO_PLAN_TILE_LDS_DMA;
  *tile_m = bm[t];
  *tile_n = (t == 3 && !rs) ? 256 : bn[t];
  return FMSMO_OK;
}

extern "C" int fmsmo_grouped_gemm_i8_dq(const int8_t* a, int64_t lda, const int8_t* b,
                                        int64_t ldb, int64_t ldb_e, const int32_t* offsets,
                                        int num_experts, int64_t total_rows, const float* a_scale,
                                        const float* w_scale, const void* bias, int bias_dtype,
                                        int epilogue, void* y, int y_dtype, int64_t ldy, int64_t N,
                                        int64_t K, fmsmo_stream_t stream) {
  int rc = check_gemm(a, lda, b, ldb, y, ldy, total_rows, N, K);
  if (rc) return rc;
  if (!offsets || !a_scale || !w_scale) return FMSMO_ERR_NULL;
  if (num_experts <= 0 || ldb_e < N * ldb) return FMSMO_ERR_SHAPE;
  if ((int64_t)num_experts * ldb_e >= (1ll << 40)) return FMSMO_ERR_UNSUPPORTED;
  if (K % 64 || ldb_e % 16) return FMSMO_ERR_ALIGN;
  if (y_dtype < 0 || y_dtype > 2 || (bias && (bias_dtype < 0 || bias_dtype > 2))) return FMSMO_ERR_UNSUPPORTED;
  if (epilogue < FMSMO_EPI_REF_F16 || epilogue > FMSMO_EPI_F32_MULADD) return FMSMO_ERR_UNSUPPORTED;
  if (total_rows == 0) return FMSMO_OK;
  GemmArgs g{};
  g.a = (const uint8_t*)a; g.b = (const uint8_t*)b; g.lda = lda; g.ldb = ldb;
  g.M = (int)total_rows; g.N = (int)N; g.K = (int)K;
  g.offsets = offsets; g.num_experts = num_experts; g.ldb_e = ldb_e;
  g.grid_m = div_up(total_rows, TileBig::BM) + num_experts;  // upper bound on row tiles
  if (epilogue == FMSMO_EPI_REF_F16)
    return launch_dq<MMA_I8, true, int, true>(g, a_scale, 1, w_scale, 1, bias, bias_dtype, y,
                                              y_dtype, ldy, (hipStream_t)stream);
  return launch_dq<MMA_I8, false, int, true>(g, a_scale, 1, w_scale, 1, bias, bias_dtype, y,
                                             y_dtype, ldy, (hipStream_t)stream, true,
                                             epilogue == FMSMO_EPI_F32_MULADD);
}


extern "C" int fmsmo_bmm_i8_dq(const int8_t* a, int64_t lda, const int8_t* b, int64_t ldb,
                               int64_t stride_b, const float* a_scale, const float* b_scale,
                               const float* bias, void* y, int y_dtype, int64_t ldy, int64_t batch,
                               int64_t M, int64_t N, int64_t K, fmsmo_stream_t stream) {
  return launch_bmm<MMA_I8, int>(a, lda, b, ldb, stride_b, a_scale, b_scale, bias, y, y_dtype, ldy,
                                 batch, M, N, K, (hipStream_t)stream);
}

