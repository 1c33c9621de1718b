// e4m3 entry points of the tiled MFMA GEMMs (fused dequantizing epilogue, batched variant).
#include "gemm_launch.hpp"

static int gemm_fp8_dq_impl(const uint8_t* a, int64_t lda, const uint8_t* b, int64_t ldb,
                            const float* a_scale, int64_t a_scale_n, const float* w_scale,
                            int64_t w_scale_n, const void* bias, int bias_dtype, void* y,
                            int y_dtype, int64_t ldy, int64_t M, int64_t N, int64_t K,
                            void* workspace, int64_t workspace_bytes, fmsmo_stream_t stream) {
  int rc = check_gemm(a, lda, b, ldb, y, ldy, M, N, K);
  if (rc) return rc;
  rc = check_dq(a_scale, a_scale_n, w_scale, w_scale_n, bias, bias_dtype, y_dtype, M, N);
  if (rc) return rc;
  if (M == 0) return FMSMO_OK;
  if ((M <= 16 && K % 128 == 0) || fmsmo_gemv_batch_ok(M, K))
    return fmsmo_gemv_dispatch(FMSMO_OP_E4M3, a, lda, b, ldb, a_scale, a_scale_n, w_scale,
                               w_scale_n, bias, bias_dtype, FMSMO_EPI_F32, y, y_dtype, ldy, M, N, K,
                               (hipStream_t)stream);
  GemmArgs g{};
  g.a = a; g.b = b; g.lda = lda; g.ldb = ldb;
  g.M = (int)M; g.N = (int)N; g.K = (int)K;
  const int as = a_scale_n == 1 ? 0 : 1, ws = w_scale_n == 1 ? 0 : 1;
  const SplitPlan plan = plan_split_k(M, N, K, workspace ? workspace_bytes : 0);
  if (plan.splits > 1 && workspace && workspace_bytes >= plan.ws_bytes && aligned16(workspace) &&
      plan.splits * M * lda < (1ll << 31))
    return launch_split_k<MMA_FP8, false, float>(plan, g, workspace, a_scale, as, w_scale, ws, bias,
                                                 bias_dtype, y, y_dtype, ldy, (hipStream_t)stream);
  return launch_dq<MMA_FP8, false, float, false>(g, a_scale, as, w_scale, ws, bias, bias_dtype, y,
                                                 y_dtype, ldy, (hipStream_t)stream);
}

extern "C" int fmsmo_gemm_fp8_dq(const uint8_t* a, int64_t lda, const uint8_t* b, int64_t ldb,
                                 const float* a_scale, int64_t a_scale_n, const float* w_scale,
                                 int64_t w_scale_n, const void* bias, int bias_dtype, void* y,
                                 int y_dtype, int64_t ldy, int64_t M, int64_t N, int64_t K,
                                 fmsmo_stream_t stream) {
  return gemm_fp8_dq_impl(a, lda, b, ldb, a_scale, a_scale_n, w_scale, w_scale_n, bias, bias_dtype,
                          y, y_dtype, ldy, M, N, K, nullptr, 0, stream);
}

extern "C" int fmsmo_gemm_fp8_dq_ws(const uint8_t* a, int64_t lda, const uint8_t* b, int64_t ldb,
                                    const float* a_scale, int64_t a_scale_n, const float* w_scale,
                                    int64_t w_scale_n, const void* bias, int bias_dtype, void* y,
                                    int y_dtype, int64_t ldy, int64_t M, int64_t N, int64_t K,
                                    void* workspace, int64_t workspace_bytes,
                                    fmsmo_stream_t stream) {
  return gemm_fp8_dq_impl(a, lda, b, ldb, a_scale, a_scale_n, w_scale, w_scale_n, bias, bias_dtype,
                          y, y_dtype, ldy, M, N, K, workspace, workspace_bytes, stream);
}

extern "C" int fmsmo_bmm_fp8_dq(const uint8_t* a, int64_t lda, const uint8_t* b, int64_t ldb,
                                int64_t stride_b, const float* a_scale, const float* b_scale,
                                const float* bias, void* y, int y_dtype, int64_t ldy, int64_t batch,
                                int64_t M, int64_t N, int64_t K, fmsmo_stream_t stream) {
  return launch_bmm<MMA_FP8, float>(a, lda, b, ldb, stride_b, a_scale, b_scale, bias, y, y_dtype,
                                    ldy, batch, M, N, K, (hipStream_t)stream);
}
