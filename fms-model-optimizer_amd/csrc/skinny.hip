// Skinny-M (decode, M <= 16) W8A8 linear: stream the weight matrix once from HBM.
//
// y[M,N] = dequant( x_q[M,K] . W_q[N,K]^T ).  The weights (N*K bytes) dominate the traffic, so
// the kernel is organised around reading every weight line exactly once with as many bytes in
// flight as possible:
//   * a block owns RG groups of 16 weight rows; its NW waves split K between them;
//   * per 128-byte K step a lane fetches 2 x 16 B of its weight row straight into MFMA operand
//     registers (no LDS round trip: rows are the MFMA "A" rows, and the MFMA sums over k, so any
//     assignment of k-bytes to lanes is valid as long as x uses the same one);
//   * the (tiny, L2-resident) activations are the MFMA "B" operand, padded to 16 columns;
//   * 16x16 MFMA blocks (int8: 2 x v_mfma_i32_16x16x64_i8, fp8: v_mfma_f32_16x16x128_f8f6f4)
//     do the dot products, so the vector ALUs stay free and the loop is pure load + MFMA;
//   * the NW partial 16x16 blocks are reduced through LDS and dequantized by the first 256
//     threads.
#include "common.hpp"

namespace fmsmo {

struct GemvArgs {
  const uint8_t* a;  // [M,K] quantized activations
  const uint8_t* b;  // [N,K] quantized weights
  int64_t lda, ldb;
  int M, N, K;
  const float* a_scale;
  const float* w_scale;
  int a_stride, w_stride;
  const void* bias;
  int bias_dtype;
  int ref_f16;
  void* y;
  int y_dtype;
  int64_t ldy;
};

template <int OP, int RG, int NW>
__global__ __launch_bounds__(NW * 64) void gemv_kernel(GemvArgs g) {
  typedef typename std::conditional<OP == FMSMO_OP_I8, int, float>::type AccT;
  typedef AccT Acc4 __attribute__((ext_vector_type(4)));
  __shared__ AccT red[NW][RG][256];

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int r = lane & 15, kg = lane >> 4;
  const int n0 = blockIdx.x * (RG * 16);
  const int kslice = g.K / NW;  // multiple of 128 (checked on the host)
  const int kbeg = wave * kslice;

  const uint8_t* xp = g.a + (int64_t)min(r, g.M - 1) * g.lda + kbeg + kg * 16;
  const uint8_t* wp[RG];
#pragma unroll
  for (int i = 0; i < RG; ++i)
    wp[i] = g.b + (int64_t)min(n0 + i * 16 + r, g.N - 1) * g.ldb + kbeg + kg * 16;

  Acc4 acc[RG];
#pragma unroll
  for (int i = 0; i < RG; ++i) acc[i] = Acc4{0, 0, 0, 0};

  constexpr int UNROLL = 4 / RG > 0 ? 4 / RG : 1;  // ~8 x 16 B weight loads in flight per lane
  int k = 0;
  auto step = [&](int kk) {
    const v4i x0 = *(const v4i*)(xp + kk);
    const v4i x1 = *(const v4i*)(xp + kk + 64);
#pragma unroll
    for (int i = 0; i < RG; ++i) {
      const v4i w0 = __builtin_nontemporal_load((const v4i*)(wp[i] + kk));
      const v4i w1 = __builtin_nontemporal_load((const v4i*)(wp[i] + kk + 64));
      if constexpr (OP == FMSMO_OP_I8) {
        acc[i] = __builtin_amdgcn_mfma_i32_16x16x64_i8(w0, x0, acc[i], 0, 0, 0);
        acc[i] = __builtin_amdgcn_mfma_i32_16x16x64_i8(w1, x1, acc[i], 0, 0, 0);
      } else {
        const v8i w = {w0[0], w0[1], w0[2], w0[3], w1[0], w1[1], w1[2], w1[3]};
        const v8i x = {x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
        acc[i] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(w, x, acc[i], 0, 0, 0, 0, 0, 0);
      }
    }
  };
  for (; k + 128 * UNROLL <= kslice; k += 128 * UNROLL) {
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) step(k + u * 128);
  }
  for (; k < kslice; k += 128) step(k);

  // acc[i][v] = partial C(n = n0 + 16 i + 4 (lane / 16) + v, m = lane % 16)
#pragma unroll
  for (int i = 0; i < RG; ++i)
#pragma unroll
    for (int v = 0; v < 4; ++v) red[wave][i][(kg * 4 + v) * 16 + r] = acc[i][v];
  __syncthreads();

  for (int o = threadIdx.x; o < RG * 256; o += NW * 64) {
    const int i = o >> 8, e = o & 255;
    AccT s = red[0][i][e];
#pragma unroll
    for (int w = 1; w < NW; ++w) s += red[w][i][e];
    const int n = n0 + i * 16 + (e >> 4), m = e & 15;
    if (n < g.N && m < g.M) {
      const float as = g.a_scale[g.a_stride ? m : 0], ws = g.w_scale[g.w_stride ? n : 0];
      float b = 0.f;
      if (g.bias) {
        b = g.bias_dtype == FMSMO_F16 ? f16_to_f32(((const u16*)g.bias)[n])
            : g.bias_dtype == FMSMO_BF16 ? bf16_to_f32(((const u16*)g.bias)[n])
                                         : ((const float*)g.bias)[n];
      }
      float out;
      if (g.ref_f16) {
        const float sc = round_to<FMSMO_F16>(__fmul_rn(as, ws));
        out = round_to<FMSMO_F16>(__fadd_rn(__fmul_rn((float)s, sc), b));
      } else {
        out = __fmaf_rn((float)s, __fmul_rn(as, ws), b);
      }
      const int64_t idx = (int64_t)m * g.ldy + n;
      if (g.y_dtype == FMSMO_F16) ((u16*)g.y)[idx] = f32_to_f16(out);
      else if (g.y_dtype == FMSMO_BF16) ((u16*)g.y)[idx] = f32_to_bf16(out);
      else ((float*)g.y)[idx] = out;
    }
  }
}

}  // namespace fmsmo

using namespace fmsmo;

int fmsmo_check_launch();

template <int OP, int RG>
static void launch_gemv(const GemvArgs& g, int nw, hipStream_t st) {
  dim3 grid(div_up(g.N, RG * 16));
  switch (nw) {
    case 8: hipLaunchKernelGGL((gemv_kernel<OP, RG, 8>), grid, dim3(512), 0, st, g); break;
    case 4: hipLaunchKernelGGL((gemv_kernel<OP, RG, 4>), grid, dim3(256), 0, st, g); break;
    case 2: hipLaunchKernelGGL((gemv_kernel<OP, RG, 2>), grid, dim3(128), 0, st, g); break;
    default: hipLaunchKernelGGL((gemv_kernel<OP, RG, 1>), grid, dim3(64), 0, st, g); break;
  }
}

int fmsmo_gemv_dispatch(int op, const void* a, int64_t lda, const void* b, int64_t ldb,
                        const float* a_scale, int64_t a_scale_n, const float* w_scale,
                        int64_t w_scale_n, const void* bias, int bias_dtype, int epilogue,
                        void* y, int y_dtype, int64_t ldy, int64_t M, int64_t N, int64_t K,
                        hipStream_t st) {
  GemvArgs g{};
  g.a = (const uint8_t*)a; g.b = (const uint8_t*)b; g.lda = lda; g.ldb = ldb;
  g.M = (int)M; g.N = (int)N; g.K = (int)K;
  g.a_scale = a_scale; g.w_scale = w_scale;
  g.a_stride = a_scale_n == 1 ? 0 : 1; g.w_stride = w_scale_n == 1 ? 0 : 1;
  g.bias = bias; g.bias_dtype = bias_dtype; g.ref_f16 = epilogue == FMSMO_EPI_REF_F16;
  g.y = y; g.y_dtype = y_dtype; g.ldy = ldy;
  int nw = 8;
  while (nw > 1 && K % (128 * nw)) nw >>= 1;
  // enough row groups per block to amortise the activation re-reads, while keeping >= 2 blocks
  // per compute unit (256 CUs)
  const int64_t groups = (N + 15) / 16;
  const int rg = groups >= 4 * 512 ? 4 : groups >= 2 * 512 ? 2 : 1;
  if (op == FMSMO_OP_I8) {
    if (rg == 4) launch_gemv<FMSMO_OP_I8, 4>(g, nw, st);
    else if (rg == 2) launch_gemv<FMSMO_OP_I8, 2>(g, nw, st);
    else launch_gemv<FMSMO_OP_I8, 1>(g, nw, st);
  } else {
    if (rg == 4) launch_gemv<FMSMO_OP_E4M3, 4>(g, nw, st);
    else if (rg == 2) launch_gemv<FMSMO_OP_E4M3, 2>(g, nw, st);
    else launch_gemv<FMSMO_OP_E4M3, 1>(g, nw, st);
  }
  return fmsmo_check_launch();
}

static int check_gemv(const void* a, int64_t lda, const void* b, int64_t ldb, const float* a_scale,
                      int64_t a_scale_n, const float* w_scale, int64_t w_scale_n, const void* bias,
                      int bias_dtype, const void* y, int y_dtype, int64_t ldy, int64_t M, int64_t N,
                      int64_t K) {
  if (!a || !b || !y || !a_scale || !w_scale) return FMSMO_ERR_NULL;
  if (M < 0 || N <= 0 || K <= 0 || lda < K || ldb < K || ldy < N) return FMSMO_ERR_SHAPE;
  if ((a_scale_n != 1 && a_scale_n != M) || (w_scale_n != 1 && w_scale_n != N)) return FMSMO_ERR_SHAPE;
  if (M > 16 || K % 128) return FMSMO_ERR_UNSUPPORTED;
  if (N >= (1 << 30) || N * ldb >= (1ll << 40)) return FMSMO_ERR_UNSUPPORTED;
  if (y_dtype < 0 || y_dtype > 2 || (bias && (bias_dtype < 0 || bias_dtype > 2))) return FMSMO_ERR_UNSUPPORTED;
  if (lda % 16 || ldb % 16 || (((uintptr_t)a) & 15) || (((uintptr_t)b) & 15)) return FMSMO_ERR_ALIGN;
  return FMSMO_OK;
}

extern "C" int fmsmo_gemv_i8_dq(const int8_t* a, int64_t lda, const int8_t* b, int64_t ldb,
                                const float* a_scale, int64_t a_scale_n, const float* w_scale,
                                int64_t w_scale_n, const void* bias, int bias_dtype, int epilogue,
                                void* y, int y_dtype, int64_t ldy, int64_t M, int64_t N,
                                int64_t K, fmsmo_stream_t stream) {
  int rc = check_gemv(a, lda, b, ldb, a_scale, a_scale_n, w_scale, w_scale_n, bias, bias_dtype, y,
                      y_dtype, ldy, M, N, K);
  if (rc) return rc;
  if (epilogue != FMSMO_EPI_REF_F16 && epilogue != FMSMO_EPI_F32) return FMSMO_ERR_UNSUPPORTED;
  if (M == 0) return FMSMO_OK;
  return fmsmo_gemv_dispatch(FMSMO_OP_I8, a, lda, b, ldb, a_scale, a_scale_n, w_scale, w_scale_n,
                             bias, bias_dtype, epilogue, y, y_dtype, ldy, M, N, K,
                             (hipStream_t)stream);
}

extern "C" int fmsmo_gemv_fp8_dq(const uint8_t* a, int64_t lda, const uint8_t* b, int64_t ldb,
                                 const float* a_scale, int64_t a_scale_n, const float* w_scale,
                                 int64_t w_scale_n, const void* bias, int bias_dtype, void* y,
                                 int y_dtype, int64_t ldy, int64_t M, int64_t N, int64_t K,
                                 fmsmo_stream_t stream) {
  int rc = check_gemv(a, lda, b, ldb, a_scale, a_scale_n, w_scale, w_scale_n, bias, bias_dtype, y,
                      y_dtype, ldy, M, N, K);
  if (rc) return rc;
  if (M == 0) return FMSMO_OK;
  return fmsmo_gemv_dispatch(FMSMO_OP_E4M3, a, lda, b, ldb, a_scale, a_scale_n, w_scale, w_scale_n,
                             bias, bias_dtype, FMSMO_EPI_F32, y, y_dtype, ldy, M, N, K,
                             (hipStream_t)stream);
}
