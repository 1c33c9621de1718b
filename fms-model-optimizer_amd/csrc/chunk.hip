// Chunked reduced-precision-accumulation matmuls (int8 -> int32 and e4m3/f16/bf16/f32 -> fp32).
//
// D[M,N] = sum over K-chunks of round_trunc( A_chunk . B_chunk^T ) (+ C).  Every chunk is
// multiplied into a FRESH MFMA accumulator (the C operand is the inline constant 0 for the
// first MFMA of the chunk), the chunk result is range-clamped / LSB-rounded on the vector ALU,
// and only then added to the running accumulator -- the same order of operations as the
// reference's Triton kernels, whose BLOCK_SIZE_K equals the chunk size.
//
// Two kernels.  K (in bytes) a multiple of 64: the pipelined tile kernel of gemm_tile.hpp
// (128x128 block, 4-stage DMA ring) with its chunk hook.  Any other K: the simple kernel below.
//
// Simple kernel tiling: 128x128 block, 4 waves of 64x64 (2x2 MFMA 32x32 blocks each); K advances in 64-byte
// stages through two LDS buffers filled with bounds-checked 16-byte loads (zero fill past M, N
// and K, which is what "the K tail is masked to 0" means).  One MFMA k-step is 32 bytes of K
// for every operand type, so chunk boundaries (multiples of 32 bytes) always fall between
// k-steps.
#include "gemm_tile.hpp"

namespace fmsmo {

typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));

struct ChunkArgs {
  const uint8_t* a;
  const uint8_t* b;
  int64_t lda, ldb;  // bytes
  int M, N, Kb;      // Kb = K in bytes
  int chunk_bytes;
  int trun_bits, max_acc_bits, dl16, tta;
  const void* c_in;
  int64_t ldc;  // row stride of c_in (elements)
};

// What happens to a finished accumulator element.  One functor type per accumulator type with the
// mode, the output dtype and the bias dtype as run-time fields: the switch is on wave-uniform
// values in a 64-element epilogue behind a K loop of thousands of MFMAs, and it keeps the number
// of instantiations of the pipelined kernel (operand types x interleaving schedules) unchanged.
//   CHUNK_EPI_RAW        d[m,n] = acc                                  (int32 / fp32 out)
//   FMSMO_EPI_REF_F16    f16( f32(acc) * f16(as ws) + b )              (iaddmm_int's plain branch)
//   FMSMO_EPI_F32        fma( f32(acc), as ws, b )
//   FMSMO_EPI_F32_MULADD ( f32(acc) * (as ws) ) + b, every step rounded (iaddmm_int's chunk loop)
//   FMSMO_EPI_SEQ_OUT    T( T( (f32(acc) * as) * ws ) + T(b) ), T = output dtype
//                        (LinearFuncFPxFwdBwd / LinearFuncINT8FwdFP32Bwd: descale, cast, add bias)
enum { CHUNK_EPI_RAW = -1 };
template <class AccT>
struct EpiChunk {
  static constexpr bool UNIFORM_ROWS = false;
  void* y;
  int64_t ldy;
  const float* a_scale;
  const float* w_scale;
  const void* bias;
  int a_stride, w_stride;
  int mode, out_dt, bias_dt;
  struct Col {
    float ws, b;
  };
  struct Row {
    float as;
  };
  __device__ __forceinline__ float to_out_grid(float v) const {
    return out_dt == FMSMO_F16 ? round_to<FMSMO_F16>(v) : out_dt == FMSMO_BF16 ? round_to<FMSMO_BF16>(v) : v;
  }
  __device__ __forceinline__ Col col(int n, int, int) const {
    Col c{1.0f, -0.0f};
    if (mode == CHUNK_EPI_RAW) return c;
    c.ws = w_scale[w_stride ? n : 0];
    if (bias) {
      c.b = bias_dt == FMSMO_F16 ? load_as_f32<FMSMO_F16>(bias, n)
            : bias_dt == FMSMO_BF16 ? load_as_f32<FMSMO_BF16>(bias, n) : load_as_f32<FMSMO_F32>(bias, n);
      if (mode == FMSMO_EPI_SEQ_OUT) c.b = to_out_grid(c.b);
    }
    return c;
  }
  __device__ __forceinline__ Row row(int m) const {
    return Row{mode == CHUNK_EPI_RAW ? 1.0f : a_scale[a_stride ? m : 0]};
  }
  __device__ __forceinline__ void store(int m, int n, AccT v, Row r, Col c) const {
    const int64_t idx = (int64_t)m * ldy + n;
    if (mode == CHUNK_EPI_RAW) {
      ((AccT*)y)[idx] = v;
      return;
    }
    float t;
    if (mode == FMSMO_EPI_REF_F16) {
      const float sc = round_to<FMSMO_F16>(__fmul_rn(r.as, c.ws));
      t = __fadd_rn(__fmul_rn((float)v, sc), c.b);
      if (out_dt != FMSMO_F32) t = round_to<FMSMO_F16>(t);  // the fp16 accumulator dtype, then the output dtype
    } else if (mode == FMSMO_EPI_F32) {
      t = __fmaf_rn((float)v, __fmul_rn(r.as, c.ws), c.b);
    } else if (mode == FMSMO_EPI_F32_MULADD) {
      t = __fadd_rn(__fmul_rn((float)v, __fmul_rn(r.as, c.ws)), c.b);
    } else {
      t = to_out_grid(__fmul_rn(__fmul_rn((float)v, r.as), c.ws));
      if (bias) t = __fadd_rn(t, c.b);
    }
    if (out_dt == FMSMO_F16) store_from_f32<FMSMO_F16>(y, idx, t);
    else if (out_dt == FMSMO_BF16) store_from_f32<FMSMO_BF16>(y, idx, t);
    else ((float*)y)[idx] = t;
  }
};

template <int OP>
struct ChunkMma;
template <>
struct ChunkMma<FMSMO_OP_I8> {
  typedef int Elem;
  typedef v16i Acc;
  __device__ static __forceinline__ Acc mma(const v4i& a, const v4i& b, const Acc& c) {
    return __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0);
  }
};
template <>
struct ChunkMma<FMSMO_OP_E4M3> {
  typedef float Elem;
  typedef v16f Acc;
  __device__ static __forceinline__ Acc mma(const v4i& a, const v4i& b, const Acc& c) {
    // two K=16 MFMAs on the low / high 8 bytes of the lane's 16-byte operand chunk
    const long a0 = ((long)(unsigned)a[1] << 32) | (unsigned)a[0];
    const long a1 = ((long)(unsigned)a[3] << 32) | (unsigned)a[2];
    const long b0 = ((long)(unsigned)b[1] << 32) | (unsigned)b[0];
    const long b1 = ((long)(unsigned)b[3] << 32) | (unsigned)b[2];
    Acc t = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(a0, b0, c, 0, 0, 0);
    return __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(a1, b1, t, 0, 0, 0);
  }
};
template <>
struct ChunkMma<FMSMO_OP_F16> {
  typedef float Elem;
  typedef v16f Acc;
  __device__ static __forceinline__ Acc mma(const v4i& a, const v4i& b, const Acc& c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, a),
                                                  __builtin_bit_cast(v8h, b), c, 0, 0, 0);
  }
};
template <>
struct ChunkMma<FMSMO_OP_BF16> {
  typedef float Elem;
  typedef v16f Acc;
  __device__ static __forceinline__ Acc mma(const v4i& a, const v4i& b, const Acc& c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, a),
                                                   __builtin_bit_cast(v8bf, b), c, 0, 0, 0);
  }
};

template <>
struct ChunkMma<FMSMO_OP_F32> {
  typedef float Elem;
  typedef v16f Acc;
  __device__ static __forceinline__ Acc mma(const v4i& a, const v4i& b, const Acc& c) {
    // four K=2 fp32 MFMAs, one per float of the lane's 16-byte operand chunk
    Acc t = c;
#pragma unroll
    for (int e = 0; e < 4; ++e)
      t = __builtin_amdgcn_mfma_f32_32x32x2f32(__int_as_float(a[e]), __int_as_float(b[e]), t, 0, 0, 0);
    return t;
  }
};

template <int OP>
__global__ __launch_bounds__(256) void chunk_matmul_kernel(ChunkArgs g, EpiChunk<typename ChunkMma<OP>::Elem> epi) {
  typedef ChunkMma<OP> MM;
  typedef typename MM::Acc Acc;
  typedef typename MM::Elem Elem;
  constexpr int BM = 128, BN = 128, BK = 64, CPR = 4;
  __shared__ __attribute__((aligned(16))) uint8_t lds[2][(BM + BN) * BK];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int row0 = blockIdx.y * BM, col0 = blockIdx.x * BN;

  // loader: thread -> (row = tid / 4 + 64 j, 16-byte chunk = tid % 4), swizzled position in LDS
  const int lr = tid >> 2, lc = tid & 3;
  auto sw = [](int r) { return ((r >> 1) & 3) ^ ((r >> 3) & 1); };
  v4i stage_reg[4];
  auto gload = [&](int k0) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int ra = row0 + lr + 64 * j, rb = col0 + lr + 64 * j;
      const int kb = k0 + lc * 16;
      const bool kin = kb + 16 <= g.Kb;
      stage_reg[j] = (ra < g.M && kin) ? *(const v4i*)(g.a + (int64_t)ra * g.lda + kb) : v4i{0, 0, 0, 0};
      stage_reg[2 + j] = (rb < g.N && kin) ? *(const v4i*)(g.b + (int64_t)rb * g.ldb + kb) : v4i{0, 0, 0, 0};
    }
  };
  auto lstore = [&](int buf) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int r = lr + 64 * j;
      const int pos = lc ^ sw(r);
      *(v4i*)(&lds[buf][r * BK + pos * 16]) = stage_reg[j];
      *(v4i*)(&lds[buf][BM * BK + r * BK + pos * 16]) = stage_reg[2 + j];
    }
  };

  const int fr = lane & 31, fg = lane >> 5, fsw = sw(fr);

  Acc acc[2][2], tmp[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        tmp[i][j][v] = 0;
        Elem init = 0;
        if (g.c_in) {
          const int m = row0 + wm * 64 + i * 32 + (v >> 2) * 8 + fg * 4 + (v & 3);
          const int n = col0 + wn * 64 + j * 32 + fr;
          if (m < g.M && n < g.N) init = ((const Elem*)g.c_in)[(int64_t)m * g.ldc + n];
        }
        acc[i][j][v] = init;
      }

  const int t = g.dl16 ? 14 : g.trun_bits;
  const unsigned round_bit = t > 0 ? 1u << (t - 1) : 0u;
  const unsigned mask = ~((1u << t) - 1u);
  const int lo = g.max_acc_bits < 32 ? -(1 << (g.max_acc_bits - 1)) : (int)0x80000000;
  const int hi = g.max_acc_bits < 32 ? (1 << (g.max_acc_bits - 1)) - 1 : 0x7fffffff;
  const bool post = g.dl16 || t > 0 || g.max_acc_bits < 32;

  auto finish_chunk = [&]() {
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          Elem p = tmp[i][j][v];
          if (post) {
            if constexpr (OP == FMSMO_OP_I8) p = trunc_i32(p, lo, hi, (int)round_bit, t);
            else p = trunc_f32(p, round_bit, mask, g.dl16);
          }
          if (g.tta) {
            if constexpr (OP == FMSMO_OP_I8) acc[i][j][v] = (int)((unsigned)acc[i][j][v] + (unsigned)p);
            else acc[i][j][v] += p;
            tmp[i][j][v] = 0;
          } else {
            acc[i][j][v] = p;   // the running accumulator itself was rounded
            tmp[i][j][v] = p;
          }
        }
  };
  if (!g.tta) {
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) tmp[i][j] = acc[i][j];
  }

  const int nstage = (g.Kb + BK - 1) / BK;
  gload(0);
  lstore(0);
  __syncthreads();
  int in_chunk = 0;  // bytes of the current chunk already multiplied
  for (int st = 0; st < nstage; ++st) {
    const int cur = st & 1;
    if (st + 1 < nstage) gload((st + 1) * BK);
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const int c = (2 * s + fg) ^ fsw;
      v4i af[2], bf[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) af[i] = *(const v4i*)(&lds[cur][(wm * 64 + i * 32 + fr) * BK + c * 16]);
#pragma unroll
      for (int j = 0; j < 2; ++j) bf[j] = *(const v4i*)(&lds[cur][BM * BK + (wn * 64 + j * 32 + fr) * BK + c * 16]);
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) tmp[i][j] = MM::mma(af[i], bf[j], tmp[i][j]);
      in_chunk += 32;
      if (in_chunk == g.chunk_bytes) {
        finish_chunk();
        in_chunk = 0;
      }
    }
    if (st + 1 < nstage) {
      lstore(cur ^ 1);
      __syncthreads();
    }
  }
  if (in_chunk != 0) finish_chunk();  // zero-padded K tail

#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int m = row0 + wm * 64 + i * 32 + (v >> 2) * 8 + fg * 4 + (v & 3);
      if (m < g.M) {
        const auto rowctx = epi.row(m);
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int n = col0 + wn * 64 + j * 32 + fr;
          if (n < g.N) epi.store(m, n, acc[i][j][v], rowctx, epi.col(n, 0, g.N));
        }
      }
    }
}

}  // namespace fmsmo

using namespace fmsmo;
int fmsmo_check_launch();

// Pipelined path: the tile GEMM kernel with the chunk hook.  Needs whole 64-byte K stages and
// 32-bit row offsets; the K tail inside the last chunk (K not a multiple of the chunk) is
// finished after the loop like any chunk.
template <int MMA, class Epi>
static bool launch_chunk_tile(const ChunkArgs& c, const Epi& epi, hipStream_t st) {
  if (c.Kb % 64 || c.chunk_bytes % 32 || (int64_t)c.M * c.lda >= (1ll << 31) ||
      (int64_t)c.N * c.ldb >= (1ll << 31))
    return false;
  GemmArgs g{};
  g.a = c.a; g.b = c.b; g.lda = c.lda; g.ldb = c.ldb;
  g.M = c.M; g.N = c.N; g.K = c.Kb;
  g.grid_m = div_up(c.M, 128); g.grid_n = div_up(c.N, 128); g.group_m = 8;
  const bool fast = c.tta && !c.dl16 && c.max_acc_bits >= 32;
  ChunkTrunc<false> k{};
  k.chunk_ks = c.chunk_bytes / 32;
  k.t = c.dl16 ? 14 : c.trun_bits;
  k.round_bit = k.t > 0 ? 1u << (k.t - 1) : 0u;
  k.mask = ~((1u << k.t) - 1u);
  k.lo = c.max_acc_bits < 32 ? -(1 << (c.max_acc_bits - 1)) : (int)0x80000000;
  k.hi = c.max_acc_bits < 32 ? (1 << (c.max_acc_bits - 1)) - 1 : 0x7fffffff;
  k.post = c.dl16 || k.t > 0 || c.max_acc_bits < 32;
  k.dl16 = c.dl16; k.tta = c.tta; k.c_in = c.c_in; k.ldc = c.ldc;
  dim3 grid((unsigned)(g.grid_m * g.grid_n)), block(256);
  // the schedules that round one block while the matrix unit multiplies the others: a chunk of one
  // 64-byte stage (every operand type), of several stages or of one 32-byte k-step (int8)
  const int sched = !fast ? 0 : c.chunk_bytes == 64 ? 1 : MMA != MMA_I8 ? 0 : c.chunk_bytes == 32 ? 3
                    : c.chunk_bytes % 64 == 0 ? 2 : 0;
#define LAUNCH_SCHED(SV)                                                                             \
  {                                                                                                  \
    ChunkTrunc<true, SV> kf{};                                                                       \
    kf.chunk_ks = k.chunk_ks; kf.t = k.t; kf.round_bit = k.round_bit; kf.mask = k.mask;              \
    kf.lo = k.lo; kf.hi = k.hi; kf.post = k.post; kf.dl16 = 0; kf.tta = 1;                           \
    kf.c_in = k.c_in; kf.ldc = k.ldc;                                                                \
    hipLaunchKernelGGL((gemm_tile_kernel<128, 128, 64, 4, 2, 2, MMA, 1, false, Epi, ChunkTrunc<true, SV>>), \
                       grid, block, 0, st, g, epi, kf);                                              \
  }
  if (sched == 1) {
    LAUNCH_SCHED(1)
  } else if (sched == 2) {
    if constexpr (MMA == MMA_I8) LAUNCH_SCHED(2)
  } else if (sched == 3) {
    if constexpr (MMA == MMA_I8) LAUNCH_SCHED(3)
  } else if (fast) {
    ChunkTrunc<true> kf{};
    kf.chunk_ks = k.chunk_ks; kf.t = k.t; kf.round_bit = k.round_bit; kf.mask = k.mask;
    kf.lo = k.lo; kf.hi = k.hi; kf.post = k.post; kf.dl16 = 0; kf.tta = 1;
    kf.c_in = k.c_in; kf.ldc = k.ldc;
    hipLaunchKernelGGL((gemm_tile_kernel<128, 128, 64, 4, 2, 2, MMA, 1, false, Epi, ChunkTrunc<true>>),
                       grid, block, 0, st, g, epi, kf);
  } else {
    hipLaunchKernelGGL((gemm_tile_kernel<128, 128, 64, 4, 2, 2, MMA, 1, false, Epi, ChunkTrunc<false>>),
                       grid, block, 0, st, g, epi, k);
  }
  return true;
}

static int check_chunk(const void* a, int64_t lda, const void* b, int64_t ldb, const void* d,
                       int64_t ldd, int64_t M, int64_t N, int64_t K, int64_t esz, int chunk_size,
                       int min_chunk) {
  if (!a || !b || !d) return FMSMO_ERR_NULL;
  if (M < 0 || N <= 0 || K <= 0 || lda < K || ldb < K || ldd < N) return FMSMO_ERR_SHAPE;
  if (M >= (1 << 30) || N >= (1 << 30) || K * esz >= (1ll << 31)) return FMSMO_ERR_UNSUPPORTED;
  if (chunk_size < min_chunk || (chunk_size & (chunk_size - 1))) return FMSMO_ERR_UNSUPPORTED;
  if ((K * esz) % 16 || (lda * esz) % 16 || (ldb * esz) % 16 || (((uintptr_t)a) & 15) ||
      (((uintptr_t)b) & 15))
    return FMSMO_ERR_ALIGN;
  return FMSMO_OK;
}

static int check_chunk_dq(const float* a_scale, int64_t a_scale_n, const float* w_scale,
                          int64_t w_scale_n, const void* bias, int bias_dtype, int epilogue,
                          int y_dtype, int64_t M, int64_t N) {
  if (!a_scale || !w_scale) return FMSMO_ERR_NULL;
  if ((a_scale_n != 1 && a_scale_n != M) || (w_scale_n != 1 && w_scale_n != N)) return FMSMO_ERR_SHAPE;
  if (y_dtype < 0 || y_dtype > 2 || (bias && (bias_dtype < 0 || bias_dtype > 2))) return FMSMO_ERR_UNSUPPORTED;
  if (epilogue < FMSMO_EPI_REF_F16 || epilogue > FMSMO_EPI_SEQ_OUT) return FMSMO_ERR_UNSUPPORTED;
  return FMSMO_OK;
}

static int run_chunk_i8(const ChunkArgs& g, const EpiChunk<int>& epi, hipStream_t st) {
  if (launch_chunk_tile<MMA_I8>(g, epi, st)) return fmsmo_check_launch();
  dim3 grid(div_up(g.N, 128), div_up(g.M, 128));
  hipLaunchKernelGGL((chunk_matmul_kernel<FMSMO_OP_I8>), grid, dim3(256), 0, st, g, epi);
  return fmsmo_check_launch();
}

static int run_chunk_fp(int op_dtype, const ChunkArgs& g, const EpiChunk<float>& epi, hipStream_t st) {
  const bool done = op_dtype == FMSMO_OP_E4M3 ? launch_chunk_tile<MMA_FP8_K32>(g, epi, st)
                    : op_dtype == FMSMO_OP_F16 ? launch_chunk_tile<MMA_F16>(g, epi, st)
                    : op_dtype == FMSMO_OP_BF16 ? launch_chunk_tile<MMA_BF16>(g, epi, st)
                                                : launch_chunk_tile<MMA_F32>(g, epi, st);
  if (done) return fmsmo_check_launch();
  dim3 grid(div_up(g.N, 128), div_up(g.M, 128));
  if (op_dtype == FMSMO_OP_E4M3)
    hipLaunchKernelGGL((chunk_matmul_kernel<FMSMO_OP_E4M3>), grid, dim3(256), 0, st, g, epi);
  else if (op_dtype == FMSMO_OP_F16)
    hipLaunchKernelGGL((chunk_matmul_kernel<FMSMO_OP_F16>), grid, dim3(256), 0, st, g, epi);
  else if (op_dtype == FMSMO_OP_F32)
    hipLaunchKernelGGL((chunk_matmul_kernel<FMSMO_OP_F32>), grid, dim3(256), 0, st, g, epi);
  else
    hipLaunchKernelGGL((chunk_matmul_kernel<FMSMO_OP_BF16>), grid, dim3(256), 0, st, g, epi);
  return fmsmo_check_launch();
}

static ChunkArgs chunk_args_i8(const int8_t* a, int64_t lda, const int8_t* b, int64_t ldb, int64_t M,
                               int64_t N, int64_t K, int chunk_size, int chunk_trun_bits,
                               int max_acc_bits, int tta, const void* c_in, int64_t ldc) {
  ChunkArgs g{};
  g.a = (const uint8_t*)a; g.b = (const uint8_t*)b; g.lda = lda; g.ldb = ldb;
  g.M = (int)M; g.N = (int)N; g.Kb = (int)K; g.chunk_bytes = chunk_size;
  g.trun_bits = chunk_trun_bits; g.max_acc_bits = max_acc_bits; g.dl16 = 0;
  g.tta = tta != 0; g.c_in = c_in; g.ldc = ldc;
  return g;
}

extern "C" int fmsmo_matmul_chunk_i8(const int8_t* a, int64_t lda, const int8_t* b, int64_t ldb,
                                     const int32_t* c_in, int32_t* d, int64_t ldd, int64_t M,
                                     int64_t N, int64_t K, int chunk_size, int chunk_trun_bits,
                                     int max_acc_bits, int truncate_then_accumulate,
                                     fmsmo_stream_t stream) {
  int rc = check_chunk(a, lda, b, ldb, d, ldd, M, N, K, 1, chunk_size, 32);
  if (rc) return rc;
  if (chunk_trun_bits < 0 || chunk_trun_bits > 31 || max_acc_bits < 2 || max_acc_bits > 32)
    return FMSMO_ERR_UNSUPPORTED;
  if (M == 0) return FMSMO_OK;
  // Nothing to round or clamp: int32 addition wraps and is associative, so the chunked sum is
  // the plain int32 GEMM.
  if (chunk_trun_bits == 0 && max_acc_bits == 32 && !c_in)
    return fmsmo_gemm_i8_i32(a, lda, b, ldb, d, ldd, M, N, K, stream);
  const ChunkArgs g = chunk_args_i8(a, lda, b, ldb, M, N, K, chunk_size, chunk_trun_bits, max_acc_bits,
                                    truncate_then_accumulate, c_in, ldd);
  EpiChunk<int> epi{};
  epi.y = d; epi.ldy = ldd; epi.mode = CHUNK_EPI_RAW;
  return run_chunk_i8(g, epi, (hipStream_t)stream);
}

extern "C" int fmsmo_matmul_chunk_i8_dq(const int8_t* a, int64_t lda, const int8_t* b, int64_t ldb,
                                        const float* a_scale, int64_t a_scale_n,
                                        const float* w_scale, int64_t w_scale_n, const void* bias,
                                        int bias_dtype, int epilogue, void* y, int y_dtype,
                                        int64_t ldy, int64_t M, int64_t N, int64_t K,
                                        int chunk_size, int chunk_trun_bits, int max_acc_bits,
                                        int truncate_then_accumulate, fmsmo_stream_t stream) {
  int rc = check_chunk(a, lda, b, ldb, y, ldy, M, N, K, 1, chunk_size, 32);
  if (rc) return rc;
  rc = check_chunk_dq(a_scale, a_scale_n, w_scale, w_scale_n, bias, bias_dtype, epilogue, y_dtype, M, N);
  if (rc) return rc;
  if (chunk_trun_bits < 0 || chunk_trun_bits > 31 || max_acc_bits < 2 || max_acc_bits > 32)
    return FMSMO_ERR_UNSUPPORTED;
  if (M == 0) return FMSMO_OK;
  // nothing to round or clamp: the plain int8 GEMM with the same epilogue, where it has it
  if (chunk_trun_bits == 0 && max_acc_bits == 32 && epilogue != FMSMO_EPI_SEQ_OUT && K % 16 == 0)
    return fmsmo_gemm_i8_dq(a, lda, b, ldb, a_scale, a_scale_n, w_scale, w_scale_n, bias, bias_dtype,
                            epilogue, y, y_dtype, ldy, M, N, K, stream);
  const ChunkArgs g = chunk_args_i8(a, lda, b, ldb, M, N, K, chunk_size, chunk_trun_bits, max_acc_bits,
                                    truncate_then_accumulate, nullptr, 0);
  EpiChunk<int> epi{y, ldy, a_scale, w_scale, bias, a_scale_n == 1 ? 0 : 1, w_scale_n == 1 ? 0 : 1,
                    epilogue, y_dtype, bias ? bias_dtype : FMSMO_F32};
  return run_chunk_i8(g, epi, (hipStream_t)stream);
}

static int chunk_args_fp(const void* a, int64_t lda, const void* b, int64_t ldb, int op_dtype,
                         const void* d, int64_t ldd, int64_t M, int64_t N, int64_t K, int chunk_size,
                         int chunk_trun_bits, int clamp_dl16, int tta, const void* c_in, int64_t ldc,
                         ChunkArgs* out) {
  if (op_dtype != FMSMO_OP_E4M3 && op_dtype != FMSMO_OP_F16 && op_dtype != FMSMO_OP_BF16 &&
      op_dtype != FMSMO_OP_F32)
    return FMSMO_ERR_UNSUPPORTED;
  const int esz = op_dtype == FMSMO_OP_E4M3 ? 1 : op_dtype == FMSMO_OP_F32 ? 4 : 2;
  int rc = check_chunk(a, lda, b, ldb, d, ldd, M, N, K, esz, chunk_size, esz == 1 ? 32 : 16);
  if (rc) return rc;
  if (chunk_trun_bits < 0 || chunk_trun_bits > 22) return FMSMO_ERR_UNSUPPORTED;
  ChunkArgs g{};
  g.a = (const uint8_t*)a; g.b = (const uint8_t*)b; g.lda = lda * esz; g.ldb = ldb * esz;
  g.M = (int)M; g.N = (int)N; g.Kb = (int)(K * esz); g.chunk_bytes = chunk_size * esz;
  g.trun_bits = chunk_trun_bits; g.max_acc_bits = 32; g.dl16 = clamp_dl16 != 0;
  g.tta = tta != 0; g.c_in = c_in; g.ldc = ldc;
  *out = g;
  return FMSMO_OK;
}

extern "C" int fmsmo_matmul_chunk_fp(const void* a, int64_t lda, const void* b, int64_t ldb,
                                     int op_dtype, const float* c_in, float* d, int64_t ldd,
                                     int64_t M, int64_t N, int64_t K, int chunk_size,
                                     int chunk_trun_bits, int clamp_dl16,
                                     int truncate_then_accumulate, fmsmo_stream_t stream) {
  ChunkArgs g{};
  int rc = chunk_args_fp(a, lda, b, ldb, op_dtype, d, ldd, M, N, K, chunk_size, chunk_trun_bits,
                         clamp_dl16, truncate_then_accumulate, c_in, ldd, &g);
  if (rc) return rc;
  if (M == 0) return FMSMO_OK;
  EpiChunk<float> epi{};
  epi.y = d; epi.ldy = ldd; epi.mode = CHUNK_EPI_RAW;
  return run_chunk_fp(op_dtype, g, epi, (hipStream_t)stream);
}

extern "C" int fmsmo_matmul_chunk_fp_dq(const void* a, int64_t lda, const void* b, int64_t ldb,
                                        int op_dtype, const float* a_scale, int64_t a_scale_n,
                                        const float* w_scale, int64_t w_scale_n, const void* bias,
                                        int bias_dtype, int epilogue, void* y, int y_dtype,
                                        int64_t ldy, int64_t M, int64_t N, int64_t K,
                                        int chunk_size, int chunk_trun_bits, int clamp_dl16,
                                        int truncate_then_accumulate, fmsmo_stream_t stream) {
  ChunkArgs g{};
  int rc = chunk_args_fp(a, lda, b, ldb, op_dtype, y, ldy, M, N, K, chunk_size, chunk_trun_bits,
                         clamp_dl16, truncate_then_accumulate, nullptr, 0, &g);
  if (rc) return rc;
  rc = check_chunk_dq(a_scale, a_scale_n, w_scale, w_scale_n, bias, bias_dtype, epilogue, y_dtype, M, N);
  if (rc) return rc;
  if (M == 0) return FMSMO_OK;
  EpiChunk<float> epi{y, ldy, a_scale, w_scale, bias, a_scale_n == 1 ? 0 : 1, w_scale_n == 1 ? 0 : 1,
                      epilogue, y_dtype, bias ? bias_dtype : FMSMO_F32};
  return run_chunk_fp(op_dtype, g, epi, (hipStream_t)stream);
}
