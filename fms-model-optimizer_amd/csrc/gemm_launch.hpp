// Host-side launch helpers shared by the GEMM translation units (int8 and e4m3 entry points are
// compiled separately to keep the build parallel): argument checks, tile choice, launchers.
#pragma once
#include "gemm_rs.hpp"
#include "gemm_k128.hpp"
#include <algorithm>
#include <cmath>
#include <cstdlib>

using namespace fmsmo;

int fmsmo_check_launch();
// Device buffer of 6 x 64 bit that later register-staged GEMM launches of this thread fill with
// block 0's clock readings (null = off); defined in gemm.hip.
unsigned long long*& fmsmo_clock_probe();
bool fmsmo_gemv_batch_ok(int64_t M, int64_t K);
int fmsmo_gemv_dispatch(int op, const void* a, int64_t lda, const void* b, int64_t ldb,
                        const float* a_scale, int64_t a_scale_n, const float* w_scale,
                        int64_t w_scale_n, const void* bias, int bias_dtype, int epilogue,
                        void* y, int y_dtype, int64_t ldy, int64_t M, int64_t N, int64_t K,
                        hipStream_t st);

namespace {

bool aligned16(const void* p) { return (((uintptr_t)p) & 15) == 0; }

int check_gemm(const void* a, int64_t lda, const void* b, int64_t ldb, const void* c,
               int64_t ldc, int64_t M, int64_t N, int64_t K) {
  if (!a || !b || !c) return FMSMO_ERR_NULL;
  if (M < 0 || N <= 0 || K <= 0 || lda < K || ldb < K || ldc < N) return FMSMO_ERR_SHAPE;
  // 32-bit byte offsets inside the kernels
  if ((M > 0 && (M * lda) >= (1ll << 31)) || N * ldb >= (1ll << 31) || M >= (1 << 30) ||
      N >= (1 << 30))
    return FMSMO_ERR_UNSUPPORTED;
  if (K % 16 || lda % 16 || ldb % 16 || !aligned16(a) || !aligned16(b)) return FMSMO_ERR_ALIGN;
  return FMSMO_OK;
}

// Tile shapes.  K is consumed in stages of BK bytes; a K that is not a multiple of BK is handled
// by the caller-visible rule "K % 64 == 0" for the MFMA path (all transformer shapes), anything
// else goes to the slow generic kernel.
struct TileBig { static constexpr int BM = 256, BN = 256, BK = 64, NST = 4, WGM = 2, WGN = 2; };
struct TileWide { static constexpr int BM = 128, BN = 256, BK = 64, NST = 4, WGM = 2, WGN = 2; };
struct TileMid { static constexpr int BM = 128, BN = 128, BK = 64, NST = 4, WGM = 2, WGN = 2; };
// The same tiles with stages of 128 bytes of K (whole 128-byte lines per row and request, half as
// many barriers): K % 128 == 0, one block per compute unit (128 / 120 KiB of LDS).  Pipelines of
// three stages lose a third against five; six (tall) and five (square) change nothing.
struct TileMidK { static constexpr int BM = 128, BN = 128, BK = 128, NST = 4, WGM = 2, WGN = 2; };
struct TileTallK { static constexpr int BM = 128, BN = 64, BK = 128, NST = 5, WGM = 2, WGN = 2; };

// A few hundred rows through a projection whose 128 x 64 tiles fill half a round of the 256
// compute units or more run as ONE pass of those tiles rather than as K slices with a second
// kernel: no partial sums to write and read back.  A block walks K in ~0.41 us per 128-byte stage (one
// round: 4.4 us + 3.3 us per 1024 of K whatever the rows), so the slices win again on long
// reductions.  us from a HIP graph, int8, before -> after (e4m3 within 5 % of these):
//   N = 4096, K = 4096: M = 129 17.5 -> 14.7, 256 21.4 -> 17.0, 512 25.7 -> 18.3 (vendor GEMM, int32
//   out: 18.1); N = 6144: 129 20.9 -> 16.1, 256 22.1 -> 17.3; N = 2048: 512 22.6 -> 16.1, 1024 25.9 ->
//   17.5; N = 1024: 1024 21.9 -> 15.6; K = 2048, N = 4096: 129 / 256 / 512 14.4 / 18.2 / 22.9 -> 9.5 /
//   10.7 / 11.3; K = 8192: 512 36.4 -> 31.6; half a round at K = 5120 / 8192 loses (256 rows: 21.1 ->
//   22.8, 24.5 -> 29.1) and so does K = 14336 (512 rows 48.2 -> 51.3): those keep the slices.
inline bool use_tall_tiles(int64_t M, int64_t N, int64_t K) {
  static const char* off = getenv("FMSMO_TALL");  // FMSMO_TALL=0 disables (tuning aid)
  if (off && off[0] == '0') return false;
  if (M <= 16 || M > 1024 || K % 128) return false;
  const int64_t tiles = (int64_t)div_up(M, TileTallK::BM) * div_up(N, TileTallK::BN);
  if (tiles > 256) return false;
  // three quarters of a round or more: also for a single row of tiles (batches of 17 .. 128 tokens
  // that the decode kernels do not take, through a wide projection; us, M = 33 / 64 / 128: N = 14336,
  // K = 8192 39.4 / 39.6 / 42.5 -> 32.2 / 33.8 / 38.3; N = 13824, K = 5120 26.2 / 28.1 -> 20.7 / 23.2;
  // N = 14336, K = 4096, M = 65 / 128 23.7 / 25.1 -> 19.6 / 20.1)
  if (tiles >= 192) return K <= 8192;
  return M > 128 && tiles >= 96 && K <= 4096;
}

// Pick the tile shape by (relative kernel efficiency) x (fill of the last round of tiles over
// the 256 compute units).  The efficiencies are measured loop efficiencies of the shapes
// (bigger tiles move fewer bytes per MFMA); 128x128 tiles fit two blocks per CU.  Shape 3 is the
// register-staged kernel with 256x192 tiles (K % 128 == 0 only): 8 % slower per operation than
// 256x256, but e.g. N = 6144 at M = 4096 then makes 512 tiles, two full rounds, instead of 384.
// Shape 4 is the same kernel with 256x128 tiles (the tile of the probabilities x values batched
// matmul): 0.85 of the 256x256 rate where both fill their rounds (4096 x 4096 x 4096: 73 -> 85 us),
// but 2048 rows x 4096 columns make 256 tiles instead of 128 (us, int8 / e4m3: K = 4096 45.8 ->
// 43.4 / 42.2 -> 38.7, K = 12800 141 -> 123 / 130 -> 114).
constexpr double EFF_RS128 = 0.85;
int pick_tile(int M, int N, bool rs192_ok) {
  static const char* force = getenv("FMSMO_TILE");  // tuning aid: 0 = 256x256, 1 = 128x256, 2 = 128x128, 3 = 256x192, 4 = 256x128
  if (force && force[0] >= '0' && force[0] <= '4') return (force[0] == '4' && !rs192_ok) ? 2 : force[0] - '0';
  // Fitted to measurements on the Llama / Granite shapes: relative loop efficiency of the three
  // tile shapes, and a sub-linear penalty for a partially filled last round (idle CUs leave
  // power, hence clock, to the busy ones).
  const double eff[5] = {1.0, 0.76, 0.70, 0.92, EFF_RS128};
  const int bm[5] = {256, 128, 128, 256, 256}, bn[5] = {256, 256, 128, 192, 128};
  int best = 0;
  double best_score = -1;
  for (int t = 0; t < (rs192_ok ? 5 : 3); ++t) {
    const long tiles = (long)div_up(M, bm[t]) * div_up(N, bn[t]);
    const long slots = (t == 2 && tiles > 256) ? 512 : 256;  // two 128x128 blocks fit per CU
    const long rounds = (tiles + slots - 1) / slots;
    const double fill = (double)tiles / (double)(rounds * slots);
    const double pad = ((double)M * N) / ((double)div_up(M, bm[t]) * bm[t] * (double)div_up(N, bn[t]) * bn[t]);
    const double score = eff[t] * pow(fill, 0.6) * pad;
    if (score > best_score) { best_score = score; best = t; }
  }
  return best;
}

template <class Tile, int OP, bool GROUPED, class Epi>
void launch_tile(const GemmArgs& g0, const Epi& epi, hipStream_t st) {
  GemmArgs g = g0;
  g.grid_n = div_up(g.N, Tile::BN);
  if (!GROUPED) g.grid_m = div_up(g.M, Tile::BM);
  g.group_m = 4;
  dim3 grid((unsigned)(g.grid_m * g.grid_n)), block(Tile::WGM * Tile::WGN * 64);
  hipLaunchKernelGGL(
      (gemm_tile_kernel<Tile::BM, Tile::BN, Tile::BK, Tile::NST, Tile::WGM, Tile::WGN, OP, 1,
                        GROUPED, Epi>),
      grid, block, 0, st, g, epi, NoChunk{});
}

// 256x256 tiles with K a multiple of 128 run the register-staged pipeline (gemm_rs.hpp: whole
// 128-byte lines, half the L2 -> L1 traffic).  FMSMO_RS=0 / 1 forces the choice for tuning.
static bool use_register_staged(int op) {
  static const char* force = getenv("FMSMO_RS");
  if (force && (force[0] == '0' || force[0] == '1')) return force[0] == '1';
  (void)op;
  return true;
}
// Compute units of the current device (the grid of the persistent blocks).
inline int compute_units() {
  static thread_local int cached_dev = -1, cached = 0;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) dev = 0;
  if (dev != cached_dev) {
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 1) cus = 256;
    cached_dev = dev;
    cached = cus;
  }
  return cached;
}

template <int OP, bool GROUPED = false, int BN = 256, class Epi>
void launch_rs(const GemmArgs& g0, const Epi& epi, hipStream_t st) {
  GemmArgs g = g0;
  g.clk = fmsmo_clock_probe();
  g.grid_n = div_up(g.N, BN);
  if (!GROUPED) g.grid_m = div_up(g.M, 256);
  g.group_m = 4;
  dim3 grid((unsigned)(g.grid_m * g.grid_n)), block(256);
  // mixture-of-experts mode: grid_m is only an upper bound on the row tiles (the row counts live
  // on the device); the blocks are persistent, one per compute unit, and count the tiles themselves
  if (GROUPED && g.rows_per_group == 0) grid.x = (unsigned)std::min<long>((long)grid.x, compute_units());
  if constexpr (OP == MMA_FP8) {
    // e4m3: the 16 x 16 x 128 matrix instruction (more work per joule under the power limit: the
    // four Llama-3-8B shapes at 4096 rows +1 ... +4 %) unless FMSMO_MFMA16=0 asks for 32 x 32 x 64
    // (tuning aid).  int8 stays with 32 x 32 x 32: its 16 x 16 x 64 form issues four times as many
    // instructions per slab and lost 3 ... 25 % in this kernel.
    static const char* force16 = getenv("FMSMO_MFMA16");
    if (!(force16 && force16[0] == '0')) {
      hipLaunchKernelGGL((gemm_rs_kernel<OP, Epi, GROUPED, BN, true>), grid, block, 0, st, g, epi);
      return;
    }
  }
  hipLaunchKernelGGL((gemm_rs_kernel<OP, Epi, GROUPED, BN, false>), grid, block, 0, st, g, epi);
}

// Reduction of exactly 128 bytes (attention scores): persistent blocks over 128 x 256 tiles, two
// per compute unit (FMSMO_K128_BLOCKS sets the grid, for tuning).
template <int OP, class Epi>
void launch_k128(const GemmArgs& g0, int batch, int M, const Epi& epi, hipStream_t st) {
  GemmArgs g = g0;
  g.grid_n = div_up(g.N, 256);
  g.grid_m = batch * div_up(M, 128);
  g.group_m = 4;
  static const int env_blocks = getenv("FMSMO_K128_BLOCKS") ? atoi(getenv("FMSMO_K128_BLOCKS")) : 0;
  const long tiles = (long)g.grid_m * g.grid_n;
  long blocks = env_blocks > 0 ? env_blocks : 512;
  if (blocks > tiles) blocks = tiles;
  hipLaunchKernelGGL((gemm_k128_kernel<OP, Epi>), dim3((unsigned)blocks), dim3(256), 0, st, g, epi);
}

// Generic fallback (any K % 16 == 0): one thread per output element, 4-byte dot products.
template <int OP, class Epi>
__global__ void gemm_simple_kernel(GemmArgs g, Epi epi) {
  const int n = blockIdx.x * blockDim.x + threadIdx.x;
  const int m = blockIdx.y;
  if (n >= g.N) return;
  const uint8_t* ar = g.a + (int64_t)m * g.lda;
  const uint8_t* br = g.b + (int64_t)n * g.ldb;
  typename Epi::Col c = epi.col(n, 0, g.N);
  typename Epi::Row r = epi.row(m);
  if constexpr (OP == MMA_I8) {
    int acc = 0;
    for (int k = 0; k < g.K; k += 4)
      acc = __builtin_amdgcn_sdot4(*(const int*)(ar + k), *(const int*)(br + k), acc, false);
    epi.store(m, n, acc, r, c);
  } else {
    float acc = 0.f;
    for (int k = 0; k < g.K; k += 4) {
      const uint32_t av = *(const uint32_t*)(ar + k), bv = *(const uint32_t*)(br + k);
      acc = __fmaf_rn(__builtin_amdgcn_cvt_f32_fp8(av, 0), __builtin_amdgcn_cvt_f32_fp8(bv, 0), acc);
      acc = __fmaf_rn(__builtin_amdgcn_cvt_f32_fp8(av, 1), __builtin_amdgcn_cvt_f32_fp8(bv, 1), acc);
      acc = __fmaf_rn(__builtin_amdgcn_cvt_f32_fp8(av, 2), __builtin_amdgcn_cvt_f32_fp8(bv, 2), acc);
      acc = __fmaf_rn(__builtin_amdgcn_cvt_f32_fp8(av, 3), __builtin_amdgcn_cvt_f32_fp8(bv, 3), acc);
    }
    epi.store(m, n, acc, r, c);
  }
}

template <int OP, class Epi>
void launch_any(const GemmArgs& g, const Epi& epi, hipStream_t st) {
  if (use_tall_tiles(g.M, g.N, g.K)) {
    launch_tile<TileTallK, OP, false>(g, epi, st);
  } else if (g.K % 64 == 0) {
    switch (pick_tile(g.M, g.N, g.K % 128 == 0 && use_register_staged(OP))) {
      case 0:
        if (g.K % 128 == 0 && use_register_staged(OP)) launch_rs<OP>(g, epi, st);
        else launch_tile<TileBig, OP, false>(g, epi, st);
        break;
      case 1: launch_tile<TileWide, OP, false>(g, epi, st); break;
      case 3:
        if (g.K % 128 == 0 && use_register_staged(OP)) launch_rs<OP, false, 192>(g, epi, st);
        else launch_tile<TileBig, OP, false>(g, epi, st);
        break;
      case 4: launch_rs<OP, false, 128>(g, epi, st); break;  // only offered when K % 128 == 0
      default:
        // one round of 128 x 128 tiles: stages of 128 bytes (us, 1024 rows, N = 4096: K = 4096 29.0 ->
        // 25.6, 5120 36.8 -> 31.2; 512 rows, N = 6144, K = 4096: 28.0 -> 23.5); more than a round keeps
        // the 64-byte stages, whose blocks fit two to a compute unit
        if (g.K % 128 == 0 && (long)div_up(g.M, TileMidK::BM) * div_up(g.N, TileMidK::BN) <= 256)
          launch_tile<TileMidK, OP, false>(g, epi, st);
        else
          launch_tile<TileMid, OP, false>(g, epi, st);
        break;
    }
  } else {
    dim3 grid(div_up(g.N, 64), (unsigned)g.M), block(64);
    hipLaunchKernelGGL((gemm_simple_kernel<OP, Epi>), grid, block, 0, st, g, epi);
  }
}

// A last round of 256x256 tiles that fills at most a quarter of the compute units costs most of
// a round.  Columns to cut off so that the remaining tiles make full rounds (0 = leave the GEMM
// whole); the cut columns then run as a second, small GEMM with the tile shape that suits them.
// Taken only when at least 1024 columns are cut: a narrower second GEMM is a latency-bound launch
// that costs as much as the sparse round it replaces (us, whole -> cut: 2048 x 25600 x 4096, 32
// tiles over 3 rounds, int8 263 -> 248, e4m3 224 -> 204; 4096 x 8448 x 8192, 16 tiles over 2
// rounds, one column tile cut: 316 -> 321).  FMSMO_TAIL_SPLIT=0 switches this off (tuning aid).
inline int tail_split_columns(int M, int N, int K) {
  static const char* off = getenv("FMSMO_TAIL_SPLIT");
  if (off && off[0] == '0') return 0;
  if (K % 128 || !use_register_staged(0) || pick_tile(M, N, true) != 0) return 0;
  const long gm = div_up(M, 256), gn = div_up(N, 256), tiles = gm * gn;
  if (tiles <= 256) return 0;
  const long last = tiles % 256;
  if (last == 0 || last > 64) return 0;
  const long cut = (last + gm - 1) / gm;  // column tiles
  if (cut < 4 || cut >= gn) return 0;
  return (int)(N - (gn - cut) * 256);
}

template <int OP, bool REF, class AccT, bool GROUPED>
int launch_dq(const GemmArgs& g, const float* a_scale, int a_stride, const float* w_scale,
              int w_stride, const void* bias, int bias_dtype, void* y, int y_dtype, int64_t ldy,
              hipStream_t st, bool may_split = true, int muladd = 0) {
  if (!bias) bias_dtype = FMSMO_F32;
  if constexpr (!GROUPED) {
    const int tail = may_split ? tail_split_columns(g.M, g.N, g.K) : 0;
    if (tail > 0) {
      const int64_t n0 = g.N - tail;
      GemmArgs g1 = g, g2 = g;
      g1.N = (int)n0;
      g2.N = tail;
      g2.b = g.b + n0 * g.ldb;
      const int64_t ysz = y_dtype == FMSMO_F32 ? 4 : 2, bsz = bias_dtype == FMSMO_F32 ? 4 : 2;
      int rc = launch_dq<OP, REF, AccT, false>(g1, a_scale, a_stride, w_scale, w_stride, bias, bias_dtype,
                                               y, y_dtype, ldy, st, false, muladd);
      if (rc) return rc;
      return launch_dq<OP, REF, AccT, false>(
          g2, a_scale, a_stride, w_scale + (w_stride ? n0 : 0), w_stride,
          bias ? (const void*)((const char*)bias + n0 * bsz) : nullptr, bias_dtype,
          (void*)((char*)y + n0 * ysz), y_dtype, ldy, st, false, muladd);
    }
  }
#define GO(OUT, BIAS)                                                                         \
  {                                                                                           \
    EpiDequant<OUT, BIAS, REF, AccT, OP == MMA_I8 || OUT == FMSMO_F32> epi{y, ldy, a_scale, w_scale, bias, a_stride, w_stride, muladd}; \
    if constexpr (GROUPED) {                                                                  \
      if (g.K % 128 == 0 && use_register_staged(OP)) launch_rs<OP, true>(g, epi, st);         \
      else launch_tile<TileBig, OP, true>(g, epi, st);                                        \
    } else                                                                                    \
      launch_any<OP>(g, epi, st);                                                             \
  }
#define GO_BIAS(OUT)                            \
  switch (bias_dtype) {                         \
    case FMSMO_F16: GO(OUT, FMSMO_F16) break;   \
    case FMSMO_BF16: GO(OUT, FMSMO_BF16) break; \
    default: GO(OUT, FMSMO_F32) break;          \
  }
  switch (y_dtype) {
    case FMSMO_F16: GO_BIAS(FMSMO_F16) break;
    case FMSMO_BF16: GO_BIAS(FMSMO_BF16) break;
    case FMSMO_F32: GO_BIAS(FMSMO_F32) break;
    default: return FMSMO_ERR_UNSUPPORTED;
  }
#undef GO
#undef GO_BIAS
  return fmsmo_check_launch();
}

int check_dq(const float* a_scale, int64_t a_scale_n, const float* w_scale, int64_t w_scale_n,
             const void* bias, int bias_dtype, int y_dtype, int64_t M, int64_t N) {
  if (!a_scale || !w_scale) return FMSMO_ERR_NULL;
  if ((a_scale_n != 1 && a_scale_n != M) || (w_scale_n != 1 && w_scale_n != N)) return FMSMO_ERR_SHAPE;
  if (y_dtype < 0 || y_dtype > 2 || (bias && (bias_dtype < 0 || bias_dtype > 2))) return FMSMO_ERR_UNSUPPORTED;
  return FMSMO_OK;
}

}  // namespace

// ---------------------------------------------------------------------------------- split K
// Few output tiles and a long reduction (a batch of tens to hundreds of tokens through a
// projection with few output columns) leave most compute units idle: 17 x 4096 x 14336 is 32 tiles
// of 128 x 128.  With a caller-provided workspace the reduction is cut into slices that run as
// the uniform "groups" of the grouped kernels (A and B advance along K per group, the partial
// sums of group s land in rows [s M, (s + 1) M) of the workspace) and a second kernel adds the
// slices in a fixed order and applies the dequantizing epilogue.  int32 partial sums are exact, so
// the int8 result is bit-identical to the single-pass one.
namespace {

struct SplitPlan {
  int splits;
  int64_t k_len, ws_bytes;
  bool rs;  // 256 x 128 tiles of the register-staged kernel instead of 128 x 128 LDS-DMA tiles
  bool tall = false;  // 128 x 64 tiles with 128-byte stages
};

// `limit` > 0: the workspace at hand; a plan that needs more is passed over for the next one (the
// register-staged slices need more partial sums than the 128 x 128 ones: more, shorter slices).
inline SplitPlan plan_split_k(int64_t M, int64_t N, int64_t K, int64_t limit = 0) {
  SplitPlan p{1, K, 0, false};
  static const char* off = getenv("FMSMO_SPLIT_K");  // FMSMO_SPLIT_K=0 disables (tuning aid)
  if (off && off[0] == '0') return p;
  if (M <= 16 || M > 1024 || K % 128 || use_tall_tiles(M, N, K)) return p;
  // Long reductions under a few hundred rows: 256 x 128 tiles of the register-staged kernel carry
  // the slices (us, 128 x 128 LDS-DMA tiles -> these, N = 4096, K = 14336: M = 384 51.4 -> 49.0,
  // 512 54.6 -> 48.3, 768 84.7 -> 68.2, 1024 87.6 -> 77.8; at K = 4096 they lose, M = 512 25.5 ->
  // 27.7, and below 384 rows their 256-row tiles are half empty)
  if (K >= 8192 && M >= 384 && use_register_staged(0)) {
    const int64_t t = (int64_t)div_up(M, 256) * div_up(N, 128);
    // a full round of 128 x 128 tiles runs faster in one pass with 128-byte stages than as two
    // slices (1024 x 4096, us: K = 8192 53.4 -> 42.6, K = 14336 80.0 -> 72.5)
    const bool full_round = (int64_t)div_up(M, TileMidK::BM) * div_up(N, TileMidK::BN) == 256;
    if (t <= 128 && !full_round) {
      int s = (int)(256 / t);
      while (s > 1 && (K % (s * 128) != 0 || K / s < 512)) --s;
      if (s >= 2 && (limit <= 0 || (int64_t)s * M * N * 4 <= limit)) {
        p.splits = s;
        p.k_len = K / s;
        p.ws_bytes = (int64_t)s * M * N * 4;
        p.rs = true;
        return p;
      }
    }
  }
  // Slices of at least 1024 on 128 x 64 tiles with 128-byte stages: twice the blocks of the
  // 128 x 128 tiles for the same partial sums, or the same blocks for half of them (us, 128 x 128
  // tiles with 64-byte stages -> these, M = 65 / 100 / 128: N = 4096, K = 4096 15.8 / 16.9 / 16.5 ->
  // 13.4 / 14.2 / 14.9; N = 2048 13.2 / 13.5 / 11.9 -> 9.4 / 9.9 / 9.7; N = 1000 12.6 / 13.0 / 12.7 ->
  // 10.3 / 10.8 / 10.7; N = 4096, K = 2048 12.8 / 14.4 / 13.6 -> 10.1 / 11.5 / 11.4; K = 5120 17.3 /
  // 19.4 / 17.9 -> 13.8 / 15.5 / 16.3; K = 8192 18.9 / 19.6 / 18.3 -> 17.4 / 18.5 / 17.2; N = 1024,
  // K = 8192 14.3 / 14.6 / 13.1 -> 10.6 / 11.2 / 11.2; K = 14336, N = 4096, M = 33 / 128 / 256 22.7 /
  // 25.1 / 34.1 -> 22.1 / 24.3 / 33.0).  At most 256 blocks of 128 x 64 partial sums: 8 MiB.
  const int64_t tiles_t = (int64_t)div_up(M, TileTallK::BM) * div_up(N, TileTallK::BN);
  if (tiles_t <= 128) {
    int s = (int)(256 / tiles_t);
    while (s > 1 && (K % (s * 128) != 0 || K / s < 1024)) --s;
    if (s >= 2) {
      p.splits = s;
      p.k_len = K / s;
      p.ws_bytes = (int64_t)s * M * N * 4;
      p.tall = true;
      return p;
    }
  }
  // shorter reductions: 128 x 128 tiles, slices of at least 512
  const int64_t tiles = (int64_t)div_up(M, TileMid::BM) * div_up(N, TileMid::BN);
  if (tiles > 128) return p;
  int s = (int)(256 / tiles);  // one block per compute unit; 512 and 1024 blocks measured slower
  while (s > 1 && (K % (s * 128) != 0 || K / s < 512)) --s;
  // Slices of 512 are mostly prologue and partial-sum traffic (as many bytes as the weights at
  // 128 rows): from K = 4096 on, half as many slices of 1024 are faster while 64 blocks remain
  // (us, M = 65 / 100 / 128: N = 4096, K = 4096 16.4 / 18.8 / 18.1 -> 15.8 / 17.2 / 16.5; N = 2048
  // 13.8 / 15.1 / 14.1 -> 13.2 / 13.5 / 11.8; N = 1024, K = 8192 15.5 / 16.7 / 15.4 -> 14.2 / 14.6 /
  // 13.1; N = 1000, K = 4096, where 32 blocks would remain, 12.7 -> 14.1; K = 2048 no difference)
  if (K >= 4096 && K / s <= 512 && s >= 4 && s % 2 == 0 && tiles * (s / 2) >= 64) s /= 2;
  if (s < 2) return p;
  p.splits = s;
  p.k_len = K / s;
  p.ws_bytes = (int64_t)s * M * N * 4;
  return p;
}

template <class AccT, class Epi>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const AccT* __restrict__ ws, int S, int M,
                                                            int N, Epi epi) {
  const int n = blockIdx.x * 256 + threadIdx.x, m = blockIdx.y;
  if (n >= N) return;
  AccT sum = ws[(int64_t)m * N + n];
  for (int s = 1; s < S; ++s) sum += ws[((int64_t)s * M + m) * N + n];
  epi.store(m, n, sum, epi.row(m), epi.col(n, 0, N));
}

// c = sum over K slices (int32, exact), see above.  The caller has checked the operands.
inline int launch_split_k_i32(const SplitPlan& p, const GemmArgs& g0, void* workspace, int32_t* c, int64_t ldc,
                              hipStream_t st) {
  GemmArgs g = g0;
  g.K = (int)p.k_len;
  g.num_experts = p.splits;
  g.rows_per_group = g0.M;
  g.M = p.splits * g0.M;
  g.lda_e = p.k_len;
  g.ldb_e = p.k_len;
  g.grid_m = p.splits * div_up(g0.M, p.rs ? 256 : TileMid::BM);
  if (p.rs) launch_rs<MMA_I8, true, 128>(g, EpiStoreI32{(int32_t*)workspace, g0.N}, st);
  else if (p.tall) launch_tile<TileTallK, MMA_I8, true>(g, EpiStoreI32{(int32_t*)workspace, g0.N}, st);
  else launch_tile<TileMid, MMA_I8, true>(g, EpiStoreI32{(int32_t*)workspace, g0.N}, st);
  dim3 grid(div_up(g0.N, 256), (unsigned)g0.M), block(256);
  EpiStoreI32 epi{c, ldc};
  hipLaunchKernelGGL((splitk_reduce_kernel<int, EpiStoreI32>), grid, block, 0, st, (const int*)workspace,
                     p.splits, g0.M, g0.N, epi);
  return fmsmo_check_launch();
}

// y = epilogue( sum over K slices ), see above.  The caller has checked the operands.
template <int OP, bool REF, class AccT>
int launch_split_k(const SplitPlan& p, const GemmArgs& g0, void* workspace, const float* a_scale,
                   int a_stride, const float* w_scale, int w_stride, const void* bias,
                   int bias_dtype, void* y, int y_dtype, int64_t ldy, hipStream_t st, int muladd = 0) {
  GemmArgs g = g0;
  g.K = (int)p.k_len;
  g.num_experts = p.splits;
  g.rows_per_group = g0.M;
  g.M = p.splits * g0.M;
  g.lda_e = p.k_len;
  g.ldb_e = p.k_len;
  g.grid_m = p.splits * div_up(g0.M, p.rs ? 256 : TileMid::BM);
  if (p.rs) {
    if constexpr (OP == MMA_I8) launch_rs<OP, true, 128>(g, EpiStoreI32{(int32_t*)workspace, g0.N}, st);
    else launch_rs<OP, true, 128>(g, EpiStoreF32{(float*)workspace, g0.N}, st);
  } else if (p.tall) {
    if constexpr (OP == MMA_I8) launch_tile<TileTallK, OP, true>(g, EpiStoreI32{(int32_t*)workspace, g0.N}, st);
    else launch_tile<TileTallK, OP, true>(g, EpiStoreF32{(float*)workspace, g0.N}, st);
  } else if constexpr (OP == MMA_I8) launch_tile<TileMid, OP, true>(g, EpiStoreI32{(int32_t*)workspace, g0.N}, st);
  else launch_tile<TileMid, OP, true>(g, EpiStoreF32{(float*)workspace, g0.N}, st);
  if (!bias) bias_dtype = FMSMO_F32;
  dim3 grid(div_up(g0.N, 256), (unsigned)g0.M), block(256);
#define GO(OUT, BIAS)                                                                         \
  {                                                                                           \
    EpiDequant<OUT, BIAS, REF, AccT, OP == MMA_I8 || OUT == FMSMO_F32> epi{y, ldy, a_scale, w_scale, bias, a_stride, w_stride, muladd}; \
    hipLaunchKernelGGL((splitk_reduce_kernel<AccT, decltype(epi)>), grid, block, 0, st,       \
                       (const AccT*)workspace, p.splits, g0.M, g0.N, epi);                    \
  }
#define GO_BIAS(OUT)                            \
  switch (bias_dtype) {                         \
    case FMSMO_F16: GO(OUT, FMSMO_F16) break;   \
    case FMSMO_BF16: GO(OUT, FMSMO_BF16) break; \
    default: GO(OUT, FMSMO_F32) break;          \
  }
  switch (y_dtype) {
    case FMSMO_F16: GO_BIAS(FMSMO_F16) break;
    case FMSMO_BF16: GO_BIAS(FMSMO_BF16) break;
    case FMSMO_F32: GO_BIAS(FMSMO_F32) break;
    default: return FMSMO_ERR_UNSUPPORTED;
  }
#undef GO
#undef GO_BIAS
  return fmsmo_check_launch();
}

}  // namespace

// ------------------------------------------------------------------------------ batched matmul
namespace {

// Batches are the "groups" of the grouped kernels with a uniform row count: the rows of A (and of
// y) of all batches are stacked, B advances by stride_b per batch, the bias by N.
template <int OP, class AccT>
int launch_bmm(const void* a, int64_t lda, const void* b, int64_t ldb, int64_t stride_b,
               const float* a_scale, const float* b_scale, const float* bias, void* y, int y_dtype,
               int64_t ldy, int64_t batch, int64_t M, int64_t N, int64_t K, hipStream_t st) {
  int rc = check_gemm(a, lda, b, ldb, y, ldy, batch * M, N, K);
  if (rc) return rc;
  if (!a_scale || !b_scale) return FMSMO_ERR_NULL;
  if (batch <= 0 || M <= 0 || stride_b < N * ldb) return FMSMO_ERR_SHAPE;
  if (batch * stride_b >= (1ll << 40) || batch >= (1 << 20)) return FMSMO_ERR_UNSUPPORTED;
  if (K % 64 || stride_b % 16) return FMSMO_ERR_ALIGN;
  if (y_dtype < 0 || y_dtype > 2) return FMSMO_ERR_UNSUPPORTED;
  GemmArgs g{};
  g.a = (const uint8_t*)a; g.b = (const uint8_t*)b; g.lda = lda; g.ldb = ldb;
  g.M = (int)(batch * M); g.N = (int)N; g.K = (int)K;
  g.num_experts = (int)batch; g.ldb_e = stride_b; g.rows_per_group = (int)M;
  g.lda_e = M * lda;
  // small per-batch outputs (attention heads: N or M of 128) take the 128x128 tile
  const bool mid = N <= 128 || M <= 128;
  // probabilities x values: many rows, one head dimension of columns, a long reduction whose
  // A operand is read exactly once -- 256 x 128 tiles of the register-staged pipeline (whole
  // 128-byte lines of P), every block starting its reduction at a different slab: with all blocks
  // sweeping K in step, rows a power of two apart ask for the same memory channels at the same
  // time (4096 x 128 x 4096 per head, 32 heads: 0.144 ms in step, 0.118 ms staggered).  Operands
  // that several tiles share (the large GEMMs) want the opposite: their tiles meet in L2 because
  // they sweep K together (K = 14336: 205 -> 255 us when staggered).
  const bool tall = N > 64 && N <= 128 && M >= 256 && K % 128 == 0 && K >= 512 && use_register_staged(OP);
  g.k_rotate = tall ? 5 : 0;
#define GO(OUT)                                                                             \
  {                                                                                         \
    EpiDequant<OUT, FMSMO_F32, false, AccT> epi{y, ldy, a_scale, b_scale, bias, 0, 0};      \
    if (tall) {                                                                             \
      g.grid_m = (int)batch * div_up(M, 256);                                               \
      launch_rs<OP, true, 128>(g, epi, st);                                                 \
    } else if (mid) {                                                                       \
      g.grid_m = (int)batch * div_up(M, TileMid::BM);                                       \
      launch_tile<TileMid, OP, true>(g, epi, st);                                           \
    } else {                                                                                \
      g.grid_m = (int)batch * div_up(M, 256);                                               \
      if (K == 128 && use_register_staged(OP)) {                                            \
        launch_k128<OP>(g, (int)batch, (int)M, EpiScaleBias<OUT, AccT>{y, ldy, a_scale, b_scale, bias}, st); \
      }                                                                                     \
      else if (K % 128 == 0 && use_register_staged(OP)) launch_rs<OP, true>(g, epi, st);    \
      else launch_tile<TileBig, OP, true>(g, epi, st);                                      \
    }                                                                                       \
  }
  switch (y_dtype) {
    case FMSMO_F16: GO(FMSMO_F16) break;
    case FMSMO_BF16: GO(FMSMO_BF16) break;
    default: GO(FMSMO_F32) break;
  }
#undef GO
  return fmsmo_check_launch();
}

}  // namespace
