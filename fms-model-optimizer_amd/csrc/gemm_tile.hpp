// LDS-tiled MFMA GEMM core for gfx950:  C[M,N] = A[M,K] . B[N,K]^T with 1-byte operands.
//
// Data movement: both operands are K-contiguous, so a tile is a set of rows of BK bytes.  Tiles
// go HBM/L2 -> LDS with global_load_lds_dwordx4 (no VGPR staging); each wave instruction moves
// 64 x 16 B = 1 KiB that lands contiguously in LDS, i.e. 1024/BK whole rows, so every row is
// fetched as one BK-byte run (full 128-byte lines for BK = 128).  The 16-byte chunks of a row
// are XOR-permuted on the way in (the lane picks which global chunk it fetches) so that the
// ds_read_b128 operand fetches of the MFMA phase are bank-conflict free.
//
// Math: each wave owns a (BM/WGM) x (BN/WGN) sub-tile built from 32x32 MFMA blocks
// (v_mfma_i32_32x32x32_i8, or v_mfma_f32_32x32x64_f8f6f4 with both operands e4m3).  The MFMA
// sums over k, so any assignment of k-bytes to (lane group, register byte) is valid as long as
// A and B use the same one; the loaders exploit that and never transpose anything.
//
// Pipeline: NSTAGE LDS buffers.  The DMA of stage kt+NSTAGE is issued during the last MFMA k-step
// of stage kt, so every stage has NSTAGE-1 full iterations (> 1 us) to arrive from L2/HBM.
// One barrier per stage; the barrier, the DMA issue and the first operand reads of the next
// stage are hidden under MFMAs whose operands were read earlier (register double buffering).
#pragma once
#include "common.hpp"
#include <type_traits>
#include <utility>

namespace fmsmo {

enum { MMA_I8 = 0, MMA_FP8 = 1, MMA_FP8_K32 = 2, MMA_F16 = 3, MMA_BF16 = 4, MMA_F32 = 5 };

struct GemmArgs {
  const uint8_t* a;
  const uint8_t* b;
  int64_t lda, ldb;  // bytes
  int M, N, K;
  int grid_m, grid_n;  // tiles along M and N (grid_m is an upper bound in grouped mode)
  int group_m;         // tile-order grouping along M
  // grouped (mixture-of-experts) mode
  const int32_t* offsets;
  int num_experts;
  int64_t ldb_e;  // bytes between experts in B
  int rows_per_group;  // > 0: every group owns this many rows (batched matmul, split K), offsets unused
  int64_t lda_e;       // uniform groups: bytes between groups in A (rows * lda for stacked batches,
                       // the K slice length when the groups are slices of one reduction)
  int k_rotate;  // register-staged kernel: block b starts its reduction at slab (b * k_rotate) % slabs
  // optional clock probe (register-staged kernel): block 0 stores {core clock counter, 100 MHz
  // wall clock} at its start, after its K loop and after its epilogue; null = off
  unsigned long long* clk;
};

// 16-byte chunk c of row r is stored at chunk position c ^ swz(r).  Depends on r & 15 only.
template <int CPR, int SWZ>
__device__ __forceinline__ int swz(int r) {
  if constexpr (SWZ == 0) return 0;
  if constexpr (CPR == 8) {
    if constexpr (SWZ == 1) return (r & 7) ^ ((r >> 3) & 1);
    if constexpr (SWZ == 2) return (r & 7);
    return (r >> 1) & 7;
  } else {  // CPR == 4
    if constexpr (SWZ == 1) return ((r >> 1) & 3) ^ ((r >> 3) & 1);
    if constexpr (SWZ == 2) return (r >> 1) & 3;
    return (r >> 2) & 3;
  }
}

template <int OP>
struct Mma;
template <>
struct Mma<MMA_I8> {
  typedef v4i Frag;
  typedef v16i Acc;
  typedef int Elem;
  static constexpr int KSTEP = 32;  // bytes of K per MFMA
  __device__ static __forceinline__ Acc mma(const Frag& a, const Frag& b, const Acc& c) {
    return __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0);
  }
};
template <>
struct Mma<MMA_FP8> {
  typedef v8i Frag;
  typedef v16f Acc;
  typedef float Elem;
  static constexpr int KSTEP = 64;
  __device__ static __forceinline__ Acc mma(const Frag& a, const Frag& b, const Acc& c) {
    // cbsz = blgp = 0: both operands OCP e4m3; zero scale operands select the unscaled form.
    return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0);
  }
};

// 32-byte k-steps for the chunked-accumulation kernels (chunk boundaries are multiples of 32
// bytes of K for every operand type): two legacy K=16 e4m3 MFMAs, one K=16 f16 / bf16 MFMA, four
// K=2 fp32 MFMAs per 16-byte lane operand.
template <>
struct Mma<MMA_FP8_K32> {
  typedef v4i Frag;
  typedef v16f Acc;
  typedef float Elem;
  static constexpr int KSTEP = 32;
  __device__ static __forceinline__ Acc mma(const Frag& a, const Frag& b, const Acc& c) {
    const long a0 = ((long)(unsigned)a[1] << 32) | (unsigned)a[0];
    const long a1 = ((long)(unsigned)a[3] << 32) | (unsigned)a[2];
    const long b0 = ((long)(unsigned)b[1] << 32) | (unsigned)b[0];
    const long b1 = ((long)(unsigned)b[3] << 32) | (unsigned)b[2];
    Acc t = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(a0, b0, c, 0, 0, 0);
    return __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(a1, b1, t, 0, 0, 0);
  }
};
template <>
struct Mma<MMA_F16> {
  typedef v4i Frag;
  typedef v16f Acc;
  typedef float Elem;
  static constexpr int KSTEP = 32;
  typedef _Float16 v8h __attribute__((ext_vector_type(8)));
  __device__ static __forceinline__ Acc mma(const Frag& a, const Frag& b, const Acc& c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, a),
                                                  __builtin_bit_cast(v8h, b), c, 0, 0, 0);
  }
};
template <>
struct Mma<MMA_BF16> {
  typedef v4i Frag;
  typedef v16f Acc;
  typedef float Elem;
  static constexpr int KSTEP = 32;
  typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
  __device__ static __forceinline__ Acc mma(const Frag& a, const Frag& b, const Acc& c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, a),
                                                   __builtin_bit_cast(v8bf, b), c, 0, 0, 0);
  }
};
template <>
struct Mma<MMA_F32> {
  typedef v4i Frag;
  typedef v16f Acc;
  typedef float Elem;
  static constexpr int KSTEP = 32;
  __device__ static __forceinline__ Acc mma(const Frag& a, const Frag& b, const Acc& c) {
    Acc t = c;
#pragma unroll
    for (int e = 0; e < 4; ++e)
      t = __builtin_amdgcn_mfma_f32_32x32x2f32(__int_as_float(a[e]), __int_as_float(b[e]), t, 0, 0, 0);
    return t;
  }
};

// ---- chunked accumulation: every `chunk_ks` MFMA k-steps the partial product is range-clamped /
// LSB-rounded and folded into the running accumulator (or the running accumulator itself is
// rounded when tta == 0).
struct NoChunk {
  static constexpr bool enabled = false;
  static constexpr bool fast = false;
  static constexpr bool one_stage = false;
};
// FAST = the common configuration (truncate-then-accumulate, no integer clamp, no DL16 clamp):
// three vector ALU operations per accumulator element and chunk.
// ONE_STAGE (with FAST) = the schedules that interleave the rounding of one 32x32 block with the
// MFMAs of the others inside one wave (see the loop in gemm_tile_kernel): integers with any chunk
// of one k-step or of whole LDS stages, floating point with a chunk of exactly one stage.
// SCHED: 1 = a chunk is one stage, 2 = several whole stages, 3 = one k-step (integers only); each is
// a kernel of its own (one kernel holding all three loops runs out of registers).
template <bool FAST, int SCHED = 0>
struct ChunkTrunc {
  static_assert(FAST || SCHED == 0, "the interleaved schedules exist for the fast configuration only");
  static constexpr bool enabled = true;
  static constexpr bool fast = FAST;
  static constexpr bool one_stage = SCHED != 0;
  static constexpr int sched = SCHED;
  int chunk_ks;           // MFMA k-steps (32 bytes of K) per chunk
  int t, lo, hi;          // LSBs to round away; integer clamp range
  unsigned round_bit, mask;
  int post, dl16, tta;
  const void* c_in;       // optional initial accumulator [M, N], same element type as the output
  int64_t ldc;
};
__device__ __forceinline__ int trunc_i32(int p, int lo, int hi, int round_bit, int t) {
  p = max(min(p, hi), lo);
  // (p + 2^(t-1)) >> t << t with two's-complement wrap on the add, arithmetic right shift
  p = (int)((unsigned)p + (unsigned)round_bit);
  return (int)((unsigned)(p >> t) << t);
}
__device__ __forceinline__ float trunc_f32(float p, unsigned round_bit, unsigned mask, int dl16) {
  float x = __uint_as_float((__float_as_uint(p) + round_bit) & mask);
  if (dl16) {
    x = x >= 8581545984.0f ? __builtin_inff() : x;
    x = x <= -8581545984.0f ? -__builtin_inff() : x;
    x = fabsf(x) < 4.665707820095122e-10f ? 0.0f : x;
  }
  return x;
}

// Position `pid` of the tile sequence: column-major inside groups of `group_m` tile rows (the
// second half of tile_of_block below, for blocks that walk the sequence themselves).
__device__ __forceinline__ void tile_of_pid(int pid, int grid_m, int grid_n, int group_m, int& tm, int& tn) {
  const int in_group = group_m * grid_n;
  const int gid = pid / in_group;
  const int first_m = gid * group_m;
  const int gsz = min(grid_m - first_m, group_m);
  const int r = pid - gid * in_group;
  tm = first_m + r % gsz;
  tn = r / gsz;
}

// Map the hardware block id to a tile.  Work-groups are dealt round-robin to the 8 XCDs (each
// with a private L2), so block b runs on XCD b % 8; give every XCD one contiguous span of the
// tile sequence, and order that sequence in column-major groups of `group_m` tile rows so the
// tiles resident on an XCD at the same time share A rows and B rows.
__device__ __forceinline__ void tile_of_block(int bid, int nblk, int grid_m, int grid_n,
                                              int group_m, int& tm, int& tn) {
  const int per = nblk >> 3, rem = nblk & 7;
  const int xcd = bid & 7, idx = bid >> 3;
  const int pid = (xcd < rem ? xcd * (per + 1) : rem * (per + 1) + (xcd - rem) * per) + idx;
  const int in_group = group_m * grid_n;
  const int gid = pid / in_group;
  const int first_m = gid * group_m;
  const int gsz = min(grid_m - first_m, group_m);
  const int r = pid - gid * in_group;
  tm = first_m + r % gsz;
  tn = r / gsz;
}

template <int BM, int BN, int BK, int NSTAGE, int WGM, int WGN, int OP, int SWZ, bool GROUPED,
          class Epi, class Chk = NoChunk>
// (two blocks per compute unit for the scheduled chunk hooks; the generic hook keeps a second
// accumulator set and would spill at 256 registers)
__global__ __launch_bounds__(WGM* WGN * 64, (Chk::enabled && Chk::fast) ? 2 : 1) void gemm_tile_kernel(GemmArgs g, Epi epi, Chk chk) {
#if defined(__HIP_DEVICE_COMPILE__)  // the host pass only needs the launch stub
  typedef Mma<OP> MM;
  typedef typename MM::Frag Frag;
  typedef typename MM::Acc Acc;
  constexpr int THREADS = WGM * WGN * 64;
  constexpr int CPR = BK / 16;              // 16-byte chunks per tile row
  constexpr int RPI = THREADS / CPR;        // tile rows moved by one block-wide load instruction
  constexpr int NIA = BM / RPI, NIB = BN / RPI;
  constexpr int TM = BM / WGM, TN = BN / WGN;  // wave sub-tile
  constexpr int FM = TM / 32, FN = TN / 32;    // 32x32 MFMA blocks per wave
  constexpr int NKS = BK / MM::KSTEP;          // MFMA k-steps per stage
  constexpr int CL = MM::KSTEP / 32;           // 16-byte chunks per lane per k-step
  static_assert(RPI % 16 == 0 && BM % RPI == 0 && BN % RPI == 0, "loader shape");
  static_assert(TM % 32 == 0 && TN % 32 == 0, "wave tile");

  constexpr int STAGE_BYTES = (BM + BN) * BK;
  __shared__ __attribute__((aligned(16))) uint8_t lds[NSTAGE][STAGE_BYTES];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WGN, wn = wave % WGN;

  int tile_m, tile_n;
  int row_lo = 0, row_hi = g.M, expert = 0;
  int64_t a_adj = 0;
  if constexpr (GROUPED) {
    if (g.rows_per_group > 0) {
      // batched matmul: every group has the same number of rows, the grid is exact
      const int nt = (g.rows_per_group + BM - 1) / BM;
      tile_of_block(blockIdx.x, gridDim.x, g.num_experts * nt, g.grid_n, g.group_m, tile_m, tile_n);
      expert = tile_m / nt;
      row_lo = expert * g.rows_per_group + (tile_m - expert * nt) * BM;
      row_hi = (expert + 1) * g.rows_per_group;
      // rows are numbered as stacked groups (that is how the output is laid out); A may be laid
      // out differently
      a_adj = (int64_t)expert * (g.lda_e - (int64_t)g.rows_per_group * g.lda);
    } else {
      // The launch grid is an upper bound (the host cannot see the expert sizes).  Count the
      // real row tiles and map only the first real_tiles block ids, so that every XCD gets an
      // equal share of real work; the surplus blocks are the last to be dispatched and exit at
      // once.
      int real_m = 0;
      for (int e = 0; e < g.num_experts; ++e) real_m += (g.offsets[e + 1] - g.offsets[e] + BM - 1) / BM;
      const int real_tiles = real_m * g.grid_n;
      if ((int)blockIdx.x >= real_tiles) return;  // uniform for the whole block
      tile_of_block(blockIdx.x, real_tiles, real_m, g.grid_n, g.group_m, tile_m, tile_n);
      int t = tile_m;
      for (int e = 0; e < g.num_experts; ++e) {
        const int lo = g.offsets[e], hi = g.offsets[e + 1];
        const int nt = (hi - lo + BM - 1) / BM;
        if (t < nt) {
          row_lo = lo + t * BM;
          row_hi = hi;
          expert = e;
          break;
        }
        t -= nt;
      }
    }
  } else {
    tile_of_block(blockIdx.x, gridDim.x, g.grid_m, g.grid_n, g.group_m, tile_m, tile_n);
    row_lo = tile_m * BM;
  }
  const int col_lo = tile_n * BN;

  const uint8_t* __restrict__ A = g.a + a_adj;
  const uint8_t* __restrict__ B = g.b + (GROUPED ? (int64_t)expert * g.ldb_e : 0);

  // ---- global -> LDS loader addressing (per thread, constant over the K loop)
  const int ld_row = tid / CPR;
  const int ld_pos = tid % CPR;
  const int ld_chunk = ld_pos ^ swz<CPR, SWZ>(ld_row);
  uint32_t a_off[NIA], b_off[NIB];
#pragma unroll
  for (int j = 0; j < NIA; ++j) {
    const int r = min(row_lo + ld_row + j * RPI, row_hi - 1);  // clamp: rows past the end re-read
    a_off[j] = (uint32_t)r * (uint32_t)g.lda + ld_chunk * 16;  // the last valid row, never stored
  }
#pragma unroll
  for (int j = 0; j < NIB; ++j) {
    const int r = min(col_lo + ld_row + j * RPI, g.N - 1);
    b_off[j] = (uint32_t)r * (uint32_t)g.ldb + ld_chunk * 16;
  }

  // DMA instructions j in [j0, j1) of a stage (A rows first, then B rows).  Buffer addressing:
  // per-lane 32-bit row/chunk offset (constant over K) + scalar K offset, so the loop needs no
  // vector address arithmetic.
  const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc((void*)A, 0, -1, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc((void*)B, 0, -1, 0x00020000);
  auto issue_part = [&](int stage, int k0, auto j0_c, auto j1_c) {
    constexpr int J0 = decltype(j0_c)::value, J1 = decltype(j1_c)::value;
    uint8_t* la = &lds[0][0] + stage * STAGE_BYTES + wave * 1024;
#pragma unroll
    for (int j = J0; j < J1; ++j) {
      if (j < NIA)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, FMSMO_LPTR(la + j * THREADS * 16), 16,
                                                 a_off[j], k0, 0, 0);
      else
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, FMSMO_LPTR(la + j * THREADS * 16), 16,
                                                 b_off[j - NIA], k0, 0, 0);
    }
  };

  // ---- LDS -> MFMA operand addressing
  const int fr = lane & 31, fg = lane >> 5;
  const int fsw = swz<CPR, SWZ>(fr);
  int a_rd[NKS][CL], b_rd[NKS][CL];
#pragma unroll
  for (int s = 0; s < NKS; ++s)
#pragma unroll
    for (int e = 0; e < CL; ++e) {
      const int c = s * 2 * CL + fg * CL + e;
      a_rd[s][e] = (wm * TM + fr) * BK + ((c ^ fsw) * 16);
      b_rd[s][e] = BM * BK + (wn * TN + fr) * BK + ((c ^ fsw) * 16);
    }

  Acc acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0;

  // chunked accumulation: MFMAs run into `work`, finished chunks are folded into `acc`
  typedef typename MM::Elem Elem;
  Acc work[Chk::enabled ? FM : 1][Chk::enabled ? FN : 1];
  int ks_cnt = 0;
  if constexpr (Chk::enabled) {
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int j = 0; j < FN; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          Elem init = 0;
          if (chk.c_in) {
            const int m = row_lo + wm * TM + i * 32 + (v >> 2) * 8 + (lane >> 5) * 4 + (v & 3);
            const int n = col_lo + wn * TN + j * 32 + (lane & 31);
            if (m < row_hi && n < g.N) init = ((const Elem*)chk.c_in)[(int64_t)m * chk.ldc + n];
          }
          acc[i][j][v] = chk.tta ? init : (Elem)0;
          work[i][j][v] = chk.tta ? (Elem)0 : init;
        }
  }
  auto finish_chunk = [&](auto post_c, auto tta_c) __attribute__((always_inline)) {
    constexpr bool POST = decltype(post_c)::value, TTA = decltype(tta_c)::value;
    if constexpr (Chk::enabled) {
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            Elem p = work[i][j][v];
            if constexpr (POST) {
              if constexpr (std::is_same<Elem, int>::value) p = trunc_i32(p, chk.lo, chk.hi, (int)chk.round_bit, chk.t);
              else p = trunc_f32(p, chk.round_bit, chk.mask, chk.dl16);
            }
            if constexpr (TTA) {
              if constexpr (std::is_same<Elem, int>::value) acc[i][j][v] = (int)((unsigned)acc[i][j][v] + (unsigned)p);
              else acc[i][j][v] += p;
              work[i][j][v] = 0;
            } else {
              work[i][j][v] = p;  // the running accumulator itself is rounded
            }
          }
    }
  };
  auto finish_any = [&]() __attribute__((always_inline)) {
    if constexpr (Chk::fast) {
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            // (p + 2^(t-1)) with the low t bits cleared: same bits for two's-complement integers
            // ((p + r) >> t << t) and for fp32 patterns; work is overwritten by the next chunk
            if constexpr (std::is_same<Elem, int>::value) {
              acc[i][j][v] = (int)((unsigned)acc[i][j][v] + (((unsigned)work[i][j][v] + chk.round_bit) & chk.mask));
            } else {
              acc[i][j][v] += __uint_as_float((__float_as_uint(work[i][j][v]) + chk.round_bit) & chk.mask);
            }
          }
    } else if constexpr (Chk::enabled) {
      if (chk.tta) {
        if (chk.post) finish_chunk(std::true_type{}, std::true_type{});
        else finish_chunk(std::false_type{}, std::true_type{});
      } else if (chk.post) {
        finish_chunk(std::true_type{}, std::false_type{});
      }
    }
  };
  auto chunk_tick = [&]() __attribute__((always_inline)) {
    if constexpr (Chk::enabled) {
      if (++ks_cnt == chk.chunk_ks) {
        finish_any();
        ks_cnt = 0;
      }
    }
  };

  auto read_frags = [&](const uint8_t* ls, int s, Frag* af, Frag* bf) {
#pragma unroll
    for (int i = 0; i < FM; ++i) {
      if constexpr (CL == 1) {
        af[i] = *(const v4i*)(ls + a_rd[s][0] + i * 32 * BK);
      } else {
        const v4i lo = *(const v4i*)(ls + a_rd[s][0] + i * 32 * BK);
        const v4i hi = *(const v4i*)(ls + a_rd[s][1] + i * 32 * BK);
        af[i] = Frag{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      }
    }
#pragma unroll
    for (int j = 0; j < FN; ++j) {
      if constexpr (CL == 1) {
        bf[j] = *(const v4i*)(ls + b_rd[s][0] + j * 32 * BK);
      } else {
        const v4i lo = *(const v4i*)(ls + b_rd[s][0] + j * 32 * BK);
        const v4i hi = *(const v4i*)(ls + b_rd[s][1] + j * 32 * BK);
        bf[j] = Frag{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      }
    }
  };
  auto mma_step = [&](const Frag* af, const Frag* bf) {
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int j = 0; j < FN; ++j) {
        if constexpr (Chk::enabled) work[i][j] = MM::mma(af[i], bf[j], work[i][j]);
        else acc[i][j] = MM::mma(af[i], bf[j], acc[i][j]);
      }
  };
  // first k-step of a chunk in FAST mode: the MFMA's C operand is the constant 0, so `work` needs
  // no clearing between chunks
  auto mma_step_fresh = [&](const Frag* af, const Frag* bf) {
    Acc zero;
#pragma unroll
    for (int v = 0; v < 16; ++v) zero[v] = 0;
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int j = 0; j < FN; ++j) work[i][j] = MM::mma(af[i], bf[j], zero);
  };
  auto mma_any = [&](const Frag* af, const Frag* bf) __attribute__((always_inline)) {
    if constexpr (Chk::fast) {
      if (ks_cnt == 0) mma_step_fresh(af, bf);
      else mma_step(af, bf);
    } else {
      mma_step(af, bf);
    }
  };
  // Instruction-order hints (DS read = 0x100, MFMA = 0x008, VMEM = 0x020): the operand reads of
  // the next k-step go between the first MFMAs of the current one, so their latency is covered
  // by the remaining MFMAs; the DMA instructions are spread evenly behind them (the texture
  // path takes ~16 cycles per 1 KiB wave instruction and is shared by the whole CU, so bursts
  // of DMA issue would stall the in-order wave and starve the MFMA pipe).
  constexpr int NRD = (FM + FN) * CL, NMMA = FM * FN, NLD = NIA + NIB;
  // DMA instructions [NLD * S / NKS, NLD * (S + 1) / NKS) are issued during k-step S
  static_assert(NSTAGE >= 3, "pipeline needs at least three LDS stages");
  auto interleave = [&](auto ldp_c) {
    constexpr int LDP = decltype(ldp_c)::value;  // DMA instructions issued in this k-step
    constexpr int PER = (NMMA / 2) / NRD > 0 ? (NMMA / 2) / NRD : 1;
#pragma unroll
    for (int r = 0; r < NRD; ++r) {
      __builtin_amdgcn_sched_group_barrier(0x008, PER, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    constexpr int REST = NMMA - PER * NRD > 0 ? NMMA - PER * NRD : 0;
    if constexpr (REST >= LDP && LDP > 0) {
      constexpr int MPL = REST / LDP;  // MFMAs per DMA instruction
#pragma unroll
      for (int r = 0; r < LDP; ++r) {
        __builtin_amdgcn_sched_group_barrier(0x008, MPL, 0);
        __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
      }
      if constexpr (REST - MPL * LDP > 0) __builtin_amdgcn_sched_group_barrier(0x008, REST - MPL * LDP, 0);
    } else if constexpr (REST > 0) {
      __builtin_amdgcn_sched_group_barrier(0x008, REST, 0);
    }
  };

  Frag fa[2][FM], fb[2][FN];
  const int nk = g.K / BK;

  // One K-stage.  PAR = parity of kt * NKS, so that operand-register buffer indices are static.
  // While stage kt is multiplied, the DMA of stage kt+NSTAGE-1 refills the buffer that stage
  // kt-1 occupied (free since the barrier at the end of stage kt-1).  Stages past the end of K
  // are "phantom": their DMA re-reads the last real stage into a buffer nobody consumes, which
  // keeps the loop body and the vmcnt bookkeeping uniform.
  auto stage = [&](int kt, auto par_c) {
    constexpr int PAR = decltype(par_c)::value;
    const int cur = kt % NSTAGE;
    const int fill = (kt + NSTAGE - 1) % NSTAGE;
    const int fill_k0 = min(kt + NSTAGE - 1, nk - 1) * BK;
    const uint8_t* ls = &lds[0][0] + cur * STAGE_BYTES;
    auto dma = [&](auto s_c) {
      constexpr int S = decltype(s_c)::value;
      issue_part(fill, fill_k0, std::integral_constant<int, NLD * S / NKS>{},
                 std::integral_constant<int, NLD * (S + 1) / NKS>{});
    };
    [&]<int... S>(std::integer_sequence<int, S...>) {
      (
          [&] {
            read_frags(ls, S + 1, fa[(PAR + S + 1) & 1], fb[(PAR + S + 1) & 1]);
            dma(std::integral_constant<int, S>{});
            mma_any(fa[(PAR + S) & 1], fb[(PAR + S) & 1]);
            interleave(std::integral_constant<int, NLD * (S + 1) / NKS - NLD * S / NKS>{});
            chunk_tick();
          }(),
          ...);
    }(std::make_integer_sequence<int, NKS - 1>{});
    // Last k-step: its operands are already in registers.  Wait until this wave's share of
    // stage kt+1 has landed (younger DMA may stay in flight) and until its own LDS reads of
    // stage kt have returned, then barrier: stage kt+1 is now complete for all waves and buffer
    // `cur` may be refilled during the next stage.
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"((NSTAGE - 3) * NLD + NLD * (NKS - 1) / NKS)
                 : "memory");
    const int nxt = (kt + 1) % NSTAGE;
    read_frags(&lds[0][0] + nxt * STAGE_BYTES, 0, fa[(PAR + NKS) & 1], fb[(PAR + NKS) & 1]);
    dma(std::integral_constant<int, NKS - 1>{});
    mma_any(fa[(PAR + NKS - 1) & 1], fb[(PAR + NKS - 1) & 1]);
    interleave(std::integral_constant<int, NLD - NLD * (NKS - 1) / NKS>{});
    chunk_tick();
  };

#pragma unroll
  for (int st = 0; st < NSTAGE - 1; ++st)
    issue_part(st, min(st, nk - 1) * BK, std::integral_constant<int, 0>{},
               std::integral_constant<int, NLD>{});
  asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"((NSTAGE - 2) * NLD) : "memory");
  if constexpr (Chk::one_stage) {
    // Chunk == stage: the fragments of all k-steps of a chunk are register resident (two sets:
    // the stage being multiplied and the one being read), and the rounding of one 32x32 block is
    // issued between the MFMAs of the others, so that one wave keeps both units busy.  With all
    // MFMAs of a chunk issued before any rounding (the generic schedule) the units take turns, and
    // only a second resident wave overlaps them -- which a problem with about one tile per compute
    // unit does not have.
    Frag ca[2][NKS][FM], cb[2][NKS][FN];
    constexpr bool INT = std::is_same<Elem, int>::value;
    auto stage_top = [&](int kt, auto par_c) {
      constexpr int PAR = decltype(par_c)::value;
      // stage kt + 1 has landed for every wave; its fragments go to the other register set, and
      // the buffer of stage kt - 1 (last read a stage ago) is refilled with stage kt + 3
      asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"((NSTAGE - 3) * NLD) : "memory");
      const uint8_t* ls = &lds[0][0] + ((kt + 1) % NSTAGE) * STAGE_BYTES;
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) read_frags(ls, ks, ca[PAR ^ 1][ks], cb[PAR ^ 1][ks]);
      issue_part((kt + NSTAGE - 1) % NSTAGE, min(kt + NSTAGE - 1, nk - 1) * BK,
                 std::integral_constant<int, 0>{}, std::integral_constant<int, NLD>{});
      __builtin_amdgcn_sched_barrier(0);
    };
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) read_frags(&lds[0][0], ks, ca[0][ks], cb[0][ks]);
    if constexpr (INT) {
      // Integers: with R the running sum (a multiple of 2^t) and r the rounding bit, a chunk's
      // MFMAs started from C = R + r leave W = R + p + r, and (W & mask) = R + ((p + r) & mask) is
      // the new running sum: ONE operation per element and chunk, W <- (W & mask) | r, turns the
      // accumulator into the next chunk's C operand (low bits are zero, so OR adds r), and the
      // matrix unit does the accumulation.  8 such operations take as long as one MFMA, and a
      // chunk has 8 MFMAs and 64 elements per lane: the steady state below issues 8 operations in
      // front of every MFMA.  Block b's k-steps are two MFMA slots apart, its 16 operations follow
      // its second MFMA by a slot or more and are complete before its next first MFMA:
      //   slot       0       1       2       3       4       5       6       7
      //   rounding   b1 hi'  b2 lo'  b2 hi'  b3 lo'  b3 hi'  b0 lo   b0 hi   b1 lo    (' = previous chunk)
      //   MFMA       b0 k0   b1 k0   b0 k1   b1 k1   b2 k0   b3 k0   b2 k1   b3 k1
      // (a chunk of several stages rounds behind its last stage only; a chunk of one k-step has a
      // table of its own below)
      // Rounding an accumulator that holds C = R + r changes nothing, so the first chunk runs the
      // same code.  An initial accumulator enters as its multiple of 2^t; its low bits are added
      // at the end (adding a multiple of 2^t commutes with clearing the low bits).
      static_assert(NKS == 2 && FM == 2 && FN == 2, "the slot table is written for 2 k-steps x 4 blocks");
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int jj = 0; jj < FN; ++jj)
#pragma unroll
          for (int v = 0; v < 16; ++v)
            work[i][jj][v] = (int)(((unsigned)acc[i][jj][v] & chk.mask) | chk.round_bit);
      // (one v_and_or_b32: the instruction takes a single scalar operand, so the rounding bit
      // lives in a vector register)
      unsigned rbv = chk.round_bit;
      asm volatile("" : "+v"(rbv));
      auto rnd = [&](auto b_c, auto h_c) {
        constexpr int I = decltype(b_c)::value / FN, J = decltype(b_c)::value % FN, H = decltype(h_c)::value;
#pragma unroll
        for (int v = H * 8; v < H * 8 + 8; ++v)
          work[I][J][v] = (int)(((unsigned)work[I][J][v] & chk.mask) | rbv);
        __builtin_amdgcn_sched_barrier(0);
      };
      auto mm = [&](auto par_c, auto b_c, auto ks_c) {
        constexpr int PAR = decltype(par_c)::value, KS = decltype(ks_c)::value;
        constexpr int I = decltype(b_c)::value / FN, J = decltype(b_c)::value % FN;
        work[I][J] = MM::mma(ca[PAR][KS][I], cb[PAR][KS][J], work[I][J]);
        __builtin_amdgcn_sched_barrier(0);
      };
      typedef std::integral_constant<int, 0> I0;
      typedef std::integral_constant<int, 1> I1;
      typedef std::integral_constant<int, 2> I2;
      typedef std::integral_constant<int, 3> I3;
      if constexpr (Chk::sched == 1) {
        // a chunk is one stage: the table as it stands
        auto chunk_stage = [&](int kt, auto par_c) {
          stage_top(kt, par_c);
          rnd(I1{}, I1{}); mm(par_c, I0{}, I0{});
          rnd(I2{}, I0{}); mm(par_c, I1{}, I0{});
          rnd(I2{}, I1{}); mm(par_c, I0{}, I1{});
          rnd(I3{}, I0{}); mm(par_c, I1{}, I1{});
          rnd(I3{}, I1{}); mm(par_c, I2{}, I0{});
          rnd(I0{}, I0{}); mm(par_c, I3{}, I0{});
          rnd(I0{}, I1{}); mm(par_c, I2{}, I1{});
          rnd(I1{}, I0{}); mm(par_c, I3{}, I1{});
        };
        int kt = 0;
        for (; kt + 1 < nk; kt += 2) {
          chunk_stage(kt, I0{});
          chunk_stage(kt + 1, I1{});
        }
        if (kt < nk) chunk_stage(kt, I0{});
      } else if constexpr (Chk::sched == 2) {
        // a chunk is several whole stages: the roundings run only behind a chunk's last stage
        // (slots 5 - 7 of that stage, slots 0 - 4 of the following one)
        const int spc = chk.chunk_ks / NKS;
        int phase = 0;  // stage index inside the chunk
        auto chunk_stage = [&](int kt, auto par_c) {
          stage_top(kt, par_c);
          const bool prev_end = phase == 0, this_end = phase + 1 == spc;
          phase = this_end ? 0 : phase + 1;
          if (prev_end) rnd(I1{}, I1{});
          mm(par_c, I0{}, I0{});
          if (prev_end) rnd(I2{}, I0{});
          mm(par_c, I1{}, I0{});
          if (prev_end) rnd(I2{}, I1{});
          mm(par_c, I0{}, I1{});
          if (prev_end) rnd(I3{}, I0{});
          mm(par_c, I1{}, I1{});
          if (prev_end) rnd(I3{}, I1{});
          mm(par_c, I2{}, I0{});
          if (this_end) rnd(I0{}, I0{});
          mm(par_c, I3{}, I0{});
          if (this_end) rnd(I0{}, I1{});
          mm(par_c, I2{}, I1{});
          if (this_end) rnd(I1{}, I0{});
          mm(par_c, I3{}, I1{});
        };
        int kt = 0;
        for (; kt + 1 < nk; kt += 2) {
          chunk_stage(kt, I0{});
          chunk_stage(kt + 1, I1{});
        }
        if (kt < nk) chunk_stage(kt, I0{});
      } else {
        // a chunk is one k-step (32 bytes of K): 16 roundings per MFMA, the vector ALU is the
        // bound (half the MFMA rate at best).  Per k-step: MFMA b0, round b2', MFMA b1, round b3',
        // MFMA b2, round b0, MFMA b3, round b1 (' = of the previous k-step).
        auto chunk_stage = [&](int kt, auto par_c) {
          stage_top(kt, par_c);
          [&]<int... KS>(std::integer_sequence<int, KS...>) {
            (
                [&] {
                  typedef std::integral_constant<int, KS> CK;
                  mm(par_c, I0{}, CK{}); rnd(I2{}, I0{}); rnd(I2{}, I1{});
                  mm(par_c, I1{}, CK{}); rnd(I3{}, I0{}); rnd(I3{}, I1{});
                  mm(par_c, I2{}, CK{}); rnd(I0{}, I0{}); rnd(I0{}, I1{});
                  mm(par_c, I3{}, CK{}); rnd(I1{}, I0{}); rnd(I1{}, I1{});
                }(),
                ...);
          }(std::make_integer_sequence<int, NKS>{});
        };
        int kt = 0;
        for (; kt + 1 < nk; kt += 2) {
          chunk_stage(kt, I0{});
          chunk_stage(kt + 1, I1{});
        }
        if (kt < nk) chunk_stage(kt, I0{});
      }
      // the sum of the rounded chunks, plus the low bits of the initial accumulator (read again
      // here: holding it in registers through the loop would cost 64 of them)
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int jj = 0; jj < FN; ++jj)
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            unsigned low = 0;
            if (chk.c_in) {
              const int m = row_lo + wm * TM + i * 32 + (v >> 2) * 8 + (lane >> 5) * 4 + (v & 3);
              const int n = col_lo + wn * TN + jj * 32 + (lane & 31);
              if (m < row_hi && n < g.N) low = (unsigned)((const int*)chk.c_in)[(int64_t)m * chk.ldc + n] & ~chk.mask;
            }
            acc[i][jj][v] = (int)(((unsigned)work[i][jj][v] & chk.mask) + low);
          }
    } else {
      // Floating point: the rounding works on the bits of the chunk's own sum, which is then added
      // in fp32 -- three operations per element (integer add, and, float add).  Block b's MFMAs
      // start from C = 0; block b - 1 is folded into `acc` while they run.
      Acc zero;
#pragma unroll
      for (int v = 0; v < 16; ++v) zero[v] = 0;
      auto fold = [&](auto b_c) {
        constexpr int I = decltype(b_c)::value / FN, J = decltype(b_c)::value % FN;
#pragma unroll
        for (int v = 0; v < 16; ++v)
          acc[I][J][v] += __uint_as_float((__float_as_uint(work[I][J][v]) + chk.round_bit) & chk.mask);
      };
      auto chunk_stage = [&](int kt, auto par_c) {
        constexpr int PAR = decltype(par_c)::value;
        stage_top(kt, par_c);
        [&]<int... B>(std::integer_sequence<int, B...>) {
          (
              [&] {
                constexpr int I = B / FN, J = B % FN;
                work[I][J] = MM::mma(ca[PAR][0][I], cb[PAR][0][J], zero);
#pragma unroll
                for (int ks = 1; ks < NKS; ++ks)
                  work[I][J] = MM::mma(ca[PAR][ks][I], cb[PAR][ks][J], work[I][J]);
                __builtin_amdgcn_sched_barrier(0);
                // block B - 1 of this chunk, or the last block of the previous one (zeros before
                // the first chunk: a zero block folds to zero)
                fold(std::integral_constant<int, (B + NMMA - 1) % NMMA>{});
                __builtin_amdgcn_sched_barrier(0);
              }(),
              ...);
        }(std::make_integer_sequence<int, NMMA>{});
      };
      int kt = 0;
      for (; kt + 1 < nk; kt += 2) {
        chunk_stage(kt, std::integral_constant<int, 0>{});
        chunk_stage(kt + 1, std::integral_constant<int, 1>{});
      }
      if (kt < nk) chunk_stage(kt, std::integral_constant<int, 0>{});
      fold(std::integral_constant<int, NMMA - 1>{});
    }
  } else {
  read_frags(&lds[0][0], 0, fa[0], fb[0]);
  {
    int kt = 0;
    if constexpr (NKS % 2 == 0) {
      for (; kt < nk; ++kt) stage(kt, std::integral_constant<int, 0>{});
    } else {
      for (; kt + 1 < nk; kt += 2) {
        stage(kt, std::integral_constant<int, 0>{});
        stage(kt + 1, std::integral_constant<int, 1>{});
      }
      if (kt < nk) stage(kt, std::integral_constant<int, 0>{});
    }
  }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // no DMA may be in flight when LDS is released
  if constexpr (Chk::enabled && !Chk::one_stage) {
    if (ks_cnt != 0) finish_any();  // K ended inside a chunk
    if (!chk.tta) {
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) acc[i][j] = work[i][j];
    }
  }

  // ---- epilogue: acc[i][j][v] is C(row, col) with
  //      row = 32 i + 8 (v / 4) + 4 (lane / 32) + v % 4,   col = 32 j + lane % 32
  const int m_base = row_lo + wm * TM + fg * 4;
  const int n_base = col_lo + wn * TN + fr;
  typename Epi::Col colctx[FN];
#pragma unroll
  for (int j = 0; j < FN; ++j) colctx[j] = epi.col(min(n_base + j * 32, g.N - 1), expert, g.N);
  // Whole tiles take a branch-free path.  The row operands (token scales) of up to two row blocks
  // are requested before the blocks' first store: a load may not be moved across a store through an
  // unrelated pointer, so requested block by block their latency is paid once per block.  Tiles cut
  // by the last row test rows in the groups of 8 that the accumulator layout makes wave-uniform
  // (whole groups store without per-lane tests, groups past the end are skipped by a scalar
  // branch); per-lane tests around every store would put each store into a basic block of its own.
  const bool cols_full = col_lo + BN <= g.N;
  const bool interior = (row_lo + BM <= row_hi) && cols_full;
  const int rows_left = row_hi - row_lo - wm * TM;  // valid rows from this wave's first row on; uniform
  constexpr int RBB = FM % 2 == 0 ? 2 : 1;
#pragma unroll
  for (int i0 = 0; i0 < FM; i0 += RBB) {
    if (rows_left - i0 * 32 <= 0) break;
    typename Epi::Row rowctx[RBB][16];
#pragma unroll
    for (int i = 0; i < RBB; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v)
        rowctx[i][v] = epi.row(min(m_base + (i0 + i) * 32 + (v >> 2) * 8 + (v & 3), row_hi - 1));
    if (interior) {
#pragma unroll
      for (int i = 0; i < RBB; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int m = m_base + (i0 + i) * 32 + (v >> 2) * 8 + (v & 3);
#pragma unroll
          for (int j = 0; j < FN; ++j) epi.store(m, n_base + j * 32, acc[i0 + i][j][v], rowctx[i][v], colctx[j]);
        }
    } else {
#pragma unroll
      for (int i = 0; i < RBB; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int left = rows_left - (i0 + i) * 32 - q * 8;
          if (left >= 8 && cols_full) {
#pragma unroll
            for (int vv = 0; vv < 4; ++vv) {
              const int v = q * 4 + vv, m = m_base + (i0 + i) * 32 + q * 8 + vv;
#pragma unroll
              for (int j = 0; j < FN; ++j) epi.store(m, n_base + j * 32, acc[i0 + i][j][v], rowctx[i][v], colctx[j]);
            }
          } else if (left > 0) {
#pragma unroll
            for (int vv = 0; vv < 4; ++vv) {
              const int v = q * 4 + vv, m = m_base + (i0 + i) * 32 + q * 8 + vv;
              if (m < row_hi) {
#pragma unroll
                for (int j = 0; j < FN; ++j) {
                  const int n = n_base + j * 32;
                  if (n < g.N) epi.store(m, n, acc[i0 + i][j][v], rowctx[i][v], colctx[j]);
                }
              }
            }
          }
        }
    }
  }
#endif  // __HIP_DEVICE_COMPILE__
}

// ------------------------------------------------------------------------------ epilogues
struct EpiStoreI32 {
  int32_t* c;
  int64_t ldc;
  struct Col {};
  struct Row {};
  __device__ __forceinline__ Col col(int, int, int) const { return Col{}; }
  __device__ __forceinline__ Row row(int) const { return Row{}; }
  __device__ __forceinline__ void store(int m, int n, int v, Row, Col) const {
    c[(int64_t)m * ldc + n] = v;
  }
};

struct EpiStoreF32 {
  float* c;
  int64_t ldc;
  struct Col {};
  struct Row {};
  __device__ __forceinline__ Col col(int, int, int) const { return Col{}; }
  __device__ __forceinline__ Row row(int) const { return Row{}; }
  __device__ __forceinline__ void store(int m, int n, float v, Row, Col) const {
    c[(int64_t)m * ldc + n] = v;
  }
};

// y = acc * (a_scale[m] x w_scale[n]) + bias[n], see FMSMO_EPI_* in fmsmo_hip.h.
// MULADD_SWITCH: whether the fp32-scale form looks at `muladd` at all.  The e4m3 GEMMs never ask
// for the separate multiply and add; without the test their 256 stores per lane are one straight
// run (the block-uniform test per element cost them 0.5 ... 1.5 % of the whole launch).  Their
// fp32-output instances keep the switch: without it the register allocation of the 256 x 256
// tile came out four registers short.
template <int OUT, int BIAS, bool REF_F16, class AccT, bool MULADD_SWITCH = true>
struct EpiDequant {
  static constexpr bool UNIFORM_ROWS = false;
  void* y;
  int64_t ldy;
  const float* a_scale;
  const float* w_scale;
  const void* bias;
  int a_stride, w_stride;  // 0 = one value for all rows / columns, 1 = per row / column
  int muladd = 0;          // fp32-scale form only: separate multiply and add instead of one fma
  struct Col {
    float ws, b;
  };
  struct Row {
    float as;
  };
  __device__ __forceinline__ Col col(int n, int expert, int N) const {
    Col c;
    const int64_t o = (int64_t)expert * N + n;
    c.ws = w_scale[w_stride ? o : 0];
    c.b = bias ? load_as_f32<BIAS>(bias, o) : -0.0f;  // no bias: x + (-0) == x, the sign of a zero product included
    return c;
  }
  __device__ __forceinline__ Row row(int m) const { return Row{a_scale[a_stride ? m : 0]}; }
  __device__ __forceinline__ void store(int m, int n, AccT v, Row r, Col c) const {
    const int64_t idx = (int64_t)m * ldy + n;
    if constexpr (REF_F16) {
      // separate fp32 multiply and add (no fma), scale product rounded to fp16 first; a 16-bit
      // output is the fp16 accumulator dtype of from_fms_mo cast to the output dtype, an fp32
      // output is the fp32 accumulator dtype of from_torch_iW (no fp16 rounding of the result)
      const float sc = round_to<FMSMO_F16>(__fmul_rn(r.as, c.ws));
      const float t = __fadd_rn(__fmul_rn((float)v, sc), c.b);
      if constexpr (OUT == FMSMO_F32) ((float*)y)[idx] = t;
      else if constexpr (OUT == FMSMO_F16) __builtin_nontemporal_store(f32_to_f16(t), &((u16*)y)[idx]);
      else store_from_f32<OUT>(y, idx, f16_to_f32(f32_to_f16(t)));
    } else {
      const float sc = __fmul_rn(r.as, c.ws);
      const float t = (MULADD_SWITCH && muladd) ? __fadd_rn(__fmul_rn((float)v, sc), c.b) : __fmaf_rn((float)v, sc, c.b);
      store_from_f32<OUT>(y, idx, t);
    }
  }
};

// y = acc * (a_scale[0] * w_scale[0]) + bias[n]: the batched matmuls' epilogue, one scale for the
// whole batch (EpiDequant's fp32-scale arithmetic with nothing to fetch per row).
template <int OUT, class AccT>
struct EpiScaleBias {
  static constexpr bool UNIFORM_ROWS = true;
  static constexpr int OUT_DT = OUT;
  void* y;
  int64_t ldy;
  const float* a_scale;
  const float* w_scale;
  const float* bias;
  struct Col {
    float b;
  };
  struct Row {
    float sc;
  };
  __device__ __forceinline__ Col col(int n, int expert, int N) const {
    return Col{bias ? bias[(int64_t)expert * N + n] : -0.0f};
  }
  __device__ __forceinline__ Row row(int) const { return Row{__fmul_rn(a_scale[0], w_scale[0])}; }
  __device__ __forceinline__ float value(AccT v, Row r, Col c) const { return __fmaf_rn((float)v, r.sc, c.b); }
  __device__ __forceinline__ void store(int m, int n, AccT v, Row r, Col c) const {
    store_from_f32<OUT>(y, (int64_t)m * ldy + n, value(v, r, c));
  }
};

}  // namespace fmsmo
