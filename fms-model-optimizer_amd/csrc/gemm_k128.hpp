// Batched C = A . B^T with a reduction of exactly 128 bytes (attention scores: Q . K^T with a head
// dimension of 128), 1-byte operands, 128 x 256 tiles.
//
// Such a tile reads 48 KiB, multiplies for half a microsecond and writes 64 KiB (16-bit output):
// the work is the epilogue and the launch is bound by how well loads, conversion arithmetic and
// stores of neighbouring tiles overlap, not by the matrix units.  One tile per block leaves a
// memory latency, a barrier and a block launch in front of every epilogue with nothing to hide
// them behind (two blocks share a compute unit).  Here a block walks the tiles  blockIdx.x,
// blockIdx.x + gridDim.x, ...:  the operands of its next tile are requested (into registers) before
// the current tile is converted and written (after its MFMAs, when the fragment registers are
// free: two blocks per compute unit leave 256 registers per lane), so the next tile's memory
// latency runs under the current tile's epilogue; the row / column operands of the epilogue are
// fetched before those requests (loads return in order: fetched after them, the epilogue would
// wait for the whole next tile first).
//
// LDS layout, operand fragments and accumulator layout are those of gemm_rs.hpp (rows of 128
// bytes, 16-byte chunk c of row r at position c ^ swz(r); 32 x 32 MFMA blocks).
#pragma once
#include "gemm_tile.hpp"

namespace fmsmo {

template <int OP, class Epi>
__global__ __launch_bounds__(256, 2) void gemm_k128_kernel(GemmArgs g, Epi epi) {
#if defined(__HIP_DEVICE_COMPILE__)
  typedef Mma<OP> MM;
  typedef typename MM::Frag Frag;
  typedef typename MM::Acc Acc;
  constexpr int BM = 128, BN = 256, BK = 128, CPR = 8;
  constexpr int TM = BM / 2, TN = BN / 2, FM = TM / 32, FN = TN / 32;
  constexpr int NKS = BK / MM::KSTEP;  // MFMA k-steps (int8 4, e4m3 2)
  constexpr int CL = MM::KSTEP / 32;   // 16-byte chunks per lane per k-step
  constexpr int NJ = BM / 32, NJB = BN / 32;
  __shared__ __attribute__((aligned(16))) uint8_t lds[(BM + BN) * BK];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int nt = (g.rows_per_group + BM - 1) / BM;  // row tiles per batch entry
  const int total = g.num_experts * nt * g.grid_n;

  struct Where {
    int row_lo, row_hi, col_lo, expert;
  };
  auto locate = [&](int tile) {
    int tile_m, tile_n;
    tile_of_block(tile, total, g.num_experts * nt, g.grid_n, g.group_m, tile_m, tile_n);
    Where w;
    w.expert = tile_m / nt;
    w.row_lo = w.expert * g.rows_per_group + (tile_m - w.expert * nt) * BM;
    w.row_hi = (w.expert + 1) * g.rows_per_group;
    w.col_lo = tile_n * BN;
    return w;
  };

  // ---- global -> registers: thread -> (row = tid / 8 + 32 j, 16-byte chunk = tid % 8); rows past
  // the batch entry's last row / past N read as zero through the descriptors' range check
  const int ld_row = tid >> 3, ld_chunk = tid & 7;
  v4i sta[NJ], stb[NJB];
  auto request = [&](const Where& w) {
    const int64_t a_adj = (int64_t)w.expert * (g.lda_e - (int64_t)g.rows_per_group * g.lda);
    const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(g.a + a_adj), 0, (int)((int64_t)(w.row_hi - 1) * g.lda + g.K), 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(g.b + (int64_t)w.expert * g.ldb_e), 0, (int)((int64_t)(g.N - 1) * g.ldb + g.K), 0x00020000);
    const int va = (w.row_lo + ld_row) * (int)g.lda + ld_chunk * 16;
    const int vb = (w.col_lo + ld_row) * (int)g.ldb + ld_chunk * 16;
#pragma unroll
    for (int j = 0; j < NJB; ++j) {
      if (j < NJ)
        sta[j] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrc_a, va, j * 32 * (int)g.lda, 0));
      stb[j] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrc_b, vb, j * 32 * (int)g.ldb, 0));
    }
  };
  const int wr = ld_row * BK + ((ld_chunk ^ swz<CPR, 1>(ld_row)) * 16);

  // ---- LDS -> MFMA operand addressing
  const int fr = lane & 31, fg = lane >> 5;
  const int fsw = swz<CPR, 1>(fr);
  int a_rd[NKS][CL], b_rd[NKS][CL];
#pragma unroll
  for (int s = 0; s < NKS; ++s)
#pragma unroll
    for (int e = 0; e < CL; ++e) {
      const int c = s * 2 * CL + fg * CL + e;
      a_rd[s][e] = (wm * TM + fr) * BK + ((c ^ fsw) * 16);
      b_rd[s][e] = BM * BK + (wn * TN + fr) * BK + ((c ^ fsw) * 16);
    }
  auto frag = [&](const int (&rd)[NKS][CL], int s, int blk) -> Frag {
    if constexpr (CL == 1) {
      return *(const v4i*)(lds + rd[s][0] + blk * 32 * BK);
    } else {
      const v4i lo = *(const v4i*)(lds + rd[s][0] + blk * 32 * BK);
      const v4i hi = *(const v4i*)(lds + rd[s][1] + blk * 32 * BK);
      return Frag{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    }
  };

  int tile = blockIdx.x;
  if (tile >= total) return;
  Where cur = locate(tile);
  request(cur);
  while (true) {
    // the tile's operands into LDS (waits for its requests)
#pragma unroll
    for (int j = 0; j < NJB; ++j) {
      if (j < NJ) *(v4i*)(lds + wr + j * 32 * BK) = sta[j];
      *(v4i*)(lds + BM * BK + wr + j * 32 * BK) = stb[j];
    }
    __syncthreads();

    // epilogue operands of this tile are fetched before the next tile's requests (see above)
    const int m_base = cur.row_lo + wm * TM + fg * 4;
    const int n_base = cur.col_lo + wn * TN + fr;
    typename Epi::Col colctx[FN];
#pragma unroll
    for (int j = 0; j < FN; ++j) colctx[j] = epi.col(min(n_base + j * 32, g.N - 1), cur.expert, g.N);
    constexpr int NROW = Epi::UNIFORM_ROWS ? 1 : FM * 16;  // one scale for all rows: nothing per row
    typename Epi::Row rowctx[NROW];
#pragma unroll
    for (int i = 0; i < NROW; ++i)
      rowctx[i] = epi.row(min(m_base + (i >> 4) * 32 + ((i & 15) >> 2) * 8 + (i & 3), cur.row_hi - 1));
    __builtin_amdgcn_sched_barrier(0);

    // multiply (one set of fragment registers: the matrix work is a small part of a tile)
    Acc acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int j = 0; j < FN; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][j][v] = 0;
#pragma unroll
    for (int s = 0; s < NKS; ++s) {
      Frag fa[FM], fb[FN];
#pragma unroll
      for (int i = 0; i < FM; ++i) fa[i] = frag(a_rd, s, i);
#pragma unroll
      for (int j = 0; j < FN; ++j) fb[j] = frag(b_rd, s, j);
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) acc[i][j] = MM::mma(fa[i], fb[j], acc[i][j]);
      __builtin_amdgcn_sched_barrier(0);
    }

    // the next tile's operands are requested now that the fragment registers are free; they
    // arrive while this tile is converted and stored
    const int next = tile + (int)gridDim.x;
    const bool has_next = next < total;
    Where nxt = cur;
    if (has_next) {
      __syncthreads();  // every wave has read its fragments: the slab may be overwritten
      nxt = locate(next);
      request(nxt);
    }
    __builtin_amdgcn_sched_barrier(0);

    // ---- epilogue: acc[i][j][v] is C(row, col) with
    //      row = 32 i + 8 (v / 4) + 4 (lane / 32) + v % 4,   col = 32 j + lane % 32
    // (a wave store instruction covers two 64-byte runs of two output rows; writing 8 or 16 bytes
    // per lane -- accumulators transposed by swapping the MFMA operands, with or without a pass
    // through LDS to make whole 256-byte runs -- measured slower: 0.27 -> 0.49 / 0.35 ms on 32
    // heads of 4096 x 4096 scores)
    const bool interior = (cur.row_lo + BM <= cur.row_hi) && (cur.col_lo + BN <= g.N);
#pragma unroll
    for (int i = 0; i < FM; ++i) {
      if (interior) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int m = m_base + i * 32 + (v >> 2) * 8 + (v & 3);
#pragma unroll
          for (int j = 0; j < FN; ++j)
            epi.store(m, n_base + j * 32, acc[i][j][v], rowctx[Epi::UNIFORM_ROWS ? 0 : i * 16 + v], colctx[j]);
        }
      } else {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int m = m_base + i * 32 + (v >> 2) * 8 + (v & 3);
          if (m < cur.row_hi) {
#pragma unroll
            for (int j = 0; j < FN; ++j) {
              const int n = n_base + j * 32;
              if (n < g.N) epi.store(m, n, acc[i][j][v], rowctx[Epi::UNIFORM_ROWS ? 0 : i * 16 + v], colctx[j]);
            }
          }
        }
      }
    }
    if (!has_next) break;
    tile = next;
    cur = nxt;
  }
#endif  // __HIP_DEVICE_COMPILE__
}

}  // namespace fmsmo
