// Register-staged MFMA GEMM for gfx950: C[M,N] = A[M,K] . B[N,K]^T, 1-byte operands, 256x256 tile.
//
// Why a second pipeline: with 64-byte K stages (gemm_tile.hpp) every 128-byte L2 line is requested
// twice, one stage apart, and the 64 KiB of lines a stage touches do not survive in the vector L1;
// the L2 -> L1 traffic is therefore twice the operand bytes and, with all 256 CUs active, that is
// what bounds the loop.  Here K advances in slabs of 128 bytes (whole lines, fetched once).  A
// 256x256 slab is 64 KiB, so only two fit in LDS; the third pipeline level is the register file:
// the slab after next is fetched with plain buffer loads (8 rows x 128 B per wave instruction)
// into 64 VGPRs per lane and written to LDS (ds_write_b128, XOR-swizzled) as soon as the buffer it
// replaces has been read for the last time.
//
// Per slab: NKS MFMA k-steps with register double-buffered operand fragments.  At the start of
// the last k-step every wave holds its last fragments of the current buffer, so after one
// barrier the buffer is refilled (from the staging registers) and the staging registers are
// re-loaded (slab + 3), all interleaved with the MFMAs of that k-step.  One barrier per slab.
// Rows past M / N read as zero through the buffer descriptor's range check.
#pragma once
#include "gemm_tile.hpp"

namespace fmsmo {

// The 16 x 16 x 128 form of the e4m3 matrix instruction: a lane holds row lane % 16 and the K group
// lane / 16 (four groups of 32 bytes), so one instruction covers a whole 128-byte slab.  Under the
// part's power limit it does more work per joule than 32 x 32 x 64 (the same loop of matrix
// instructions alone on the same Gaussian codes: 4570 against 4000 TFLOP/s), and a GEMM of this
// size runs against that limit, not against issue slots.  (int8 has 16 x 16 x 64, 3630 against
// 3430 TOPS in that loop; in this kernel its four times as many instructions per slab lost
// 3 ... 25 %, so int8 keeps the 32 x 32 x 32 form and there is no int8 specialization.)
template <int OP>
struct Mma16;
template <>
struct Mma16<MMA_FP8> {
  typedef v8i Frag;
  typedef v4f Acc;
  typedef float Elem;
  static constexpr int KSTEP = 128;
  __device__ static __forceinline__ Acc mma(const Frag& a, const Frag& b, const Acc& c) {
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0);
  }
};

// (A reduction of a single slab, K == 128, has its own kernel: gemm_k128.hpp.)
template <int OP, class Epi, bool GROUPED = false, int BN_ = 256, bool B16 = false>
__global__ __launch_bounds__(256, 1) void gemm_rs_kernel(GemmArgs g, Epi epi) {
#if defined(__HIP_DEVICE_COMPILE__)
  typedef typename std::conditional<B16, Mma16<OP>, Mma<OP>>::type MM;
  typedef typename MM::Frag Frag;
  typedef typename MM::Acc Acc;
  static_assert(BN_ == 256 || BN_ == 192 || BN_ == 128, "tile width");
  constexpr int BM = 256, BN = BN_, BK = 128, CPR = 8;
  constexpr bool LOOPS = GROUPED;  // the block may walk several tiles
  constexpr int RB = B16 ? 16 : 32;     // rows of a matrix-instruction block
  constexpr int KG = 64 / RB;           // K groups of lanes
  constexpr int NACC = RB * RB / 64;    // accumulator registers per block
  constexpr int TM = BM / 2, TN = BN / 2, FM = TM / RB, FN = TN / RB;
  constexpr int NKS = BK / MM::KSTEP;   // MFMA k-steps per slab (32 x 32: int8 4, e4m3 2; 16 x 16: 2, 1)
  constexpr int CL = MM::KSTEP / KG / 16;  // 16-byte chunks per lane per k-step
  // LDS: [A of buffer 0][A of buffer 1][B of buffer 0][B of buffer 1], 32 KiB apart.  Both buffers
  // of an operand lie within the 64 KiB that the 16-bit offset field of an LDS instruction spans,
  // so one address register per operand fragment serves both (buffers 64 KiB apart needed a second
  // set of address registers, which the persistent blocks' tile loop had no room for).
  constexpr int SLAB = BM * BK;      // buffer 1 of an operand follows buffer 0
  constexpr int BOFF = 2 * BM * BK;  // operand B follows both buffers of A
  constexpr int NJ = BM / 32, NJB = BN / 32;  // row groups of 32 per thread: A, B
  static_assert(NKS == 1 || NKS % 2 == 0, "fragment buffers alternate per k-step");
  __shared__ __attribute__((aligned(16))) uint8_t lds[BOFF + BM * BK + BN * BK];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  int tile_m, tile_n;
  int row_lo, row_hi = g.M, expert = 0;
  int64_t a_adj = 0;
  // Mixture-of-experts mode: the blocks are persistent.  The host launches one block per compute
  // unit (it does not know the row counts); the real tiles -- counted here from `offsets` -- are
  // dealt to the 8 XCDs in contiguous spans of the tile sequence, and the blocks of an XCD take
  // their span's tiles in turn (block slot, slot + slots, ...), so that the tiles resident on an
  // XCD at one time are neighbours in the sequence and share A and B panels in its L2.  One tile
  // per block left the order of the tiles to the dispatcher, which hands out work-groups in
  // order, round-robin over the XCDs: with tiles of uneven cost (row tiles cut by an expert's
  // end store less) compute units waited 5 us per tile for their turn.
  [[maybe_unused]] int real_m = 0, p_next = 0, p_end = 0, p_step = 1;  // this block's positions in the tile sequence
  if constexpr (GROUPED) {
    if (g.rows_per_group > 0) {
      // batched matmul: every group has the same number of rows, the grid is exact
      const int nt = (g.rows_per_group + BM - 1) / BM;
      tile_of_block(blockIdx.x, gridDim.x, g.num_experts * nt, g.grid_n, g.group_m, tile_m, tile_n);
      expert = tile_m / nt;
      row_lo = expert * g.rows_per_group + (tile_m - expert * nt) * BM;
      row_hi = (expert + 1) * g.rows_per_group;
      // rows are numbered as stacked groups (the layout of the output); A may be laid out
      // differently: shift its base so that stacked row numbers address the group's rows
      a_adj = (int64_t)expert * (g.lda_e - (int64_t)g.rows_per_group * g.lda);
    } else {
      for (int e = 0; e < g.num_experts; ++e) real_m += (g.offsets[e + 1] - g.offsets[e] + BM - 1) / BM;
      const int real_tiles = real_m * g.grid_n;
      const int nx = min(8, (int)gridDim.x);
      const int xcd = blockIdx.x % nx;
      p_step = ((int)gridDim.x - xcd + nx - 1) / nx;  // blocks on this XCD
      const int per = real_tiles / nx, rem = real_tiles % nx;
      const int lo = xcd < rem ? xcd * (per + 1) : rem * (per + 1) + (xcd - rem) * per;
      p_end = lo + per + (xcd < rem ? 1 : 0);
      p_next = lo + blockIdx.x / nx;
      if (p_next >= p_end) return;  // uniform for the whole block
    }
  } else {
    tile_of_block(blockIdx.x, gridDim.x, g.grid_m, g.grid_n, g.group_m, tile_m, tile_n);
    row_lo = tile_m * BM;
  }

  // ---- global -> register staging: thread -> (row = tid / 8 + 32 j, 16-byte chunk = tid % 8)
  const int ld_row = tid >> 3, ld_chunk = tid & 7;
  // (mixture-of-experts mode re-makes it per tile so that it ends with the expert's last row: the
  // rows of a cut tile past that row then load as zeros instead of the next expert's tokens, and
  // matrix instructions on zeros draw far less power than on live codes)
  __amdgpu_buffer_rsrc_t rsrc_a;
  // per tile (a persistent block re-assigns them): B descriptor of the tile's expert, first
  // column, byte offsets of the thread's first A and B rows
  __amdgpu_buffer_rsrc_t rsrc_b;
  int col_lo, va, vb;
  const int sa32 = 32 * (int)g.lda, sb32 = 32 * (int)g.ldb;
  const int nslab = g.K / BK;
  // slabs past the end: never used.  With k_rotate the block walks the slabs from its own
  // starting point (all blocks sweeping K in step would ask for the same address bits 7.. of
  // rows a power of two apart at the same time).
  const int s0 = g.k_rotate ? (int)((blockIdx.x * (unsigned)g.k_rotate) % (unsigned)nslab) : 0;
  auto slab_k0 = [&](int s) {
    int t = min(s, nslab - 1) + s0;
    if (t >= nslab) t -= nslab;
    return t * BK;
  };
  // Staging sets.  Two of them where the registers allow it (int8 with 32 x 32 blocks: 16-byte
  // fragments): set t % 2 carries slab t, so a slab's loads are in flight for two slab times before
  // they are needed instead of one -- the loop otherwise waits on them (the operand lines that miss
  // the L2 come from the memory side and take longer than a slab lasts when the fabric is busy).
  constexpr int NSET = (OP == MMA_I8 && !B16) ? 2 : 1;
  v4i sta[NSET][NJ], stb[NSET][NJB];
  // The loads keep their program order (a scheduling barrier that only memory instructions may
  // not cross follows each one): the compiler's vmcnt bookkeeping is exact only if the order in
  // the prologue and in the loop is the same.
  constexpr int NOT_VMEM = 0x7ff & ~(0x010 | 0x020 | 0x040);
  auto load_a = [&](int j, int k0) {
    sta[0][j] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrc_a, va, j * sa32 + k0, 0));
    __builtin_amdgcn_sched_barrier(NOT_VMEM);
  };
  auto load_b = [&](int j, int k0) {
    stb[0][j] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrc_b, vb, j * sb32 + k0, 0));
    __builtin_amdgcn_sched_barrier(NOT_VMEM);
  };
  auto load_slab = [&](int s) {
    const int k0 = slab_k0(s);
#pragma unroll
    for (int j = 0; j < (NJ > NJB ? NJ : NJB); ++j) {
      if (j < NJ) load_a(j, k0);
      if (j < NJB) load_b(j, k0);
    }
  };
  // LDS position of the thread's chunk: row-major [row][128 B], chunk c of row r at c ^ swz(r);
  // swz depends on r % 16 only, so it is the same for all 8 row groups
  const int wr = ld_row * BK + ((ld_chunk ^ swz<CPR, 1>(ld_row)) * 16);
  auto store_slab = [&](uint8_t* buf, int wr_t) {
#pragma unroll
    for (int j = 0; j < (NJ > NJB ? NJ : NJB); ++j) {
      if (j < NJ) *(v4i*)(buf + wr_t + j * 32 * BK) = sta[0][j];
      if (j < NJB) *(v4i*)(buf + BOFF + wr_t + j * 32 * BK) = stb[0][j];
    }
  };

  // ---- LDS -> MFMA operand addressing
  const int fr = lane % RB, fg = lane / RB;
  const int fsw = swz<CPR, 1>(fr);
  int a_rd[NKS][CL], b_rd[NKS][CL];
#pragma unroll
  for (int s = 0; s < NKS; ++s)
#pragma unroll
    for (int e = 0; e < CL; ++e) {
      const int c = (s * KG + fg) * CL + e;
      a_rd[s][e] = (wm * TM + fr) * BK + ((c ^ fsw) * 16);
      b_rd[s][e] = BOFF + (wn * TN + fr) * BK + ((c ^ fsw) * 16);
    }
  // operand fragments are kept as their 16-byte halves so that single reads can be placed
  // between MFMAs; index r enumerates the reads of one k-step: A (i, e) first, then B (j, e)
  // (a slab of one k-step keeps a single set: a fragment is re-read right after its last use)
  constexpr int NFB = NKS == 1 ? 1 : 2;
  v4i ha[NFB][FM][CL], hb[NFB][FN][CL];
  constexpr int NRD = (FM + FN) * CL, NMMA = FM * FN;
  auto read_one = [&](const uint8_t* ls, int s, int buf, auto r_c) {
    constexpr int R = decltype(r_c)::value;
    if constexpr (R < FM * CL) {
      ha[buf][R / CL][R % CL] = *(const v4i*)(ls + a_rd[s][R % CL] + (R / CL) * RB * BK);
    } else {
      constexpr int Q = R - FM * CL;
      hb[buf][Q / CL][Q % CL] = *(const v4i*)(ls + b_rd[s][Q % CL] + (Q / CL) * RB * BK);
    }
  };
  auto read_all = [&](const uint8_t* ls, int s, int buf) {
    [&]<int... R>(std::integer_sequence<int, R...>) {
      (read_one(ls, s, buf, std::integral_constant<int, R>{}), ...);
    }(std::make_integer_sequence<int, NRD>{});
  };
  auto frag_a = [&](int buf, int i) -> Frag {
    if constexpr (CL == 1) return ha[buf][i][0];
    else return Frag{ha[buf][i][0][0], ha[buf][i][0][1], ha[buf][i][0][2], ha[buf][i][0][3],
                     ha[buf][i][1][0], ha[buf][i][1][1], ha[buf][i][1][2], ha[buf][i][1][3]};
  };
  auto frag_b = [&](int buf, int j) -> Frag {
    if constexpr (CL == 1) return hb[buf][j][0];
    else return Frag{hb[buf][j][0][0], hb[buf][j][0][1], hb[buf][j][0][2], hb[buf][j][0][3],
                     hb[buf][j][1][0], hb[buf][j][1][1], hb[buf][j][1][2], hb[buf][j][1][3]};
  };

  Acc acc[FM][FN];
  auto mma_step = [&](int buf) {
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int j = 0; j < FN; ++j) acc[i][j] = MM::mma(frag_a(buf, i), frag_b(buf, j), acc[i][j]);
  };

  // One k-step in explicit order.  Behind MFMA r (a full scheduling barrier closes every group):
  // read r of the fragments for the following k-step (from `rd_ls`, k-step `RS`, into buffer RB)
  // and the staging pairs [P0, P1) spread evenly over the FM x FN MFMAs.  A pair = write one staged
  // 16-byte chunk into `wr_buf`, then re-load its registers from slab `k0`.  Pair p < NJ is
  // operand A row group p, pair p >= NJ operand B row group p - NJ.
  auto pair = [&](uint8_t* wr_buf, int k0, auto p_c, auto set_c) {
    constexpr int P = decltype(p_c)::value, ST = decltype(set_c)::value;
    if constexpr (P < NJ) {
      *(v4i*)(wr_buf + wr + P * 32 * BK) = sta[ST][P];
      sta[ST][P] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrc_a, va, P * sa32 + k0, 0));
    } else {
      *(v4i*)(wr_buf + BOFF + wr + (P - NJ) * 32 * BK) = stb[ST][P - NJ];
      stb[ST][P - NJ] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrc_b, vb, (P - NJ) * sb32 + k0, 0));
    }
  };
  auto kstep = [&](auto mb_c, const uint8_t* rd_ls, auto rs_c, auto rb_c, uint8_t* wr_buf, int k0,
                   auto p0_c, auto p1_c, auto set_c) {
    constexpr int MB = decltype(mb_c)::value, RS = decltype(rs_c)::value, RB = decltype(rb_c)::value;
    constexpr int P0 = decltype(p0_c)::value, P1 = decltype(p1_c)::value, NP = P1 - P0;
    [&]<int... R>(std::integer_sequence<int, R...>) {
      (
          [&] {
            constexpr int I = R / FN, J = R % FN;
            acc[I][J] = MM::mma(frag_a(MB, I), frag_b(MB, J), acc[I][J]);
            // two fragment reads behind each of the first MFMAs: the last one must be back
            // well before the k-step ends (its consumers are the first MFMAs of the next one)
            if constexpr (2 * R < NRD) read_one(rd_ls, RS, RB, std::integral_constant<int, 2 * R>{});
            if constexpr (2 * R + 1 < NRD) read_one(rd_ls, RS, RB, std::integral_constant<int, 2 * R + 1>{});
            if constexpr (NP > 0) {
              constexpr int PA = P0 + R * NP / NMMA, PB = P0 + (R + 1) * NP / NMMA;
              if constexpr (PB > PA) pair(wr_buf, k0, std::integral_constant<int, PA>{}, set_c);
              if constexpr (PB > PA + 1) pair(wr_buf, k0, std::integral_constant<int, PA + 1>{}, set_c);
            }
            __builtin_amdgcn_sched_barrier(0);
          }(),
          ...);
    }(std::make_integer_sequence<int, NMMA>{});
  };
  // Staging pairs [0, NP0) are handled in the last k-step of a slab, [NP0, NPAIR) in the first
  // k-step of the next one (int8 MFMAs are half as long as e4m3 ones: 16 of them cannot hide 16
  // buffer loads and 16 LDS writes).
  constexpr int NPAIR = NJ + NJB;
  constexpr int NP0 = OP == MMA_I8 ? NPAIR / 2 : NPAIR;
  auto pairs_now = [&](uint8_t* wr_buf, int k0, auto p0_c, auto p1_c) {  // no MFMAs to hide behind
    [&]<int... P>(std::integer_sequence<int, P...>) {
      (pair(wr_buf, k0, std::integral_constant<int, decltype(p0_c)::value + P>{}, std::integral_constant<int, 0>{}), ...);
    }(std::make_integer_sequence<int, decltype(p1_c)::value - decltype(p0_c)::value>{});
  };
  typedef std::integral_constant<int, 0> C0;
  typedef std::integral_constant<int, 1> C1;
  typedef std::integral_constant<int, NP0> CNP0;
  typedef std::integral_constant<int, NPAIR> CNP;

  for (;;) {  // one pass per tile: a single one except for the persistent blocks
  if constexpr (GROUPED) {
    if (g.rows_per_group == 0) {
      tile_of_pid(p_next, real_m, g.grid_n, g.group_m, tile_m, tile_n);
      int t = tile_m;
      row_lo = 0;
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
  }
  col_lo = tile_n * BN;
  rsrc_a = __builtin_amdgcn_make_buffer_rsrc((void*)(g.a + a_adj), 0, (int)((int64_t)(row_hi - 1) * g.lda + g.K), 0x00020000);
  rsrc_b = __builtin_amdgcn_make_buffer_rsrc((void*)(g.b + (GROUPED ? (int64_t)expert * g.ldb_e : 0)), 0,
                                             (int)((int64_t)(g.N - 1) * g.ldb + g.K), 0x00020000);
  {
    // (persistent blocks: derived from an opaque copy of the thread id, or the compiler hoists
    // these products out of the tile loop and holds them in registers the K loop has no room for)
    int t_id = tid;
    if constexpr (LOOPS) asm volatile("" : "+v"(t_id));
    va = (row_lo + (t_id >> 3)) * (int)g.lda + (t_id & 7) * 16;
    vb = (col_lo + (t_id >> 3)) * (int)g.ldb + (t_id & 7) * 16;
  }
  if (blockIdx.x == 0 && tid == 0 && g.clk) { g.clk[0] = clock64(); g.clk[1] = wall_clock64(); }
#pragma unroll
  for (int i = 0; i < FM; ++i)
#pragma unroll
    for (int j = 0; j < FN; ++j)
#pragma unroll
      for (int v = 0; v < NACC; ++v) acc[i][j][v] = 0;

  // ---- prologue: slab 0 into LDS; slab 1: pairs [0, NP0) into LDS and their registers re-loaded
  // with slab 2, pairs [NP0, NPAIR) still staged (the first k-step of the loop writes them)
  // (slabs 0 and 1 are fetched together: the accumulators and fragments are not live yet, so
  // there are registers for a second staging set)
  {
    load_slab(0);
    v4i ta[NJ], tb[NJB];
    const int k1 = slab_k0(1);
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      ta[j] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrc_a, va, j * sa32 + k1, 0));
      if (j < NJB)
        tb[j] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrc_b, vb, j * sb32 + k1, 0));
    }
    int wr_t = wr;  // (persistent blocks: opaque, so that the addresses below are formed here)
    if constexpr (LOOPS) asm volatile("" : "+v"(wr_t));
    store_slab(lds, wr_t);
    // slab 1: pairs [0, NP0) go to LDS, the rest stay staged
    [&]<int... P>(std::integer_sequence<int, P...>) {
      (
          [&] {
            if constexpr (P < NP0) {
              if constexpr (P < NJ) *(v4i*)(lds + SLAB + wr_t + P * 32 * BK) = ta[P];
              else *(v4i*)(lds + SLAB + BOFF + wr_t + (P - NJ) * 32 * BK) = tb[P - NJ];
            } else {
              // (slab 1 belongs to set 1 where there are two)
              if constexpr (P < NJ) sta[NSET - 1][P] = ta[P];
              else stb[NSET - 1][P - NJ] = tb[P - NJ];
            }
          }(),
          ...);
    }(std::make_integer_sequence<int, NPAIR>{});
    const int k2 = slab_k0(2), k3p = slab_k0(3);
    // one set: its pairs [0, NP0) take slab 2.  Two sets: set 0 takes all of slab 2, the pairs
    // [0, NP0) of set 1 take slab 3
    [&]<int... P>(std::integer_sequence<int, P...>) {
      (
          [&] {
            if constexpr (P < NJ) sta[0][P] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrc_a, va, P * sa32 + k2, 0));
            else stb[0][P - NJ] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrc_b, vb, (P - NJ) * sb32 + k2, 0));
            __builtin_amdgcn_sched_barrier(NOT_VMEM);
          }(),
          ...);
    }(std::make_integer_sequence<int, NSET == 2 ? NPAIR : NP0>{});
    if constexpr (NSET == 2) {
      [&]<int... P>(std::integer_sequence<int, P...>) {
        (
            [&] {
              if constexpr (P < NJ) sta[1][P] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrc_a, va, P * sa32 + k3p, 0));
              else stb[1][P - NJ] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrc_b, vb, (P - NJ) * sb32 + k3p, 0));
              __builtin_amdgcn_sched_barrier(NOT_VMEM);
            }(),
            ...);
      }(std::make_integer_sequence<int, NP0>{});
    }
  }
  __syncthreads();
  read_all(lds, 0, 0);

  if constexpr (NKS == 1) {
    // One k-step per slab (16 x 16 x 128): FM x FN matrix instructions on a single set of
    // fragments, re-read one by one as the instructions release them.  Entering slab s the
    // fragments of slab s are in registers except A[HM ..] (below), buffer (s + 1) % 2 holds slab
    // s + 1 and the staging registers hold slab s + 2.
    //   row 0 of the blocks, and behind its instructions the reads of A[HM ..] of slab s;
    //   barrier: every wave has all of slab s in registers and has written its part of slab s + 1;
    //   rows 1 .. HM - 1 row by row, A[i - 1] re-read (slab s + 1) once row i is under way;
    //   rows HM .. FM - 1 column by column, B[j] re-read once column j is done;
    //   spread over everything behind the barrier: the staged slab goes into buffer s % 2 and the
    //   staging registers are re-loaded with slab s + 3.
    // Every re-read is at least FN - 1 instructions ahead of its use.  (All rows in row order left
    // all FN fragments of B, and the last one of A, to be re-read behind the last row: 18 KiB per
    // wave in the time of 8 instructions, more than twice what the LDS delivers.)
    constexpr int HM = FM / 2, NCOL = FM - HM;
    constexpr int NQ = (FM - 1) * FN;     // instructions behind the barrier
    constexpr int NQP = NQ - NCOL;        // ... that carry staging pairs (not the last column)
    constexpr int NDR = NCOL * CL;        // reads of A[HM ..] behind row 0
    static_assert(FM >= 4 && FM % 2 == 0 && NPAIR <= NQP && CL <= NCOL, "schedule of a one-k-step slab");
    for (int s = 0; s < nslab; ++s) {
      uint8_t* cur = lds + (s & 1) * SLAB;
      const uint8_t* nxt = lds + ((s + 1) & 1) * SLAB;
      const int k3 = slab_k0(s + 3);
      [&]<int... J>(std::integer_sequence<int, J...>) {
        (
            [&] {
              acc[0][J] = MM::mma(frag_a(0, 0), frag_b(0, J), acc[0][J]);
              constexpr int R0 = J * NDR / FN, R1 = (J + 1) * NDR / FN;
              if constexpr (R1 > R0) read_one(cur, 0, 0, std::integral_constant<int, HM * CL + R0>{});
              if constexpr (R1 > R0 + 1) read_one(cur, 0, 0, std::integral_constant<int, HM * CL + R0 + 1>{});
              static_assert(R1 <= R0 + 2, "at most two reads behind an instruction of row 0");
              __builtin_amdgcn_sched_barrier(0);
            }(),
            ...);
      }(std::make_integer_sequence<int, FN>{});
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
      __builtin_amdgcn_sched_barrier(0);
      [&]<int... Q>(std::integer_sequence<int, Q...>) {
        (
            [&] {
              constexpr bool BYROW = Q < (HM - 1) * FN;
              constexpr int Q2 = Q - (HM - 1) * FN;
              constexpr int I = BYROW ? 1 + Q / FN : HM + Q2 % NCOL;
              constexpr int J = BYROW ? Q % FN : Q2 / NCOL;
              acc[I][J] = MM::mma(frag_a(0, I), frag_b(0, J), acc[I][J]);
              if constexpr (BYROW) {
                // fragment A[I - 1]: its CL reads behind the first CL instructions of row I
                if constexpr (J < CL) read_one(nxt, 0, 0, std::integral_constant<int, (I - 1) * CL + J>{});
              } else {
                // A[HM - 1] behind the first instructions of the columns, B[J] behind column J
                if constexpr (Q2 < CL) read_one(nxt, 0, 0, std::integral_constant<int, (HM - 1) * CL + Q2>{});
                if constexpr (I == FM - 1) {
                  read_one(nxt, 0, 0, std::integral_constant<int, FM * CL + J * CL>{});
                  if constexpr (CL > 1) read_one(nxt, 0, 0, std::integral_constant<int, FM * CL + J * CL + 1>{});
                }
              }
              if constexpr (Q < NQP) {
                constexpr int PA = Q * NPAIR / NQP, PB = (Q + 1) * NPAIR / NQP;
                if constexpr (PB > PA) pair(cur, k3, std::integral_constant<int, PA>{}, C0{});
                if constexpr (PB > PA + 1) pair(cur, k3, std::integral_constant<int, PA + 1>{}, C0{});
              }
              __builtin_amdgcn_sched_barrier(0);
            }(),
            ...);
      }(std::make_integer_sequence<int, NQ>{});
    }
  } else {
    // One slab.  PAR = s % 2 as a constant (it names staging sets, i.e. registers).
    auto slab = [&](int s, auto par_c) {
      constexpr int PAR = decltype(par_c)::value;
      // staging set and reload distance: one set carries every slab (written one slab after its
      // reload); with two, set t % 2 carries slab t (written two slabs after its reload)
      typedef std::integral_constant<int, NSET == 2 ? (PAR ^ 1) : 0> SetFirst;
      typedef std::integral_constant<int, NSET == 2 ? PAR : 0> SetLast;
      // (two staging sets: the loop is unrolled by two and PAR == s % 2, a constant)
      uint8_t* cur = lds + (NSET == 2 ? PAR : (s & 1)) * SLAB;
      uint8_t* nxt = lds + (NSET == 2 ? PAR ^ 1 : ((s + 1) & 1)) * SLAB;
      // first k-step: the rest of the staged slab s + 1 goes into `nxt`, its registers re-loaded
      kstep(C0{}, cur, C1{}, C1{}, nxt, slab_k0(s + 1 + NSET), CNP0{}, CNP{}, SetFirst{});
      // middle k-steps
      [&]<int... KS>(std::integer_sequence<int, KS...>) {
        (kstep(std::integral_constant<int, (KS + 1) & 1>{}, cur, std::integral_constant<int, KS + 2>{},
               std::integral_constant<int, KS & 1>{}, nxt, 0, C0{}, C0{}, C0{}),
         ...);
      }(std::make_integer_sequence<int, NKS - 2>{});
      // Last k-step.  Its fragments are in registers once the LDS counter drains; after the
      // barrier nobody reads `cur` any more: the staged slab s + 2 starts to go into it, and the
      // first fragments of slab s + 1 are read from `nxt`.
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
      __builtin_amdgcn_sched_barrier(0);
      kstep(std::integral_constant<int, (NKS - 1) & 1>{}, nxt, C0{}, C0{}, cur, slab_k0(s + 2 + NSET), C0{}, CNP0{},
            SetLast{});
    };
    if constexpr (NSET == 2) {
      int s = 0;
      for (; s + 1 < nslab; s += 2) {
        slab(s, C0{});
        slab(s + 1, C1{});
      }
      if (s < nslab) slab(s, C0{});
    } else {
      for (int s = 0; s < nslab; ++s) slab(s, C0{});
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  if (blockIdx.x == 0 && tid == 0 && g.clk) { g.clk[2] = clock64(); g.clk[3] = wall_clock64(); }

  // ---- epilogue: acc[i][j][v] is C(row, col) with
  //      row = 32 i + 8 (v / 4) + 4 (lane / 32) + v % 4,   col = 32 j + lane % 32   (32 x 32 blocks)
  //      row = 16 i + 4 (lane / 16) + v,                   col = 16 j + lane % 16   (16 x 16 blocks)
  int e_lane = lane;
  if constexpr (LOOPS) asm volatile("" : "+v"(e_lane));  // as above
  const int m_base = row_lo + wm * TM + (e_lane / RB) * 4;
  const int n_base = col_lo + wn * TN + e_lane % RB;
  typename Epi::Col colctx[FN];
#pragma unroll
  for (int j = 0; j < FN; ++j) colctx[j] = epi.col(min(n_base + j * RB, g.N - 1), expert, g.N);
  // Rows are tested in groups that a wave's accumulator layout makes uniform (8 rows of a 32 x 32
  // block, 16 of a 16 x 16 one): a group wholly below row_hi stores without any per-lane test, a
  // group wholly past it is skipped by a scalar branch, and only the one group that row_hi cuts
  // tests every lane.  (Per-lane tests around every store put each store into a basic block of its
  // own: a row tile with 200 of its 256 rows valid then took twice as long to store as a full one.)
  const bool cols_full = col_lo + BN <= g.N;
  const int rows_left = row_hi - row_lo - wm * TM;  // valid rows from this wave's first row on; uniform
  // whole tile: one straight run of stores (the row groups' branches cost the dense shapes 1 %; the
  // persistent blocks have no registers for a third copy of the stores)
  const bool interior = !GROUPED && cols_full && row_lo + BM <= row_hi;
  if (interior) {
    // All row operands (the token scales) are requested before the first store: the compiler may
    // not move a load across a store through an unrelated pointer, so fetched row block by row
    // block their latency was paid FM times, between the blocks' stores.
    if constexpr (B16) {
      typename Epi::Row rowctx[FM][4];
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int v = 0; v < 4; ++v) rowctx[i][v] = epi.row(m_base + i * 16 + v);
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int v = 0; v < 4; ++v)
#pragma unroll
          for (int j = 0; j < FN; ++j)
            epi.store(m_base + i * 16 + v, n_base + j * 16, acc[i][j][v], rowctx[i][v], colctx[j]);
    } else {
      // (two row blocks at a time: 64 operands at once left some instances without registers; the
      // e4m3 instance with 32 x 32 blocks, kept for comparisons, has none for more than one block)
      constexpr int RBB = OP == MMA_I8 ? 2 : 1;
      static_assert(FM % RBB == 0, "row blocks in batches");
#pragma unroll
      for (int i0 = 0; i0 < FM; i0 += RBB) {
        typename Epi::Row rowctx[RBB][16];
#pragma unroll
        for (int i = 0; i < RBB; ++i)
#pragma unroll
          for (int v = 0; v < 16; ++v) rowctx[i][v] = epi.row(m_base + (i0 + i) * 32 + (v >> 2) * 8 + (v & 3));
#pragma unroll
        for (int i = 0; i < RBB; ++i)
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            const int m = m_base + (i0 + i) * 32 + (v >> 2) * 8 + (v & 3);
#pragma unroll
            for (int j = 0; j < FN; ++j) epi.store(m, n_base + j * 32, acc[i0 + i][j][v], rowctx[i][v], colctx[j]);
          }
      }
    }
  } else if constexpr (B16) {
    typename Epi::Row rowctx_all[FM][4];  // (all row operands first, as above; rows past the end take the last row's)
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int v = 0; v < 4; ++v) rowctx_all[i][v] = epi.row(min(m_base + i * 16 + v, row_hi - 1));
#pragma unroll
    for (int i = 0; i < FM; ++i) {
      const int left = rows_left - i * 16;
      if (left <= 0) break;
      typename Epi::Row(&rowctx)[4] = rowctx_all[i];
      if (left >= 16 && cols_full) {
#pragma unroll
        for (int v = 0; v < 4; ++v)
#pragma unroll
          for (int j = 0; j < FN; ++j)
            epi.store(m_base + i * 16 + v, n_base + j * 16, acc[i][j][v], rowctx[v], colctx[j]);
      } else {
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const int m = m_base + i * 16 + v;
          if (m < row_hi) {
#pragma unroll
            for (int j = 0; j < FN; ++j) {
              const int n = n_base + j * 16;
              if (n < g.N) epi.store(m, n, acc[i][j][v], rowctx[v], colctx[j]);
            }
          }
        }
      }
    }
  } else
#pragma unroll
  for (int i = 0; i < FM; ++i) {
    if (rows_left - i * 32 <= 0) break;
    typename Epi::Row rowctx[16];
#pragma unroll
    for (int v = 0; v < 16; ++v)
      rowctx[v] = epi.row(min(m_base + i * 32 + (v >> 2) * 8 + (v & 3), row_hi - 1));
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int left = rows_left - i * 32 - q * 8;
      if (left >= 8 && cols_full) {
#pragma unroll
        for (int vv = 0; vv < 4; ++vv) {
          const int v = q * 4 + vv, m = m_base + i * 32 + q * 8 + vv;
#pragma unroll
          for (int j = 0; j < FN; ++j) epi.store(m, n_base + j * 32, acc[i][j][v], rowctx[v], colctx[j]);
        }
      } else if (left > 0) {
#pragma unroll
        for (int vv = 0; vv < 4; ++vv) {
          const int v = q * 4 + vv, m = m_base + i * 32 + q * 8 + vv;
          if (m < row_hi) {
#pragma unroll
            for (int j = 0; j < FN; ++j) {
              const int n = n_base + j * 32;
              if (n < g.N) epi.store(m, n, acc[i][j][v], rowctx[v], colctx[j]);
            }
          }
        }
      }
    }
  }
  if (blockIdx.x == 0 && tid == 0 && g.clk) { g.clk[4] = clock64(); g.clk[5] = wall_clock64(); }
  if constexpr (!GROUPED) {
    break;
  } else {
    if (g.rows_per_group > 0) break;
    p_next += p_step;
    if (p_next >= p_end) break;
    __syncthreads();  // every wave has read its last fragments: the slabs may be overwritten
  }
  }  // tiles
#endif  // __HIP_DEVICE_COMPILE__
}

}  // namespace fmsmo
