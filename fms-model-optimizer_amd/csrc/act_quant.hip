// Fused activation quantizers: one pass over x (read 2-4 B, write 1 B per element).
//
// One 256-thread block per token row.  The row is pulled from HBM once with 16-byte loads and
// kept in registers while the block reduces |x| (wave butterfly + one LDS exchange); the scale
// is then formed and the row is quantized straight from registers and written with 8-byte
// (int8 / e4m3) stores.  Rows longer than 16384 elements are read a second time (L2 hit).
//
// Every division is IEEE correctly rounded in fp32 on operands widened from the compute dtype T
// and then rounded to T, which equals the correctly rounded T division torch performs.
#include "quant_math.hpp"

#include <type_traits>

namespace fmsmo {

constexpr int AQ_THREADS = 256;
constexpr int AQ_MAXCHUNK = 8;   // chunks cached in registers per thread

__device__ __forceinline__ float block_max(float v, float* red) {
  v = wave_max(v);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float r = red[0];
#pragma unroll
  for (int w = 1; w < AQ_THREADS / 64; ++w) r = fmaxf(r, red[w]);
  __syncthreads();
  return r;
}

// ------------------------------------------------------------------ int8, dynamic per token
template <int XT, int T>
__global__ __launch_bounds__(AQ_THREADS) void quant_i8_pertoken_kernel(
    const void* __restrict__ x, int64_t ldx, const void* __restrict__ smooth, int smooth_dtype,
    int saturate, int8_t* __restrict__ q, int64_t ldq, float* __restrict__ scale, int K) {
  __shared__ float red[AQ_THREADS / 64];
  const int row = blockIdx.x;
  const size_t xrow = (size_t)row * ldx;
  const int nchunk = K / AQ_VEC;
  float v[AQ_MAXCHUNK][8];
  float amax = 0.0f;

  auto fetch = [&](int c, float (&e)[8]) {
    load8<XT>(x, xrow + (size_t)c * AQ_VEC, e);
    if (smooth) {
      float d[8];
      if (smooth_dtype == FMSMO_F16) load8<FMSMO_F16>(smooth, (size_t)c * AQ_VEC, d);
      else if (smooth_dtype == FMSMO_BF16) load8<FMSMO_BF16>(smooth, (size_t)c * AQ_VEC, d);
      else load8<FMSMO_F32>(smooth, (size_t)c * AQ_VEC, d);
#pragma unroll
      for (int i = 0; i < 8; ++i) e[i] = round_to<T>(e[i] / d[i]);
    }
  };

#pragma unroll
  for (int i = 0; i < AQ_MAXCHUNK; ++i) {
    const int c = threadIdx.x + i * AQ_THREADS;
    if (c < nchunk) {
      fetch(c, v[i]);
#pragma unroll
      for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(v[i][j]));
    }
  }
  for (int c = threadIdx.x + AQ_MAXCHUNK * AQ_THREADS; c < nchunk; c += AQ_THREADS) {
    float e[8];
    fetch(c, e);
#pragma unroll
    for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(e[j]));
  }
  amax = block_max(amax, red);

  // s = rnd_T( max(amax, rnd_T(1e-5)) / 127 )
  const float s = round_to<T>(fmaxf(amax, round_to<T>(1e-5f)) / 127.0f);
  if (threadIdx.x == 0) scale[row] = s;

  auto emit = [&](int c, const float (&e)[8]) {
    uint8_t b[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      float r = __builtin_rintf(round_to<T>(e[j] / s));
      if (saturate) r = fminf(fmaxf(r, -127.0f), 127.0f);
      b[j] = (uint8_t)(int)r;  // two's-complement truncation: 128 -> 0x80 = -128
    }
    store8((uint8_t*)q, (size_t)row * ldq + (size_t)c * AQ_VEC, b);
  };
#pragma unroll
  for (int i = 0; i < AQ_MAXCHUNK; ++i) {
    const int c = threadIdx.x + i * AQ_THREADS;
    if (c < nchunk) emit(c, v[i]);
  }
  for (int c = threadIdx.x + AQ_MAXCHUNK * AQ_THREADS; c < nchunk; c += AQ_THREADS) {
    float e[8];
    fetch(c, e);
    emit(c, e);
  }
}

// ------------------------------------------------------------------ int8, dynamic per token,
// 16-bit compute dtype (x, the SmoothQuant scale and every intermediate in fp16 or bf16).
//
// Blocks walk rows with a stride of gridDim.x and fetch the next row while they work on the
// current one, so the bytes in flight per compute unit stay constant for the life of the kernel
// (the launcher gives that resident grid to the instances whose per-block set-up is worth keeping;
// the others get one row per block, see row_walk_grid).
// The SmoothQuant scale (or its reciprocal) of the thread's columns lives in registers for all
// rows of the block, and the divided row is kept as packed 16-bit values.
//
// fp16 divisions do not use the IEEE fp32 sequence.  For fp16 operands e, s the quotient is never
// closer than 2^-23 (relative) to a rounding boundary of the fp16 grid without lying exactly on
// it (e - m s is a non-zero multiple of the product's last bit, m has 12 significant bits, s 11),
// so any faithfully rounded fp32 quotient that is exact when e / s is representable rounds to
// the same fp16 value as the correctly rounded one.  q1 = fma(fma(-q0, s, e), r, q0) with
// q0 = e r, r = rcp(s) (1 ulp) is such a quotient: the inner fma is exact, the correction
// carries a relative error of 2^-23 on a term of 2 ulp.  The same holds for bf16 (boundaries at
// least 2^-17 apart from any inexact quotient) as long as nothing leaves the fp32 normal range:
// a block whose bf16 divisors fall outside 2^-60 .. 2^60, and any row whose maximum comes out
// inf / NaN (zero or non-finite operands, overflow), is computed with plain IEEE divisions.
// Quotients below 2^-66 may round differently, which can change neither q nor the scale.
template <int T, int NCH, bool SMOOTH, int TH = AQ_THREADS, bool KEEP = true>
__global__ __launch_bounds__(TH) void quant_i8_pertoken16_kernel(
    const u16* __restrict__ x, int64_t ldx, const u16* __restrict__ smooth, int saturate,
    int8_t* __restrict__ q, int64_t ldq, float* __restrict__ scale, int M, int K) {
  // reciprocals of the divisors stay in registers across rows while the row is short enough
  constexpr bool KEEP_RCP = SMOOTH && KEEP;
  __shared__ float red[2][TH / 64];
  const int nchunk = K / AQ_VEC;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;

  // divisors of this thread's columns, packed as loaded
  v4i sm[SMOOTH ? NCH : 1];
  float sr[KEEP_RCP ? NCH : 1][8];
  bool ieee_block = false;
  // bf16 divisors outside 2^-60 .. 2^60 (zero, subnormal, inf and NaN among them) are outside the
  // fast quotient's proof: a thread that holds one reports NaN as its row maximum, which sends
  // every row of the block down the IEEE path -- the rows' own reduction carries the flag, the
  // set-up needs no barrier.  The test is on the packed exponent fields (biased 67 .. 186;
  // 2^60 itself counts as outside, which only costs speed).
  [[maybe_unused]] bool bad_divisor = false;
  if constexpr (SMOOTH) {
    us2 worst = {0, 0};
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int c = threadIdx.x + i * TH;
      if (c < nchunk) {
        sm[i] = *(const v4i*)(smooth + (size_t)c * AQ_VEC);
        if constexpr (T == FMSMO_BF16) {
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            // (a borrow out of the low half only happens when that half is already out of range)
            const uint32_t ex = (((uint32_t)sm[i][j] >> 7) & 0x00ff00ffu) - 0x00430043u;
            us2 e2;
            __builtin_memcpy(&e2, &ex, 4);
            worst = __builtin_elementwise_max(worst, e2);
          }
        }
        if constexpr (KEEP_RCP) {
#pragma unroll
          for (int j = 0; j < 8; ++j)
            sr[i][j] = __builtin_amdgcn_rcpf(cvt16<T>((u16)((uint32_t)sm[i][j >> 1] >> ((j & 1) * 16))));
        }
      }
    }
    if constexpr (T == FMSMO_BF16) bad_divisor = worst[0] > 119 || worst[1] > 119;
  }

  const float nz = opaque_neg_zero();
  v4i cur[NCH], nxt[NCH];
  auto load_row = [&](int row, v4i (&dst)[NCH]) {
    const u16* xr = x + (size_t)row * ldx;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int c = threadIdx.x + i * TH;
      if (c < nchunk) dst[i] = __builtin_nontemporal_load((const v4i*)(xr + (size_t)c * AQ_VEC));
    }
  };
  // cur <- rnd_T(cur / smooth), packed.  The quotient of a zero / non-finite operand comes out NaN
  // instead of its IEEE value; the caller detects that from the row maximum.
  auto divide_row = [&]() {
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int c = threadIdx.x + i * TH;
      if (c < nchunk) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          uint32_t d = (uint32_t)sm[i][j];
          // long rows: keep the compiler from hoisting the 2 x NCH x 8 widened divisors and
          // reciprocals out of the row loop (that costs 128 registers and halves the occupancy)
          if constexpr (!KEEP_RCP) asm volatile("" : "+v"(d));
          const uint32_t w = (uint32_t)cur[i][j];
          const float lo = cvt16<T>((u16)(w & 0xffff)), hi = cvt16<T>((u16)(w >> 16));
          const float dl = cvt16<T>((u16)(d & 0xffff)), dh = cvt16<T>((u16)(d >> 16));
          float rl, rh;
          if constexpr (KEEP_RCP) {
            rl = sr[i][2 * j], rh = sr[i][2 * j + 1];
          } else {
            rl = __builtin_amdgcn_rcpf(dl), rh = __builtin_amdgcn_rcpf(dh);
          }
          cur[i][j] = (int)pack16<T>(div16_mix<T>(lo, dl, rl, nz), div16_mix<T>(hi, dh, rh, nz));
        }
      }
      __builtin_amdgcn_sched_barrier(0);  // one chunk at a time: keeps the live ranges short
    }
  };
  // max |cur| over the row.  |e| is monotone in its bit pattern, so the maximum is taken on the
  // packed 15-bit magnitudes, two per instruction (a NaN outranks inf).
  int parity = 0;
  auto row_amax_bits = [&]() -> uint32_t {
    us2 amax2 = {0, 0};
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int c = threadIdx.x + i * TH;
      if (c < nchunk) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint32_t mag = (uint32_t)cur[i][j] & 0x7fff7fffu;
          us2 m2;
          __builtin_memcpy(&m2, &mag, 4);
          amax2 = __builtin_elementwise_max(amax2, m2);
        }
      }
    }
    if constexpr (SMOOTH && T == FMSMO_BF16) {
      if (bad_divisor) amax2 = us2{0x7fff, 0x7fff};
    }
    uint32_t v = wave_max_u32((uint32_t)(amax2[0] > amax2[1] ? amax2[0] : amax2[1]));
    float* rb = red[parity];
    parity ^= 1;
    if (lane == 0) rb[wave] = __uint_as_float(v);
    __syncthreads();
#pragma unroll
    for (int w = 0; w < TH / 64; ++w) {
      const uint32_t o = __float_as_uint(rb[w]);
      v = o > v ? o : v;
    }
    return v;
  };
  constexpr uint32_t INF_BITS = T == FMSMO_F16 ? 0x7c00u : 0x7f80u;

  int row = blockIdx.x;
  if (row < M) load_row(row, cur);
  const float floor_T = cvt16<T>(to16<T>(1e-5f));
  for (; row < M; row += gridDim.x) {
    const int nrow = row + gridDim.x;
    if (nrow < M) load_row(nrow, nxt);

    uint32_t abits = INF_BITS;
    if (!ieee_block) {
      if constexpr (SMOOTH) divide_row();
      abits = row_amax_bits();
    }
    if (abits >= INF_BITS) {
      // divisors outside the fast path's range, zero / non-finite operands or overflow in the
      // row: IEEE divisions, straight from memory (block-uniform branch)
      quant_i8_row_ieee16<T, TH>(x + (size_t)row * ldx, SMOOTH ? smooth : nullptr, saturate,
                                 q + (size_t)row * ldq, scale + row, K, red[0]);
#pragma unroll
      for (int i = 0; i < NCH; ++i) cur[i] = nxt[i];
      continue;
    }
    const float amax = cvt16<T>((u16)abits);

    // s = rnd_T( max(amax, rnd_T(1e-5)) / 127 ): finite and non-zero, so the quotients below
    // need no special-case fix-up unless the row overflowed the 16-bit range (amax = inf)
    const float s = cvt16<T>(to16<T>(fmaxf(amax, floor_T) / 127.0f));
    const float rs = __builtin_amdgcn_rcpf(s);
    if (threadIdx.x == 0) scale[row] = s;
    int8_t* qr = q + (size_t)row * ldq;
    {
#pragma unroll
      for (int i = 0; i < NCH; ++i) {
        const int c = threadIdx.x + i * TH;
        if (c < nchunk) {
          uint32_t code[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const uint32_t w = (uint32_t)cur[i][j];
            const float ql = div16_mix<T>(cvt16<T>((u16)(w & 0xffff)), s, rs, nz);
            const float qh = div16_mix<T>(cvt16<T>((u16)(w >> 16)), s, rs, nz);
            code[j] = rint_codes_packed<T>(pack16<T>(ql, qh), saturate != 0);
          }
          // bytes 0 and 2 of each code word -> 8 consecutive int8
          const uint32_t o0 = __builtin_amdgcn_perm(code[1], code[0], 0x06040200u);
          const uint32_t o1 = __builtin_amdgcn_perm(code[3], code[2], 0x06040200u);
          *(uint2*)(qr + (size_t)c * AQ_VEC) = make_uint2(o0, o1);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
#pragma unroll
    for (int i = 0; i < NCH; ++i) cur[i] = nxt[i];
  }
}

// ------------------------------------------------------------------ int8, dynamic per token,
// fp16 x with an fp32 SmoothQuant scale: torch promotes x / smooth to fp32 and the whole
// quantizer then runs in fp32.
//
// Same row-walking structure as the 16-bit kernel.  Divisions use the correctly rounded fp32
// sequence without its range-scaling steps: r1 = rcp(s) refined once, q0 = x r1, two residual
// corrections q <- fma(fma(-s, q, x), r1, q).  That is the IEEE result whenever no intermediate
// leaves the normal range, which holds for fp16 x (6e-8 .. 65504) and 2^-60 <= |s| <= 2^60;
// a block that sees a divisor outside that range, or a row whose maximum is not finite, takes
// the plain IEEE division instead.  Quotients by the row scale only feed rint(); where they
// underflow they are far below 0.5.
// bf16 x (XT = FMSMO_BF16) reaches below fp16's range: a row whose maximum quotient is under
// 2^-80 (and not zero) also takes the IEEE division, because the residuals of its corrections
// could fall below the smallest fp32 subnormal; elements that small inside an ordinary row
// quantize to zero whichever way their last bit is rounded.
template <int NCH, bool KEEP, int TH = AQ_THREADS, int XT = FMSMO_F16>
__global__ __launch_bounds__(TH) void quant_i8_pertoken_f16x_f32s_kernel(
    const u16* __restrict__ x, int64_t ldx, const float* __restrict__ smooth, int saturate,
    int8_t* __restrict__ q, int64_t ldq, float* __restrict__ scale, int M, int K) {
  __shared__ float red[2][TH / 64];
  const int nchunk = K / AQ_VEC;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;

  // divisors (and refined reciprocals) of this thread's columns; kept across rows for short rows,
  // re-read from L2 per row otherwise
  // A thread that holds a divisor outside 2^-60 .. 2^60 (or NaN) reports NaN as its row maximum:
  // the row's own reduction then sends the whole row down the IEEE path, and the set-up needs no
  // barrier.
  float sv[KEEP ? NCH : 1][8], sr[KEEP ? NCH : 1][8];
  int bad = 0;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = threadIdx.x + i * TH;
    if (c < nchunk) {
      const float4 a = *(const float4*)(smooth + (size_t)c * AQ_VEC);
      const float4 b = *(const float4*)(smooth + (size_t)c * AQ_VEC + 4);
      const float d[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float m = fabsf(d[j]);
        bad |= !(m >= 8.6736174e-19f && m <= 1.1529215e18f);
        if constexpr (KEEP) {
          sv[i][j] = d[j];
          sr[i][j] = rcp_refined(d[j]);
        }
      }
    }
  }
  constexpr bool ieee_block = false;

  const float nz = opaque_neg_zero();
  v4i cur[NCH], nxt[NCH];
  float e[NCH][8];
  auto load_row = [&](int row, v4i (&dst)[NCH]) {
    const u16* xr = x + (size_t)row * ldx;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int c = threadIdx.x + i * TH;
      if (c < nchunk) dst[i] = __builtin_nontemporal_load((const v4i*)(xr + (size_t)c * AQ_VEC));
    }
  };
  // e <- x / smooth (fp32); returns the thread's max |e|
  auto divide_row = [&](auto ieee_tag) -> float {
    constexpr bool IEEE = decltype(ieee_tag)::value;
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int c = threadIdx.x + i * TH;
      if (c < nchunk) {
        float d[8];
        if constexpr (!KEEP || IEEE) {
          const float4 a = *(const float4*)(smooth + (size_t)c * AQ_VEC);
          const float4 b = *(const float4*)(smooth + (size_t)c * AQ_VEC + 4);
          d[0] = a.x; d[1] = a.y; d[2] = a.z; d[3] = a.w; d[4] = b.x; d[5] = b.y; d[6] = b.z; d[7] = b.w;
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float xv = cvt16<XT>((u16)((uint32_t)cur[i][j >> 1] >> ((j & 1) * 16)));
          if constexpr (IEEE) e[i][j] = xv / d[j];
          else if constexpr (KEEP) e[i][j] = div32_fast_mix(xv, sv[i][j], sr[i][j], nz);
          else e[i][j] = div32_fast_mix(xv, d[j], rcp_refined(d[j]), nz);
          amax = fmaxf(amax, fabsf(e[i][j]));
        }
      }
    }
    if constexpr (!IEEE) {
      if (bad) amax = __builtin_nanf("");
    }
    return amax;
  };
  int parity = 0;
  auto block_amax = [&](float v) -> float {
    // NaN must survive the reduction (it selects the IEEE path): compare bit patterns of |v|
    uint32_t b = __float_as_uint(v) & 0x7fffffffu;
    b = wave_max_u32(b);
    float* rb = red[parity];
    parity ^= 1;
    if (lane == 0) rb[wave] = __uint_as_float(b);
    __syncthreads();
    uint32_t r = __float_as_uint(rb[0]);
#pragma unroll
    for (int w = 1; w < TH / 64; ++w) r = max(r, __float_as_uint(rb[w]));
    return __uint_as_float(r);
  };

  int row = blockIdx.x;
  if (row < M) load_row(row, cur);
  for (; row < M; row += gridDim.x) {
    const int nrow = row + gridDim.x;
    if (nrow < M) load_row(nrow, nxt);

    float amax;
    bool ieee = ieee_block;
    if (!ieee) {
      amax = block_amax(divide_row(std::false_type{}));
      ieee = !(amax < __builtin_inff());  // inf or NaN somewhere in the row
      if constexpr (XT == FMSMO_BF16) ieee = ieee || (amax != 0.0f && amax < 8.271806e-25f);
    }
    if (ieee) {
      // fmaxf drops NaN like the generic kernel does
      float v = divide_row(std::true_type{});
      amax = block_amax(v);
    }
    const float s = fmaxf(amax, 1e-5f) / 127.0f;
    const float rs = rcp_refined(s);
    if (threadIdx.x == 0) scale[row] = s;
    int8_t* qr = q + (size_t)row * ldq;
    // (the two block-uniform choices are made outside the element loops: tested per element they
    // cut the unrolled code into one basic block per element, which serializes the quotients)
    auto emit_row = [&](auto ieee_tag, auto sat_tag) {
      constexpr bool IEEE = decltype(ieee_tag)::value, SAT = decltype(sat_tag)::value;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int c = threadIdx.x + i * TH;
      if (c < nchunk) {
        uint32_t code[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          float r = IEEE ? e[i][j] / s : div32_fast(e[i][j], s, rs);
          if constexpr (SAT) r = fminf(fmaxf(r, -127.0f), 127.0f);  // the bounds are integers
          // |r| <= 128.5 in every finite row: the addition of 1.5 * 2^23 itself rounds r to the
          // nearest integer, ties to even, and leaves it in two's complement in the low mantissa
          // bits
          code[j] = __float_as_uint(r + 12582912.0f);
        }
        // byte 0 of each code word -> 8 consecutive int8
        uint32_t o[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const uint32_t lo = __builtin_amdgcn_perm(code[4 * h + 1], code[4 * h], 0x0c0c0400u);
          const uint32_t hi = __builtin_amdgcn_perm(code[4 * h + 3], code[4 * h + 2], 0x0c0c0400u);
          o[h] = __builtin_amdgcn_perm(hi, lo, 0x05040100u);
        }
        *(uint2*)(qr + (size_t)c * AQ_VEC) = make_uint2(o[0], o[1]);
      }
    }
    };
    if (ieee) {
      if (saturate) emit_row(std::true_type{}, std::true_type{});
      else emit_row(std::true_type{}, std::false_type{});
    } else {
      if (saturate) emit_row(std::false_type{}, std::true_type{});
      else emit_row(std::false_type{}, std::false_type{});
    }
#pragma unroll
    for (int i = 0; i < NCH; ++i) cur[i] = nxt[i];
  }
}

// ------------------------------------------------------------------ int8, static per tensor
template <int XT>
__global__ __launch_bounds__(AQ_THREADS) void quant_i8_static_kernel(
    const void* __restrict__ x, int64_t ldx, float scale, float zp, float sym, int pt_native,
    int8_t* __restrict__ q, int64_t ldq, int K) {
  const int row = blockIdx.x;
  const int nchunk = K / AQ_VEC;
  const float inv_scale = 1.0f / scale;
  // x / scale: the IEEE fp32 sequence is r1 = refined rcp, q = x r1, two residual corrections,
  // wrapped in range scaling and a special-case fix-up.  Without the wrapping the same operations
  // give the same quotient whenever no intermediate leaves the normal range: |scale| within
  // 2^-20 .. 2^20 and x zero or within 2^-100 .. 2^100 (always, for fp16 x) with a finite result.
  const float r1 = rcp_refined(scale);
  const bool fast = fabsf(scale) >= 9.5367431640625e-07f && fabsf(scale) <= 1048576.0f;
  for (int c = threadIdx.x; c < nchunk; c += AQ_THREADS) {
    float e[8];
    load8<XT>(x, (size_t)row * ldx + (size_t)c * AQ_VEC, e);
    uint8_t b[8];
    float qv[8];
    if (!pt_native) {
      bool ok = fast;
      if (fast) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          qv[j] = div32_fast(e[j], scale, r1);
          ok = ok && fabsf(qv[j]) < __builtin_inff();
          if constexpr (XT != FMSMO_F16) {
            // |x| in [2^-100, 2^100): one unsigned compare on the exponent field
            const uint32_t mag = __float_as_uint(e[j]) & 0x7fffffffu;
            ok = ok && (mag == 0u || mag - 0x0d800000u < 0x64000000u);
          }
        }
      }
      if (__builtin_expect(!ok, 0)) {  // one rarely taken branch per 8 elements
#pragma unroll
        for (int j = 0; j < 8; ++j) qv[j] = e[j] / scale;
      }
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      // ((x/s + zp) - 128) + sym, each step rounded to fp32, then round-half-even and clamp
      float t;
      if (pt_native)  // torch.quantize_per_tensor: rint(x * (1/scale)) + zero_point
        t = __builtin_rintf(__fmul_rn(e[j], inv_scale)) + (zp - 128.0f + sym);
      else
        t = __builtin_rintf(__fadd_rn(__fadd_rn(__fadd_rn(qv[j], zp), -128.0f), sym));
      t = fminf(fmaxf(t, -128.0f), 127.0f);
      b[j] = (uint8_t)(int)t;
    }
    store8((uint8_t*)q, (size_t)row * ldq + (size_t)c * AQ_VEC, b);
  }
}

// ------------------------------------------------------------------ int8, multiplicative scale
// The quantize half of the W8A8 accelerator op: the scale is  levels / clip  as torch evaluates
// "number / tensor", i.e. rnd_T( rnd_T(1 / clip) * levels )  (the reflected division of a Python
// scalar by a tensor is reciprocal-then-multiply), and the codes are  rint( rnd_T( rnd_T(x / sq) * scale ) [- zp] ),  every
// intermediate rounded to T as torch's elementwise kernels do.  Products of two 16-bit floats are
// exact in fp32, so rounding the fp32 product to T is the correctly rounded T product.
//   mode 0: per token, scale_m = 127 / max_k |x/sq|, codes clamped to +-127
//   mode 1: per tensor symmetric, scale = 127 / clip[0], codes clamped to +-127
//   mode 2: per tensor asymmetric, scale = 255 / (clip[0] - clip[1]), zp = clip[1] * scale, codes
//           clamped to [0, 255] and stored minus 128
// a_scale receives 1 / scale_m per row (mode 0) or { 1 / scale, zp } (modes 1 and 2).
template <int T>
__device__ __forceinline__ float levels_over(float levels, float clip) {
  return round_to<T>(__fmul_rn(round_to<T>(1.0f / clip), levels));
}

template <int XT, int T>
__global__ __launch_bounds__(AQ_THREADS) void quant_i8_mulscale_kernel(
    const void* __restrict__ x, int64_t ldx, const void* __restrict__ smooth,
    const void* __restrict__ clip, int meta_dtype, int mode, int8_t* __restrict__ q, int64_t ldq,
    float* __restrict__ a_scale, int K) {
  __shared__ float red[AQ_THREADS / 64];
  const int row = blockIdx.x;
  const size_t xrow = (size_t)row * ldx;
  const int nchunk = K / AQ_VEC;
  float v[AQ_MAXCHUNK][8];

  auto meta = [&](const void* p, size_t i) {
    return meta_dtype == FMSMO_F16 ? load_as_f32<FMSMO_F16>(p, i)
           : meta_dtype == FMSMO_BF16 ? load_as_f32<FMSMO_BF16>(p, i)
                                      : load_as_f32<FMSMO_F32>(p, i);
  };
  auto fetch = [&](int c, float (&e)[8]) {
    load8<XT>(x, xrow + (size_t)c * AQ_VEC, e);
    if (smooth) {
      float d[8];
      if (meta_dtype == FMSMO_F16) load8<FMSMO_F16>(smooth, (size_t)c * AQ_VEC, d);
      else if (meta_dtype == FMSMO_BF16) load8<FMSMO_BF16>(smooth, (size_t)c * AQ_VEC, d);
      else load8<FMSMO_F32>(smooth, (size_t)c * AQ_VEC, d);
#pragma unroll
      for (int i = 0; i < 8; ++i) e[i] = round_to<T>(e[i] / d[i]);
    }
  };

  float sx, zp = 0.0f, lo = -127.0f, hi = 127.0f, shift = 0.0f;
  if (mode == 0) {
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < AQ_MAXCHUNK; ++i) {
      const int c = threadIdx.x + i * AQ_THREADS;
      if (c < nchunk) {
        fetch(c, v[i]);
#pragma unroll
        for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(v[i][j]));
      }
    }
    for (int c = threadIdx.x + AQ_MAXCHUNK * AQ_THREADS; c < nchunk; c += AQ_THREADS) {
      float e[8];
      fetch(c, e);
#pragma unroll
      for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(e[j]));
    }
    amax = block_max(amax, red);
    // a row of zeros has no scale (127 / 0): it is quantized to zeros with a zero output scale
    sx = amax > 0.0f ? levels_over<T>(127.0f, amax) : 0.0f;
    if (threadIdx.x == 0) a_scale[row] = (sx > 0.0f) ? 1.0f / sx : 0.0f;
  } else {
#pragma unroll
    for (int i = 0; i < AQ_MAXCHUNK; ++i) {
      const int c = threadIdx.x + i * AQ_THREADS;
      if (c < nchunk) fetch(c, v[i]);
    }
    const float cv = meta(clip, 0);
    if (mode == 1) {
      sx = levels_over<T>(127.0f, cv);
    } else {
      const float cvn = meta(clip, 1);
      sx = levels_over<T>(255.0f, round_to<T>(__fsub_rn(cv, cvn)));
      zp = round_to<T>(__fmul_rn(cvn, sx));
      lo = 0.0f; hi = 255.0f; shift = 128.0f;
    }
    if (row == 0 && threadIdx.x == 0) { a_scale[0] = 1.0f / sx; a_scale[1] = zp; }
  }

  auto emit = [&](int c, const float (&e)[8]) {
    uint8_t b[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      float t = round_to<T>(__fmul_rn(e[j], sx));
      if (mode == 2) t = round_to<T>(__fsub_rn(t, zp));
      t = fminf(fmaxf(__builtin_rintf(t), lo), hi) - shift;
      b[j] = (uint8_t)(int)t;
    }
    store8((uint8_t*)q, (size_t)row * ldq + (size_t)c * AQ_VEC, b);
  };
#pragma unroll
  for (int i = 0; i < AQ_MAXCHUNK; ++i) {
    const int c = threadIdx.x + i * AQ_THREADS;
    if (c < nchunk) emit(c, v[i]);
  }
  for (int c = threadIdx.x + AQ_MAXCHUNK * AQ_THREADS; c < nchunk; c += AQ_THREADS) {
    float e[8];
    fetch(c, e);
    emit(c, e);
  }
}

// ------------------------------------------------------------------ int8, multiplicative scale,
// 16-bit compute dtype (x, the SmoothQuant scale, the clip values and every intermediate in fp16
// or in bf16): the row-walking structure of quant_i8_pertoken16_kernel.  Blocks walk rows with a
// stride of gridDim.x and fetch the next row while they work on the current one; the divisors of
// the thread's columns stay in registers; the divided row is kept as packed 16-bit values and its
// maximum is taken on the packed magnitudes.  The division uses the same fast quotient (see there
// for why it rounds like the IEEE one); rows or blocks it does not cover -- divisors outside its
// range, a zero or non-finite divisor, inf / NaN anywhere in the divided row, a row maximum whose
// reciprocal overflows -- take mulscale_row_ieee16, which repeats the generic kernel's arithmetic.
// The products  rnd_T(e * scale)  are exact in fp32 (two 16-bit significands), so one rounding to T
// gives the correctly rounded T product; fp16 does it, the zero-point subtraction and the clamp
// on packed pairs, and rounds to integer by adding 1536 (mode 2: 1536 - 128, which also folds the
// shift to signed storage into the same single rounding).
template <int T, int TH>
__device__ __forceinline__ void mulscale_row_ieee16(const u16* __restrict__ xr, const u16* __restrict__ smooth,
                                                    int mode, float sx, float zp, int8_t* __restrict__ qr,
                                                    float* __restrict__ scale_out, int K, float* red) {
  const int nchunk = K / AQ_VEC;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  auto chunk = [&](int c, float (&e)[8]) {
    load8<T>(xr, (size_t)c * AQ_VEC, e);
    if (smooth) {
      float d[8];
      load8<T>(smooth, (size_t)c * AQ_VEC, d);
#pragma unroll
      for (int i = 0; i < 8; ++i) e[i] = round_to<T>(e[i] / d[i]);
    }
  };
  float lo = -127.0f, hi = 127.0f, shift = 0.0f;
  if (mode == 2) { lo = 0.0f; hi = 255.0f; shift = 128.0f; }
  if (mode == 0) {
    float amax = 0.0f;
#pragma unroll 1
    for (int c = threadIdx.x; c < nchunk; c += TH) {
      float e[8];
      chunk(c, e);
#pragma unroll
      for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(e[j]));
    }
    amax = wave_max(amax);
    __syncthreads();
    if (lane == 0) red[wave] = amax;
    __syncthreads();
    amax = red[0];
#pragma unroll
    for (int w = 1; w < TH / 64; ++w) amax = fmaxf(amax, red[w]);
    __syncthreads();
    sx = amax > 0.0f ? levels_over<T>(127.0f, amax) : 0.0f;
    if (threadIdx.x == 0) *scale_out = (sx > 0.0f) ? 1.0f / sx : 0.0f;
  }
#pragma unroll 1
  for (int c = threadIdx.x; c < nchunk; c += TH) {
    float e[8];
    chunk(c, e);
    uint8_t b[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      float t = round_to<T>(__fmul_rn(e[j], sx));
      if (mode == 2) t = round_to<T>(__fsub_rn(t, zp));
      t = fminf(fmaxf(__builtin_rintf(t), lo), hi) - shift;
      b[j] = (uint8_t)(int)t;
    }
    store8((uint8_t*)qr, (size_t)c * AQ_VEC, b);
  }
}

template <int T, int MODE, int NCH, bool SMOOTH, int TH = AQ_THREADS, bool KEEP = true>
__global__ __launch_bounds__(TH) void quant_i8_mulscale16_kernel(
    const u16* __restrict__ x, int64_t ldx, const u16* __restrict__ smooth,
    const u16* __restrict__ clip, int8_t* __restrict__ q, int64_t ldq,
    float* __restrict__ a_scale, int M, int K) {
  constexpr bool KEEP_RCP = SMOOTH && KEEP;
  constexpr int mode = MODE;
  __shared__ float red[2][TH / 64];
  const int nchunk = K / AQ_VEC;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;

  v4i sm[SMOOTH ? NCH : 1];
  float sr[KEEP_RCP ? NCH : 1][8];
  bool ieee_block = false;
  // bf16 divisors outside 2^-60 .. 2^60 (zero, subnormal, inf and NaN among them) are outside the
  // fast quotient's proof: a thread that holds one reports NaN as its row maximum, which sends
  // every row of the block down the IEEE path -- the rows' own reduction carries the flag, the
  // set-up needs no barrier.  The test is on the packed exponent fields (biased 67 .. 186;
  // 2^60 itself counts as outside, which only costs speed).
  [[maybe_unused]] bool bad_divisor = false;
  if constexpr (SMOOTH) {
    us2 worst = {0, 0};
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int c = threadIdx.x + i * TH;
      if (c < nchunk) {
        sm[i] = *(const v4i*)(smooth + (size_t)c * AQ_VEC);
        if constexpr (T == FMSMO_BF16) {
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            // (a borrow out of the low half only happens when that half is already out of range)
            const uint32_t ex = (((uint32_t)sm[i][j] >> 7) & 0x00ff00ffu) - 0x00430043u;
            us2 e2;
            __builtin_memcpy(&e2, &ex, 4);
            worst = __builtin_elementwise_max(worst, e2);
          }
        }
        if constexpr (KEEP_RCP) {
#pragma unroll
          for (int j = 0; j < 8; ++j)
            sr[i][j] = __builtin_amdgcn_rcpf(cvt16<T>((u16)((uint32_t)sm[i][j >> 1] >> ((j & 1) * 16))));
        }
      }
    }
    if constexpr (T == FMSMO_BF16) bad_divisor = worst[0] > 119 || worst[1] > 119;
  }

  // per-tensor modes: one scale (and zero point) for all rows
  float sx = 0.0f, zp = 0.0f;
  if (mode != 0) {
    const float cv = cvt16<T>(clip[0]);
    if (mode == 1) {
      sx = levels_over<T>(127.0f, cv);
    } else {
      const float cvn = cvt16<T>(clip[1]);
      sx = levels_over<T>(255.0f, round_to<T>(__fsub_rn(cv, cvn)));
      zp = round_to<T>(__fmul_rn(cvn, sx));
    }
    if (blockIdx.x == 0 && threadIdx.x == 0) { a_scale[0] = 1.0f / sx; a_scale[1] = zp; }
    // clip values that give an infinite or NaN scale or zero point: every row the IEEE way
    if (!(fabsf(sx) <= 3.0e38f) || !(fabsf(zp) <= 3.0e38f)) ieee_block = true;
  }

  const float nz = opaque_neg_zero();
  v4i cur[NCH], nxt[NCH];
  auto load_row = [&](int row, v4i (&dst)[NCH]) {
    const u16* xr = x + (size_t)row * ldx;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int c = threadIdx.x + i * TH;
      if (c < nchunk) dst[i] = __builtin_nontemporal_load((const v4i*)(xr + (size_t)c * AQ_VEC));
    }
  };
  auto divide_row = [&]() {
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int c = threadIdx.x + i * TH;
      if (c < nchunk) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          uint32_t d = (uint32_t)sm[i][j];
          if constexpr (!KEEP_RCP) asm volatile("" : "+v"(d));
          const uint32_t w = (uint32_t)cur[i][j];
          const float lo = cvt16<T>((u16)(w & 0xffff)), hi = cvt16<T>((u16)(w >> 16));
          const float dl = cvt16<T>((u16)(d & 0xffff)), dh = cvt16<T>((u16)(d >> 16));
          float rl, rh;
          if constexpr (KEEP_RCP) {
            rl = sr[i][2 * j], rh = sr[i][2 * j + 1];
          } else {
            rl = __builtin_amdgcn_rcpf(dl), rh = __builtin_amdgcn_rcpf(dh);
          }
          cur[i][j] = (int)pack16<T>(div16_mix<T>(lo, dl, rl, nz), div16_mix<T>(hi, dh, rh, nz));
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  int parity = 0;
  auto row_amax_bits = [&]() -> uint32_t {
    us2 amax2 = {0, 0};
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int c = threadIdx.x + i * TH;
      if (c < nchunk) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint32_t mag = (uint32_t)cur[i][j] & 0x7fff7fffu;
          us2 m2;
          __builtin_memcpy(&m2, &mag, 4);
          amax2 = __builtin_elementwise_max(amax2, m2);
        }
      }
    }
    if constexpr (SMOOTH && T == FMSMO_BF16) {
      if (bad_divisor) amax2 = us2{0x7fff, 0x7fff};
    }
    uint32_t v = wave_max_u32((uint32_t)(amax2[0] > amax2[1] ? amax2[0] : amax2[1]));
    float* rb = red[parity];
    parity ^= 1;
    if (lane == 0) rb[wave] = __uint_as_float(v);
    __syncthreads();
#pragma unroll
    for (int w = 0; w < TH / 64; ++w) {
      const uint32_t o = __float_as_uint(rb[w]);
      v = o > v ? o : v;
    }
    return v;
  };
  constexpr uint32_t INF_BITS = T == FMSMO_F16 ? 0x7c00u : 0x7f80u;

  int row = blockIdx.x;
  if (row < M) load_row(row, cur);
  for (; row < M; row += gridDim.x) {
    const int nrow = row + gridDim.x;
    if (nrow < M) load_row(nrow, nxt);

    uint32_t abits = INF_BITS;
    if (!ieee_block) {
      if constexpr (SMOOTH) divide_row();
      abits = row_amax_bits();
    }
    float s_row = sx;
    if (abits < INF_BITS && mode == 0) {
      const float amax = cvt16<T>((u16)abits);
      s_row = amax > 0.0f ? levels_over<T>(127.0f, amax) : 0.0f;
      if (!(s_row <= 3.0e38f)) abits = INF_BITS;  // 1 / amax overflowed T: the IEEE path's business
    }
    if (abits >= INF_BITS) {
      mulscale_row_ieee16<T, TH>(x + (size_t)row * ldx, SMOOTH ? smooth : nullptr, mode, sx, zp,
                                 q + (size_t)row * ldq, a_scale + row, K, red[0]);
#pragma unroll
      for (int i = 0; i < NCH; ++i) cur[i] = nxt[i];
      continue;
    }
    if (mode == 0 && threadIdx.x == 0) a_scale[row] = (s_row > 0.0f) ? 1.0f / s_row : 0.0f;
    int8_t* qr = q + (size_t)row * ldq;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int c = threadIdx.x + i * TH;
      if (c < nchunk) {
        uint32_t code[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint32_t w = (uint32_t)cur[i][j];
          if constexpr (T == FMSMO_F16) {
            hf2 h;
            __builtin_memcpy(&h, &w, 4);
            const _Float16 s16 = (_Float16)s_row, z16 = (_Float16)zp;
            h = h * hf2{s16, s16};
            if (mode == 2) h = h - hf2{z16, z16};
            const _Float16 lo16 = mode == 2 ? (_Float16)0.0f : (_Float16)-127.0f;
            const _Float16 hi16 = mode == 2 ? (_Float16)255.0f : (_Float16)127.0f;
            h = __builtin_elementwise_min(__builtin_elementwise_max(h, hf2{lo16, lo16}), hf2{hi16, hi16});
            const _Float16 magic = mode == 2 ? (_Float16)1408.0f : (_Float16)1536.0f;
            h = h + hf2{magic, magic};
            __builtin_memcpy(&code[j], &h, 4);
          } else {
            float tl = round_to<T>(__fmul_rn(cvt16<T>((u16)(w & 0xffff)), s_row));
            float th = round_to<T>(__fmul_rn(cvt16<T>((u16)(w >> 16)), s_row));
            float lo = -127.0f, hi = 127.0f, shift = 0.0f;
            if (mode == 2) {
              tl = round_to<T>(__fsub_rn(tl, zp));
              th = round_to<T>(__fsub_rn(th, zp));
              lo = 0.0f; hi = 255.0f; shift = 128.0f;
            }
            const int cl = (int)(fminf(fmaxf(__builtin_rintf(tl), lo), hi) - shift);
            const int ch = (int)(fminf(fmaxf(__builtin_rintf(th), lo), hi) - shift);
            code[j] = ((uint32_t)cl & 0xffu) | (((uint32_t)ch & 0xffu) << 16);
          }
        }
        const uint32_t o0 = __builtin_amdgcn_perm(code[1], code[0], 0x06040200u);
        const uint32_t o1 = __builtin_amdgcn_perm(code[3], code[2], 0x06040200u);
        *(uint2*)(qr + (size_t)c * AQ_VEC) = make_uint2(o0, o1);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int i = 0; i < NCH; ++i) cur[i] = nxt[i];
  }
}

// ------------------------------------------------------------------ int8, static per tensor,
// evaluated in the compute dtype T, for the operands of a batched matmul:
//   q = clamp( rint( rnd_T( rnd_T(x / scale) + offset ) ), -128, 127 )
// x is [batch][R][C].  The plain kernel writes q [batch][R][ldq]; the transposing kernel writes
// q [batch][C][ldq] (q[c][r] = code of x[r][c]) so that an operand stored with its reduction
// dimension outermost becomes reduction-contiguous for the MFMA kernels.  Columns of q past the
// data are filled with zeros (they pad the reduction dimension of the matmul).
// The division by the (scalar) scale without the IEEE sequence where that is exact: the 16-bit
// quotient of quant_i8_pertoken16_kernel when the scale is itself a value of T, the refined fp32
// quotient of the fp16-x / fp32-scale kernel when x is fp16; both need a scale of 2^-60 .. 2^60.
// A quotient that comes out inf or NaN (non-finite x, overflow) is redone with the IEEE division.
struct AffineDiv {
  float s, r;
  bool fast;
};
template <int XT, int T>
__device__ __forceinline__ AffineDiv affine_div(float scale) {
  AffineDiv d;
  d.s = scale;
  const float m = fabsf(scale);
  d.fast = m >= 8.6736174e-19f && m <= 1.1529215e18f;
  if constexpr (T == FMSMO_F32) {
    d.fast = d.fast && XT == FMSMO_F16;
    d.r = rcp_refined(scale);
  } else {
    d.fast = d.fast && XT == T && round_to<T>(scale) == scale;
    d.r = __builtin_amdgcn_rcpf(scale);
  }
  return d;
}
template <int T>
__device__ __forceinline__ float affine_code(float e, const AffineDiv& d, float offset) {
  float q;
  if (d.fast) {
    if constexpr (T == FMSMO_F32) q = div32_fast(e, d.s, d.r);
    else q = div16<T, false>(e, d.s, d.r);
    if (__builtin_expect(!(fabsf(q) < __builtin_inff()), 0)) q = e / d.s;
  } else {
    q = e / d.s;
  }
  const float t = round_to<T>(__fadd_rn(round_to<T>(q), offset));
  return fminf(fmaxf(__builtin_rintf(t), -128.0f), 127.0f);
}

// 8 consecutive elements starting at column c of a row; vec: the 16-byte load is legal
template <int XT>
__device__ __forceinline__ void load8_guard(const void* x, size_t row_elem, int c, int C, bool vec,
                                            float (&e)[8]) {
  if (vec && c + 8 <= C) {
    load8<XT>(x, row_elem + c, e);
  } else {
#pragma unroll
    for (int j = 0; j < 8; ++j) e[j] = (c + j < C) ? load_as_f32<XT>(x, row_elem + c + j) : 0.0f;
  }
}

template <int XT, int T>
__global__ __launch_bounds__(AQ_THREADS) void quant_i8_affine_kernel(
    const void* __restrict__ x, int64_t ldx, int64_t stride_x, float scale, float offset, bool vec,
    int8_t* __restrict__ q, int64_t ldq, int64_t stride_q, int C) {
  const size_t xrow = (size_t)blockIdx.y * stride_x + (size_t)blockIdx.x * ldx;
  uint8_t* qrow = (uint8_t*)q + (size_t)blockIdx.y * stride_q + (size_t)blockIdx.x * ldq;
  const AffineDiv dv = affine_div<XT, T>(scale);
  for (int c = threadIdx.x * 8; c < (int)ldq; c += AQ_THREADS * 8) {
    uint8_t b[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    if (c < C) {
      float e[8];
      load8_guard<XT>(x, xrow, c, C, vec, e);
#pragma unroll
      for (int j = 0; j < 8; ++j)
        b[j] = (c + j < C) ? (uint8_t)(int)affine_code<T>(e[j], dv, offset) : (uint8_t)0;
    }
    store8(qrow, (size_t)c, b);
  }
}

template <int XT, int T>
__global__ __launch_bounds__(256) void quant_i8_affine_t_kernel(
    const void* __restrict__ x, int64_t ldx, int64_t stride_x, float scale, float offset, bool vec,
    int8_t* __restrict__ q, int64_t ldq, int64_t stride_q, int R, int C) {
  __shared__ __attribute__((aligned(16))) uint8_t tile[64][80];  // [c][r], rows 16-byte aligned
  const int r0 = blockIdx.x * 64, c0 = blockIdx.y * 64;
  const size_t xb = (size_t)blockIdx.z * stride_x;
  const int cl = (threadIdx.x & 7) * 8;
  const AffineDiv dv = affine_div<XT, T>(scale);
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int rl = (threadIdx.x >> 3) + 32 * i;
    const int r = r0 + rl, c = c0 + cl;
    float e[8];
    if (r < R && c < C) load8_guard<XT>(x, xb + (size_t)r * ldx, c, C, vec, e);
#pragma unroll
    for (int j = 0; j < 8; ++j)
      tile[cl + j][rl] =
          (r < R && c + j < C) ? (uint8_t)(int)affine_code<T>(e[j], dv, offset) : (uint8_t)0;
  }
  __syncthreads();
  const int oc = threadIdx.x >> 2, chunk = threadIdx.x & 3;
  if (c0 + oc < C)
    *(uint4*)((uint8_t*)q + (size_t)blockIdx.z * stride_q + (size_t)(c0 + oc) * ldq + r0 + chunk * 16) =
        *(const uint4*)&tile[oc][chunk * 16];
}

// ------------------------------------------------------------------ e4m3, per token
// Dynamic scale from an abs-max (a value of x's dtype XT): max(amax / 448, floor), formed in
// fp32 or -- in_xt -- with quotient and floor both rounded to XT (a python-scalar clamp bound
// leaves a tensor in its dtype, so the bound acts as its rounded value).
template <int XT>
__device__ __forceinline__ float fp8_dynamic_scale(float amax, float floor_v, int in_xt) {
  if (in_xt) return fmaxf(round_to<XT>(amax / 448.0f), round_to<XT>(floor_v));
  return fmaxf(amax / 448.0f, floor_v);
}

// scale[0] <- dynamic per-tensor scale from the per-column abs-max vector (one block).
template <int XT>
__global__ __launch_bounds__(AQ_THREADS) void fp8_tensor_scale_kernel(
    const float* __restrict__ col_amax, int K, float scale_floor, int scale_in_xt,
    float* __restrict__ scale) {
  __shared__ float red[AQ_THREADS / 64];
  // NaN abs-max entries order above inf as unsigned bit patterns, like torch's amax propagates them
  uint32_t b = 0;
  for (int k = threadIdx.x; k < K; k += AQ_THREADS) b = max(b, __float_as_uint(col_amax[k]));
  b = wave_max_u32(b);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = __uint_as_float(b);
  __syncthreads();
  if (threadIdx.x == 0) {
    uint32_t m = 0;
    for (int w = 0; w < AQ_THREADS / 64; ++w) m = max(m, __float_as_uint(red[w]));
    scale[0] = fp8_dynamic_scale<XT>(__uint_as_float(m), scale_floor, scale_in_xt);
  }
}

template <int XT>
__global__ __launch_bounds__(AQ_THREADS) void quant_fp8_pertoken_kernel(
    const void* __restrict__ x, int64_t ldx, int variant, int static_scale,
    uint8_t* __restrict__ q, int64_t ldq, float* __restrict__ scale, int K, float scale_floor,
    int scale_in_xt) {
  __shared__ float red[AQ_THREADS / 64];
  const int row = blockIdx.x;
  const size_t xrow = (size_t)row * ldx;
  const int nchunk = K / AQ_VEC;
  float v[AQ_MAXCHUNK][8];
  float amax = 0.0f;
#pragma unroll
  for (int i = 0; i < AQ_MAXCHUNK; ++i) {
    const int c = threadIdx.x + i * AQ_THREADS;
    if (c < nchunk) {
      load8<XT>(x, xrow + (size_t)c * AQ_VEC, v[i]);
#pragma unroll
      for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(v[i][j]));
    }
  }
  float s;
  if (static_scale) {
    s = scale[0];
  } else {
    for (int c = threadIdx.x + AQ_MAXCHUNK * AQ_THREADS; c < nchunk; c += AQ_THREADS) {
      float e[8];
      load8<XT>(x, xrow + (size_t)c * AQ_VEC, e);
#pragma unroll
      for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(e[j]));
    }
    amax = block_max(amax, red);
    s = fp8_dynamic_scale<XT>(amax, scale_floor, scale_in_xt);
    if (threadIdx.x == 0) scale[row] = s;
  }
  auto emit = [&](int c, const float (&e)[8]) {
    uint8_t b[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      float t;
      if (variant == FMSMO_FP8_LINEAR) {
        t = fminf(fmaxf(e[j] / s, -448.0f), 448.0f);
      } else {
        t = round_to<XT>(e[j] / s);
      }
      uint8_t code = f32_to_e4m3_sw(t);
      // DL8 flush: |v| < 0.0087890625 = 4.5 * 2^-9, i.e. the subnormal codes 1..4 (k * 2^-9)
      if (variant == FMSMO_FP8_FPXACC_DL8 && (code & 0x7f) <= 0x04) code = 0x00;
      b[j] = code;
    }
    store8(q, (size_t)row * ldq + (size_t)c * AQ_VEC, b);
  };
#pragma unroll
  for (int i = 0; i < AQ_MAXCHUNK; ++i) {
    const int c = threadIdx.x + i * AQ_THREADS;
    if (c < nchunk) emit(c, v[i]);
  }
  for (int c = threadIdx.x + AQ_MAXCHUNK * AQ_THREADS; c < nchunk; c += AQ_THREADS) {
    float e[8];
    load8<XT>(x, xrow + (size_t)c * AQ_VEC, e);
    emit(c, e);
  }
}

// ------------------------------------------------------------------ e4m3, per token, 16-bit x
// Row-walking variant of the kernel above (dynamic scale, fp16 / bf16 x, K <= 16384): next row
// prefetched, packed abs-max, divisions from a refined reciprocal (fp32 quotients for the
// FP8Linear recipe, 16-bit-rounded quotients for the FPx recipe, see div32_fast / div16), and the
// hardware OCP e4m3 conversion on values clamped to +-448 (torch maps (448, 464] to 448 and
// finite rows cannot exceed that).  Rows whose maximum is inf / NaN take the IEEE + software
// encoder route of the generic kernel.
// The recipe (VAR: FMSMO_FP8_LINEAR / _FPXACC / _FPXACC_DL8) is a compile-time fact: no
// per-element variant tests, the fp16 -> fp32 widening of the FP8Linear quotient folded into its
// fmas, the clamp a single median.
template <int XT, int NCH, int VAR>
__global__ __launch_bounds__(AQ_THREADS) void quant_fp8_pertoken16_kernel(
    const u16* __restrict__ x, int64_t ldx, uint8_t* __restrict__ q, int64_t ldq,
    float* __restrict__ scale, int M, int K, float scale_floor, int scale_in_xt,
    int fixed_scale) {
  constexpr int variant = VAR;
  constexpr bool LIN = VAR == FMSMO_FP8_LINEAR;
  __shared__ float red[2][AQ_THREADS / 64];
  const int nchunk = K / AQ_VEC;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  constexpr uint32_t INF_BITS = XT == FMSMO_F16 ? 0x7c00u : 0x7f80u;
  // fixed_scale: one scale for every row, read from scale[0] (nothing is written there); the row
  // maximum still decides between the fast quotients and the IEEE route of non-finite rows
  const float s_fixed = fixed_scale ? scale[0] : 0.0f;

  v4i cur[NCH], nxt[NCH];
  auto load_row = [&](int row, v4i (&dst)[NCH]) {
    const u16* xr = x + (size_t)row * ldx;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int c = threadIdx.x + i * AQ_THREADS;
      if (c < nchunk) dst[i] = __builtin_nontemporal_load((const v4i*)(xr + (size_t)c * AQ_VEC));
    }
  };
  int parity = 0;
  int row = blockIdx.x;
  if (row < M) load_row(row, cur);
  for (; row < M; row += gridDim.x) {
    const int nrow = row + gridDim.x;
    if (nrow < M) load_row(nrow, nxt);

    us2 amax2 = {0, 0};
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int c = threadIdx.x + i * AQ_THREADS;
      if (c < nchunk) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint32_t mag = (uint32_t)cur[i][j] & 0x7fff7fffu;
          us2 m2;
          __builtin_memcpy(&m2, &mag, 4);
          amax2 = __builtin_elementwise_max(amax2, m2);
        }
      }
    }
    const uint32_t v = wave_max_u32((uint32_t)(amax2[0] > amax2[1] ? amax2[0] : amax2[1]));
    float* rb = red[parity];
    parity ^= 1;
    if (lane == 0) rb[wave] = __uint_as_float(v);
    __syncthreads();
    const uint32_t abits = max(max(__float_as_uint(rb[0]), __float_as_uint(rb[1])),
                               max(__float_as_uint(rb[2]), __float_as_uint(rb[3])));
    const float amax = cvt16<XT>((u16)abits);

    float s = s_fixed;
    if (!fixed_scale) {
      s = fp8_dynamic_scale<XT>(amax, scale_floor, scale_in_xt);
      if (threadIdx.x == 0) scale[row] = s;
    }
    uint8_t* qr = q + (size_t)row * ldq;

    // a fixed scale outside the range where the refined reciprocal is exact takes the IEEE route
    const bool fast = abits < INF_BITS &&
                      (!fixed_scale || (s >= 0x1p-60f && s <= 0x1p60f && amax <= s * 0x1p100f));
    if (fast) {
      const float r1 = rcp_refined(s);
      [[maybe_unused]] const float nz = opaque_neg_zero();
#pragma unroll
      for (int i = 0; i < NCH; ++i) {
        const int c = threadIdx.x + i * AQ_THREADS;
        if (c < nchunk) {
          float t[8];
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const float xv = cvt16<XT>((u16)((uint32_t)cur[i][j >> 1] >> ((j & 1) * 16)));
            if constexpr (LIN) {
              // (the row is finite here, so the median of three is the clamp)
              if constexpr (XT == FMSMO_F16) t[j] = div32_fast_mix(xv, s, r1, nz);
              else t[j] = div32_fast(xv, s, r1);
              t[j] = __builtin_copysignf(__builtin_amdgcn_fmed3f(t[j], -448.0f, 448.0f), xv);
            } else {
              t[j] = cvt16<XT>(to16<XT>(div16<XT, false>(xv, s, r1)));
              // the residual corrections lose the sign of a zero quotient; s > 0
              t[j] = __builtin_copysignf(__builtin_amdgcn_fmed3f(t[j], -448.0f, 448.0f), xv);
              // DL8: the codes 1..4 (|t| up to the tie 4.5 * 2^-9, which rounds to code 4) flush to +0
              if constexpr (VAR == FMSMO_FP8_FPXACC_DL8) t[j] = fabsf(t[j]) <= 0.0087890625f ? 0.0f : t[j];
            }
          }
          int o0 = 0, o1 = 0;
          o0 = __builtin_amdgcn_cvt_pk_fp8_f32(t[0], t[1], o0, false);
          o0 = __builtin_amdgcn_cvt_pk_fp8_f32(t[2], t[3], o0, true);
          o1 = __builtin_amdgcn_cvt_pk_fp8_f32(t[4], t[5], o1, false);
          o1 = __builtin_amdgcn_cvt_pk_fp8_f32(t[6], t[7], o1, true);
          *(uint2*)(qr + (size_t)c * AQ_VEC) = make_uint2((uint32_t)o0, (uint32_t)o1);
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < NCH; ++i) {
        const int c = threadIdx.x + i * AQ_THREADS;
        if (c < nchunk) {
          uint8_t b[8];
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const float xv = cvt16<XT>((u16)((uint32_t)cur[i][j >> 1] >> ((j & 1) * 16)));
            float t;
            if (variant == FMSMO_FP8_LINEAR) t = fminf(fmaxf(xv / s, -448.0f), 448.0f);
            else t = round_to<XT>(xv / s);
            uint8_t code = f32_to_e4m3_sw(t);
            if (variant == FMSMO_FP8_FPXACC_DL8 && (code & 0x7f) <= 0x04) code = 0x00;
            b[j] = code;
          }
          store8(qr, (size_t)c * AQ_VEC, b);
        }
      }
    }
#pragma unroll
    for (int i = 0; i < NCH; ++i) cur[i] = nxt[i];
  }
}

}  // namespace fmsmo

using namespace fmsmo;

extern thread_local char g_fmsmo_last_error[256];
int fmsmo_check_launch();

static bool aligned16(const void* p) { return (((uintptr_t)p) & 15) == 0; }

// Blocks of AQ_THREADS threads the current device keeps resident for a row-walking kernel (its
// grid size); asked of the runtime once per kernel and device.
static int64_t resident_blocks(const void* kernel, int threads = AQ_THREADS) {
  struct Entry { const void* k; int dev; int64_t n; };
  static thread_local Entry cache[64];
  static thread_local int used = 0;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) dev = 0;
  for (int i = 0; i < used; ++i)
    if (cache[i].k == kernel && cache[i].dev == dev) return cache[i].n;
  int per_cu = 0, cus = 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, threads, 0) != hipSuccess || per_cu < 1)
    per_cu = 2;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 1)
    cus = 256;
  const int64_t n = (int64_t)per_cu * cus;
  if (used < 64) cache[used++] = Entry{kernel, dev, n};
  return n;
}

// Grid of a row-walking kernel.  Blocks that keep nothing across rows run one row each and leave
// the order to the dispatcher (measured 2 ... 18 % faster than a resident grid that walks the rows:
// a resident grid is rarely a divisor of the row count, and its last turn runs part-filled); blocks
// with a set-up worth keeping -- checked bf16 divisors, refined fp32 reciprocals, the longest
// rows -- stay resident and walk.
static int64_t row_walk_grid(int64_t M, int64_t resident, bool one_row_per_block) {
  return one_row_per_block || M < resident ? M : resident;
}

extern "C" int fmsmo_quant_act_i8_pertoken(const void* x, int x_dtype, int64_t ldx,
                                           const void* smooth, int smooth_dtype,
                                           int compute_dtype, int saturate, int8_t* q, int64_t ldq,
                                           float* scale, int64_t M, int64_t K,
                                           fmsmo_stream_t stream) {
  if (!x || !q || !scale) return FMSMO_ERR_NULL;
  if (M < 0 || K <= 0 || ldx < K || ldq < K || M > 0x7fffffff || K > 0x7fffffff) return FMSMO_ERR_SHAPE;
  if (x_dtype < 0 || x_dtype > 2 || compute_dtype < 0 || compute_dtype > 2) return FMSMO_ERR_UNSUPPORTED;
  if (smooth && (smooth_dtype < 0 || smooth_dtype > 2)) return FMSMO_ERR_UNSUPPORTED;
  if (K % 8 || ldx % 8 || ldq % 8 || !aligned16(x) || (((uintptr_t)q) & 7)) return FMSMO_ERR_ALIGN;
  if (smooth && !aligned16(smooth)) return FMSMO_ERR_ALIGN;
  if (M == 0) return FMSMO_OK;
  hipStream_t st = (hipStream_t)stream;
  // 16-bit fast path: x, the divisor and the compute dtype all fp16 (or all bf16), row cached in
  // registers (K <= 32768)
  if (x_dtype != FMSMO_F32 && compute_dtype == x_dtype && (!smooth || smooth_dtype == x_dtype) &&
      K <= 2 * AQ_MAXCHUNK * AQ_THREADS * AQ_VEC) {
    const int64_t per_thread = div_up(K, AQ_THREADS * AQ_VEC);
    const int nch = per_thread <= 1 ? 1 : per_thread <= 2 ? 2 : per_thread <= 4 ? 4 : per_thread <= 8 ? 8 : 16;
    // rows longer than 8192 elements: 512-thread blocks with 4 chunks per thread (more, shorter
    // lanes: 45 vs 49 us at K = 14336 with the SmoothQuant divide, 34 vs 38 us without)
#define LAUNCH16(T, NCH, SM, TH, KEEP)                                                           \
  {                                                                                              \
    const int64_t resident =                                                                     \
        resident_blocks((const void*)quant_i8_pertoken16_kernel<T, NCH, SM, TH, KEEP>, TH);      \
    dim3 grid16((unsigned)row_walk_grid(M, resident, !(SM) || (T == FMSMO_F16 && NCH <= 4))),    \
        block16(TH);                                                                             \
    hipLaunchKernelGGL((quant_i8_pertoken16_kernel<T, NCH, SM, TH, KEEP>), grid16, block16, 0,   \
                       st, (const u16*)x, ldx, (const u16*)smooth, saturate, q, ldq, scale,      \
                       (int)M, (int)K);                                                          \
  }
    // divisors with rows of up to 8192 elements: fp16 blocks run one row each and keep nothing;
    // bf16 blocks (costlier reciprocals, checked divisors) keep theirs across rows once they walk
    // several, i.e. beyond the resident grid
#define SMOOTH16(T, NCH)                                                                         \
  if (T == FMSMO_F16 ||                                                                          \
      M <= resident_blocks((const void*)quant_i8_pertoken16_kernel<T, NCH, true, 256, false>, 256)) \
    LAUNCH16(T, NCH, true, 256, false)                                                           \
  else                                                                                           \
    LAUNCH16(T, NCH, true, 256, true)
#define PICK16(T)                                                                                        \
  switch (nch * 2 + (smooth ? 1 : 0)) {                                                                  \
    case 2: LAUNCH16(T, 1, false, 256, true); break;  case 3: SMOOTH16(T, 1); break;   \
    case 4: LAUNCH16(T, 2, false, 256, true); break;  case 5: SMOOTH16(T, 2); break;   \
    case 8: LAUNCH16(T, 4, false, 256, true); break;  case 9: SMOOTH16(T, 4); break;   \
    case 16: LAUNCH16(T, 4, false, 512, true); break; case 17: LAUNCH16(T, 4, true, 512, false); break; \
    case 32: LAUNCH16(T, 8, false, 512, true); break;                                                   \
    default: LAUNCH16(T, 8, true, 512, false); break; /* 16384 < K <= 32768 */                          \
  }
    if (x_dtype == FMSMO_F16) { PICK16(FMSMO_F16) } else { PICK16(FMSMO_BF16) }
#undef PICK16
#undef SMOOTH16
#undef LAUNCH16
    return fmsmo_check_launch();
  }
  // fp16 / bf16 x promoted to fp32 by an fp32 SmoothQuant scale
  if (x_dtype != FMSMO_F32 && smooth && smooth_dtype == FMSMO_F32 && compute_dtype == FMSMO_F32 &&
      K <= AQ_MAXCHUNK * AQ_THREADS * AQ_VEC) {
    const int64_t per_thread = div_up(K, AQ_THREADS * AQ_VEC);
#define LAUNCH32(NCH, KEEP, TH)                                                                   \
  {                                                                                               \
    if (x_dtype == FMSMO_F16) {                                                                   \
      const int64_t resident =                                                                    \
          resident_blocks((const void*)quant_i8_pertoken_f16x_f32s_kernel<NCH, KEEP, TH>, TH);    \
      dim3 grid32((unsigned)row_walk_grid(M, resident, false)), block32(TH);                      \
      hipLaunchKernelGGL((quant_i8_pertoken_f16x_f32s_kernel<NCH, KEEP, TH>), grid32, block32, 0, \
                         st, (const u16*)x, ldx, (const float*)smooth, saturate, q, ldq, scale,   \
                         (int)M, (int)K);                                                         \
    } else {                                                                                      \
      const int64_t resident = resident_blocks(                                                   \
          (const void*)quant_i8_pertoken_f16x_f32s_kernel<NCH, KEEP, TH, FMSMO_BF16>, TH);        \
      dim3 grid32((unsigned)row_walk_grid(M, resident, false)), block32(TH);                      \
      hipLaunchKernelGGL((quant_i8_pertoken_f16x_f32s_kernel<NCH, KEEP, TH, FMSMO_BF16>), grid32, \
                         block32, 0, st, (const u16*)x, ldx, (const float*)smooth, saturate, q,   \
                         ldq, scale, (int)M, (int)K);                                             \
    }                                                                                             \
  }
    if (per_thread <= 1) LAUNCH32(1, true, 256)
    else if (per_thread <= 2) LAUNCH32(2, true, 256)
    else if (per_thread <= 4) LAUNCH32(4, false, 256)
    else LAUNCH32(4, false, 512)
#undef LAUNCH32
    return fmsmo_check_launch();
  }
  dim3 grid((unsigned)M), block(AQ_THREADS);
#define LAUNCH(XT, T)                                                                          \
  hipLaunchKernelGGL((quant_i8_pertoken_kernel<XT, T>), grid, block, 0, st, x, ldx, smooth,    \
                     smooth_dtype, saturate, q, ldq, scale, (int)K)
#define DISPATCH_T(XT)                                                      \
  switch (compute_dtype) {                                                  \
    case FMSMO_F16: LAUNCH(XT, FMSMO_F16); break;                           \
    case FMSMO_BF16: LAUNCH(XT, FMSMO_BF16); break;                         \
    default: LAUNCH(XT, FMSMO_F32); break;                                  \
  }
  switch (x_dtype) {
    case FMSMO_F16: DISPATCH_T(FMSMO_F16); break;
    case FMSMO_BF16: DISPATCH_T(FMSMO_BF16); break;
    default: DISPATCH_T(FMSMO_F32); break;
  }
#undef LAUNCH
#undef DISPATCH_T
  return fmsmo_check_launch();
}

extern "C" int fmsmo_quant_act_i8_static(const void* x, int x_dtype, int64_t ldx, float scale,
                                         int zp, int sym, int8_t* q, int64_t ldq, int64_t M,
                                         int64_t K, fmsmo_stream_t stream) {
  if (!x || !q) return FMSMO_ERR_NULL;
  if (M < 0 || K <= 0 || ldx < K || ldq < K || M > 0x7fffffff || K > 0x7fffffff) return FMSMO_ERR_SHAPE;
  if (x_dtype < 0 || x_dtype > 2) return FMSMO_ERR_UNSUPPORTED;
  if (K % 8 || ldx % 8 || ldq % 8 || !aligned16(x) || (((uintptr_t)q) & 7)) return FMSMO_ERR_ALIGN;
  if (M == 0) return FMSMO_OK;
  hipStream_t st = (hipStream_t)stream;
  dim3 grid((unsigned)M), block(AQ_THREADS);
#define LAUNCH(XT)                                                                           \
  hipLaunchKernelGGL((quant_i8_static_kernel<XT>), grid, block, 0, st, x, ldx, scale,        \
                     (float)zp, (float)(sym & 1), (sym >> 1) & 1, q, ldq, (int)K)
  switch (x_dtype) {
    case FMSMO_F16: LAUNCH(FMSMO_F16); break;
    case FMSMO_BF16: LAUNCH(FMSMO_BF16); break;
    default: LAUNCH(FMSMO_F32); break;
  }
#undef LAUNCH
  return fmsmo_check_launch();
}

extern "C" int fmsmo_quant_act_i8_mulscale(const void* x, int x_dtype, int64_t ldx,
                                           const void* smooth, const void* clip, int meta_dtype,
                                           int compute_dtype, int mode, int8_t* q, int64_t ldq,
                                           float* a_scale, int64_t M, int64_t K,
                                           fmsmo_stream_t stream) {
  if (!x || !q || !a_scale) return FMSMO_ERR_NULL;
  if (mode < 0 || mode > 2) return FMSMO_ERR_UNSUPPORTED;
  if (mode != 0 && !clip) return FMSMO_ERR_NULL;
  if (M < 0 || K <= 0 || ldx < K || ldq < K || M > 0x7fffffff || K > 0x7fffffff) return FMSMO_ERR_SHAPE;
  if (x_dtype < 0 || x_dtype > 2 || meta_dtype < 0 || meta_dtype > 2 || compute_dtype < 0 ||
      compute_dtype > 2)
    return FMSMO_ERR_UNSUPPORTED;
  // the compute dtype is the promotion of x's and the metadata's dtype, as torch would choose it
  if (compute_dtype != FMSMO_F32 && compute_dtype != x_dtype) return FMSMO_ERR_UNSUPPORTED;
  if (K % 8 || ldx % 8 || ldq % 8 || !aligned16(x) || (((uintptr_t)q) & 7) ||
      (smooth && !aligned16(smooth)))
    return FMSMO_ERR_ALIGN;
  if (M == 0) return FMSMO_OK;
  hipStream_t st = (hipStream_t)stream;
  // 16-bit fast path: x, the metadata and the compute dtype all fp16 (or all bf16)
  if (x_dtype != FMSMO_F32 && compute_dtype == x_dtype && meta_dtype == x_dtype &&
      K <= 2 * AQ_MAXCHUNK * AQ_THREADS * AQ_VEC) {
    const int64_t per_thread = div_up(K, AQ_THREADS * AQ_VEC);
    const int nch = per_thread <= 1 ? 1 : per_thread <= 2 ? 2 : per_thread <= 4 ? 4 : per_thread <= 8 ? 8 : 16;
#define LAUNCH16M(T, MD, NCH, SM, TH, KEEP)                                                      \
  {                                                                                              \
    const int64_t resident =                                                                     \
        resident_blocks((const void*)quant_i8_mulscale16_kernel<T, MD, NCH, SM, TH, KEEP>, TH);  \
    dim3 grid16((unsigned)row_walk_grid(M, resident, (SM) ? (T == FMSMO_F16 && NCH <= 4)         \
                                                          : TH == 256)),                         \
        block16(TH);                                                                             \
    hipLaunchKernelGGL((quant_i8_mulscale16_kernel<T, MD, NCH, SM, TH, KEEP>), grid16, block16,  \
                       0, st, (const u16*)x, ldx, (const u16*)smooth, (const u16*)clip, q, ldq,  \
                       a_scale, (int)M, (int)K);                                                 \
  }
#define LAUNCH16(T, NCH, SM, TH, KEEP)                    \
  if (mode == 0) LAUNCH16M(T, 0, NCH, SM, TH, KEEP)       \
  else if (mode == 1) LAUNCH16M(T, 1, NCH, SM, TH, KEEP)  \
  else LAUNCH16M(T, 2, NCH, SM, TH, KEEP)
    // (as in fmsmo_quant_act_i8_pertoken: fp16 blocks keep nothing, bf16 blocks keep their
    // reciprocals once they walk several rows)
#define SMOOTH16(T, NCH)                                                                         \
  if (T == FMSMO_F16 ||                                                                          \
      M <= resident_blocks((const void*)quant_i8_mulscale16_kernel<T, 0, NCH, true, 256, false>, 256)) \
    LAUNCH16(T, NCH, true, 256, false)                                                           \
  else                                                                                           \
    LAUNCH16(T, NCH, true, 256, true)
#define PICK16(T)                                                                                        \
  switch (nch * 2 + (smooth ? 1 : 0)) {                                                                  \
    case 2: LAUNCH16(T, 1, false, 256, true); break;  case 3: SMOOTH16(T, 1); break;   \
    case 4: LAUNCH16(T, 2, false, 256, true); break;  case 5: SMOOTH16(T, 2); break;   \
    case 8: LAUNCH16(T, 4, false, 256, true); break;  case 9: SMOOTH16(T, 4); break;   \
    case 16: LAUNCH16(T, 4, false, 512, true); break; case 17: LAUNCH16(T, 4, true, 512, false); break; \
    case 32: LAUNCH16(T, 8, false, 512, true); break;                                                   \
    default: LAUNCH16(T, 8, true, 512, false); break; /* 16384 < K <= 32768 */                          \
  }
    if (x_dtype == FMSMO_F16) { PICK16(FMSMO_F16) } else { PICK16(FMSMO_BF16) }
#undef PICK16
#undef SMOOTH16
#undef LAUNCH16
#undef LAUNCH16M
    return fmsmo_check_launch();
  }
  dim3 grid((unsigned)M), block(AQ_THREADS);
#define LAUNCH(XT, T)                                                                        \
  hipLaunchKernelGGL((quant_i8_mulscale_kernel<XT, T>), grid, block, 0, st, x, ldx, smooth,  \
                     clip, meta_dtype, mode, q, ldq, a_scale, (int)K)
  if (compute_dtype == FMSMO_F32) {
    switch (x_dtype) {
      case FMSMO_F16: LAUNCH(FMSMO_F16, FMSMO_F32); break;
      case FMSMO_BF16: LAUNCH(FMSMO_BF16, FMSMO_F32); break;
      default: LAUNCH(FMSMO_F32, FMSMO_F32); break;
    }
  } else if (x_dtype == FMSMO_F16) {
    LAUNCH(FMSMO_F16, FMSMO_F16);
  } else {
    LAUNCH(FMSMO_BF16, FMSMO_BF16);
  }
#undef LAUNCH
  return fmsmo_check_launch();
}

extern "C" int fmsmo_quant_i8_affine(const void* x, int x_dtype, int64_t ldx, int64_t stride_x,
                                     float scale, float offset, int compute_dtype, int transpose,
                                     int8_t* q, int64_t ldq, int64_t stride_q, int64_t batch,
                                     int64_t R, int64_t C, fmsmo_stream_t stream) {
  if (!x || !q) return FMSMO_ERR_NULL;
  if (batch <= 0 || R <= 0 || C <= 0 || ldx < C || batch > 65535 || R > 0x7fffffff ||
      C > 0x7fffffff || stride_x < 0 || stride_q < 0)
    return FMSMO_ERR_SHAPE;
  if (x_dtype < 0 || x_dtype > 2 || compute_dtype < 0 || compute_dtype > 2) return FMSMO_ERR_UNSUPPORTED;
  if (compute_dtype != FMSMO_F32 && compute_dtype != x_dtype) return FMSMO_ERR_UNSUPPORTED;
  if (transpose) {
    if (ldq < R || ldq % 64 || stride_q % 16 || !aligned16(q)) return FMSMO_ERR_ALIGN;
    if (C > 65535 * 64ll) return FMSMO_ERR_SHAPE;
  } else {
    if (ldq < C || ldq % 8 || stride_q % 8 || (((uintptr_t)q) & 7)) return FMSMO_ERR_ALIGN;
    if (ldq > 0x7fffffff) return FMSMO_ERR_SHAPE;
  }
  const int esz = x_dtype == FMSMO_F32 ? 4 : 2;
  const bool vec = aligned16(x) && (ldx * esz) % 16 == 0 && (stride_x * esz) % 16 == 0;
  hipStream_t st = (hipStream_t)stream;
#define LAUNCH(XT, T)                                                                          \
  if (transpose)                                                                               \
    hipLaunchKernelGGL((quant_i8_affine_t_kernel<XT, T>),                                      \
                       dim3((unsigned)(ldq / 64), (unsigned)div_up(C, 64), (unsigned)batch),   \
                       dim3(256), 0, st, x, ldx, stride_x, scale, offset, vec, q, ldq,         \
                       stride_q, (int)R, (int)C);                                              \
  else                                                                                         \
    hipLaunchKernelGGL((quant_i8_affine_kernel<XT, T>), dim3((unsigned)R, (unsigned)batch),    \
                       dim3(AQ_THREADS), 0, st, x, ldx, stride_x, scale, offset, vec, q, ldq,  \
                       stride_q, (int)C)
  if (compute_dtype == FMSMO_F32) {
    switch (x_dtype) {
      case FMSMO_F16: LAUNCH(FMSMO_F16, FMSMO_F32); break;
      case FMSMO_BF16: LAUNCH(FMSMO_BF16, FMSMO_F32); break;
      default: LAUNCH(FMSMO_F32, FMSMO_F32); break;
    }
  } else if (x_dtype == FMSMO_F16) {
    LAUNCH(FMSMO_F16, FMSMO_F16);
  } else {
    LAUNCH(FMSMO_BF16, FMSMO_BF16);
  }
#undef LAUNCH
  return fmsmo_check_launch();
}

// Shared launcher of the e4m3 quantizer entry points.  scale_mode: 0 one dynamic scale per row
// (written to scale[M]); 1 scale[0] given by the caller, any value; 2 scale[0] is a dynamic
// per-tensor scale that fp8_tensor_scale_kernel has left there (a value the variant's own rule
// produces from the tensor's abs-max, so no quotient exceeds the e4m3 range).
static int launch_quant_fp8(const void* x, int x_dtype, int64_t ldx, int variant, int scale_mode,
                            float scale_floor, int scale_in_xt, uint8_t* q, int64_t ldq,
                            float* scale, int64_t M, int64_t K, hipStream_t st) {
  // the row-walking kernel clamps to +-448 before the hardware conversion: right for the
  // FP8Linear recipe with any scale, and for the unclamped FPx recipe when the scale comes from
  // the data's own maximum
  const bool walk_ok = scale_mode == 0 || scale_mode == 2 || variant == FMSMO_FP8_LINEAR;
  if (x_dtype != FMSMO_F32 && walk_ok && K <= AQ_MAXCHUNK * AQ_THREADS * AQ_VEC) {
    const int64_t per_thread = div_up(K, AQ_THREADS * AQ_VEC);
    dim3 block16(AQ_THREADS);
#define LAUNCH8V(XT, NCH, VAR)                                                                    \
  hipLaunchKernelGGL((quant_fp8_pertoken16_kernel<XT, NCH, VAR>), grid16, block16, 0, st,         \
                     (const u16*)x, ldx, q, ldq, scale, (int)M, (int)K, scale_floor, scale_in_xt, \
                     scale_mode != 0);
#define LAUNCH8(XT, NCH)                                                                          \
  {                                                                                               \
    dim3 grid16((unsigned)M); /* one row per block: see row_walk_grid */                          \
    if (variant == FMSMO_FP8_LINEAR) LAUNCH8V(XT, NCH, FMSMO_FP8_LINEAR)                          \
    else if (variant == FMSMO_FP8_FPXACC) LAUNCH8V(XT, NCH, FMSMO_FP8_FPXACC)                     \
    else LAUNCH8V(XT, NCH, FMSMO_FP8_FPXACC_DL8)                                                  \
  }
#define PICK8(XT)                                  \
  if (per_thread <= 1) LAUNCH8(XT, 1)              \
  else if (per_thread <= 2) LAUNCH8(XT, 2)         \
  else if (per_thread <= 4) LAUNCH8(XT, 4)         \
  else LAUNCH8(XT, 8)
    if (x_dtype == FMSMO_F16) { PICK8(FMSMO_F16) } else { PICK8(FMSMO_BF16) }
#undef PICK8
#undef LAUNCH8
#undef LAUNCH8V
    return fmsmo_check_launch();
  }
  dim3 grid((unsigned)M), block(AQ_THREADS);
#define LAUNCH(XT)                                                                             \
  hipLaunchKernelGGL((quant_fp8_pertoken_kernel<XT>), grid, block, 0, st, x, ldx, variant,     \
                     (int)(scale_mode != 0), q, ldq, scale, (int)K, scale_floor, scale_in_xt)
  switch (x_dtype) {
    case FMSMO_F16: LAUNCH(FMSMO_F16); break;
    case FMSMO_BF16: LAUNCH(FMSMO_BF16); break;
    default: LAUNCH(FMSMO_F32); break;
  }
#undef LAUNCH
  return fmsmo_check_launch();
}

static int check_quant_fp8(const void* x, int x_dtype, int64_t ldx, int variant, const uint8_t* q,
                           int64_t ldq, const float* scale, int64_t M, int64_t K) {
  if (!x || !q || !scale) return FMSMO_ERR_NULL;
  if (M < 0 || K <= 0 || ldx < K || ldq < K || M > 0x7fffffff || K > 0x7fffffff) return FMSMO_ERR_SHAPE;
  if (x_dtype < 0 || x_dtype > 2 || variant < 0 || variant > 2) return FMSMO_ERR_UNSUPPORTED;
  if (K % 8 || ldx % 8 || ldq % 8 || !aligned16(x) || (((uintptr_t)q) & 7)) return FMSMO_ERR_ALIGN;
  return FMSMO_OK;
}

extern "C" int fmsmo_quant_act_fp8_pertoken(const void* x, int x_dtype, int64_t ldx, int variant,
                                            int static_scale, uint8_t* q, int64_t ldq,
                                            float* scale, int64_t M, int64_t K,
                                            fmsmo_stream_t stream) {
  if (const int e = check_quant_fp8(x, x_dtype, ldx, variant, q, ldq, scale, M, K)) return e;
  if (M == 0) return FMSMO_OK;
  // the rule each variant's reference states: fp32 amax / 448 floored at 1e-12 for the FP8Linear
  // recipe, the quotient in x's dtype floored at 1e-5 for the FPx recipes
  const bool lin = variant == FMSMO_FP8_LINEAR;
  return launch_quant_fp8(x, x_dtype, ldx, variant, static_scale ? 1 : 0, lin ? 1e-12f : 1e-5f,
                          lin ? 0 : 1, q, ldq, scale, M, K, (hipStream_t)stream);
}

extern "C" int fmsmo_quant_act_fp8_dynamic(const void* x, int x_dtype, int64_t ldx, int variant,
                                           int per_tensor, const float* col_amax,
                                           float scale_floor, int scale_dtype, uint8_t* q,
                                           int64_t ldq, float* scale, int64_t M, int64_t K,
                                           fmsmo_stream_t stream) {
  if (const int e = check_quant_fp8(x, x_dtype, ldx, variant, q, ldq, scale, M, K)) return e;
  if (per_tensor && !col_amax) return FMSMO_ERR_NULL;
  if (scale_dtype != FMSMO_F32 && scale_dtype != x_dtype) return FMSMO_ERR_UNSUPPORTED;
  if (!(scale_floor > 0.0f) || !(scale_floor < 0x1p60f)) return FMSMO_ERR_UNSUPPORTED;
  // a floor that rounds to zero in x's dtype would let a zero row divide by zero
  if (scale_dtype == FMSMO_F16 && scale_floor <= 0x1p-25f) return FMSMO_ERR_UNSUPPORTED;
  if (scale_dtype == FMSMO_BF16 && scale_floor < 0x1p-126f) return FMSMO_ERR_UNSUPPORTED;
  if (M == 0) return FMSMO_OK;
  hipStream_t st = (hipStream_t)stream;
  const int in_xt = scale_dtype != FMSMO_F32;
  if (per_tensor) {
#define LAUNCH(XT)                                                                            \
  hipLaunchKernelGGL((fp8_tensor_scale_kernel<XT>), dim3(1), dim3(AQ_THREADS), 0, st, col_amax, \
                     (int)K, scale_floor, in_xt, scale)
    switch (x_dtype) {
      case FMSMO_F16: LAUNCH(FMSMO_F16); break;
      case FMSMO_BF16: LAUNCH(FMSMO_BF16); break;
      default: LAUNCH(FMSMO_F32); break;
    }
#undef LAUNCH
  }
  return launch_quant_fp8(x, x_dtype, ldx, variant, per_tensor ? 2 : 0, scale_floor, in_xt, q, ldq,
                          scale, M, K, st);
}
