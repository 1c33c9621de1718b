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
#include "quant_math.hpp"

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
  int epi;  // FMSMO_EPI_*
  void* y;
  int y_dtype;
  int64_t ldy;
  // fused decode linear: the activations arrive unquantized (fp16 / bf16) and every block
  // quantizes them itself
  const u16* x16;       // [M,K]
  int64_t ldx;
  const u16* smooth;    // [K] SmoothQuant divisors of x's dtype (fp32 when smooth_f32), or NULL
  int smooth_f32;
  int saturate;
  float* a_scale_out;   // [M] per-token scales (written by block 0), or NULL
};

// Per-token int8 quantization of up to MAXM token rows by all NT threads of a block, into LDS:
// the arithmetic of the stand-alone quantizer for a 16-bit compute dtype T (divide by the
// SmoothQuant scale, row maximum, s = rnd_T(max(amax, rnd_T(1e-5)) / 127), rint(rnd_T(x / s)),
// exact quotients from reciprocals, rows or divisors outside the fast path's range redone with
// IEEE divisions).  A decode step has a handful of tokens: quantizing them again in every block
// costs a few KB of L2 reads and saves a kernel launch in front of every linear layer.
template <int T, int NT, int KMAX, int MAXM>
__device__ __forceinline__ void quantize_rows_to_lds(const GemvArgs& g, uint8_t (*xq)[KMAX], float* sc,
                                                     float* red) {
  constexpr int NCH = (KMAX / AQ_VEC + NT - 1) / NT;
  const int nchunk = g.K / AQ_VEC;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  constexpr uint32_t INF_BITS = T == FMSMO_F16 ? 0x7c00u : 0x7f80u;
  const float floor_T = cvt16<T>(to16<T>(1e-5f));
  const float sat_hi = g.saturate ? 127.0f : 3.0e38f;
  for (int m = 0; m < g.M; ++m) {
    const u16* xr = g.x16 + (size_t)m * g.ldx;
    v4i cur[NCH];
    int bad = 0;
    us2 amax2 = {0, 0};
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int c = threadIdx.x + i * NT;
      if (c < nchunk) {
        cur[i] = *(const v4i*)(xr + (size_t)c * AQ_VEC);
        if (g.smooth) {
          const v4i sm = *(const v4i*)(g.smooth + (size_t)c * AQ_VEC);
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const uint32_t w = (uint32_t)cur[i][j], d = (uint32_t)sm[j];
            const float dl = cvt16<T>((u16)(d & 0xffff)), dh = cvt16<T>((u16)(d >> 16));
            if constexpr (T == FMSMO_BF16)
              bad |= !(fabsf(dl) >= 8.6736174e-19f && fabsf(dl) <= 1.1529215e18f) ||
                     !(fabsf(dh) >= 8.6736174e-19f && fabsf(dh) <= 1.1529215e18f);
            const u16 el = to16<T>(div16<T, false>(cvt16<T>((u16)(w & 0xffff)), dl, __builtin_amdgcn_rcpf(dl)));
            const u16 eh = to16<T>(div16<T, false>(cvt16<T>((u16)(w >> 16)), dh, __builtin_amdgcn_rcpf(dh)));
            cur[i][j] = (int)((uint32_t)el | ((uint32_t)eh << 16));
          }
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint32_t mag = (uint32_t)cur[i][j] & 0x7fff7fffu;
          us2 m2;
          __builtin_memcpy(&m2, &mag, 4);
          amax2 = __builtin_elementwise_max(amax2, m2);
        }
      }
    }
    // non-negative floats order like their bit patterns (a NaN outranks inf)
    // (a divisor outside the fast path's range marks the row for the IEEE routine)
    float v = wave_max(__uint_as_float(bad ? 0xffffu : (uint32_t)(amax2[0] > amax2[1] ? amax2[0] : amax2[1])));
    if (lane == 0) red[wave] = v;
    __syncthreads();
    v = red[0];
#pragma unroll
    for (int w = 1; w < NT / 64; ++w) v = fmaxf(v, red[w]);
    __syncthreads();
    const uint32_t abits = __float_as_uint(v);
    if (abits >= INF_BITS) {
      quant_i8_row_ieee16<T, NT>(xr, g.smooth, g.saturate, (int8_t*)xq[m], sc + m, g.K, red);
      continue;
    }
    const float s = cvt16<T>(to16<T>(fmaxf(cvt16<T>((u16)abits), floor_T) / 127.0f));
    const float rs = __builtin_amdgcn_rcpf(s);
    if (threadIdx.x == 0) sc[m] = s;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int c = threadIdx.x + i * NT;
      if (c < nchunk) {
        uint32_t code[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint32_t w = (uint32_t)cur[i][j];
          float ql = div16<T, false>(cvt16<T>((u16)(w & 0xffff)), s, rs);
          float qh = div16<T, false>(cvt16<T>((u16)(w >> 16)), s, rs);
          if (g.saturate) {
            ql = fminf(fmaxf(ql, -sat_hi), sat_hi);
            qh = fminf(fmaxf(qh, -sat_hi), sat_hi);
          }
          code[j] = rint_codes<T>(to16<T>(ql), to16<T>(qh));
        }
        const uint32_t o0 = __builtin_amdgcn_perm(code[1], code[0], 0x06040200u);
        const uint32_t o1 = __builtin_amdgcn_perm(code[3], code[2], 0x06040200u);
        *(uint2*)(&xq[m][(size_t)c * AQ_VEC]) = make_uint2(o0, o1);
      }
    }
  }
  __syncthreads();
  if (blockIdx.x == 0 && g.a_scale_out && threadIdx.x < g.M) g.a_scale_out[threadIdx.x] = sc[threadIdx.x];
}

// The FP8Linear recipe for one token row by all NT threads of a block, into LDS:
// s = max(amax / 448, 1e-12) in fp32, q = e4m3( clamp(f32(x) / s, -448, 448) ), IEEE divisions
// (a row is a few thousand elements); rows whose maximum is inf / NaN use the software encoder,
// like the stand-alone quantizer.
template <int XT, int NT, int KMAX>
__device__ __forceinline__ void quantize_row_fp8_to_lds(const GemvArgs& g, uint8_t (*xq)[KMAX], float* sc,
                                                        float* red) {
  constexpr int NCH = (KMAX / AQ_VEC + NT - 1) / NT;
  const int nchunk = g.K / AQ_VEC;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  constexpr uint32_t INF_BITS = XT == FMSMO_F16 ? 0x7c00u : 0x7f80u;
  v4i cur[NCH];
  us2 amax2 = {0, 0};
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = threadIdx.x + i * NT;
    if (c < nchunk) {
      cur[i] = *(const v4i*)(g.x16 + (size_t)c * AQ_VEC);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t mag = (uint32_t)cur[i][j] & 0x7fff7fffu;
        us2 m2;
        __builtin_memcpy(&m2, &mag, 4);
        amax2 = __builtin_elementwise_max(amax2, m2);
      }
    }
  }
  float v = wave_max(__uint_as_float((uint32_t)(amax2[0] > amax2[1] ? amax2[0] : amax2[1])));
  if (lane == 0) red[wave] = v;
  __syncthreads();
  v = red[0];
#pragma unroll
  for (int w = 1; w < NT / 64; ++w) v = fmaxf(v, red[w]);
  const uint32_t abits = __float_as_uint(v);
  const float s = fmaxf(cvt16<XT>((u16)abits) / 448.0f, 1e-12f);
  if (threadIdx.x == 0) sc[0] = s;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = threadIdx.x + i * NT;
    if (c < nchunk) {
      float t[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float xv = cvt16<XT>((u16)((uint32_t)cur[i][j >> 1] >> ((j & 1) * 16)));
        t[j] = fminf(fmaxf(xv / s, -448.0f), 448.0f);
      }
      if (abits < INF_BITS) {
        int o0 = 0, o1 = 0;
        o0 = __builtin_amdgcn_cvt_pk_fp8_f32(t[0], t[1], o0, false);
        o0 = __builtin_amdgcn_cvt_pk_fp8_f32(t[2], t[3], o0, true);
        o1 = __builtin_amdgcn_cvt_pk_fp8_f32(t[4], t[5], o1, false);
        o1 = __builtin_amdgcn_cvt_pk_fp8_f32(t[6], t[7], o1, true);
        *(uint2*)(&xq[0][(size_t)c * AQ_VEC]) = make_uint2((uint32_t)o0, (uint32_t)o1);
      } else {
        uint8_t b[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) b[j] = f32_to_e4m3_sw(t[j]);
        store8(&xq[0][0], (size_t)c * AQ_VEC, b);
      }
    }
  }
  __syncthreads();
  if (blockIdx.x == 0 && g.a_scale_out && threadIdx.x == 0) g.a_scale_out[0] = sc[0];
}

// The two quantizers above for up to MAXM token rows of KROW elements, split in two so that the
// caller can issue other loads (the head of a weight stream) between the rows' loads and their
// use: rows_request() issues the loads, rows_finish_i8 / rows_finish_fp8 do the arithmetic and
// leave codes (row stride xstride bytes) and scales in LDS; they end with a barrier.
// Threads are dealt to the rows so that a wave stays inside one row: with at least as many threads
// as a row has 16-byte chunks, RPP rows are worked on at once, one chunk per thread; otherwise
// every thread takes QCH chunks of one row at a time.
template <int NT, int KROW, int MAXM_>
struct RowsPlan {
  static constexpr int MAXM = MAXM_;
  static constexpr int CPR = KROW / AQ_VEC;            // chunks per row
  static constexpr int TPR = NT >= CPR ? CPR : NT;     // threads per row
  static constexpr int RPP = NT / TPR;                 // rows per pass
  static constexpr int QCH = (CPR + TPR - 1) / TPR;    // chunks per thread and row
  static constexpr int NPASS = (MAXM + RPP - 1) / RPP;
  static constexpr int WPR = TPR / 64;                 // waves per row
  static constexpr int NTHREADS = NT;
  static_assert(TPR % 64 == 0 && NT % TPR == 0 && KROW % AQ_VEC == 0, "a wave stays inside one row");
};

template <class P>
__device__ __forceinline__ void rows_request(const GemvArgs& g, v4i (&cur)[P::NPASS][P::QCH], v4i (&sm)[P::QCH]) {
  const int tr = threadIdx.x % P::TPR, rs = threadIdx.x / P::TPR;
#pragma unroll
  for (int i = 0; i < P::QCH; ++i) {
    const int c = tr + i * P::TPR;
    sm[i] = v4i{0, 0, 0, 0};
    if (c < P::CPR && g.smooth) sm[i] = *(const v4i*)(g.smooth + (size_t)c * AQ_VEC);
  }
#pragma unroll
  for (int j = 0; j < P::NPASS; ++j) {
    const int m = j * P::RPP + rs;
#pragma unroll
    for (int i = 0; i < P::QCH; ++i) {
      const int c = tr + i * P::TPR;
      cur[j][i] = v4i{0, 0, 0, 0};
      if (m < g.M && c < P::CPR) cur[j][i] = *(const v4i*)(g.x16 + (size_t)m * g.ldx + (size_t)c * AQ_VEC);
    }
  }
}

// red: P::MAXM * P::WPR floats, followed by NT / 64 for the IEEE routine; sc: P::MAXM
template <int T, class P>
__device__ __forceinline__ void rows_finish_i8(const GemvArgs& g, v4i (&cur)[P::NPASS][P::QCH],
                                               const v4i (&sm)[P::QCH], uint8_t* xq, int xstride, float* sc,
                                               float* red) {
  const int tr = threadIdx.x % P::TPR, rs = threadIdx.x / P::TPR;
  const int lane = threadIdx.x & 63, wrow = tr >> 6;
  constexpr uint32_t INF_BITS = T == FMSMO_F16 ? 0x7c00u : 0x7f80u;
  const float floor_T = cvt16<T>(to16<T>(1e-5f));
#pragma unroll
  for (int j = 0; j < P::NPASS; ++j) {
    const int m = j * P::RPP + rs;  // uniform in a wave
    int bad = 0;
    us2 amax2 = {0, 0};
    if (m < g.M) {
#pragma unroll
      for (int i = 0; i < P::QCH; ++i) {
        const int c = tr + i * P::TPR;
        if (c < P::CPR) {
          if (g.smooth) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const uint32_t w = (uint32_t)cur[j][i][q], d = (uint32_t)sm[i][q];
              const float dl = cvt16<T>((u16)(d & 0xffff)), dh = cvt16<T>((u16)(d >> 16));
              if constexpr (T == FMSMO_BF16)
                bad |= !(fabsf(dl) >= 8.6736174e-19f && fabsf(dl) <= 1.1529215e18f) ||
                       !(fabsf(dh) >= 8.6736174e-19f && fabsf(dh) <= 1.1529215e18f);
              const u16 el = to16<T>(div16<T, false>(cvt16<T>((u16)(w & 0xffff)), dl, __builtin_amdgcn_rcpf(dl)));
              const u16 eh = to16<T>(div16<T, false>(cvt16<T>((u16)(w >> 16)), dh, __builtin_amdgcn_rcpf(dh)));
              cur[j][i][q] = (int)((uint32_t)el | ((uint32_t)eh << 16));
            }
          }
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const uint32_t mag = (uint32_t)cur[j][i][q] & 0x7fff7fffu;
            us2 m2;
            __builtin_memcpy(&m2, &mag, 4);
            amax2 = __builtin_elementwise_max(amax2, m2);
          }
        }
      }
      // non-negative floats order like their bit patterns (a NaN outranks inf; a divisor outside
      // the fast path's range marks the row for the IEEE routine)
      const float v = wave_max(__uint_as_float(bad ? 0xffffu : (uint32_t)(amax2[0] > amax2[1] ? amax2[0] : amax2[1])));
      if (lane == 0) red[m * P::WPR + wrow] = v;
    }
  }
  __syncthreads();
  // every thread forms every row's maximum itself (broadcast reads; no second barrier)
  uint32_t rowbits[P::MAXM];
  uint32_t off_fast = 0;  // (uniform) rows for the IEEE routine
#pragma unroll
  for (int m = 0; m < P::MAXM; ++m) {
    rowbits[m] = 0;
    if (m < g.M) {
      float v = red[m * P::WPR];
#pragma unroll
      for (int w = 1; w < P::WPR; ++w) v = fmaxf(v, red[m * P::WPR + w]);
      rowbits[m] = __float_as_uint(v);
      if (rowbits[m] >= INF_BITS) off_fast |= 1u << m;
    }
  }
  if (off_fast)
    for (int m = 0; m < g.M; ++m)  // by the whole block, with scratch of their own
      if (off_fast >> m & 1)
        quant_i8_row_ieee16<T, P::NTHREADS>(g.x16 + (size_t)m * g.ldx, g.smooth, g.saturate,
                                            (int8_t*)(xq + (size_t)m * xstride), sc + m, g.K, red + P::MAXM * P::WPR);
#pragma unroll
  for (int j = 0; j < P::NPASS; ++j) {
    const int m = j * P::RPP + rs;
    uint32_t abits = 0;
#pragma unroll
    for (int q = 0; q < P::RPP; ++q)
      if (j * P::RPP + q < P::MAXM && rs == q) abits = rowbits[j * P::RPP + q];
    if (m < g.M && abits < INF_BITS) {
      const float s = cvt16<T>(to16<T>(fmaxf(cvt16<T>((u16)abits), floor_T) / 127.0f));
      const float rcp_s = __builtin_amdgcn_rcpf(s);
      if (tr == 0) sc[m] = s;
#pragma unroll
      for (int i = 0; i < P::QCH; ++i) {
        const int c = tr + i * P::TPR;
        if (c < P::CPR) {
          uint32_t code[4];
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const uint32_t w = (uint32_t)cur[j][i][q];
            float ql = div16<T, false>(cvt16<T>((u16)(w & 0xffff)), s, rcp_s);
            float qh = div16<T, false>(cvt16<T>((u16)(w >> 16)), s, rcp_s);
            if (g.saturate) {
              ql = fminf(fmaxf(ql, -127.0f), 127.0f);
              qh = fminf(fmaxf(qh, -127.0f), 127.0f);
            }
            code[q] = rint_codes<T>(to16<T>(ql), to16<T>(qh));
          }
          const uint32_t o0 = __builtin_amdgcn_perm(code[1], code[0], 0x06040200u);
          const uint32_t o1 = __builtin_amdgcn_perm(code[3], code[2], 0x06040200u);
          *(uint2*)(xq + (size_t)m * xstride + (size_t)c * AQ_VEC) = make_uint2(o0, o1);
        }
      }
    }
  }
  __syncthreads();
  if (blockIdx.x == 0 && g.a_scale_out && (int)threadIdx.x < g.M) g.a_scale_out[threadIdx.x] = sc[threadIdx.x];
}

// fp32 SmoothQuant divisors: torch promotes x / smooth to fp32 and the whole quantizer then runs in
// fp32 (scale max(amax, 1e-5) / 127, quotients, rint), as in the stand-alone quantizer's kernel for
// that case: fast correctly rounded divisions while every divisor lies in 2^-60 .. 2^60 and the
// row maximum is finite (for bf16 x: and not below 2^-80), IEEE divisions otherwise.
template <class P>
__device__ __forceinline__ void rows_request_f32s(const GemvArgs& g, v4i (&cur)[P::NPASS][P::QCH],
                                                  float (&sd)[P::QCH][8]) {
  const int tr = threadIdx.x % P::TPR, rs = threadIdx.x / P::TPR;
  const float* smooth = (const float*)g.smooth;
#pragma unroll
  for (int i = 0; i < P::QCH; ++i) {
    const int c = tr + i * P::TPR;
#pragma unroll
    for (int q = 0; q < 8; ++q) sd[i][q] = 1.0f;
    if (c < P::CPR) {
      const float4 a = *(const float4*)(smooth + (size_t)c * AQ_VEC);
      const float4 b = *(const float4*)(smooth + (size_t)c * AQ_VEC + 4);
      sd[i][0] = a.x, sd[i][1] = a.y, sd[i][2] = a.z, sd[i][3] = a.w;
      sd[i][4] = b.x, sd[i][5] = b.y, sd[i][6] = b.z, sd[i][7] = b.w;
    }
  }
#pragma unroll
  for (int j = 0; j < P::NPASS; ++j) {
    const int m = j * P::RPP + rs;
#pragma unroll
    for (int i = 0; i < P::QCH; ++i) {
      const int c = tr + i * P::TPR;
      cur[j][i] = v4i{0, 0, 0, 0};
      if (m < g.M && c < P::CPR) cur[j][i] = *(const v4i*)(g.x16 + (size_t)m * g.ldx + (size_t)c * AQ_VEC);
    }
  }
}

// red: 2 * P::MAXM * P::WPR floats; sc: P::MAXM
template <int XT, class P>
__device__ __forceinline__ void rows_finish_i8_f32s(const GemvArgs& g, const v4i (&cur)[P::NPASS][P::QCH],
                                                    const float (&sd)[P::QCH][8], uint8_t* xq, int xstride,
                                                    float* sc, float* red) {
  const int tr = threadIdx.x % P::TPR, rs = threadIdx.x / P::TPR;
  const int lane = threadIdx.x & 63, wrow = tr >> 6;
  const float nz = opaque_neg_zero();
  int bad = 0;
#pragma unroll
  for (int i = 0; i < P::QCH; ++i)
#pragma unroll
    for (int q = 0; q < 8; ++q) {  // (chunks past the row hold ones)
      const float a = fabsf(sd[i][q]);
      bad |= !(a >= 8.6736174e-19f && a <= 1.1529215e18f);  // outside 2^-60 .. 2^60, or NaN
    }
  const bool ieee_block = __syncthreads_or(bad) != 0;
  float e[P::NPASS][P::QCH][8];
  // e <- x / smooth of the thread's rows; the waves' maxima of |e| (a thread's maximum drops NaN,
  // bit patterns of non-negative floats order like the floats)
  auto divide = [&](int j, bool ieee) -> float {
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < P::QCH; ++i) {
      const int c = tr + i * P::TPR;
      if (c < P::CPR) {
#pragma unroll
        for (int q = 0; q < 8; ++q) {
          const float xv = cvt16<XT>((u16)((uint32_t)cur[j][i][q >> 1] >> ((q & 1) * 16)));
          e[j][i][q] = ieee ? xv / sd[i][q] : div32_fast_mix(xv, sd[i][q], rcp_refined(sd[i][q]), nz);
          amax = fmaxf(amax, fabsf(e[j][i][q]));
        }
      }
    }
    return amax;
  };
  auto row_maxima = [&](float* buf, uint32_t (&rowbits)[P::MAXM]) {
    __syncthreads();
#pragma unroll
    for (int m = 0; m < P::MAXM; ++m) {
      rowbits[m] = 0;
      if (m < g.M) {
        uint32_t v = __float_as_uint(buf[m * P::WPR]);
#pragma unroll
        for (int w = 1; w < P::WPR; ++w) v = max(v, __float_as_uint(buf[m * P::WPR + w]));
        rowbits[m] = v;
      }
    }
  };
#pragma unroll
  for (int j = 0; j < P::NPASS; ++j) {
    const int m = j * P::RPP + rs;  // uniform in a wave
    if (m < g.M) {
      const uint32_t b = wave_max_u32(__float_as_uint(divide(j, ieee_block)) & 0x7fffffffu);
      if (lane == 0) red[m * P::WPR + wrow] = __uint_as_float(b);
    }
  }
  uint32_t rowbits[P::MAXM];
  row_maxima(red, rowbits);
  // rows that take the IEEE divisions (uniform over the block)
  uint32_t ieee_rows = 0;
#pragma unroll
  for (int m = 0; m < P::MAXM; ++m) {
    const float amax = __uint_as_float(rowbits[m]);
    bool ieee = ieee_block || !(amax < __builtin_inff());
    if constexpr (XT == FMSMO_BF16) ieee = ieee || (amax != 0.0f && amax < 8.271806e-25f);
    if (m < g.M && ieee) ieee_rows |= 1u << m;
  }
  if (ieee_rows && !ieee_block) {  // redo those rows (with every divisor in range the first pass was the fast one)
    float* red2 = red + P::MAXM * P::WPR;
#pragma unroll
    for (int j = 0; j < P::NPASS; ++j) {
      const int m = j * P::RPP + rs;
      if (m < g.M && (ieee_rows >> m & 1)) {
        const uint32_t b = wave_max_u32(__float_as_uint(divide(j, true)) & 0x7fffffffu);
        if (lane == 0) red2[m * P::WPR + wrow] = __uint_as_float(b);
      }
    }
    uint32_t again[P::MAXM];
    row_maxima(red2, again);
#pragma unroll
    for (int m = 0; m < P::MAXM; ++m)
      if (ieee_rows >> m & 1) rowbits[m] = again[m];
  }
#pragma unroll
  for (int j = 0; j < P::NPASS; ++j) {
    const int m = j * P::RPP + rs;
    uint32_t abits = 0;
    bool ieee = false;
#pragma unroll
    for (int q = 0; q < P::RPP; ++q)
      if (j * P::RPP + q < P::MAXM && rs == q) {
        abits = rowbits[j * P::RPP + q];
        ieee = ieee_rows >> (j * P::RPP + q) & 1;
      }
    if (m < g.M) {
      const float s = fmaxf(__uint_as_float(abits), 1e-5f) / 127.0f;
      const float rcp_s = rcp_refined(s);
      if (tr == 0) sc[m] = s;
#pragma unroll
      for (int i = 0; i < P::QCH; ++i) {
        const int c = tr + i * P::TPR;
        if (c < P::CPR) {
          uint32_t code[8];
#pragma unroll
          for (int q = 0; q < 8; ++q) {
            float r = ieee ? e[j][i][q] / s : div32_fast(e[j][i][q], s, rcp_s);
            if (g.saturate) r = fminf(fmaxf(r, -127.0f), 127.0f);
            // |r| <= 128.5 in every finite row: adding 1.5 * 2^23 rounds to the nearest integer,
            // ties to even, and leaves it in two's complement in the low mantissa bits
            code[q] = __float_as_uint(r + 12582912.0f);
          }
          uint32_t o[2];
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            const uint32_t lo = __builtin_amdgcn_perm(code[4 * h + 1], code[4 * h], 0x0c0c0400u);
            const uint32_t hi = __builtin_amdgcn_perm(code[4 * h + 3], code[4 * h + 2], 0x0c0c0400u);
            o[h] = __builtin_amdgcn_perm(hi, lo, 0x05040100u);
          }
          *(uint2*)(xq + (size_t)m * xstride + (size_t)c * AQ_VEC) = make_uint2(o[0], o[1]);
        }
      }
    }
  }
  __syncthreads();
  if (blockIdx.x == 0 && g.a_scale_out && (int)threadIdx.x < g.M) g.a_scale_out[threadIdx.x] = sc[threadIdx.x];
}

template <int XT, class P>
__device__ __forceinline__ void rows_finish_fp8(const GemvArgs& g, const v4i (&cur)[P::NPASS][P::QCH], uint8_t* xq,
                                                int xstride, float* sc, float* red) {
  const int tr = threadIdx.x % P::TPR, rs = threadIdx.x / P::TPR;
  const int lane = threadIdx.x & 63, wrow = tr >> 6;
  constexpr uint32_t INF_BITS = XT == FMSMO_F16 ? 0x7c00u : 0x7f80u;
#pragma unroll
  for (int j = 0; j < P::NPASS; ++j) {
    const int m = j * P::RPP + rs;
    if (m < g.M) {
      us2 amax2 = {0, 0};
#pragma unroll
      for (int i = 0; i < P::QCH; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q) {  // (chunks past the row are zero)
          const uint32_t mag = (uint32_t)cur[j][i][q] & 0x7fff7fffu;
          us2 m2;
          __builtin_memcpy(&m2, &mag, 4);
          amax2 = __builtin_elementwise_max(amax2, m2);
        }
      const float v = wave_max(__uint_as_float((uint32_t)(amax2[0] > amax2[1] ? amax2[0] : amax2[1])));
      if (lane == 0) red[m * P::WPR + wrow] = v;
    }
  }
  __syncthreads();
#pragma unroll
  for (int j = 0; j < P::NPASS; ++j) {
    const int m = j * P::RPP + rs;
    if (m < g.M) {
      float v = red[m * P::WPR];
#pragma unroll
      for (int w = 1; w < P::WPR; ++w) v = fmaxf(v, red[m * P::WPR + w]);
      const uint32_t abits = __float_as_uint(v);
      const float s = fmaxf(cvt16<XT>((u16)abits) / 448.0f, 1e-12f);
      if (tr == 0) sc[m] = s;
      const bool finite = abits < INF_BITS;
#pragma unroll
      for (int i = 0; i < P::QCH; ++i) {
        const int c = tr + i * P::TPR;
        if (c < P::CPR) {
          float t[8];
#pragma unroll
          for (int q = 0; q < 8; ++q) {
            const float xv = cvt16<XT>((u16)((uint32_t)cur[j][i][q >> 1] >> ((q & 1) * 16)));
            t[q] = fminf(fmaxf(xv / s, -448.0f), 448.0f);
          }
          uint8_t* dst = xq + (size_t)m * xstride;
          if (finite) {
            int o0 = 0, o1 = 0;
            o0 = __builtin_amdgcn_cvt_pk_fp8_f32(t[0], t[1], o0, false);
            o0 = __builtin_amdgcn_cvt_pk_fp8_f32(t[2], t[3], o0, true);
            o1 = __builtin_amdgcn_cvt_pk_fp8_f32(t[4], t[5], o1, false);
            o1 = __builtin_amdgcn_cvt_pk_fp8_f32(t[6], t[7], o1, true);
            *(uint2*)(dst + (size_t)c * AQ_VEC) = make_uint2((uint32_t)o0, (uint32_t)o1);
          } else {
            uint8_t b[8];
#pragma unroll
            for (int q = 0; q < 8; ++q) b[q] = f32_to_e4m3_sw(t[q]);
            store8(dst, (size_t)c * AQ_VEC, b);
          }
        }
      }
    }
  }
  __syncthreads();
  if (blockIdx.x == 0 && g.a_scale_out && (int)threadIdx.x < g.M) g.a_scale_out[threadIdx.x] = sc[threadIdx.x];
}

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
      const float as = g.a_scale ? g.a_scale[g.a_stride ? m : 0] : 1.f, ws = g.w_scale ? g.w_scale[g.w_stride ? n : 0] : 1.f;
      float b = -0.f;  // no bias: adding -0 changes nothing, not even the sign of a zero product
      if (g.bias) {
        b = g.bias_dtype == FMSMO_F16 ? f16_to_f32(((const u16*)g.bias)[n])
            : g.bias_dtype == FMSMO_BF16 ? bf16_to_f32(((const u16*)g.bias)[n])
                                         : ((const float*)g.bias)[n];
      }
      float out;
      if (g.epi == FMSMO_EPI_REF_F16) {
        const float sc = round_to<FMSMO_F16>(__fmul_rn(as, ws));
        out = __fadd_rn(__fmul_rn((float)s, sc), b);
        if (g.y_dtype != FMSMO_F32) out = round_to<FMSMO_F16>(out);
      } else if (g.epi == FMSMO_EPI_F32_MULADD) {
        out = __fadd_rn(__fmul_rn((float)s, __fmul_rn(as, ws)), b);
      } else {
        out = __fmaf_rn((float)s, __fmul_rn(as, ws), b);
      }
      const int64_t idx = (int64_t)m * g.ldy + n;
      if (g.epi == EPI_RAW_I32) ((int*)g.y)[idx] = (int)s;
      else if (g.y_dtype == FMSMO_F16) ((u16*)g.y)[idx] = f32_to_f16(out);
      else if (g.y_dtype == FMSMO_BF16) ((u16*)g.y)[idx] = f32_to_bf16(out);
      else ((float*)g.y)[idx] = out;
    }
  }
}


// Streaming variant (K = 128 * STEPS * NW).  Weight rows must be fetched as whole 128-byte
// lines: a wave load that touches 16 rows x 64 B tops out near 4.4 TB/s on this part, 8 rows x
// 128 B per instruction reaches 6.3 TB/s (a fully contiguous stream: 6.7).  MFMA operands want
// 16 rows x 16 B per lane group instead, so every K step of 16 rows (2 KiB: two 8-row loads)
// is transposed through a tiny wave-private LDS buffer (ds_write_b128 with an XOR swizzle,
// ds_read_b128 of the operand fragments).  D steps of loads stay in flight in registers; nothing
// is shared between waves except the final 16x16 partial sums, so the only barrier is one per
// group of 16 rows.  The activation fragments of the wave's K slice stay in registers.
// MT > 1: batches of up to 16 MT tokens.  The weight stream is the same; every step feeds MT
// MFMAs (one per tile of 16 tokens) from the same weight fragment, so up to 64 tokens cost little
// more than 16 as long as their activation fragments fit in registers (MT * STEPS * 8 VGPRs).
// D steps of weight loads are in flight per wave.  Long rows want a shallow pipeline: the
// activation fragments of K = 14336 take 112 registers per lane, and with 7 of the 14 steps in
// flight the kernel spilled (12 / 32 registers for int8 / e4m3 at the 256-register limit); D = 2
// fits and is faster at every token count (us at N = 4096, 16 tokens: int8 18.9 -> 15.4, e4m3
// 23.5 -> 16.1; 4 tokens 15.8 -> 12.5; K = 12800 as 10 waves x 10 steps, D = 5 -> 2: 20.1 ->
// 11.3 at 4 tokens), also than keeping the activations in LDS with all 14 steps in flight (4
// tokens: 14.6).
// Work is dealt to the blocks in units of 8 weight rows (half an MFMA row group): block b owns the
// half groups [b H / B, (b + 1) H / B) of the H = ceil(N / 8) there are, so that N = 6144 gives
// each of 256 blocks 24 rows (whole groups only: 192 blocks of 32 rows, a quarter of the compute
// units idle).  A block walks its rows in groups of 16; when the last one is a half group, its
// upper 8 rows are neither loaded nor stored.
// HALF = false: the host has checked that every block owns whole groups only (the loads of the
// upper rows are then unconditional, which the register allocation of the long-row shapes needs).
// XT >= 0 (fused decode linear, up to MAXM tokens of dtype XT, K = NW * STEPS * 128): the block
// quantizes the token rows itself, into LDS -- their loads are issued first, the head of the
// weight stream next, and the quantizer's arithmetic runs while those weights are in flight --
// and the activation fragments of every step are read from there (rows of 16 bytes more than K,
// so that the 16 token rows of a fragment read fall into different banks; the lanes of token rows
// past M substitute zeros).  No activation registers: the weight pipeline can be as deep as with
// XS, for any number of row groups per block.
// SF32: the fused form with fp32 SmoothQuant divisors (int8 only).
template <int OP, int STEPS, int NW, int D, int MT = 1, bool HALF = false, bool XS = false, int XT = -1,
          int MAXM = 1, bool SF32 = false>
__global__ __launch_bounds__(NW * 64) void gemv_stream_kernel(GemvArgs g, int halves) {
  static_assert(STEPS % D == 0, "pipeline depth must divide the steps per group");
  static_assert(!XS || MT == 1, "streamed activations: one tile of tokens");
  constexpr bool FUSED = XT >= 0;
  static_assert(!FUSED || (MT == 1 && MAXM <= 16), "the fused form serves one tile of tokens");
  constexpr int KROW = NW * STEPS * 128;
  constexpr int XSTRIDE = KROW + 16;
  typedef RowsPlan<NW * 64, KROW, MAXM> QP;
  __shared__ __attribute__((aligned(16))) uint8_t xq[FUSED ? MAXM * XSTRIDE : 16];
  __shared__ float xsc[FUSED ? MAXM : 1];
  __shared__ float xred[FUSED ? 2 * MAXM * QP::WPR + NW : 1];
  typedef typename std::conditional<OP == FMSMO_OP_I8, int, float>::type AccT;
  typedef AccT Acc4 __attribute__((ext_vector_type(4)));
  constexpr int NRED = 2;  // exchange buffers alternate, one barrier per group
  __shared__ __attribute__((aligned(16))) uint8_t stage[NW][2][2048];
  __shared__ AccT red[NRED][NW][256 * MT];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int r = lane & 15, kg = lane >> 4;
  const int h_lo = (int)(((int64_t)blockIdx.x * halves) / gridDim.x);
  const int h_hi = (int)(((int64_t)(blockIdx.x + 1) * halves) / gridDim.x);
  const int row_lo = h_lo * 8, row_hi = min(h_hi * 8, g.N);  // this block's weight rows
  const int gcount = (h_hi - h_lo + 1) >> 1;                 // groups of 16 rows, the last maybe half
  if (gcount <= 0) return;                                    // more blocks than half groups
  const int kwave = wave * (STEPS * 128);

  // weight loads: lane -> (row = lane / 8 [+8], 16-byte chunk = lane % 8): 8 rows x 128 B each
  const int drow = lane >> 3, dpos = lane & 7;
  // per-group row pointers, clamped (branch-free) for prefetch past the end and a ragged last group
  const int64_t kcol = kwave + dpos * 16;
  auto rowptr = [&](int gi, int half) {
    const int row0 = row_lo + min(gi, gcount - 1) * 16;
    return g.b + (int64_t)min(row0 + half * 8 + drow, g.N - 1) * g.ldb + kcol;
  };
  // does group gi hold rows in its upper half? (uniform; a half group's upper rows belong to the
  // next block: not loaded, their products are never stored)
  auto is_full = [&](int gi) { return !HALF || row_lo + min(gi, gcount - 1) * 16 + 8 < row_hi; };
  const uint8_t* pc[2] = {rowptr(0, 0), rowptr(0, 1)};  // current group
  const uint8_t* pn[2] = {rowptr(1, 0), rowptr(1, 1)};  // next group
  bool fullc = is_full(0), fulln = is_full(1);
  auto load_item = [&](bool next, int s, v4i (&w)[2]) {
    w[0] = __builtin_nontemporal_load((const v4i*)((next ? pn[0] : pc[0]) + s * 128));
    if (!HALF || (next ? fulln : fullc))
      w[1] = __builtin_nontemporal_load((const v4i*)((next ? pn[1] : pc[1]) + s * 128));
  };
  // staging: row-major [16 rows][128 B], chunk c of row q stored at position c ^ (q % 8)
  const int wr0 = drow * 128 + ((dpos ^ drow) * 16);
  const int wr1 = (8 + drow) * 128 + ((dpos ^ drow) * 16);
  const int rr = r & 7;
  const int rd0 = r * 128 + ((kg ^ rr) * 16), rd1 = r * 128 + (((4 + kg) ^ rr) * 16);

  v4i wb[D][2];
  if constexpr (HALF) {  // the upper halves stay unloaded for a block whose only group is a half one
#pragma unroll
    for (int j = 0; j < D; ++j) wb[j][1] = v4i{0, 0, 0, 0};
  }
  // Activation fragments: lane (m = r, kg) holds x[m][kwave + s*128 + (h*4 + kg)*16 ...], fetched
  // through a buffer descriptor that ends with token row M - 1: the lanes of token rows past M get
  // zeros without a branch or a clamped address (column m of the MFMA's second operand only
  // reaches output column m, which is never stored).  Every block re-reads the activations from
  // L2: 16 K bytes against its (N / blocks) K weight bytes, as much as the weights at N = 4096.
  // XS = false: the fragments of the wave's whole K slice stay in registers for all the block's
  // groups.  XS = true (long rows, one group per block, so each fragment is used once): they are
  // fetched step by step beside the weights, D steps in flight, and the registers they leave free
  // go to a deeper pipeline (us at N = 4096, K = 14336, int8, 4 / 16 tokens: 12.7 / 15.5 with the
  // fragments held and two steps in flight, 11.4 / 13.8 streamed with seven; starting the blocks
  // at different K steps so that they do not all ask L2 for the same lines at once: 11.7 / 14.3).
  v4i xf[XS || FUSED ? 1 : MT][XS || FUSED ? 1 : STEPS][2];
  v4i xb[XS && !FUSED ? D : 1][2];
  v4i qcur[FUSED ? QP::NPASS : 1][FUSED ? QP::QCH : 1], qsm[FUSED && !SF32 ? QP::QCH : 1];
  float qsd[SF32 ? QP::QCH : 1][8];
  const __amdgpu_buffer_rsrc_t rsrc_x = __builtin_amdgcn_make_buffer_rsrc(
      (void*)g.a, 0, FUSED ? 0 : (int)((int64_t)(g.M - 1) * g.lda + g.K), 0x00020000);
  const int vx = r * (int)g.lda + kwave + kg * 16;
  auto load_x = [&](int t, int s, v4i (&x)[2]) {
    const int v = vx + t * 16 * (int)g.lda;
    x[0] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrc_x, v, s * 128, 0));
    x[1] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrc_x, v, s * 128 + 64, 0));
  };
  if constexpr (SF32) {
    rows_request_f32s<QP>(g, qcur, qsd);
  } else if constexpr (FUSED) {
    rows_request<QP>(g, qcur, qsm);
  } else if constexpr (XS) {
#pragma unroll
    for (int j = 0; j < D; ++j) load_x(0, j, xb[j]);
  } else {
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int s = 0; s < STEPS; ++s) load_x(t, s, xf[t][s]);
  }
  // (the activation loads go first: with the weights ahead of them the kernel measured 2 - 5 %
  // slower at 16 tokens)
#pragma unroll
  for (int j = 0; j < D; ++j) load_item(false, j, wb[j]);

  // epilogue operands of output element e = threadIdx.x (n = e / 16, m = e % 16 of the group) are
  // fetched at the top of each group so that their latency hides behind the weight stream
  const int em = min((int)(threadIdx.x & 15), g.M - 1);
  float as;
  if constexpr (FUSED) {
    if constexpr (SF32) rows_finish_i8_f32s<XT, QP>(g, qcur, qsd, xq, XSTRIDE, xsc, xred);
    else if constexpr (OP == FMSMO_OP_I8) rows_finish_i8<XT, QP>(g, qcur, qsm, xq, XSTRIDE, xsc, xred);
    else rows_finish_fp8<XT, QP>(g, qcur, xq, XSTRIDE, xsc, xred);
    as = xsc[em];
  } else {
    as = g.a_scale ? g.a_scale[g.a_stride ? em : 0] : 1.f;
  }
  // fused: the codes of this lane's token row and K positions (token rows past M: zeros)
  const bool xrow = r < g.M;
  const uint8_t* xl = xq + (FUSED ? (xrow ? r : 0) * XSTRIDE + kwave + kg * 16 : 0);

  // The last group of a block refills nothing (its prefetches would fall into the next block's
  // rows), so the group body exists twice: streaming (LAST = false) and draining (LAST = true).
  auto do_group = [&](auto last_tag, int gi) {
    constexpr bool LAST = decltype(last_tag)::value;
    const int en = min(row_lo + gi * 16 + (int)((threadIdx.x >> 4) & 15), g.N - 1);
    const float ws = g.w_scale ? g.w_scale[g.w_stride ? en : 0] : 1.f;
    float bv = -0.f;  // no bias: adding -0 changes nothing, not even the sign of a zero product
    if (g.bias) {
      bv = g.bias_dtype == FMSMO_F16 ? f16_to_f32(((const u16*)g.bias)[en])
           : g.bias_dtype == FMSMO_BF16 ? bf16_to_f32(((const u16*)g.bias)[en])
                                        : ((const float*)g.bias)[en];
    }
    Acc4 acc[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[t] = Acc4{0, 0, 0, 0};
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      uint8_t* st = &stage[wave][s & 1][0];
      *(v4i*)(st + wr0) = wb[s % D][0];
      *(v4i*)(st + wr1) = wb[s % D][1];
      __builtin_amdgcn_sched_barrier(0);  // keep the refill right behind the registers it frees
      if (!LAST || s + D < STEPS) load_item(s + D >= STEPS, (s + D) % STEPS, wb[s % D]);
      __builtin_amdgcn_sched_barrier(0);
      const v4i w0 = *(const v4i*)(st + rd0);
      const v4i w1 = *(const v4i*)(st + rd1);
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        v4i x0, x1;
        if constexpr (FUSED) {
          const v4i z = {0, 0, 0, 0};
          x0 = *(const v4i*)(xl + s * 128), x1 = *(const v4i*)(xl + s * 128 + 64);
          x0 = xrow ? x0 : z, x1 = xrow ? x1 : z;
        } else {
          x0 = XS ? xb[s % D][0] : xf[t][s][0], x1 = XS ? xb[s % D][1] : xf[t][s][1];
        }
        if constexpr (OP == FMSMO_OP_I8) {
          acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(w0, x0, acc[t], 0, 0, 0);
          acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(w1, x1, acc[t], 0, 0, 0);
        } else {
          const v8i wv = {w0[0], w0[1], w0[2], w0[3], w1[0], w1[1], w1[2], w1[3]};
          const v8i xv = {x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
          acc[t] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wv, xv, acc[t], 0, 0, 0, 0, 0, 0);
        }
      }
      if constexpr (XS && !FUSED) {  // the same K offsets serve every group: the refill wraps around
        __builtin_amdgcn_sched_barrier(0);
        if (!LAST || s + D < STEPS) load_x(0, (s + D) % STEPS, xb[s % D]);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    // acc[v] = partial C(n = 16 (group0+gi) + 4 kg + v, m = r) of this wave's K slice.  The NW
    // partials are summed by the first 256 threads; two exchange buffers alternate so that one
    // barrier per group is enough.
    if (!LAST) {
      pc[0] = pn[0], pc[1] = pn[1];
      pn[0] = rowptr(gi + 2, 0), pn[1] = rowptr(gi + 2, 1);
      if constexpr (HALF) {
        fullc = fulln;
        fulln = is_full(gi + 2);
      }
    }
    AccT* mine = &red[gi % NRED][wave][0];
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int v = 0; v < 4; ++v) mine[t * 256 + (kg * 4 + v) * 16 + r] = acc[t][v];
    __syncthreads();
    auto finish = [&](int e, float as_e, float ws_e, float bv_e) {
      AccT sum = red[gi % NRED][0][e];
#pragma unroll
      for (int w = 1; w < NW; ++w) sum += red[gi % NRED][w][e];
      const int n = row_lo + gi * 16 + ((e >> 4) & 15), m = (e >> 8) * 16 + (e & 15);
      if (n < row_hi && m < g.M) {
        float out;
        if (g.epi == FMSMO_EPI_REF_F16) {
          const float sc = round_to<FMSMO_F16>(__fmul_rn(as_e, ws_e));
          out = __fadd_rn(__fmul_rn((float)sum, sc), bv_e);
          if (g.y_dtype != FMSMO_F32) out = round_to<FMSMO_F16>(out);
        } else if (g.epi == FMSMO_EPI_F32_MULADD) {
          out = __fadd_rn(__fmul_rn((float)sum, __fmul_rn(as_e, ws_e)), bv_e);
        } else {
          out = __fmaf_rn((float)sum, __fmul_rn(as_e, ws_e), bv_e);
        }
        const int64_t idx = (int64_t)m * g.ldy + n;
        if (g.epi == EPI_RAW_I32) ((int*)g.y)[idx] = (int)sum;
        else if (g.y_dtype == FMSMO_F16) ((u16*)g.y)[idx] = f32_to_f16(out);
        else if (g.y_dtype == FMSMO_BF16) ((u16*)g.y)[idx] = f32_to_bf16(out);
        else ((float*)g.y)[idx] = out;
      }
    };
    if constexpr (MT == 1) {
      if (threadIdx.x < 256) finish(threadIdx.x, as, ws, bv);
    } else {
      // the column of output e is that of thread e % 256 (already fetched: ws, bv); its token row
      // differs per tile, so the token scale is fetched here
      static_assert(MT == 1 || (NW * 64) % 256 == 0, "outputs of a thread must share its column");
      for (int e = threadIdx.x; e < 256 * MT; e += NW * 64) {
        const int m = min((e >> 8) * 16 + (e & 15), g.M - 1);
        finish(e, g.a_scale ? g.a_scale[g.a_stride ? m : 0] : 1.f, ws, bv);
      }
    }
  };
  if constexpr (!XS) {
    for (int gi = 0; gi + 1 < gcount; ++gi) do_group(std::false_type{}, gi);
  }
  do_group(std::true_type{}, gcount - 1);  // XS: the host gives every block one group at most
}

// Row-streaming variant for M <= 2: no MFMA, no LDS.  A wave owns whole weight rows and reads
// each as one contiguous run (lane l takes the 16-byte chunks l, l + 64, ...: every wave load is
// 1 KiB of consecutive bytes, the access pattern HBM serves best), multiplies with the
// activation chunks it keeps in registers (v_dot4_i32_i8, exact; e4m3 is widened to fp32 and
// accumulated with FMAs), and reduces the 64 partial sums with a butterfly.  U rows are in
// flight per wave; rows are dealt to waves so that neighbouring waves read neighbouring rows.
// KCH = ceil(K / 1024) chunks per lane; chunks past K are zero.
template <int OP, int MR, int KCH, int U, int XT = -1>
__global__ __launch_bounds__(256) void gemv_rows_kernel(GemvArgs g) {
  typedef typename std::conditional<OP == FMSMO_OP_I8, int, float>::type AccT;
  // XT >= 0 (FMSMO_F16 / FMSMO_BF16): fused decode linear -- the block first quantizes the
  // unquantized activations into LDS (quantize_rows_to_lds) and then takes its chunks and token
  // scales from there instead of from global memory
  constexpr bool FUSED = XT >= 0;
  __shared__ __attribute__((aligned(16))) uint8_t xq[FUSED ? MR : 1][FUSED ? KCH * 1024 : 16];
  __shared__ float xsc[4];
  __shared__ float xred[4];
  const int lane = threadIdx.x & 63;
  const int wave_g = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int nwaves = gridDim.x * 4;
  const int kchunks = g.K >> 4;

  auto load_w = [&](int n0, v4i (&w)[U][KCH]) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint8_t* wp = g.b + (int64_t)min(n0 + u, g.N - 1) * g.ldb;
#pragma unroll
      for (int c = 0; c < KCH; ++c) {
        const int ch = c * 64 + lane;
        // chunks past K: re-read the row's first chunk; the zero activation chunk cancels it
        w[u][c] = __builtin_nontemporal_load((const v4i*)(wp + (int64_t)(ch < kchunks ? ch : lane % kchunks) * 16));
      }
    }
  };
  v4i w[U][KCH];
  if constexpr (FUSED) {
    // the weights of the first turn are in flight while the block quantizes its activations
    load_w(wave_g * U, w);
    if constexpr (OP == FMSMO_OP_I8) quantize_rows_to_lds<XT, 256, KCH * 1024, MR>(g, xq, xsc, xred);
    else quantize_row_fp8_to_lds<XT, 256, KCH * 1024>(g, xq, xsc, xred);
    g.a = &xq[0][0];
    g.lda = KCH * 1024;
    g.a_scale = xsc;
    g.a_stride = 1;
  }

  v4i xr[MR][KCH];
#pragma unroll
  for (int m = 0; m < MR; ++m) {
    const uint8_t* xp = g.a + (int64_t)min(m, g.M - 1) * g.lda;
#pragma unroll
    for (int c = 0; c < KCH; ++c) {
      const int ch = c * 64 + lane;
      xr[m][c] = ch < kchunks ? *(const v4i*)(xp + (int64_t)ch * 16) : v4i{0, 0, 0, 0};
    }
  }

  // e4m3: every code is an fp16 value and a product of two fp16 values is exact in fp32, so the
  // codes are widened two at a time to packed fp16 and multiplied by v_dot2_f32_f16 (fp32
  // accumulation): 6 vector instructions per 4 weight bytes, 4 where the activation chunks are
  // kept widened (XH: at most 64 registers), against 8 for conversions to fp32 and FMAs.
  constexpr bool XH = OP != FMSMO_OP_I8 && MR * KCH <= 8;
  typedef _Float16 h2 __attribute__((ext_vector_type(2)));
  h2 xh[XH ? MR : 1][XH ? KCH : 1][8];
  if constexpr (XH) {
#pragma unroll
    for (int m = 0; m < MR; ++m)
#pragma unroll
      for (int c = 0; c < KCH; ++c)
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          xh[m][c][2 * d] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(xr[m][c][d], 1.0f, false);
          xh[m][c][2 * d + 1] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(xr[m][c][d], 1.0f, true);
        }
  }

  for (int n0 = wave_g * U; n0 < g.N; n0 += nwaves * U) {
    if (!FUSED || n0 != wave_g * U) load_w(n0, w);
    AccT acc[U][MR];
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int m = 0; m < MR; ++m) {
        AccT a = 0;
#pragma unroll
        for (int c = 0; c < KCH; ++c) {
#pragma unroll
          for (int d = 0; d < 4; ++d) {
            if constexpr (OP == FMSMO_OP_I8) {
              a = __builtin_amdgcn_sdot4(w[u][c][d], xr[m][c][d], a, false);
            } else {
              const h2 w0 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w[u][c][d], 1.0f, false);
              const h2 w1 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w[u][c][d], 1.0f, true);
              h2 x0, x1;
              if constexpr (XH) {
                x0 = xh[m][c][2 * d];
                x1 = xh[m][c][2 * d + 1];
              } else {
                x0 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(xr[m][c][d], 1.0f, false);
                x1 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(xr[m][c][d], 1.0f, true);
              }
              a = __builtin_amdgcn_fdot2(w0, x0, a, false);
              a = __builtin_amdgcn_fdot2(w1, x1, a, false);
            }
          }
        }
        acc[u][m] = a;
      }
    // Transposing butterfly over the V = U * MR partial sums of a lane: each exchange halves the
    // number of values a lane still carries (the upper half of the lanes keeps the upper half of
    // the values), so V - 1 + log2(64 / V) exchanges replace 6 V.  Lane l ends with the total of
    // value index idx(l) (same in the 64 / V lanes that share its upper bits).
    constexpr int V = U * MR;
    AccT vals[V];
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int m = 0; m < MR; ++m) vals[u * MR + m] = acc[u][m];
    int idx = 0;
    {
      int width = 32;
#pragma unroll
      for (int nv = V; nv > 1; nv >>= 1, width >>= 1) {
        const int half = nv >> 1;
        const bool upper = (lane & width) != 0;
#pragma unroll
        for (int i = 0; i < half; ++i) {
          const AccT send = upper ? vals[i] : vals[i + half];
          const AccT keep = upper ? vals[i + half] : vals[i];
          vals[i] = keep + __shfl_xor(send, width, 64);
        }
        idx += upper ? half : 0;
      }
#pragma unroll
      for (; width > 0; width >>= 1) vals[0] += __shfl_xor(vals[0], width, 64);
    }
    const AccT sum = vals[0];
    const int eu = idx / MR, em = idx % MR;
    constexpr int SHARE = 64 / V;  // lanes holding the same total; the first of them writes it
    const int n = n0 + eu;
    if ((lane & (SHARE - 1)) == 0 && n < g.N && em < g.M) {
      const float as = g.a_scale ? g.a_scale[g.a_stride ? em : 0] : 1.f, ws = g.w_scale ? g.w_scale[g.w_stride ? n : 0] : 1.f;
      float bv = -0.f;  // no bias: adding -0 changes nothing, not even the sign of a zero product
      if (g.bias) {
        bv = g.bias_dtype == FMSMO_F16 ? f16_to_f32(((const u16*)g.bias)[n])
             : g.bias_dtype == FMSMO_BF16 ? bf16_to_f32(((const u16*)g.bias)[n])
                                          : ((const float*)g.bias)[n];
      }
      float out;
      if (g.epi == FMSMO_EPI_REF_F16) {
        const float sc = round_to<FMSMO_F16>(__fmul_rn(as, ws));
        out = __fadd_rn(__fmul_rn((float)sum, sc), bv);
        if (g.y_dtype != FMSMO_F32) out = round_to<FMSMO_F16>(out);
      } else if (g.epi == FMSMO_EPI_F32_MULADD) {
        out = __fadd_rn(__fmul_rn((float)sum, __fmul_rn(as, ws)), bv);
      } else {
        out = __fmaf_rn((float)sum, __fmul_rn(as, ws), bv);
      }
      const int64_t idx = (int64_t)em * g.ldy + n;
      if (g.epi == EPI_RAW_I32) ((int*)g.y)[idx] = (int)sum;
      else if (g.y_dtype == FMSMO_F16) ((u16*)g.y)[idx] = f32_to_f16(out);
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

// Batches of 17 .. 64 tokens that the weight-streaming kernel takes in one pass (their
// activation fragments must fit in registers): K = 1024 * {1, 2, 4, 5, 8} up to 32 tokens,
// K = 1024 * {1, 2, 4} up to 64.  (K = 5120, 17 / 32 tokens against the tiled kernels, us:
// N = 5120 14.5 -> 9.8 / 15.8 -> 11.2, N = 13824 27.0 -> 17.6 / 25.9 -> 19.1.)
bool fmsmo_gemv_batch_ok(int64_t M, int64_t K) {
  if (M <= 16 || M > 64 || K % 1024) return false;
  const int64_t steps = K / 1024;
  if (steps != 1 && steps != 2 && steps != 4 && steps != 5 && steps != 8) return false;
  return M <= 32 || steps <= 4;
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
  g.bias = bias; g.bias_dtype = bias_dtype; g.epi = epilogue;
  g.y = y; g.y_dtype = y_dtype; g.ldy = ldy;
  // M <= 2: whole-row streaming on the vector ALUs (at M = 4 its register use halves the
  // occupancy and the MFMA streaming kernel below is faster) (FMSMO_GEMV_KIND=1 disables it for tuning)
  {
    static const int env_kind = getenv("FMSMO_GEMV_KIND") ? atoi(getenv("FMSMO_GEMV_KIND")) : 0;
    const int kch = (int)((K + 1023) / 1024);
    const int mr = M <= 1 ? 1 : 2;
    // Where the MFMA streaming kernel below has an instantiation for K it is the faster one for
    // two e4m3 tokens (twice the widening work per weight byte; us at N = 4096, rows -> streaming:
    // K = 4096 6.2 -> 5.4, 14336 22.3 -> 12.6), for two int8 tokens from K = 8192 (7.9 -> 7.4;
    // 14336: 13.7 -> 12.1; 5120: 5.7 against 5.9), for one e4m3 token from K = 12800 (12.6 ->
    // 11.2; 8192: 7.9 both) and for one int8 token at K = 12800 (11.4 -> 10.8; 14336: 11.8 both,
    // 16384: 13.0 against 13.8).
    const int steps128 = K % 128 ? 0 : (int)(K / 128);
    const bool stream_ok = steps128 == 8 || steps128 == 16 || steps128 == 32 || steps128 == 40 ||
                           steps128 == 64 || steps128 == 100 || steps128 == 112 || steps128 == 128;
    // Rows of 14336 where N <= 4096 gives every block of the streaming kernel a single row group
    // (activations streamed beside the weights, seven steps in flight): one token 11.8 -> 11.2
    // (int8), 12.7 -> 11.9 (e4m3).
    const bool one_group = N <= 16 * 256;
    const bool prefer_stream =
        stream_ok && (op == FMSMO_OP_I8 ? (M == 2 ? kch >= 8 : (kch == 13 || (kch == 14 && one_group)))
                                        : (M == 2 || kch >= 11));
    bool handled = env_kind != 1 && M <= 2 && K >= 1024 && !prefer_stream;
    if (handled) {
      // 16 waves per CU resident (register use allows it), rows dealt round-robin to waves
      const int64_t waves_needed = N;  // at U = 1
      dim3 block(256);
#define GEMV_ROWS(OPV, MRV, KCHV, UV)                                                        \
  {                                                                                          \
    const int64_t blocks = (waves_needed + 4 * UV - 1) / (4 * UV);                           \
    dim3 grid((unsigned)(blocks < 1024 ? blocks : 1024));                                    \
    hipLaunchKernelGGL((gemv_rows_kernel<OPV, MRV, KCHV, UV>), grid, block, 0, st, g);       \
  }
#define GEMV_ROWS_M(OPV, KCHV, UV)                                   \
  if (mr == 1) GEMV_ROWS(OPV, 1, KCHV, UV)                           \
  else GEMV_ROWS(OPV, 2, KCHV, UV)
#define GEMV_ROWS_K(OPV)                                        \
  switch (kch) {                                                \
    case 1: GEMV_ROWS_M(OPV, 1, 8) break;                       \
    case 2: GEMV_ROWS_M(OPV, 2, 8) break;                       \
    case 4: GEMV_ROWS_M(OPV, 4, 4) break;                       \
    case 5: GEMV_ROWS_M(OPV, 5, 2) break;                       \
    case 8: GEMV_ROWS_M(OPV, 8, 2) break;                       \
    case 11: GEMV_ROWS_M(OPV, 11, 1) break;                     \
    case 13: GEMV_ROWS_M(OPV, 13, 1) break;                     \
    case 14: GEMV_ROWS_M(OPV, 14, 1) break;                     \
    case 16: GEMV_ROWS_M(OPV, 16, 1) break;                     \
    default: handled = false; break;                            \
  }
      if (op == FMSMO_OP_I8) { GEMV_ROWS_K(FMSMO_OP_I8) } else { GEMV_ROWS_K(FMSMO_OP_E4M3) }
#undef GEMV_ROWS_K
#undef GEMV_ROWS_M
#undef GEMV_ROWS
      if (handled) return fmsmo_check_launch();
    }
  }
  // Streaming variant when the K steps of 128 split evenly over the waves of a block in one of
  // the instantiated (waves, steps per wave, loads in flight) shapes; other K use the generic
  // kernel below.  One block per compute unit, each walking its share of the row groups: every block
  // re-reads the activations and pays one memory latency before its stream starts, so fewer,
  // longer-lived blocks win (measured: N = 28672, K = 4096 runs 26.5 us at G = 1, 21.0 us at
  // G = 7).  FMSMO_GEMV_G overrides G for tuning.
  {
    static const int env_g = getenv("FMSMO_GEMV_G") ? atoi(getenv("FMSMO_GEMV_G")) : 0;
    const int steps_total = (int)(K / 128);
    const int64_t groups = (N + 15) / 16;
    int NW = 0;
    if (steps_total % 8 == 0) NW = 8;
    else if (steps_total % 10 == 0) NW = 10;
    // K = 4096 and at most 16 tokens: 16 waves of 2 steps each instead of 8 of 4 (us at M = 4 / 16:
    // o 5.8 -> 5.5 / 6.6 -> 6.0, qkv 7.0 -> 7.0 / 8.2 -> 7.7, gate+up 21.8 -> 20.9 / 22.8 -> 21.8).
    if (M <= 16 && steps_total == 32) NW = 16;
    const int STEPS = NW ? steps_total / NW : 0;
    // one block per compute unit, the rows dealt out in units of 8 (FMSMO_GEMV_G = groups of 16
    // rows per block instead, for tuning)
    const int halves = (int)((N + 7) / 8);
    int64_t nblocks = env_g > 0 ? (groups + env_g - 1) / env_g : 256;
    if (nblocks > halves) nblocks = halves;
    const int G = halves;  // the kernels' second argument
    // every block's share begins and ends on a group boundary
    const bool whole_groups = halves % (2 * nblocks) == 0;
    dim3 grid((unsigned)nblocks), block(NW * 64);
    bool handled = true;
    // a block that owns one row group gains nothing from keeping the activations in registers
    // (FMSMO_GEMV_XS = 0 switches the streamed variant off, for tuning)
    static const int env_xs = getenv("FMSMO_GEMV_XS") ? atoi(getenv("FMSMO_GEMV_XS")) : -1;
    const bool x_ok = (M - 1) * lda + K < ((int64_t)1 << 31);  // 32-bit offsets into the activations
    const bool xs = M <= 16 && halves <= 2 * nblocks && env_xs != 0;
#define GEMV_STREAM_H(OPV, NWV, ST, DV, HV)                                                       \
  if (M <= 16) hipLaunchKernelGGL((gemv_stream_kernel<OPV, ST, NWV, DV, 1, HV>), grid, block, 0, st, g, G); \
  else if constexpr (NWV == 8 && ST <= 8) {                                                        \
    if (M <= 32) hipLaunchKernelGGL((gemv_stream_kernel<OPV, ST, NWV, DV, 2, HV>), grid, block, 0, st, g, G); \
    else if constexpr (ST <= 4) hipLaunchKernelGGL((gemv_stream_kernel<OPV, ST, NWV, DV, 4, HV>), grid, block, 0, st, g, G); \
    else handled = false;                                                                          \
  } else handled = false
#define GEMV_STREAM(OPV, NWV, ST, DV)                     \
  if (whole_groups) { GEMV_STREAM_H(OPV, NWV, ST, DV, false); } \
  else { GEMV_STREAM_H(OPV, NWV, ST, DV, true); }
// long rows: DXS steps of weights and activations in flight where every block owns one group
#define GEMV_STREAM_L(OPV, NWV, ST, DV, DXS)                                                       \
  if (xs && whole_groups) hipLaunchKernelGGL((gemv_stream_kernel<OPV, ST, NWV, DXS, 1, false, true>), grid, block, 0, st, g, G); \
  else if (xs) hipLaunchKernelGGL((gemv_stream_kernel<OPV, ST, NWV, DXS, 1, true, true>), grid, block, 0, st, g, G); \
  else { GEMV_STREAM(OPV, NWV, ST, DV) }
#define GEMV_SHAPES(OPV)                                            \
  switch (NW * 100 + STEPS) {                                       \
    case 801: GEMV_STREAM(OPV, 8, 1, 1); break;                     \
    case 802: GEMV_STREAM(OPV, 8, 2, 2); break;                     \
    case 804: GEMV_STREAM(OPV, 8, 4, 4); break;                     \
    case 805: GEMV_STREAM(OPV, 8, 5, 5); break;                     \
    case 808: GEMV_STREAM_L(OPV, 8, 8, 4, 8); break;                \
    case 814: GEMV_STREAM_L(OPV, 8, 14, 2, 7); break;               \
    case 816: GEMV_STREAM_L(OPV, 8, 16, 4, 8); break;               \
    case 1010: GEMV_STREAM_L(OPV, 10, 10, 2, 5); break;             \
    case 1602: GEMV_STREAM(OPV, 16, 2, 2); break;                   \
    default: handled = false; break;                                \
  }
    if (!x_ok) handled = false;
    else if (op == FMSMO_OP_I8) { GEMV_SHAPES(FMSMO_OP_I8) } else { GEMV_SHAPES(FMSMO_OP_E4M3) }
#undef GEMV_SHAPES
#undef GEMV_STREAM_L
#undef GEMV_STREAM
#undef GEMV_STREAM_H
    if (handled) return fmsmo_check_launch();
  }
  if (M > 16) return FMSMO_ERR_UNSUPPORTED;  // callers ask fmsmo_gemv_batch_ok first
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

// ---------------------------------------------------------------------- fused decode linear
// One token, K <= 8192: the row kernel quantizes the token in every block (measured from a HIP
// graph against the two launches, us: qkv 9.6 -> 8.3, o 8.1 -> 6.3, gate+up 23.4 -> 19.7).  With
// longer rows the quantization its 1024 small blocks repeat costs more than the launch it saves
// (K = 14336: 16.5 -> 19.6), so K = 14336 and K = 12800 take the streaming kernel's fused form:
// 256 blocks of 8 / 10 waves quantize the row once each while the head of their weight stream is
// in flight (N = 4096, int8 from fp16 / bf16 with SmoothQuant / e4m3: K = 14336 14.5 -> 11.4,
// 16.6 -> 12.7, 17.5 -> 12.2; K = 12800 13.6 -> 10.6, 15.6 -> 11.6, 16.6 -> 11.9).
// A few tokens take the same form while the quantization that all 256 blocks repeat costs less
// than the launch it saves (us, two launches -> fused, int8 from fp16 with SmoothQuant, 2 / 3 / 4
// tokens: o 8.8 -> 7.9, 9.3 -> 7.6, 8.9 -> 8.3; qkv 10.3 -> 8.5, 9.9 -> 8.8, 9.9 -> 9.3; gate+up
// 24.8 -> 21.8, 23.9 -> 22.1, 23.8 -> 22.8; down 15.8 -> 13.7, 15.9 -> 15.6, four tokens 15.9 ->
// 17.8; six tokens at K = 4096 lose as well: 8.8 -> 9.3, 10.1 -> 10.4).
extern "C" int fmsmo_decode_linear_ok(int64_t M, int64_t K) {
  if (M < 1 || M > 4 || K % 128 || K < 1024) return 0;
  if (M > 1) return K == 4096 || (M <= 3 && (K == 14336 || K == 12800));  // the streaming kernel's fused form
  if (K == 14336 || K == 12800) return 1;
  const int kch = (int)((K + 1023) / 1024);
  return kch == 1 || kch == 2 || kch == 4 || kch == 8;
}
// the same with fp32 SmoothQuant divisors (the streaming kernel's fused form only; the fp32
// quantizer is heavier: us, two launches -> fused at 1 / 2 / 4 tokens: o 8.7 -> 8.1, 9.5 -> 9.2,
// 9.6 -> 10.2; qkv 10.5 -> 8.9, 11.1 -> 9.9, 10.9 -> 11.5; gate+up 24.7 -> 23.3, 26.0 -> 23.3,
// 24.7 -> 24.7; down, one token, 17.2 -> 14.5)
extern "C" int fmsmo_decode_linear_f32s_ok(int64_t M, int64_t K) {
  if (M < 1 || M > 2) return 0;
  return K == 4096 || (M == 1 && (K == 14336 || K == 12800));
}

template <int OP, int XT>
static int decode_fused_launch(const GemvArgs& g, hipStream_t st) {
  // the streaming kernel's fused form: (waves, steps per wave, loads in flight, most tokens)
  const bool sf32 = g.smooth && g.smooth_f32;
  int shape = 0;
  if (g.K == 14336) shape = 814;
  else if (g.K == 12800) shape = 1010;
  else if (g.K == 4096 && (g.M > 1 || sf32)) shape = 1602;
  // (int8, one token, K = 4096 with at most one row group per compute unit: this form instead of
  // the row kernel's, us at N = 4096 / 1024 from bf16 with SmoothQuant: 6.6 -> 6.3 / 5.3 -> 4.6;
  // e4m3 stays with the row kernel there, whose fp32 sums are those of the two-call path)
  else if (g.K == 4096 && OP == FMSMO_OP_I8 && g.N <= 4096) shape = 1602;
  if (sf32 && (!shape || OP != FMSMO_OP_I8)) return FMSMO_ERR_UNSUPPORTED;
  if (shape) {
    const int halves = (g.N + 7) / 8;
    const int nblocks = halves < 256 ? halves : 256;
    const bool whole_groups = halves % (2 * nblocks) == 0;
    const bool one_group = halves == 2 * nblocks;  // the kernel without its loop over row groups
    dim3 grid((unsigned)nblocks);
#define STREAM_G(NWV, ST, DV, MM, SF)                                                                \
  if (whole_groups && one_group)                                                                     \
    hipLaunchKernelGGL((gemv_stream_kernel<OP, ST, NWV, DV, 1, false, true, XT, MM, SF>), grid, dim3(NWV * 64), 0, st, g, halves); \
  else if (whole_groups)                                                                             \
    hipLaunchKernelGGL((gemv_stream_kernel<OP, ST, NWV, DV, 1, false, false, XT, MM, SF>), grid, dim3(NWV * 64), 0, st, g, halves); \
  else                                                                                               \
    hipLaunchKernelGGL((gemv_stream_kernel<OP, ST, NWV, DV, 1, true, false, XT, MM, SF>), grid, dim3(NWV * 64), 0, st, g, halves)
#define STREAM_F(NWV, ST, DV, MM)                                       \
  if constexpr (OP == FMSMO_OP_I8) {                                    \
    if (sf32) { STREAM_G(NWV, ST, DV, MM, true); }                      \
    else { STREAM_G(NWV, ST, DV, MM, false); }                          \
  } else { STREAM_G(NWV, ST, DV, MM, false); }
    switch (shape) {
      case 814:
        if (g.M == 1) { STREAM_F(8, 14, 7, 1) } else if (sf32) return FMSMO_ERR_UNSUPPORTED; else { STREAM_G(8, 14, 7, 4, false); }
        break;
      case 1010:
        if (g.M == 1) { STREAM_F(10, 10, 5, 1) } else if (sf32) return FMSMO_ERR_UNSUPPORTED; else { STREAM_G(10, 10, 5, 4, false); }
        break;
      default:
        if (g.M == 1) { STREAM_F(16, 2, 2, 1) } else { STREAM_F(16, 2, 2, 4) }
        break;
    }
#undef STREAM_F
#undef STREAM_G
    return fmsmo_check_launch();
  }
  const int kch = (int)((g.K + 1023) / 1024);
#define ROWS(KCHV, UV)                                                                            \
  {                                                                                                \
    const int64_t blocks = ((int64_t)g.N + 4 * UV - 1) / (4 * UV);                                 \
    dim3 grid((unsigned)(blocks < 1024 ? blocks : 1024));                                          \
    hipLaunchKernelGGL((gemv_rows_kernel<OP, 1, KCHV, UV, XT>), grid, dim3(256), 0, st, g);         \
  }
  switch (kch) {
    case 1: ROWS(1, 8) break;
    case 2: ROWS(2, 8) break;
    case 4: ROWS(4, 4) break;
    case 8: ROWS(8, 2) break;
    default: return FMSMO_ERR_UNSUPPORTED;
  }
#undef ROWS
  return fmsmo_check_launch();
}

extern "C" int fmsmo_decode_linear_i8(const void* x, int x_dtype, int64_t ldx, const void* smooth,
                                      int smooth_dtype, int saturate, const int8_t* w, int64_t ldw,
                                      const float* w_scale, int64_t w_scale_n, const void* bias,
                                      int bias_dtype, int epilogue, void* y, int y_dtype,
                                      int64_t ldy, float* a_scale_out, int64_t M, int64_t N,
                                      int64_t K, fmsmo_stream_t stream) {
  if (!x || !w || !w_scale || !y) return FMSMO_ERR_NULL;
  if (M <= 0 || N <= 0 || K <= 0 || ldx < K || ldw < K || ldy < N) return FMSMO_ERR_SHAPE;
  if (w_scale_n != 1 && w_scale_n != N) return FMSMO_ERR_SHAPE;
  if (x_dtype != FMSMO_F16 && x_dtype != FMSMO_BF16) return FMSMO_ERR_UNSUPPORTED;
  const bool sf32 = smooth && smooth_dtype == FMSMO_F32;
  if (smooth && !sf32 && smooth_dtype != x_dtype) return FMSMO_ERR_UNSUPPORTED;
  if (!(sf32 ? fmsmo_decode_linear_f32s_ok(M, K) : fmsmo_decode_linear_ok(M, K))) return FMSMO_ERR_UNSUPPORTED;
  if (N >= (1 << 30) || N * ldw >= (1ll << 40)) return FMSMO_ERR_UNSUPPORTED;
  if (y_dtype < 0 || y_dtype > 2 || (bias && (bias_dtype < 0 || bias_dtype > 2))) return FMSMO_ERR_UNSUPPORTED;
  if (epilogue < FMSMO_EPI_REF_F16 || epilogue > FMSMO_EPI_F32_MULADD) return FMSMO_ERR_UNSUPPORTED;
  if (ldx % 8 || ldw % 16 || (((uintptr_t)x) & 15) || (((uintptr_t)w) & 15) ||
      (smooth && (((uintptr_t)smooth) & 15)))
    return FMSMO_ERR_ALIGN;
  GemvArgs g{};
  g.b = (const uint8_t*)w; g.ldb = ldw;
  g.M = (int)M; g.N = (int)N; g.K = (int)K;
  g.w_scale = w_scale; g.w_stride = w_scale_n == 1 ? 0 : 1;
  g.bias = bias; g.bias_dtype = bias_dtype; g.epi = epilogue;
  g.y = y; g.y_dtype = y_dtype; g.ldy = ldy;
  g.x16 = (const u16*)x; g.ldx = ldx; g.smooth = (const u16*)smooth; g.saturate = saturate;
  g.smooth_f32 = sf32 ? 1 : 0;
  g.a_scale_out = a_scale_out;
  return x_dtype == FMSMO_F16 ? decode_fused_launch<FMSMO_OP_I8, FMSMO_F16>(g, (hipStream_t)stream)
                              : decode_fused_launch<FMSMO_OP_I8, FMSMO_BF16>(g, (hipStream_t)stream);
}

extern "C" int fmsmo_decode_linear_fp8(const void* x, int x_dtype, int64_t ldx, const uint8_t* w,
                                       int64_t ldw, const float* w_scale, int64_t w_scale_n,
                                       const void* bias, int bias_dtype, void* y, int y_dtype,
                                       int64_t ldy, float* a_scale_out, int64_t M, int64_t N,
                                       int64_t K, fmsmo_stream_t stream) {
  if (!x || !w || !w_scale || !y) return FMSMO_ERR_NULL;
  if (M <= 0 || N <= 0 || K <= 0 || ldx < K || ldw < K || ldy < N) return FMSMO_ERR_SHAPE;
  if (w_scale_n != 1 && w_scale_n != N) return FMSMO_ERR_SHAPE;
  if ((x_dtype != FMSMO_F16 && x_dtype != FMSMO_BF16) || !fmsmo_decode_linear_ok(M, K)) return FMSMO_ERR_UNSUPPORTED;
  if (N >= (1 << 30) || N * ldw >= (1ll << 40)) return FMSMO_ERR_UNSUPPORTED;
  if (y_dtype < 0 || y_dtype > 2 || (bias && (bias_dtype < 0 || bias_dtype > 2))) return FMSMO_ERR_UNSUPPORTED;
  if (ldx % 8 || ldw % 16 || (((uintptr_t)x) & 15) || (((uintptr_t)w) & 15)) return FMSMO_ERR_ALIGN;
  GemvArgs g{};
  g.b = w; g.ldb = ldw;
  g.M = (int)M; g.N = (int)N; g.K = (int)K;
  g.w_scale = w_scale; g.w_stride = w_scale_n == 1 ? 0 : 1;
  g.bias = bias; g.bias_dtype = bias_dtype; g.epi = FMSMO_EPI_F32;
  g.y = y; g.y_dtype = y_dtype; g.ldy = ldy;
  g.x16 = (const u16*)x; g.ldx = ldx;
  g.a_scale_out = a_scale_out;
  return x_dtype == FMSMO_F16 ? decode_fused_launch<FMSMO_OP_E4M3, FMSMO_F16>(g, (hipStream_t)stream)
                              : decode_fused_launch<FMSMO_OP_E4M3, FMSMO_BF16>(g, (hipStream_t)stream);
}

namespace fmsmo {
// pure read of n16 16-byte words, block-contiguous, UNROLL loads in flight per lane
__global__ __launch_bounds__(1024) void stream_read_kernel(const v4i* __restrict__ p, int64_t n16, int* sink) {
  constexpr int UNROLL = 4;
  const int64_t per = (n16 + gridDim.x - 1) / gridDim.x;
  const int64_t lo = blockIdx.x * per, hi = lo + per < n16 ? lo + per : n16;
  v4i acc = {0, 0, 0, 0};
  int64_t i = lo + threadIdx.x;
  for (; i + (UNROLL - 1) * 1024 < hi; i += UNROLL * 1024) {
    v4i t[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) t[u] = __builtin_nontemporal_load(&p[i + u * 1024]);
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) acc ^= t[u];
  }
  for (; i < hi; i += 1024) acc ^= __builtin_nontemporal_load(&p[i]);
  if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x5ca1ab1e) sink[0] = 1;
}
}  // namespace fmsmo

extern "C" int fmsmo_debug_stream_read(const void* p, int64_t bytes, int32_t* sink, fmsmo_stream_t stream) {
  if (!p || !sink) return FMSMO_ERR_NULL;
  if (bytes <= 0 || bytes % 16) return FMSMO_ERR_SHAPE;
  if ((uintptr_t)p & 15) return FMSMO_ERR_ALIGN;
  hipLaunchKernelGGL(stream_read_kernel, dim3(256), dim3(1024), 0, (hipStream_t)stream, (const v4i*)p,
                     bytes / 16, sink);
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
  if (epilogue < FMSMO_EPI_REF_F16 || epilogue > FMSMO_EPI_F32_MULADD) return FMSMO_ERR_UNSUPPORTED;
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
