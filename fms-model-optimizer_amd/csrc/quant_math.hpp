// Arithmetic shared by the activation quantizers and the fused decode kernels: 8-element loads,
// the exact 16-bit division sequence, integer codes by the magic-number addition, and the IEEE
// fallback routine for one row.
#pragma once
#include "common.hpp"

namespace fmsmo {

constexpr int AQ_VEC = 8;  // elements per thread per chunk

template <int XT>
__device__ __forceinline__ void load8(const void* x, size_t elem, float (&v)[8]) {
  if constexpr (XT == FMSMO_F32) {
    const float4 a = *(const float4*)((const float*)x + elem);
    const float4 b = *(const float4*)((const float*)x + elem + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
  } else {
    const uint4 r = *(const uint4*)((const u16*)x + elem);
    const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if constexpr (XT == FMSMO_F16) {
        v[2 * i] = f16_to_f32((u16)(w[i] & 0xffff));
        v[2 * i + 1] = f16_to_f32((u16)(w[i] >> 16));
      } else {
        v[2 * i] = bf16_to_f32((u16)(w[i] & 0xffff));
        v[2 * i + 1] = bf16_to_f32((u16)(w[i] >> 16));
      }
    }
  }
}

__device__ __forceinline__ void store8(uint8_t* q, size_t elem, const uint8_t (&b)[8]) {
  uint2 o;
  o.x = b[0] | (b[1] << 8) | (b[2] << 16) | ((uint32_t)b[3] << 24);
  o.y = b[4] | (b[5] << 8) | (b[6] << 16) | ((uint32_t)b[7] << 24);
  *(uint2*)(q + elem) = o;
}

template <int T, bool IEEE>
__device__ __forceinline__ float div16(float e, float s, float r) {
  if constexpr (IEEE) {
    return e / s;
  } else {
    const float q0 = __fmul_rn(e, r);
    return __builtin_fmaf(__builtin_fmaf(-q0, s, e), r, q0);
  }
}
// -0.0f the compiler cannot see through: fma(e, r, nz) is e * r bit for bit, and for e widened
// from fp16 the widening folds into v_fma_mix_f32, where a plain product needs its own conversion.
__device__ __forceinline__ float opaque_neg_zero() {
  float z = -0.0f;
  asm volatile("" : "+s"(z));
  return z;
}
// div16<T, false> with the first product written as that fma (fp16 only; bf16 widens by a shift)
template <int T>
__device__ __forceinline__ float div16_mix(float e, float s, float r, float nz) {
  const float q0 = T == FMSMO_F16 ? __builtin_fmaf(e, r, nz) : __fmul_rn(e, r);
  return __builtin_fmaf(__builtin_fmaf(-q0, s, e), r, q0);
}
// fp32 division without the IEEE sequence's range scaling and fix-up: a refined reciprocal and two
// residual corrections give the correctly rounded quotient whenever no intermediate leaves the
// normal range (the callers check the ranges of their operands).
__device__ __forceinline__ float rcp_refined(float s) {
  const float r0 = __builtin_amdgcn_rcpf(s);
  return __builtin_fmaf(__builtin_fmaf(-s, r0, 1.0f), r0, r0);
}
__device__ __forceinline__ float div32_fast(float x, float s, float r1) {
  float q = __fmul_rn(x, r1);
  q = __builtin_fmaf(__builtin_fmaf(-s, q, x), r1, q);
  q = __builtin_fmaf(__builtin_fmaf(-s, q, x), r1, q);
  return q;
}
// the same for x widened from fp16: with the first product written as fma(x, r1, -0) (nz: see
// opaque_neg_zero) all three uses of x fold into v_fma_mix_f32 and no conversion is issued
__device__ __forceinline__ float div32_fast_mix(float x, float s, float r1, float nz) {
  float q = __builtin_fmaf(x, r1, nz);
  q = __builtin_fmaf(__builtin_fmaf(-s, q, x), r1, q);
  q = __builtin_fmaf(__builtin_fmaf(-s, q, x), r1, q);
  return q;
}

template <int T>
__device__ __forceinline__ float cvt16(u16 h) {
  if constexpr (T == FMSMO_F16) return f16_to_f32(h);
  else return bf16_to_f32(h);
}
template <int T>
__device__ __forceinline__ u16 to16(float f) {
  if constexpr (T == FMSMO_F16) return f32_to_f16(f);
  else return f32_to_bf16(f);
}

typedef unsigned short us2 __attribute__((ext_vector_type(2)));
typedef _Float16 hf2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
typedef float f2 __attribute__((ext_vector_type(2)));

// two floats rounded to T (nearest even), low and high half of one word, by one packed
// conversion.  For fp16 the empty asm keeps the conversion apart from the arithmetic that feeds
// it (see f32_to_f16).
template <int T>
__device__ __forceinline__ uint32_t pack16(float lo, float hi) {
  if constexpr (T == FMSMO_F16) {
    asm volatile("" : "+v"(lo), "+v"(hi));
    const hf2 h = {(_Float16)lo, (_Float16)hi};
    uint32_t r;
    __builtin_memcpy(&r, &h, 4);
    return r;
  } else {
    const f2 v = {lo, hi};
    const bf2 h = __builtin_convertvector(v, bf2);  // v_cvt_pk_bf16_f32: RNE, NaN stays NaN
    uint32_t r;
    __builtin_memcpy(&r, &h, 4);
    return r;
  }
}

// int8 code of rint(h) for a 16-bit value h with |h| <= 511, in the low byte of each half:
// h + 1536 lands in [1024, 2048), where the fp16 grid is the integers, so the addition itself
// rounds to nearest-even and the low mantissa bits are the two's-complement integer.
template <int T>
__device__ __forceinline__ uint32_t rint_codes(u16 lo, u16 hi);
// the same on a packed pair, optionally clamped to +-127 first (the bounds are integers, so
// clamping before or after the rounding gives the same code)
template <int T>
__device__ __forceinline__ uint32_t rint_codes_packed(uint32_t packed, bool saturate) {
  if constexpr (T == FMSMO_F16) {
    hf2 h;
    __builtin_memcpy(&h, &packed, 4);
    if (saturate) {
      const hf2 hi = {(_Float16)127.0f, (_Float16)127.0f};
      h = __builtin_elementwise_min(__builtin_elementwise_max(h, -hi), hi);
    }
    const hf2 magic = {(_Float16)1536.0f, (_Float16)1536.0f};
    h = h + magic;
    uint32_t r;
    __builtin_memcpy(&r, &h, 4);
    return r;
  } else {
    float lo = bf16_to_f32((u16)(packed & 0xffff)), hi = bf16_to_f32((u16)(packed >> 16));
    if (saturate) {
      lo = fminf(fmaxf(lo, -127.0f), 127.0f);
      hi = fminf(fmaxf(hi, -127.0f), 127.0f);
    }
    return rint_codes<T>(f32_to_bf16(lo), f32_to_bf16(hi));
  }
}
template <int T>
__device__ __forceinline__ uint32_t rint_codes(u16 lo, u16 hi) {
  if constexpr (T == FMSMO_F16) {
    hf2 h;
    const uint32_t packed = (uint32_t)lo | ((uint32_t)hi << 16);
    __builtin_memcpy(&h, &packed, 4);
    const hf2 magic = {(_Float16)1536.0f, (_Float16)1536.0f};
    h = h + magic;
    uint32_t r;
    __builtin_memcpy(&r, &h, 4);
    return r;
  } else {
    // same trick in fp32: r + 1.5 * 2^23 (|r| <= 511 is far inside its range)
    const uint32_t a = __float_as_uint(bf16_to_f32(lo) + 12582912.0f) & 0xffu;
    const uint32_t c = __float_as_uint(bf16_to_f32(hi) + 12582912.0f) & 0xffu;
    return a | (c << 16);
  }
}

// One row with plain IEEE divisions, chunk by chunk from memory (no register cache, so that this
// rarely taken path does not raise the register allocation of the kernels that call it).  Same
// arithmetic as the generic kernel for a 16-bit compute dtype.  `red` holds TH / 64 floats.
template <int T, int TH>
__device__ __forceinline__ void quant_i8_row_ieee16(const u16* __restrict__ xr, const u16* __restrict__ smooth,
                                                 int saturate, int8_t* __restrict__ qr, float* __restrict__ scale_out,
                                                 int K, float* red) {
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
  const float s = round_to<T>(fmaxf(amax, round_to<T>(1e-5f)) / 127.0f);
  if (threadIdx.x == 0) *scale_out = s;
#pragma unroll 1
  for (int c = threadIdx.x; c < nchunk; c += TH) {
    float e[8];
    chunk(c, e);
    uint8_t b[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      float r = __builtin_rintf(round_to<T>(e[j] / s));
      if (saturate) r = fminf(fmaxf(r, -127.0f), 127.0f);
      b[j] = (uint8_t)(int)r;
    }
    store8((uint8_t*)qr, (size_t)c * AQ_VEC, b);
  }
}

}  // namespace fmsmo
