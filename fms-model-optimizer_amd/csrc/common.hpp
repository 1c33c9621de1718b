// Shared device/host helpers for the gfx950 quantized-linear kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/fmsmo_hip.h"

namespace fmsmo {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef short s8v __attribute__((ext_vector_type(8)));
typedef unsigned short u16;

// internal epilogue code of the decode kernels: store the int32 sums themselves (beside the public
// FMSMO_EPI_* values)
constexpr int EPI_RAW_I32 = 100;

#define FMSMO_GPTR(p) ((const __attribute__((address_space(1))) void*)(p))
#define FMSMO_LPTR(p) ((__attribute__((address_space(3))) void*)(p))

// ---------------------------------------------------------------- 16-bit float conversions
// All conversions are round-to-nearest-even and keep subnormals, matching torch's casts.
__device__ __forceinline__ float f16_to_f32(u16 h) {
  _Float16 v;
  __builtin_memcpy(&v, &h, 2);
  return (float)v;
}
__device__ __forceinline__ u16 f32_to_f16(float f) {
  // Keep the conversion a separate instruction: without this the compiler folds
  // "round_to_f16(a * b)" / "(a + b)" into v_fma_mixlo_f16, which rounds the exact product or
  // sum once to fp16 instead of fp32-then-fp16 as torch does (differs at fp16 ties).
  asm volatile("" : "+v"(f));
  _Float16 v = (_Float16)f;  // v_cvt_f16_f32: RNE, overflow -> inf
  u16 h;
  __builtin_memcpy(&h, &v, 2);
  return h;
}
__device__ __forceinline__ float bf16_to_f32(u16 h) { return __uint_as_float(((uint32_t)h) << 16); }
__device__ __forceinline__ u16 f32_to_bf16(float f) {
  __bf16 v = (__bf16)f;  // v_cvt_pk_bf16_f32: RNE, NaN stays NaN
  u16 h;
  __builtin_memcpy(&h, &v, 2);
  return h;
}

// Round a float to the value grid of dtype T (T in FMSMO_F16/BF16/F32) and come back to f32.
template <int T>
__device__ __forceinline__ float round_to(float f) {
  if constexpr (T == FMSMO_F16) return f16_to_f32(f32_to_f16(f));
  else if constexpr (T == FMSMO_BF16) return bf16_to_f32(f32_to_bf16(f));
  else return f;
}
template <int T>
__device__ __forceinline__ float load_as_f32(const void* p, size_t i) {
  if constexpr (T == FMSMO_F16) return f16_to_f32(((const u16*)p)[i]);
  else if constexpr (T == FMSMO_BF16) return bf16_to_f32(((const u16*)p)[i]);
  else return ((const float*)p)[i];
}
template <int T>
__device__ __forceinline__ void store_from_f32(void* p, size_t i, float v) {
  if constexpr (T == FMSMO_F16) ((u16*)p)[i] = f32_to_f16(v);
  else if constexpr (T == FMSMO_BF16) ((u16*)p)[i] = f32_to_bf16(v);
  else ((float*)p)[i] = v;
}

// Maximum of an unsigned value over the 64 lanes of the wave (all active), same result in every
// lane.  Cross-lane
// moves are DPP modifiers of the max instructions themselves (no LDS round trips): pairs and quads
// by quad permutes, 8 and 16 lanes by the mirror patterns, then lane 15 / 31 broadcast into the
// following rows, after which lane 63 holds the maximum of all.
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t x) {
#define FMSMO_DPP_MAX(ctrl, rows)                                                             \
  {                                                                                            \
    const uint32_t y = (uint32_t)__builtin_amdgcn_update_dpp((int)x, (int)x, ctrl, rows, 0xf, false); \
    x = y > x ? y : x;                                                                         \
  }
  FMSMO_DPP_MAX(0xb1, 0xf)   // quad_perm [1,0,3,2]
  FMSMO_DPP_MAX(0x4e, 0xf)   // quad_perm [2,3,0,1]
  FMSMO_DPP_MAX(0x141, 0xf)  // row_half_mirror
  FMSMO_DPP_MAX(0x140, 0xf)  // row_mirror
  FMSMO_DPP_MAX(0x142, 0xa)  // row_bcast15 into rows 1 and 3
  FMSMO_DPP_MAX(0x143, 0xc)  // row_bcast31 into rows 2 and 3
#undef FMSMO_DPP_MAX
  return (uint32_t)__builtin_amdgcn_readlane((int)x, 63);
}

// The same for floats (fmaxf semantics: a NaN loses against a number).  All 64 lanes must be active.
__device__ __forceinline__ float wave_max(float v) {
#define FMSMO_DPP_FMAX(ctrl, rows)                                                            \
  {                                                                                            \
    const int b = __float_as_int(v);                                                           \
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(b, b, ctrl, rows, 0xf, false)));   \
  }
  FMSMO_DPP_FMAX(0xb1, 0xf)
  FMSMO_DPP_FMAX(0x4e, 0xf)
  FMSMO_DPP_FMAX(0x141, 0xf)
  FMSMO_DPP_FMAX(0x140, 0xf)
  FMSMO_DPP_FMAX(0x142, 0xa)
  FMSMO_DPP_FMAX(0x143, 0xc)
#undef FMSMO_DPP_FMAX
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}

// OCP e4m3fn encode of one float, RNE, the way torch's float->float8_e4m3fn cast does it:
// |x| <= 464 rounds into the finite range (max 448), anything above and NaN give 0x7f|sign.
__device__ __forceinline__ uint8_t f32_to_e4m3_sw(float f) {
  uint32_t u = __float_as_uint(f);
  uint8_t sign = (u >> 24) & 0x80;
  uint32_t a = u & 0x7fffffffu;
  if (a > 0x43e80000u) return sign | 0x7f;       // > 464 (incl. inf / NaN) -> NaN
  if (a < 0x3c800000u) {                          // subnormal target: < 2^-6, quantum 2^-9
    float q = __uint_as_float(a) * 512.0f;        // exact scaling
    float r = __builtin_rintf(q);                 // RNE
    return sign | (uint8_t)(int)r;                // r in [0,8]; 8 == smallest normal 0x08
  }
  // normal: keep 3 mantissa bits
  uint32_t r = a + 0x7ffffu + ((a >> 20) & 1u);
  r >>= 20;                                       // exponent(8) | mant(3)
  int e = (int)(r >> 3) - 127 + 7;
  return sign | (uint8_t)((e << 3) | (r & 7));
}

inline int div_up(int64_t a, int64_t b) { return (int)((a + b - 1) / b); }

}  // namespace fmsmo
