// Activation quantizers off the per-token fast path, each one pass over x (HBM bound, 8 elements
// per thread and 16-byte loads): the static per-tensor int8 formulas of the deploy modules
// evaluated in a chosen compute dtype, the dynamic per-tensor / per-column int8 quantizers whose
// scale comes from a column abs-max already on the device, and the FP8 (e4m3) emulation
// quantizers.  Every intermediate is rounded to the compute dtype T the way torch's elementwise
// kernels do it: the operation is carried out in fp32 on operands widened from T and rounded back
// (24 >= 2 * 11 + 2 significand bits make the double rounding of +, -, *, / harmless for fp16,
// and all the more for bf16); divisions are IEEE divisions, or a shorter sequence that gives the
// same rounded quotient (the 16-bit kernels).
#include "quant_math.hpp"

namespace fmsmo {

struct StaticArgs {
  float scale, zp, sym, lo, hi;
  int mode;
};

template <int XT, int T>
__global__ __launch_bounds__(256) void quant_i8_static_t_kernel(const void* __restrict__ x, int64_t ldx,
                                                                StaticArgs p, int8_t* __restrict__ q,
                                                                int64_t ldq, int M, int K) {
  const int cpr = K / AQ_VEC;
  const int64_t total = (int64_t)M * cpr;
  for (int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x; c < total; c += (int64_t)gridDim.x * 256) {
    const int64_t m = c / cpr;
    const int k = (int)(c - m * cpr) * AQ_VEC;
    float v[8];
    load8<XT>(x, (size_t)(m * ldx + k), v);
    uint8_t b[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      float e = round_to<T>(v[i]);
      float r;
      if (p.mode == FMSMO_SQ_RAW) {
        float t = round_to<T>(e / p.scale);
        t = round_to<T>(t + p.zp);
        t = round_to<T>(t - 128.0f);
        t = round_to<T>(t + p.sym);
        r = fminf(fmaxf(__builtin_rintf(t), -128.0f), 127.0f);
      } else if (p.mode == FMSMO_SQ_FMO) {
        e = fminf(fmaxf(e, p.lo), p.hi);
        float t = round_to<T>(e / p.scale);
        t = round_to<T>(t - p.zp);
        r = __builtin_rintf(t) - (128.0f - p.sym);
      } else {
        float t = round_to<T>(e / p.scale);
        t = round_to<T>(t + p.zp);
        r = __builtin_rintf(t);
        if (p.mode == FMSMO_SQ_U8_SHIFT) r = fminf(fmaxf(r, 0.0f), 255.0f) - 128.0f;
        else r = fminf(fmaxf(r, -127.0f), 127.0f);
      }
      b[i] = (uint8_t)(int)r;
    }
    store8((uint8_t*)q, (size_t)(m * ldq + k), b);
  }
}

// The same formulas for a 16-bit compute dtype T on contiguous x of that dtype, at memory speed: the
// kernel above spends ~30 vector instructions per element (an IEEE fp32 division, a 64-bit index
// division per chunk, one conversion pair per rounding step), this one ~13.  The quotient of two
// values of T is the three-operation sequence of the per-token quantizer (div16_mix: it rounds to
// the same T as the IEEE quotient whenever no intermediate leaves the fp32 normal range, which the
// launcher guarantees for the divisor and fp16 / bf16 x for the dividend; quotients of bf16 values
// below 2^-118 may differ in their last bit, far below anything that survives the rounding to an
// integer), passed through v_div_fixup so that zero, infinite and NaN operands give the IEEE
// result.  Every other step is the operation of the generic kernel on the same fp32 values, with
// the roundings to T done on pairs.  Integer codes come from the low mantissa bits of
// t + 1.5 * 2^23 (round to nearest even for |t| < 2^22; the launcher checks the bound where the
// formula itself does not clamp).
template <int T, int MODE>
__global__ __launch_bounds__(256) void quant_i8_static16_kernel(const u16* __restrict__ x, StaticArgs p,
                                                                float rcp_scale, int8_t* __restrict__ q,
                                                                int64_t nchunks) {
  const float nz = opaque_neg_zero();
  auto rnd2 = [](float& a, float& b) {
    const uint32_t w = pack16<T>(a, b);
    a = cvt16<T>((u16)(w & 0xffff));
    b = cvt16<T>((u16)(w >> 16));
  };
  for (int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x; c < nchunks; c += (int64_t)gridDim.x * 256) {
    const v4i raw = __builtin_nontemporal_load((const v4i*)(x + c * AQ_VEC));
    uint32_t code[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t w = (uint32_t)raw[j];
      float e0 = cvt16<T>((u16)(w & 0xffff)), e1 = cvt16<T>((u16)(w >> 16));
      if constexpr (MODE == FMSMO_SQ_FMO) {
        e0 = fminf(fmaxf(e0, p.lo), p.hi);
        e1 = fminf(fmaxf(e1, p.lo), p.hi);
      }
      float t0 = __builtin_amdgcn_div_fixupf(div16_mix<T>(e0, p.scale, rcp_scale, nz), p.scale, e0);
      float t1 = __builtin_amdgcn_div_fixupf(div16_mix<T>(e1, p.scale, rcp_scale, nz), p.scale, e1);
      rnd2(t0, t1);
      if constexpr (MODE == FMSMO_SQ_FMO) {
        t0 -= p.zp; t1 -= p.zp;
        rnd2(t0, t1);
      } else {
        t0 += p.zp; t1 += p.zp;
        rnd2(t0, t1);
        if constexpr (MODE == FMSMO_SQ_RAW) {
          t0 -= 128.0f; t1 -= 128.0f;
          rnd2(t0, t1);
          t0 += p.sym; t1 += p.sym;
          rnd2(t0, t1);
          t0 = fminf(fmaxf(t0, -128.0f), 127.0f);
          t1 = fminf(fmaxf(t1, -128.0f), 127.0f);
        } else if constexpr (MODE == FMSMO_SQ_U8_SHIFT) {
          t0 = fminf(fmaxf(t0, 0.0f), 255.0f);
          t1 = fminf(fmaxf(t1, 0.0f), 255.0f);
        } else {
          t0 = fminf(fmaxf(t0, -127.0f), 127.0f);
          t1 = fminf(fmaxf(t1, -127.0f), 127.0f);
        }
      }
      uint32_t c0 = __float_as_uint(t0 + 12582912.0f), c1 = __float_as_uint(t1 + 12582912.0f);
      if constexpr (MODE == FMSMO_SQ_FMO) {
        const uint32_t shift = (uint32_t)(128 - (int)p.sym);
        c0 -= shift; c1 -= shift;
      } else if constexpr (MODE == FMSMO_SQ_U8_SHIFT) {
        c0 ^= 0x80u; c1 ^= 0x80u;
      }
      code[j] = (c0 & 0xffu) | ((c1 & 0xffu) << 8);
    }
    *(uint2*)(q + c * AQ_VEC) = make_uint2(code[0] | (code[1] << 16), code[2] | (code[3] << 16));
  }
}

// scale[k] = rnd_T( max(amax_k, rnd_T(1e-5)) / levels ) per column, or the same of the maximum
// over all columns into scale[0] (one block).
template <int T>
__global__ __launch_bounds__(256) void dyn_scale_kernel(const float* __restrict__ col_amax, int K,
                                                        int per_column, float levels,
                                                        float* __restrict__ scale) {
  const float floor_t = round_to<T>(1e-5f);
  if (per_column) {
    const int k = blockIdx.x * 256 + threadIdx.x;
    if (k < K) scale[k] = round_to<T>(fmaxf(col_amax[k], floor_t) / levels);
    return;
  }
  __shared__ float red[4];
  float a = 0.0f;
  for (int k = threadIdx.x; k < K; k += 256) a = fmaxf(a, col_amax[k]);
  a = wave_max(a);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = a;
  __syncthreads();
  if (threadIdx.x == 0) {
    a = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    scale[0] = round_to<T>(fmaxf(a, floor_t) / levels);
  }
}

// q = int8( rint( rnd_T(x / s) ) + zp ) with s = scale[0] or scale[k]; the int8 cast wraps.
template <int T>
__global__ __launch_bounds__(256) void quant_i8_dynamic_kernel(const void* __restrict__ x, int64_t ldx,
                                                               const float* __restrict__ scale,
                                                               int per_column, float zp,
                                                               int8_t* __restrict__ q, int64_t ldq,
                                                               int M, int K) {
  const int cpr = K / AQ_VEC;
  const int64_t total = (int64_t)M * cpr;
  const float s0 = scale[0];
  for (int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x; c < total; c += (int64_t)gridDim.x * 256) {
    const int64_t m = c / cpr;
    const int k = (int)(c - m * cpr) * AQ_VEC;
    float v[8], s[8];
    load8<T>(x, (size_t)(m * ldx + k), v);
    if (per_column) load8<FMSMO_F32>(scale, (size_t)k, s);
    uint8_t b[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float t = round_to<T>(v[i] / (per_column ? s[i] : s0));
      const float r = round_to<T>(__builtin_rintf(t) + zp);
      b[i] = (uint8_t)(int)r;
    }
    store8((uint8_t*)q, (size_t)(m * ldq + k), b);
  }
}

// The per-tensor form on contiguous 16-bit x: the quotient of quant_i8_static16_kernel (the scale is
// a finite value of T by construction; one outside 2^-60 .. 2^60, which only an absurd abs-max
// gives, sends the whole launch through IEEE divisions), everything behind it as above.
template <int T>
__global__ __launch_bounds__(256) void quant_i8_dynamic16_kernel(const u16* __restrict__ x,
                                                                 const float* __restrict__ scale, float zp,
                                                                 int8_t* __restrict__ q, int64_t nchunks) {
  const float s = scale[0];
  const bool fast = fabsf(s) >= 8.6736174e-19f && fabsf(s) <= 1.1529215e18f;
  const float r = __builtin_amdgcn_rcpf(s);
  const float nz = opaque_neg_zero();
  for (int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x; c < nchunks; c += (int64_t)gridDim.x * 256) {
    const v4i raw = __builtin_nontemporal_load((const v4i*)(x + c * AQ_VEC));
    uint32_t code[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t w = (uint32_t)raw[j];
      const float e0 = cvt16<T>((u16)(w & 0xffff)), e1 = cvt16<T>((u16)(w >> 16));
      float t0, t1;
      if (fast) {
        t0 = __builtin_amdgcn_div_fixupf(div16_mix<T>(e0, s, r, nz), s, e0);
        t1 = __builtin_amdgcn_div_fixupf(div16_mix<T>(e1, s, r, nz), s, e1);
      } else {
        t0 = e0 / s;
        t1 = e1 / s;
      }
      uint32_t pk = pack16<T>(t0, t1);
      t0 = __builtin_rintf(cvt16<T>((u16)(pk & 0xffff))) + zp;
      t1 = __builtin_rintf(cvt16<T>((u16)(pk >> 16))) + zp;
      pk = pack16<T>(t0, t1);
      const uint32_t b0 = (uint32_t)(int)cvt16<T>((u16)(pk & 0xffff)) & 0xffu;
      const uint32_t b1 = (uint32_t)(int)cvt16<T>((u16)(pk >> 16)) & 0xffu;
      code[j] = b0 | (b1 << 8);
    }
    *(uint2*)(q + c * AQ_VEC) = make_uint2(code[0] | (code[1] << 16), code[2] | (code[3] << 16));
  }
}

// ---------------------------------------------------------------------------- FP8 emulation
// Multiplicative scale of max_to_scale: 448 / clamp(amax, 1e-12) where torch evaluates
// "number / tensor" as reciprocal-then-multiply in T and clamps to the fp16 maximum for T = fp16.
template <int T>
__device__ __forceinline__ float fp8e_scale(float amax) {
  const float c = fmaxf(amax, round_to<T>(1e-12f));  // rnd_f16(1e-12) == 0
  const float r = round_to<T>(1.0f / c);
  float s = round_to<T>(r * 448.0f);
  if constexpr (T == FMSMO_F16) s = fminf(s, 65504.0f);
  return s;
}

template <int T>
__device__ __forceinline__ void fp8e_chunk(const float (&v)[8], float s, bool scaled, void* y,
                                           size_t yo, uint8_t* q, size_t qo) {
  uint8_t b[8];
  float o[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    float t = scaled ? round_to<T>(v[i] * s) : v[i];
    t = fminf(fmaxf(t, -448.0f), 448.0f);
    if (v[i] != v[i]) t = v[i];  // torch.clamp keeps NaN
    b[i] = f32_to_e4m3_sw(t);
    const float f = __builtin_amdgcn_cvt_f32_fp8((int)b[i], 0);
    o[i] = scaled ? round_to<T>(f / s) : f;
  }
  if (q) store8(q, qo, b);
  if (y) {
    if constexpr (T == FMSMO_F32) {
      *(float4*)((float*)y + yo) = make_float4(o[0], o[1], o[2], o[3]);
      *(float4*)((float*)y + yo + 4) = make_float4(o[4], o[5], o[6], o[7]);
    } else {
      uint4 w;
      w.x = pack16<T>(o[0], o[1]); w.y = pack16<T>(o[2], o[3]);
      w.z = pack16<T>(o[4], o[5]); w.w = pack16<T>(o[6], o[7]);
      *(uint4*)((u16*)y + yo) = w;
    }
  }
}

// one block per row: the row abs-max, its scale, then the row again (it is still in L2)
template <int T>
__global__ __launch_bounds__(256) void fake_quant_fp8_rows_kernel(const void* __restrict__ x, int64_t ldx,
                                                                  void* __restrict__ y, int64_t ldy,
                                                                  uint8_t* __restrict__ q, int64_t ldq,
                                                                  float* __restrict__ scale,
                                                                  float* __restrict__ inv_scale, int K) {
  __shared__ float red[4];
  const int64_t m = blockIdx.x;
  const int nchunk = K / AQ_VEC;
  float a = 0.0f;
  for (int c = threadIdx.x; c < nchunk; c += 256) {
    float v[8];
    load8<T>(x, (size_t)(m * ldx + (int64_t)c * AQ_VEC), v);
#pragma unroll
    for (int i = 0; i < 8; ++i) a = fmaxf(a, fabsf(v[i]));
  }
  a = wave_max(a);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = a;
  __syncthreads();
  a = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  const float s = fp8e_scale<T>(a);
  if (threadIdx.x == 0) {
    if (scale) scale[m] = s;
    if (inv_scale) inv_scale[m] = 1.0f / s;
  }
  for (int c = threadIdx.x; c < nchunk; c += 256) {
    float v[8];
    load8<T>(x, (size_t)(m * ldx + (int64_t)c * AQ_VEC), v);
    fp8e_chunk<T>(v, s, true, y, (size_t)(m * ldy + (int64_t)c * AQ_VEC), q,
                  (size_t)(m * ldq + (int64_t)c * AQ_VEC));
  }
}

template <int T>
__global__ __launch_bounds__(256) void fp8e_tensor_scale_kernel(const float* __restrict__ col_amax, int K,
                                                                float* __restrict__ scale,
                                                                float* __restrict__ inv_scale) {
  __shared__ float red[4];
  float a = 0.0f;
  for (int k = threadIdx.x; k < K; k += 256) a = fmaxf(a, col_amax[k]);
  a = wave_max(a);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = a;
  __syncthreads();
  if (threadIdx.x == 0) {
    a = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    const float s = fp8e_scale<T>(a);
    scale[0] = s;
    if (inv_scale) inv_scale[0] = 1.0f / s;
  }
}

// saturating cast (scale == nullptr) or one scale for the whole tensor (scale[0])
template <int T>
__global__ __launch_bounds__(256) void fake_quant_fp8_tensor_kernel(const void* __restrict__ x, int64_t ldx,
                                                                    const float* __restrict__ scale,
                                                                    void* __restrict__ y, int64_t ldy,
                                                                    uint8_t* __restrict__ q, int64_t ldq,
                                                                    int M, int K) {
  const int cpr = K / AQ_VEC;
  const int64_t total = (int64_t)M * cpr;
  const float s = scale ? scale[0] : 1.0f;
  for (int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x; c < total; c += (int64_t)gridDim.x * 256) {
    const int64_t m = c / cpr;
    const int k = (int)(c - m * cpr) * AQ_VEC;
    float v[8];
    load8<T>(x, (size_t)(m * ldx + k), v);
    fp8e_chunk<T>(v, s, scale != nullptr, y, (size_t)(m * ldy + k), q, (size_t)(m * ldq + k));
  }
}

}  // namespace fmsmo

using namespace fmsmo;

int fmsmo_check_launch();

namespace {
bool al16(const void* p) { return (((uintptr_t)p) & 15) == 0; }
unsigned grid_for(int64_t M, int64_t K) {
  const int64_t blocks = (M * (K / AQ_VEC) + 255) / 256;
  return (unsigned)(blocks < 1 ? 1 : blocks > 8192 ? 8192 : blocks);
}
// Host-side rounding of a float to fp16 / bf16 (nearest even) and back.
float host_round16(float f, int t) {
  if (t == FMSMO_F16) return (float)(_Float16)f;
  uint32_t u;
  __builtin_memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return f;  // NaN
  u += 0x7fffu + ((u >> 16) & 1u);
  u &= 0xffff0000u;
  __builtin_memcpy(&f, &u, 4);
  return f;
}
// Parameters the fast 16-bit static quantizer covers (see quant_i8_static16_kernel).
bool static16_ok(const StaticArgs& p, int t) {
  const float s = fabsf(p.scale);
  if (!(s > 0.0f) || !(s < INFINITY) || host_round16(p.scale, t) != p.scale) return false;
  if (t == FMSMO_BF16 && !(s >= 8.6736174e-19f && s <= 1.1529215e18f)) return false;
  if (!(fabsf(p.zp) < 1.0e6f)) return false;
  if (p.mode == FMSMO_SQ_FMO) {
    // codes are not clamped: |clamp(x) / scale - zp| must stay far inside 2^22, and finite in T
    // (an fp16 quotient that overflows to inf takes the generic kernel's conversion of inf)
    const float m = fmaxf(fabsf(p.lo), fabsf(p.hi));
    if (!(m < INFINITY) || !(m / s + fabsf(p.zp) < (t == FMSMO_F16 ? 6.0e4f : 1.0e6f))) return false;
  }
  return true;
}
int check_rows(const void* x, int x_dtype, int64_t ldx, int64_t M, int64_t K) {
  if (!x) return FMSMO_ERR_NULL;
  if (M < 0 || K <= 0 || ldx < K || M > 0x7fffffff || K > 0x7fffffff) return FMSMO_ERR_SHAPE;
  if (x_dtype < 0 || x_dtype > 2) return FMSMO_ERR_UNSUPPORTED;
  if (K % 8 || ldx % 8 || !al16(x)) return FMSMO_ERR_ALIGN;
  return FMSMO_OK;
}
}  // namespace

extern "C" int fmsmo_quant_act_i8_static_t(const void* x, int x_dtype, int64_t ldx, int mode,
                                           int compute_dtype, float scale, float zp, int sym,
                                           float clip_lo, float clip_hi, int8_t* q, int64_t ldq,
                                           int64_t M, int64_t K, fmsmo_stream_t stream) {
  int rc = check_rows(x, x_dtype, ldx, M, K);
  if (rc) return rc;
  if (!q) return FMSMO_ERR_NULL;
  if (ldq < K) return FMSMO_ERR_SHAPE;
  if (ldq % 8 || (((uintptr_t)q) & 7)) return FMSMO_ERR_ALIGN;
  if (mode < FMSMO_SQ_RAW || mode > FMSMO_SQ_S8_NARROW || compute_dtype < 0 || compute_dtype > 2)
    return FMSMO_ERR_UNSUPPORTED;
  // torch's promotion of x's dtype with the scale's: x's own dtype or fp32
  if (compute_dtype != FMSMO_F32 && compute_dtype != x_dtype) return FMSMO_ERR_UNSUPPORTED;
  if (M == 0) return FMSMO_OK;
  StaticArgs p{scale, zp, (float)(sym ? 1 : 0), clip_lo, clip_hi, mode};
  dim3 grid(grid_for(M, K)), block(256);
  hipStream_t st = (hipStream_t)stream;
  // 16-bit compute dtype, contiguous rows, a divisor that is a finite non-zero value of that dtype
  // (inside 2^-60 .. 2^60 for bf16) and, for the formula that does not clamp its codes, clip values
  // whose quotients stay small: the fast kernel.  Anything else takes the generic one below.
  if (compute_dtype != FMSMO_F32 && ldx == K && ldq == K && static16_ok(p, compute_dtype)) {
    const int64_t nchunks = M * (K / AQ_VEC);
    const float rcp = 1.0f / scale;  // correctly rounded: at least as good as the device's rcp
#define FAST(T, MD)                                                                            \
  hipLaunchKernelGGL((quant_i8_static16_kernel<T, MD>), grid, block, 0, st, (const u16*)x, p, rcp, \
                     q, nchunks)
#define FAST_T(T)                                        \
  switch (mode) {                                        \
    case FMSMO_SQ_RAW: FAST(T, FMSMO_SQ_RAW); break;     \
    case FMSMO_SQ_FMO: FAST(T, FMSMO_SQ_FMO); break;     \
    case FMSMO_SQ_U8_SHIFT: FAST(T, FMSMO_SQ_U8_SHIFT); break; \
    default: FAST(T, FMSMO_SQ_S8_NARROW); break;         \
  }
    if (x_dtype == FMSMO_F16) { FAST_T(FMSMO_F16) } else { FAST_T(FMSMO_BF16) }
#undef FAST_T
#undef FAST
    return fmsmo_check_launch();
  }
#define LAUNCH(XT, T) \
  hipLaunchKernelGGL((quant_i8_static_t_kernel<XT, T>), grid, block, 0, st, x, ldx, p, q, ldq, (int)M, (int)K)
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

extern "C" int fmsmo_quant_act_i8_dynamic(const void* x, int x_dtype, int64_t ldx,
                                          const float* col_amax, int granularity, int levels,
                                          int zp, int8_t* q, int64_t ldq, float* scale, int64_t M,
                                          int64_t K, fmsmo_stream_t stream) {
  int rc = check_rows(x, x_dtype, ldx, M, K);
  if (rc) return rc;
  if (!q || !col_amax || !scale) return FMSMO_ERR_NULL;
  if (ldq < K || levels <= 0) return FMSMO_ERR_SHAPE;
  if (ldq % 8 || (((uintptr_t)q) & 7) || !al16(scale)) return FMSMO_ERR_ALIGN;
  if (granularity != FMSMO_DQ_PER_TENSOR && granularity != FMSMO_DQ_PER_COLUMN) return FMSMO_ERR_UNSUPPORTED;
  const int pc = granularity == FMSMO_DQ_PER_COLUMN;
  dim3 sgrid(pc ? (unsigned)((K + 255) / 256) : 1u), grid(grid_for(M, K)), block(256);
  hipStream_t st = (hipStream_t)stream;
#define LAUNCH(T)                                                                               \
  {                                                                                             \
    hipLaunchKernelGGL((dyn_scale_kernel<T>), sgrid, block, 0, st, col_amax, (int)K, pc,        \
                       (float)levels, scale);                                                   \
    if (M > 0) {                                                                                \
      if (T != FMSMO_F32 && !pc && ldx == K && ldq == K)                                        \
        hipLaunchKernelGGL((quant_i8_dynamic16_kernel<T == FMSMO_F32 ? FMSMO_F16 : T>), grid, block, 0, st, \
                           (const u16*)x, (const float*)scale, (float)zp, q, M * (K / AQ_VEC)); \
      else                                                                                      \
        hipLaunchKernelGGL((quant_i8_dynamic_kernel<T>), grid, block, 0, st, x, ldx,            \
                           (const float*)scale, pc, (float)zp, q, ldq, (int)M, (int)K);         \
    }                                                                                           \
  }
  switch (x_dtype) {
    case FMSMO_F16: LAUNCH(FMSMO_F16) break;
    case FMSMO_BF16: LAUNCH(FMSMO_BF16) break;
    default: LAUNCH(FMSMO_F32) break;
  }
#undef LAUNCH
  return fmsmo_check_launch();
}

extern "C" int fmsmo_fake_quant_fp8(const void* x, int x_dtype, int64_t ldx, int mode,
                                    const float* col_amax, void* y, int64_t ldy, uint8_t* q,
                                    int64_t ldq, float* scale, float* inv_scale, int64_t M,
                                    int64_t K, fmsmo_stream_t stream) {
  int rc = check_rows(x, x_dtype, ldx, M, K);
  if (rc) return rc;
  if (!y && !q) return FMSMO_ERR_NULL;
  if (mode < FMSMO_F8E_SAT || mode > FMSMO_F8E_PER_ROW) return FMSMO_ERR_UNSUPPORTED;
  if (mode == FMSMO_F8E_PER_TENSOR && (!col_amax || !scale)) return FMSMO_ERR_NULL;
  if ((y && ldy < K) || (q && ldq < K)) return FMSMO_ERR_SHAPE;
  if ((y && (ldy % 8 || !al16(y))) || (q && (ldq % 8 || (((uintptr_t)q) & 7)))) return FMSMO_ERR_ALIGN;
  hipStream_t st = (hipStream_t)stream;
  dim3 block(256);
#define LAUNCH(T)                                                                                  \
  {                                                                                                \
    if (mode == FMSMO_F8E_PER_ROW) {                                                               \
      if (M > 0)                                                                                   \
        hipLaunchKernelGGL((fake_quant_fp8_rows_kernel<T>), dim3((unsigned)M), block, 0, st, x,    \
                           ldx, y, ldy, q, ldq, scale, inv_scale, (int)K);                         \
    } else {                                                                                       \
      if (mode == FMSMO_F8E_PER_TENSOR)                                                            \
        hipLaunchKernelGGL((fp8e_tensor_scale_kernel<T>), dim3(1), block, 0, st, col_amax, (int)K, \
                           scale, inv_scale);                                                      \
      if (M > 0)                                                                                   \
        hipLaunchKernelGGL((fake_quant_fp8_tensor_kernel<T>), dim3(grid_for(M, K)), block, 0, st,  \
                           x, ldx, mode == FMSMO_F8E_PER_TENSOR ? (const float*)scale : nullptr,   \
                           y, ldy, q, ldq, (int)M, (int)K);                                        \
    }                                                                                              \
  }
  switch (x_dtype) {
    case FMSMO_F16: LAUNCH(FMSMO_F16) break;
    case FMSMO_BF16: LAUNCH(FMSMO_BF16) break;
    default: LAUNCH(FMSMO_F32) break;
  }
#undef LAUNCH
  return fmsmo_check_launch();
}
