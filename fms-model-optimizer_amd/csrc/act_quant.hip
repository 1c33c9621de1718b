// Fused activation quantizers: one pass over x (read 2-4 B, write 1 B per element).
//
// One 256-thread block per token row.  The row is pulled from HBM once with 16-byte loads and
// kept in registers while the block reduces |x| (wave butterfly + one LDS exchange); the scale
// is then formed and the row is quantized straight from registers and written with 8-byte
// (int8 / e4m3) stores.  Rows longer than 16384 elements are read a second time (L2 hit).
//
// Every division is IEEE correctly rounded in fp32 on operands widened from the compute dtype T
// and then rounded to T, which equals the correctly rounded T division torch performs.
#include "common.hpp"

namespace fmsmo {

constexpr int AQ_THREADS = 256;
constexpr int AQ_VEC = 8;        // elements per thread per chunk
constexpr int AQ_MAXCHUNK = 8;   // chunks cached in registers per thread

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

__device__ __forceinline__ float load_any(const void* p, int dtype, size_t i) {
  if (dtype == FMSMO_F16) return f16_to_f32(((const u16*)p)[i]);
  if (dtype == FMSMO_BF16) return bf16_to_f32(((const u16*)p)[i]);
  return ((const float*)p)[i];
}

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

__device__ __forceinline__ void store8(uint8_t* q, size_t elem, const uint8_t (&b)[8]) {
  uint2 o;
  o.x = b[0] | (b[1] << 8) | (b[2] << 16) | ((uint32_t)b[3] << 24);
  o.y = b[4] | (b[5] << 8) | (b[6] << 16) | ((uint32_t)b[7] << 24);
  *(uint2*)(q + elem) = o;
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
#pragma unroll
      for (int i = 0; i < 8; ++i)
        e[i] = round_to<T>(e[i] / load_any(smooth, smooth_dtype, (size_t)c * AQ_VEC + i));
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

// ------------------------------------------------------------------ int8, static per tensor
template <int XT>
__global__ __launch_bounds__(AQ_THREADS) void quant_i8_static_kernel(
    const void* __restrict__ x, int64_t ldx, float scale, float zp, float sym, int pt_native,
    int8_t* __restrict__ q, int64_t ldq, int K) {
  const int row = blockIdx.x;
  const int nchunk = K / AQ_VEC;
  const float inv_scale = 1.0f / scale;
  for (int c = threadIdx.x; c < nchunk; c += AQ_THREADS) {
    float e[8];
    load8<XT>(x, (size_t)row * ldx + (size_t)c * AQ_VEC, e);
    uint8_t b[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      // ((x/s + zp) - 128) + sym, each step rounded to fp32, then round-half-even and clamp
      float t;
      if (pt_native)  // torch.quantize_per_tensor: rint(x * (1/scale)) + zero_point
        t = __builtin_rintf(__fmul_rn(e[j], inv_scale)) + (zp - 128.0f + sym);
      else
        t = __builtin_rintf(__fadd_rn(__fadd_rn(__fadd_rn(e[j] / scale, zp), -128.0f), sym));
      t = fminf(fmaxf(t, -128.0f), 127.0f);
      b[j] = (uint8_t)(int)t;
    }
    store8((uint8_t*)q, (size_t)row * ldq + (size_t)c * AQ_VEC, b);
  }
}

// ------------------------------------------------------------------ e4m3, per token
template <int XT>
__global__ __launch_bounds__(AQ_THREADS) void quant_fp8_pertoken_kernel(
    const void* __restrict__ x, int64_t ldx, int variant, int static_scale,
    uint8_t* __restrict__ q, int64_t ldq, float* __restrict__ scale, int K) {
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
    if (variant == FMSMO_FP8_LINEAR) {
      s = fmaxf(amax / 448.0f, 1e-12f);
    } else {
      // (amax / 448) in x's dtype, then clamp(min=1e-5): the clamp bound is a python scalar,
      // so the result stays in x's dtype -> max against 1e-5 rounded to that dtype
      s = fmaxf(round_to<XT>(amax / 448.0f), round_to<XT>(1e-5f));
    }
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

}  // namespace fmsmo

using namespace fmsmo;

extern thread_local char g_fmsmo_last_error[256];
int fmsmo_check_launch();

static bool aligned16(const void* p) { return (((uintptr_t)p) & 15) == 0; }

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
  if (M == 0) return FMSMO_OK;
  hipStream_t st = (hipStream_t)stream;
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

extern "C" int fmsmo_quant_act_fp8_pertoken(const void* x, int x_dtype, int64_t ldx, int variant,
                                            int static_scale, uint8_t* q, int64_t ldq,
                                            float* scale, int64_t M, int64_t K,
                                            fmsmo_stream_t stream) {
  if (!x || !q || !scale) return FMSMO_ERR_NULL;
  if (M < 0 || K <= 0 || ldx < K || ldq < K || M > 0x7fffffff || K > 0x7fffffff) return FMSMO_ERR_SHAPE;
  if (x_dtype < 0 || x_dtype > 2 || variant < 0 || variant > 2) return FMSMO_ERR_UNSUPPORTED;
  if (K % 8 || ldx % 8 || ldq % 8 || !aligned16(x) || (((uintptr_t)q) & 7)) return FMSMO_ERR_ALIGN;
  if (M == 0) return FMSMO_OK;
  hipStream_t st = (hipStream_t)stream;
  dim3 grid((unsigned)M), block(AQ_THREADS);
#define LAUNCH(XT)                                                                             \
  hipLaunchKernelGGL((quant_fp8_pertoken_kernel<XT>), grid, block, 0, st, x, ldx, variant,     \
                     static_scale, q, ldq, scale, (int)K)
  switch (x_dtype) {
    case FMSMO_F16: LAUNCH(FMSMO_F16); break;
    case FMSMO_BF16: LAUNCH(FMSMO_BF16); break;
    default: LAUNCH(FMSMO_F32); break;
  }
#undef LAUNCH
  return fmsmo_check_launch();
}
