// Offline weight path: fp16 / bf16 / fp32 weights -> int8 rows (+ per-row integer sums).
//
//   t_nk = rnd_T1( W_nk * smooth_k )                      (SmoothQuant folding, optional)
//   mode FMSMO_WQ_MUL:  q_nk = rint( clamp( rnd_T2( coef_n * t_nk ), -127, 127 ) )
//   mode FMSMO_WQ_DIV:  q_nk = clamp( rint( rnd_T2( t_nk / coef_n ) ), -127, 127 )
//   row_sum_n = sum_k q_nk                                 (the "zero shift" of asymmetric activations)
//
// T1 = promote(weight dtype, smooth dtype), T2 = promote(T1, coef dtype): the dtypes in which torch
// evaluates the two expressions.  One 256-thread block per weight row, 16-byte loads, 8-byte
// stores; read 2-4 B and write 1 B per element (HBM bound, offline).
#include "common.hpp"

#include <type_traits>

namespace fmsmo {

__device__ __forceinline__ float round_dyn(float v, int t) {
  return t == FMSMO_F16 ? round_to<FMSMO_F16>(v) : t == FMSMO_BF16 ? round_to<FMSMO_BF16>(v) : v;
}
__device__ __forceinline__ float load_dyn(const void* p, int t, size_t i) {
  return t == FMSMO_F16 ? f16_to_f32(((const u16*)p)[i])
         : t == FMSMO_BF16 ? bf16_to_f32(((const u16*)p)[i])
                           : ((const float*)p)[i];
}

// 8 consecutive elements of a dtype known at run time, widened to fp32
__device__ __forceinline__ void load8_dyn(const void* p, int t, size_t i, float (&v)[8]) {
  if (t == FMSMO_F32) {
    const float4 a = *(const float4*)((const float*)p + i);
    const float4 b = *(const float4*)((const float*)p + i + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
  } else {
    const uint4 r = *(const uint4*)((const u16*)p + i);
    const uint32_t ww[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const u16 h = (u16)(ww[j >> 1] >> ((j & 1) * 16));
      v[j] = t == FMSMO_F16 ? f16_to_f32(h) : bf16_to_f32(h);
    }
  }
}

template <int WT>
__global__ __launch_bounds__(256) void quant_weight_i8_kernel(
    const void* __restrict__ w, int64_t ldw, const void* __restrict__ smooth, int smooth_dtype,
    const void* __restrict__ coef, int coef_dtype, int coef_stride, int t1, int t2, int mode,
    int8_t* __restrict__ q, int64_t ldq, int32_t* __restrict__ row_sum, int K) {
  __shared__ int red[4];
  const int row = blockIdx.x;
  const float c = load_dyn(coef, coef_dtype, coef_stride ? row : 0);
  int sum = 0;
  constexpr int U = 4;  // 16-byte groups in flight per thread
  typedef typename std::conditional<WT == FMSMO_F32, float4, uint4>::type Raw;
  for (int kb = threadIdx.x * 8; kb < K; kb += U * 256 * 8) {
    Raw ra[U], rb[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int k0 = kb + u * 256 * 8;
      if (k0 < K) {
        if constexpr (WT == FMSMO_F32) {
          ra[u] = *(const float4*)((const float*)w + (size_t)row * ldw + k0);
          rb[u] = *(const float4*)((const float*)w + (size_t)row * ldw + k0 + 4);
        } else {
          ra[u] = *(const uint4*)((const u16*)w + (size_t)row * ldw + k0);
        }
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int k0 = kb + u * 256 * 8;
      if (k0 >= K) break;
      float v[8];
      if constexpr (WT == FMSMO_F32) {
        v[0] = ra[u].x; v[1] = ra[u].y; v[2] = ra[u].z; v[3] = ra[u].w;
        v[4] = rb[u].x; v[5] = rb[u].y; v[6] = rb[u].z; v[7] = rb[u].w;
      } else {
        const uint32_t ww[4] = {ra[u].x, ra[u].y, ra[u].z, ra[u].w};
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const u16 h = (u16)(ww[i >> 1] >> ((i & 1) * 16));
          v[i] = WT == FMSMO_F16 ? f16_to_f32(h) : bf16_to_f32(h);
        }
      }
      float sm[8];
      if (smooth) load8_dyn(smooth, smooth_dtype, (size_t)k0, sm);
      uint32_t o[2] = {0, 0};
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        float t = v[i];
        if (smooth) t = round_dyn(__fmul_rn(t, sm[i]), t1);
        float r;
        if (mode == FMSMO_WQ_MUL) {
          r = __builtin_rintf(fminf(fmaxf(round_dyn(__fmul_rn(c, t), t2), -127.0f), 127.0f));
        } else {
          r = fminf(fmaxf(__builtin_rintf(round_dyn(t / c, t2)), -127.0f), 127.0f);
        }
        const int qi = (int)r;
        sum += qi;
        o[i >> 2] |= ((uint32_t)qi & 0xffu) << ((i & 3) * 8);
      }
      *(uint2*)(q + (size_t)row * ldq + k0) = make_uint2(o[0], o[1]);
    }
  }
  if (row_sum) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = sum;
    __syncthreads();
    if (threadIdx.x == 0) row_sum[row] = red[0] + red[1] + red[2] + red[3];
  }
}

// Per-column running abs-max:  out_k = max( out_k, max_m |x_mk| ).  A block covers 512 columns
// (64 lanes x 8) and a slab of rows shared out over its four waves, merged through LDS; |x| >= 0 orders like its bit pattern, so the slabs merge
// with an unsigned atomic max on the fp32 bits (a NaN, whose pattern is above infinity's, wins).
template <int XT>
__global__ __launch_bounds__(256) void absmax_cols_kernel(const void* __restrict__ x, int64_t ldx,
                                                          int M, int K, int rows_per_block,
                                                          uint32_t* __restrict__ out) {
  __shared__ uint32_t part[3][64][8];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int k0 = (blockIdx.x * 64 + lane) * 8;
  const bool live = k0 < K;
  // the four waves of a block take interleaved groups of U rows of the block's slab
  constexpr int U = 8;  // rows in flight per thread
  const int mb = blockIdx.y * rows_per_block, m1 = min(M, mb + rows_per_block);
  const int m0 = mb + wave * U;
  uint32_t bits[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  if (!live) {
  } else if constexpr (XT == FMSMO_F32) {
    float best[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int m = m0; m < m1; m += 4 * U) {
      float4 a[U], b[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int r = min(m + u, m1 - 1);  // the tail re-reads the last row
        a[u] = *(const float4*)((const float*)x + (size_t)r * ldx + k0);
        b[u] = *(const float4*)((const float*)x + (size_t)r * ldx + k0 + 4);
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const float v[8] = {a[u].x, a[u].y, a[u].z, a[u].w, b[u].x, b[u].y, b[u].z, b[u].w};
#pragma unroll
        for (int i = 0; i < 8; ++i) best[i] = fmaxf(best[i], fabsf(v[i]));
      }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) bits[i] = __float_as_uint(best[i]);
  } else {
    // 15-bit magnitudes of non-NaN 16-bit floats order like unsigned integers: packed maxima
    typedef unsigned short us2 __attribute__((ext_vector_type(2)));
    us2 best[4] = {{0, 0}, {0, 0}, {0, 0}, {0, 0}};
    for (int m = m0; m < m1; m += 4 * U) {
      uint4 r[U];
#pragma unroll
      for (int u = 0; u < U; ++u)
        r[u] = *(const uint4*)((const u16*)x + (size_t)min(m + u, m1 - 1) * ldx + k0);
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const uint32_t w[4] = {r[u].x, r[u].y, r[u].z, r[u].w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const uint32_t mag = w[i] & 0x7fff7fffu;
          us2 m2;
          __builtin_memcpy(&m2, &mag, 4);
          best[i] = __builtin_elementwise_max(best[i], m2);
        }
      }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const u16 h = best[i >> 1][i & 1];
      const float v = XT == FMSMO_F16 ? f16_to_f32(h) : bf16_to_f32(h);
      bits[i] = __float_as_uint(v);
    }
  }
  // merge the four waves, then one atomic per column and block
  if (wave > 0) {
#pragma unroll
    for (int i = 0; i < 8; ++i) part[wave - 1][lane][i] = bits[i];
  }
  __syncthreads();
  if (wave == 0 && live) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      uint32_t b = bits[i];
#pragma unroll
      for (int w = 0; w < 3; ++w) b = max(b, part[w][lane][i]);
      atomicMax(out + k0 + i, b);
    }
  }
}

// Bias with the zero-point correction of asymmetric activations folded in:
//   out_n = bias_n + (offset + a_meta[1]) * (sum_k w_nk) * a_meta[0] * w_scale_n
// a_meta = { 1 / activation scale, activation zero point } as left on the device by the
// activation quantizer; one wavefront per weight row, 16-byte loads, integer row sums.
__global__ __launch_bounds__(256) void zero_shift_bias_kernel(
    const int8_t* __restrict__ w, int64_t ldw, const float* __restrict__ w_scale, int w_scale_n,
    const float* __restrict__ a_meta, float offset, const void* __restrict__ bias, int bias_dtype,
    float* __restrict__ out, int N, int K) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= N) return;
  int sum = 0;
  for (int k0 = lane * 16; k0 < K; k0 += 64 * 16) {
    const uint4 r = *(const uint4*)(w + (size_t)row * ldw + k0);
    sum = __builtin_amdgcn_sdot4((int)r.x, 0x01010101, sum, false);
    sum = __builtin_amdgcn_sdot4((int)r.y, 0x01010101, sum, false);
    sum = __builtin_amdgcn_sdot4((int)r.z, 0x01010101, sum, false);
    sum = __builtin_amdgcn_sdot4((int)r.w, 0x01010101, sum, false);
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o, 64);
  if (lane == 0) {
    const float b = bias ? load_dyn(bias, bias_dtype, row) : 0.0f;
    const float ws = w_scale[w_scale_n > 1 ? row : 0];
    out[row] = b + (offset + a_meta[1]) * (float)sum * a_meta[0] * ws;
  }
}

}  // namespace fmsmo

using namespace fmsmo;
int fmsmo_check_launch();

static int promote(int a, int b) {
  if (a == b) return a;
  return FMSMO_F32;  // fp16 with bf16, or anything with fp32
}

extern "C" int fmsmo_quant_weight_i8(const void* w, int w_dtype, int64_t ldw, const void* smooth,
                                     int smooth_dtype, const void* coef, int coef_dtype,
                                     int64_t coef_n, int mode, int8_t* q, int64_t ldq,
                                     int32_t* row_sum, int64_t N, int64_t K,
                                     fmsmo_stream_t stream) {
  if (!w || !coef || !q) return FMSMO_ERR_NULL;
  if (N <= 0 || K <= 0 || ldw < K || ldq < K || N > 0x7fffffff || K > 0x7fffffff) return FMSMO_ERR_SHAPE;
  if (coef_n != 1 && coef_n != N) return FMSMO_ERR_SHAPE;
  if (w_dtype < 0 || w_dtype > 2 || coef_dtype < 0 || coef_dtype > 2 ||
      (smooth && (smooth_dtype < 0 || smooth_dtype > 2)) || (mode != FMSMO_WQ_MUL && mode != FMSMO_WQ_DIV))
    return FMSMO_ERR_UNSUPPORTED;
  if (K % 8 || ldw % 8 || ldq % 8 || (((uintptr_t)w) & 15) || (((uintptr_t)q) & 7) ||
      (smooth && (((uintptr_t)smooth) & 15)))
    return FMSMO_ERR_ALIGN;
  const int t1 = smooth ? promote(w_dtype, smooth_dtype) : w_dtype;
  const int t2 = promote(t1, coef_dtype);
  dim3 grid((unsigned)N), block(256);
  hipStream_t st = (hipStream_t)stream;
#define LAUNCH(WT)                                                                              \
  hipLaunchKernelGGL((quant_weight_i8_kernel<WT>), grid, block, 0, st, w, ldw, smooth,          \
                     smooth_dtype, coef, coef_dtype, coef_n == 1 ? 0 : 1, t1, t2, mode, q, ldq, \
                     row_sum, (int)K)
  switch (w_dtype) {
    case FMSMO_F16: LAUNCH(FMSMO_F16); break;
    case FMSMO_BF16: LAUNCH(FMSMO_BF16); break;
    default: LAUNCH(FMSMO_F32); break;
  }
#undef LAUNCH
  return fmsmo_check_launch();
}

extern "C" int fmsmo_zero_shift_bias(const int8_t* w, int64_t ldw, const float* w_scale,
                                     int64_t w_scale_n, const float* a_meta, float offset,
                                     const void* bias, int bias_dtype, float* out, int64_t N,
                                     int64_t K, fmsmo_stream_t stream) {
  if (!w || !w_scale || !a_meta || !out) return FMSMO_ERR_NULL;
  if (N <= 0 || K <= 0 || ldw < K || N > 0x7fffffff || K > 0x7fffffff) return FMSMO_ERR_SHAPE;
  if (w_scale_n != 1 && w_scale_n != N) return FMSMO_ERR_SHAPE;
  if (bias && (bias_dtype < 0 || bias_dtype > 2)) return FMSMO_ERR_UNSUPPORTED;
  if (K % 16 || ldw % 16 || (((uintptr_t)w) & 15)) return FMSMO_ERR_ALIGN;
  hipLaunchKernelGGL(zero_shift_bias_kernel, dim3((unsigned)div_up(N, 4)), dim3(256), 0,
                     (hipStream_t)stream, w, ldw, w_scale, (int)w_scale_n, a_meta, offset, bias,
                     bias_dtype, out, (int)N, (int)K);
  return fmsmo_check_launch();
}

extern "C" int fmsmo_absmax_cols(const void* x, int x_dtype, int64_t ldx, int64_t M, int64_t K,
                                 float* out, fmsmo_stream_t stream) {
  if (!x || !out) return FMSMO_ERR_NULL;
  if (M < 0 || K <= 0 || ldx < K || M > 0x7fffffff || K > 0x7fffffff) return FMSMO_ERR_SHAPE;
  if (x_dtype < 0 || x_dtype > 2) return FMSMO_ERR_UNSUPPORTED;
  if (K % 8 || ldx % 8 || (((uintptr_t)x) & 15)) return FMSMO_ERR_ALIGN;
  if (M == 0) return FMSMO_OK;
  // enough row slabs to occupy the chip, at least 128 rows each (32 per wave)
  const int col_blocks = div_up(K, 512);
  int slabs = (int)((M + 127) / 128);
  const int want = (1024 + col_blocks - 1) / col_blocks;
  if (slabs > want) slabs = want;
  const int rows_per_block = div_up(M, slabs);
  dim3 grid(col_blocks, div_up(M, rows_per_block)), block(256);
  hipStream_t st = (hipStream_t)stream;
#define LAUNCH(XT)                                                                             \
  hipLaunchKernelGGL((absmax_cols_kernel<XT>), grid, block, 0, st, x, ldx, (int)M, (int)K,     \
                     rows_per_block, (uint32_t*)out)
  switch (x_dtype) {
    case FMSMO_F16: LAUNCH(FMSMO_F16); break;
    case FMSMO_BF16: LAUNCH(FMSMO_BF16); break;
    default: LAUNCH(FMSMO_F32); break;
  }
#undef LAUNCH
  return fmsmo_check_launch();
}
