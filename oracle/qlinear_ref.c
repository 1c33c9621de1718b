/*
 * C restatement of the bit-level pieces of the reference's quantized-linear arithmetic.
 * TEST INFRASTRUCTURE ONLY: loaded by tests/ (ctypes) to cross-check the torch restatement in
 * qlinear_oracle.py with an independent implementation; never linked into the product.
 *
 * Each function cites the file:line of foundation-model-stack/fms-model-optimizer it follows.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

/* ---- IEEE helpers: round an fp32 value to the fp16 / bf16 grid (round-to-nearest-even) ---- */
static float bits_f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static uint32_t f_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

float ref_round_bf16(float f) {
  uint32_t u = f_bits(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return f;
  u += 0x7fffu + ((u >> 16) & 1u);
  return bits_f(u & 0xffff0000u);
}

float ref_round_f16(float f) {
  /* scale into the fp16 grid: values < 2^-14 use the fixed subnormal quantum 2^-24 */
  if (isnan(f) || isinf(f)) return f;
  float a = fabsf(f);
  if (a >= 65520.0f) return copysignf(INFINITY, f);
  int e;
  frexpf(a, &e); /* a = m * 2^e, m in [0.5,1) */
  int qexp = (a < 6.103515625e-05f) ? -24 : (e - 11); /* quantum = 2^qexp */
  float q = ldexpf(1.0f, qexp);
  float r = nearbyintf(a / q) * q; /* exact scaling, RNE under the default rounding mode */
  return copysignf(r, f);
}

static float round_T(float f, int T) { return T == 0 ? ref_round_f16(f) : (T == 1 ? ref_round_bf16(f) : f); }

/*
 * Per-token dynamic int8 quantizer, qa_dynamic_max_qfunc (fms_mo/modules/linear.py:1095-1100):
 *   amax = max|x|; scale = rnd_T(max(amax, rnd_T(1e-5)) / 127); q = wrap8(rint(rnd_T(x / scale)))
 * x holds values already on the T grid (as fp32).  T: 0 fp16, 1 bf16, 2 fp32.
 */
void ref_quant_act_pertoken(const float* x, int M, int K, int T, int8_t* q, float* scale) {
  for (int m = 0; m < M; ++m) {
    float amax = 0.f;
    for (int k = 0; k < K; ++k) amax = fmaxf(amax, fabsf(x[(size_t)m * K + k]));
    float s = round_T(fmaxf(amax, round_T(1e-5f, T)) / 127.0f, T);
    scale[m] = s;
    for (int k = 0; k < K; ++k) {
      float r = nearbyintf(round_T(x[(size_t)m * K + k] / s, T));
      q[(size_t)m * K + k] = (int8_t)(uint8_t)(int)r; /* 128 -> 0x80 */
    }
  }
}

/* Exact int32 GEMM, C = A[M,K] . B[N,K]^T (cutlass_i8i32gemm.cu:29-62). */
void ref_gemm_i8(const int8_t* a, const int8_t* b, int M, int N, int K, int32_t* c) {
  for (int m = 0; m < M; ++m)
    for (int n = 0; n < N; ++n) {
      int32_t acc = 0;
      for (int k = 0; k < K; ++k) acc += (int32_t)a[(size_t)m * K + k] * (int32_t)b[(size_t)n * K + k];
      c[(size_t)m * N + n] = acc;
    }
}

/* Epilogue of iaddmm_int (linear.py:1185-1188): f16( f32(acc) * f32(f16(sa*sw)) + bias ). */
float ref_epilogue(int32_t acc, float sa, float sw, float bias) {
  float sc = ref_round_f16(sa * sw);
  volatile float prod = (float)acc * sc; /* separate multiply and add */
  return ref_round_f16(prod + bias);
}

/* round_and_trun (fms_mo/custom_ext_kernels/triton_kernels.py:432-465) on one fp32 value. */
float ref_round_and_trun(float p, int t, int dl16) {
  if (dl16) t = 14;
  uint32_t rb = t > 0 ? (1u << (t - 1)) : 0u;
  uint32_t mask = ~((1u << t) - 1u);
  float x = bits_f((f_bits(p) + rb) & mask);
  if (dl16) {
    if (x >= 8581545984.0f) x = INFINITY;
    if (x <= -8581545984.0f) x = -INFINITY;
    if (fabsf(x) < 4.665707820095122e-10f) x = 0.0f;
  }
  return x;
}

/* Chunked int8 matmul, imatmul_kernel (triton_kernels.py:262-302), truncate_then_accumulate. */
void ref_chunk_i8(const int8_t* a, const int8_t* b, int M, int N, int K, int chunk, int t, int bits,
                  int32_t* d) {
  int32_t lo = bits < 32 ? -(1 << (bits - 1)) : INT32_MIN, hi = bits < 32 ? (1 << (bits - 1)) - 1 : INT32_MAX;
  for (int m = 0; m < M; ++m)
    for (int n = 0; n < N; ++n) {
      uint32_t acc = 0;
      for (int k0 = 0; k0 < K; k0 += chunk) {
        int32_t p = 0;
        for (int k = k0; k < K && k < k0 + chunk; ++k)
          p += (int32_t)a[(size_t)m * K + k] * (int32_t)b[(size_t)n * K + k];
        if (p < lo) p = lo;
        if (p > hi) p = hi;
        if (t) {
          int32_t r = (int32_t)((uint32_t)p + (1u << (t - 1)));
          p = (int32_t)((uint32_t)(r >> t) << t);
        }
        acc += (uint32_t)p;
      }
      d[(size_t)m * N + n] = (int32_t)acc;
    }
}

/* OCP e4m3fn encode with torch's cast semantics (RNE; |x| > 464 or NaN -> 0x7f). */
uint8_t ref_e4m3(float f) {
  uint32_t u = f_bits(f);
  uint8_t sign = (u >> 24) & 0x80;
  float a = fabsf(f);
  if (!(a <= 464.0f)) return sign | 0x7f;
  if (a < 0.015625f) return sign | (uint8_t)nearbyintf(a * 512.0f); /* subnormals, quantum 2^-9 */
  int e;
  float m = frexpf(a, &e); /* a = m 2^e, m in [0.5,1) -> 1.xxx * 2^(e-1) */
  float r = nearbyintf(m * 16.0f); /* 8..16 */
  if (r == 16.0f) { r = 8.0f; e += 1; }
  int ef = e - 1 + 7;
  return sign | (uint8_t)((ef << 3) | ((int)r - 8));
}
