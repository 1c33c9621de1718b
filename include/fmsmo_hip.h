/*
 * fmsmo_hip.h -- C ABI of the gfx950 (MI355X) quantized-linear kernels.
 *
 * Every entry point takes raw device pointers, element counts / leading dimensions in ELEMENTS,
 * small enums and a HIP stream handle (passed as void*; NULL = the default stream).  Nothing is
 * allocated, freed or synchronised inside the library: the caller owns inputs, outputs and
 * lifetimes, and kernels are enqueued asynchronously on the given stream.  Every function
 * returns FMSMO_OK (0) or a negative-free small error code; fmsmo_status_str() names it.
 *
 * Matrix convention (the one the reference's int8 GEMM extensions use): activations A are
 * [M,K] row-major, weights B are stored [N,K] row-major (nn.Linear layout, i.e. the memory the
 * reference's `W.t()` view points at), outputs are [M,N] row-major.
 *
 * Each declaration cites the interface of the reference (paths relative to the root of
 * foundation-model-stack/fms-model-optimizer) whose arithmetic it reproduces.
 */
#ifndef FMSMO_HIP_H_
#define FMSMO_HIP_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FMSMO_ABI_VERSION 2

typedef void* fmsmo_stream_t; /* hipStream_t */

/* 16/32-bit floating types of activations, scales, biases and outputs. */
enum { FMSMO_F16 = 0, FMSMO_BF16 = 1, FMSMO_F32 = 2 };

/* Element type of the 8-bit (or 16-bit) GEMM operands of the chunked matmul. */
enum { FMSMO_OP_I8 = 0, FMSMO_OP_E4M3 = 1, FMSMO_OP_F16 = 2, FMSMO_OP_BF16 = 3, FMSMO_OP_F32 = 4 };

/* Status codes. */
enum {
  FMSMO_OK = 0,
  FMSMO_ERR_NULL = 1,        /* a required pointer is NULL                          */
  FMSMO_ERR_SHAPE = 2,       /* negative size, leading dimension too small, ...     */
  FMSMO_ERR_ALIGN = 3,       /* pointer / leading dimension not 16-byte aligned     */
  FMSMO_ERR_UNSUPPORTED = 4, /* enum value or size outside what the kernels handle  */
  FMSMO_ERR_LAUNCH = 5,      /* hipLaunchKernel / hipGetLastError reported an error */
  FMSMO_ERR_SCRATCH = 6      /* the shape needs more scratch than the static buffer holds */
};

/* Epilogue arithmetic of the fused int8 GEMM. */
enum {
  /* t = f32(acc) * f32( f16(a_scale[m]*w_scale[n]) ) + f32(bias[n]), multiply and add rounded
     separately in fp32: the exact operation order of iaddmm_int's plain branch
     (fms_mo/modules/linear.py:1185-1188).  A 16-bit output is y = out( f16(t) ): the fp16 acc_dtype
     that from_fms_mo hard-wires (:777), then the cast to the activations' dtype (:1338).  An fp32
     output is y = t: the fp32 acc_dtype from_torch_iW defaults to (:955). */
  FMSMO_EPI_REF_F16 = 0,
  /* y = out( fma( f32(acc), a_scale[m]*w_scale[n], f32(bias[n]) ) ) with the scale product kept
     in fp32 (no fp16 rounding of the scale, single rounding to the output dtype). */
  FMSMO_EPI_F32 = 1,
  /* y = out( f32( f32(acc) * (a_scale[m]*w_scale[n]) ) + f32(bias[n]) ): fp32 scale product,
     multiply and add rounded separately -- `input_scale * w_scale * acc + bias` of
     QLinearCublasI8I32NT / QLinearCutlassI8I32NT.forward (fms_mo/modules/linear.py:1533-1535,
     1581-1583). */
  FMSMO_EPI_F32_MULADD = 2,
  /* The chunked matmuls' fused forms only (fmsmo_matmul_chunk_*_dq): descale, cast, add the bias
     in the output dtype T:  y = T( T( f32( f32(acc) * a_scale[m] ) * w_scale[n] ) + T(bias[n]) ),
     no addition without a bias -- `(acc * x_scale * w_scale.t()).to(org_dtype) + bias.to(org_dtype)`
     of LinearFuncFPxFwdBwd.forward and LinearFuncINT8FwdFP32Bwd.forward
     (fms_mo/modules/linear.py:1955-1975, 2180-2189). */
  FMSMO_EPI_SEQ_OUT = 3
};

int fmsmo_abi_version(void);
const char* fmsmo_status_str(int status);
/* hipGetLastError text of the most recent FMSMO_ERR_LAUNCH on this thread ("" if none). */
const char* fmsmo_last_error(void);

/*
 * Diagnostic with no counterpart in the reference: the core clock a GEMM really ran at.  After
 * this call every 256-row-tile (register-staged) GEMM launched from the calling thread has its
 * block 0 store six 64-bit values into dev6 (device memory, 8-byte aligned, valid until the probe
 * is switched off with NULL and the launches have finished):
 *   dev6[0], dev6[1]  core clock counter and constant 100 MHz counter when the block starts,
 *   dev6[2], dev6[3]  after its K loop,  dev6[4], dev6[5]  after its epilogue.
 * (dev6[4] - dev6[0]) / ((dev6[5] - dev6[1]) / 100) is the average core clock in MHz over the
 * block's life.  MFMA throughput scales with that clock; the published peak assumes 2400 MHz.
 * The pointer is read at launch time, so consecutive launches may be given different buffers.
 */
int fmsmo_debug_clock_probe(uint64_t* dev6);

/*
 * Diagnostic with no counterpart in the reference: the time a launch needs just to pull `bytes`
 * bytes (a multiple of 16, 16-byte aligned) out of device memory.  256 blocks of 1024 threads
 * read p once with 16-byte loads, one KiB of consecutive bytes per wave instruction, and write
 * nothing (sink, 4 bytes of device memory, is written only if the XOR of all words happens to
 * match a constant).  Timed in the same way as a decode linear over the same weights it gives
 * the floor that the launch and the memory system set for that linear: the decode kernels add
 * the activation reads, the reduction over the waves and the output on top of it.
 */
int fmsmo_debug_stream_read(const void* p, int64_t bytes, int32_t* sink, fmsmo_stream_t stream);

/*
 * Diagnostic with no counterpart in the reference: the matrix instructions of the GEMM kernels
 * alone.  256 blocks of 4 waves, one wave per SIMD of every compute unit; each wave loads two
 * sets of 4 + 4 operand fragments (64 bytes of K per fragment and lane, 512 bytes per lane in all)
 * from `data` (device memory, `bytes` a multiple of 4; indices wrap) and then issues nothing but
 * MFMAs from registers: per iteration 2 x 16 blocks of 32 x 32 x 64, as v_mfma_i32_32x32x32_i8
 * pairs (op_dtype = FMSMO_OP_I8) or v_mfma_f32_32x32x64_f8f6f4 (FMSMO_OP_E4M3).  Operations per
 * launch: 1024 waves x iters x 2 x 16 x 2 x 32 x 32 x 64.  clk2 (device, may be NULL) receives
 * {core clock cycles, ticks of the 100 MHz counter} of block 0's loop.  What this loop reaches on
 * given operand bits is the ceiling, under the part's power limit, of any kernel made of these
 * instructions on such operands.  sink: 4 bytes of device memory, practically never written.
 */
int fmsmo_debug_mfma_loop(int op_dtype, const void* data, int64_t bytes, int iters, uint64_t* clk2,
                          float* sink, fmsmo_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * 1. Activation quantizers (one pass over x: read 2-4 B, write 1 B per element).
 * ------------------------------------------------------------------------------------------ */

/*
 * Dynamic symmetric per-token int8 quantizer, optionally preceded by the SmoothQuant divide.
 *   x'      = smooth ? rnd_T(x / smooth[k]) : x
 *   amax_m  = max_k |x'_mk| ; s_m = rnd_T( max(amax_m, rnd_T(1e-5)) / 127 )
 *   q_mk    = int8( rint( rnd_T(x'_mk / s_m) ) )          (half-to-even)
 * T = compute_dtype (FMSMO_F16/BF16/F32) is the dtype in which torch would evaluate the
 * expression (x's dtype, or fp32 when an fp32 SmoothQuant scale promotes it).
 * saturate = 0 reproduces the reference: no clamp, 128 wraps to -128 on the int8 cast (reachable
 * only for T = bf16); saturate = 1 clamps to [-127,127].
 * scale[m] receives s_m as fp32 (exactly representable).
 * x and smooth 16-byte aligned, K and ldx multiples of 8 elements.  Rows holding NaN are not
 * specified (the reference's int8 cast of NaN is platform-defined).
 * Reference: QLinearINT8Deploy.qa_dynamic_max_qfunc (fms_mo/modules/linear.py:1085-1100), the
 * divide in QLinearINT8Deploy.forward (:1331-1334), QMaxDynamic.forward
 * (fms_mo/quant/quantizers.py:3531-3534).
 */
int fmsmo_quant_act_i8_pertoken(const void* x, int x_dtype, int64_t ldx, const void* smooth,
                                int smooth_dtype, int compute_dtype, int saturate, int8_t* q,
                                int64_t ldq, float* scale, int64_t M, int64_t K,
                                fmsmo_stream_t stream);

/*
 * Static per-tensor int8 quantizer:  q = clamp( rint( x/scale + zp - 128 + sym ), -128, 127 )
 * evaluated in fp32 in exactly that order (sym in {0,1}).  Reference: QLinearINT8Deploy.qa_raw_qfunc
 * (fms_mo/modules/linear.py:1061-1071); also the quantize step of fms_mo::q_iaddmm_dq
 * (fms_mo/custom_ext_kernels/utils.py:770) with sym = 0.
 * sym | 2 selects torch.quantize_per_tensor's arithmetic instead,
 *   q = clamp( rint( x * (1/scale) ) + (zp - 128 + (sym & 1)), -128, 127 ),
 * used by fms_mo::q_per_t_sym (custom_ext_kernels/utils.py:792-794) and qa_pt_quant_func
 * (linear.py:1043-1059).
 */
int fmsmo_quant_act_i8_static(const void* x, int x_dtype, int64_t ldx, float scale, int zp,
                              int sym, int8_t* q, int64_t ldq, int64_t M, int64_t K,
                              fmsmo_stream_t stream);

/*
 * Static per-tensor int8 quantizers evaluated in the compute dtype T = compute_dtype (torch's
 * promotion of x's dtype with the dtype of the module's scale buffer: x's own dtype for a module
 * cast to the model dtype, fp32 for fp32 quantizer buffers); every intermediate is rounded to T,
 * quotients are the IEEE quotients (contiguous rows with a 16-bit T, ldx == ldq == K, run at memory
 * speed on a shorter division sequence with the same results), rint is half-to-even:
 *   FMSMO_SQ_RAW        q = clamp( rint( (((x / scale) + zp) - 128) + sym ), -128, 127 )
 *                       QLinearINT8Deploy.qa_raw_qfunc (fms_mo/modules/linear.py:1061-1071)
 *   FMSMO_SQ_FMO        q = int8( rint( clamp(x, clip_lo, clip_hi) / scale - zp ) - (128 - sym) )
 *                       with scale = quant_stepsize, zp = quant_zero_point: clamp before round,
 *                       QLinearINT8Deploy.qa_fmo_mo_qfunc (linear.py:1073-1083)
 *   FMSMO_SQ_U8_SHIFT   q = clamp( rint( x / scale + zp ), 0, 255 ) - 128
 *   FMSMO_SQ_S8_NARROW  q = clamp( rint( x / scale + zp ), -127, 127 )
 *                       the quint8 / qint8 branches of QLinearCublasI8I32NT.forward and
 *                       QLinearCutlassI8I32NT.forward (linear.py:1505-1512, 1563-1570)
 * scale, zp, clip_lo, clip_hi are values of T (or of fp32 when T is fp32) passed as fp32.
 * x 16-byte aligned, K and ldx multiples of 8 elements.
 */
enum { FMSMO_SQ_RAW = 0, FMSMO_SQ_FMO = 1, FMSMO_SQ_U8_SHIFT = 2, FMSMO_SQ_S8_NARROW = 3 };
int fmsmo_quant_act_i8_static_t(const void* x, int x_dtype, int64_t ldx, int mode,
                                int compute_dtype, float scale, float zp, int sym, float clip_lo,
                                float clip_hi, int8_t* q, int64_t ldq, int64_t M, int64_t K,
                                fmsmo_stream_t stream);

/*
 * Dynamic symmetric int8 quantizers whose abs-max is taken over the whole tensor or per column
 * (over the tokens), in x's dtype T.  col_amax: device fp32 [K], the column abs-max of x as
 * fmsmo_absmax_cols writes it (a separate pass; nothing is read on the host).
 *   FMSMO_DQ_PER_TENSOR  s = rnd_T( max(max_k col_amax[k], rnd_T(1e-5)) / levels ); scale[0] <- s
 *   FMSMO_DQ_PER_COLUMN  s_k = rnd_T( max(col_amax[k], rnd_T(1e-5)) / levels );     scale[k] <- s_k
 *   q = int8( rint( rnd_T(x / s) ) + zp )            (no clamp; the int8 cast wraps like torch's)
 * PER_TENSOR with levels = 127 - zp: QLinearINT8Deploy.qa_dyn_max_fake_zero_shift
 * (fms_mo/modules/linear.py:1102-1113); PER_COLUMN with levels = 127, zp = 0:
 * qa_dynamic_max_qfunc with reduce dim -2 (linear.py:1085-1100).
 * scale: device fp32, 16-byte aligned, [1] or [K].
 */
enum { FMSMO_DQ_PER_TENSOR = 0, FMSMO_DQ_PER_COLUMN = 1 };
int fmsmo_quant_act_i8_dynamic(const void* x, int x_dtype, int64_t ldx, const float* col_amax,
                               int granularity, int levels, int zp, int8_t* q, int64_t ldq,
                               float* scale, int64_t M, int64_t K, fmsmo_stream_t stream);

/*
 * FP8 (OCP e4m3fn) emulation quantizers of QLinear, in x's dtype T:
 *   FMSMO_F8E_SAT         y = T( e4m3( clamp(x, -448, 448) ) )                       to_fp8_saturated
 *   FMSMO_F8E_PER_TENSOR  s = fp8 scale of max |x| (col_amax: device fp32 [K] column abs-max)
 *   FMSMO_F8E_PER_ROW     s_m = fp8 scale of max_k |x_mk|   (per token for activations, per output
 *                         channel for weights [N,K])
 *     fp8 scale(a) = rnd_T( rnd_T( 1 / max(a, rnd_T(1e-12)) ) * 448 ), for T = fp16 clamped to 65504
 *                    (max_to_scale; torch evaluates "448 / tensor" as reciprocal, then multiply)
 *     y = rnd_T( T( e4m3( clamp( rnd_T(x * s), -448, 448 ) ) ) / s )
 * Outputs, each optional except that y or q must be given: y [M,K] of x's dtype (the fake-quantized
 * tensor the reference feeds to F.linear); q [M,K] the e4m3 codes; scale fp32 [1] / [M] <- s
 * (required for PER_TENSOR); inv_scale fp32 [1] / [M] <- 1 / s (the dequantizing factor for a
 * GEMM on the codes).
 * Reference: to_fp8_saturated, max_to_scale, to_fp8_scaled, to_fp8_scaled_perCh,
 * to_fp8_scaled_perToken, class to_fp8 (fms_mo/quant/quantizers.py:5309-5488), emulate = True.
 * x and y 16-byte aligned, K, ldx, ldy, ldq multiples of 8 elements.
 */
enum { FMSMO_F8E_SAT = 0, FMSMO_F8E_PER_TENSOR = 1, FMSMO_F8E_PER_ROW = 2 };
int fmsmo_fake_quant_fp8(const void* x, int x_dtype, int64_t ldx, int mode, const float* col_amax,
                         void* y, int64_t ldy, uint8_t* q, int64_t ldq, float* scale,
                         float* inv_scale, int64_t M, int64_t K, fmsmo_stream_t stream);

/*
 * int8 quantizers with a multiplicative scale (the quantize half of the accelerator op
 * fms_mo::i8i8_aiu).  T = compute_dtype is torch's promotion of x's dtype and the metadata's
 * (meta_dtype: dtype of smooth and clip); every intermediate is rounded to T.
 *   x' = smooth ? rnd_T(x / smooth[k]) : x
 *   L / c below is torch's "number / tensor" = rnd_T( rnd_T(1 / c) * L ) (reciprocal, then multiply)
 *   FMSMO_MS_PER_TOKEN : s_m = 127 / max_k|x'_mk|;   q = clamp(rint(rnd_T(x' s_m)), -127, 127)
 *   FMSMO_MS_SYMM      : s = 127 / clip[0];          q = clamp(rint(rnd_T(x' s)), -127, 127)
 *   FMSMO_MS_ASYMM     : s = 255 / rnd_T(clip[0] - clip[1]);  zp = rnd_T(clip[1] s);
 *                        u = clamp(rint(rnd_T(rnd_T(x' s) - zp)), 0, 255);  q = u - 128
 * clip: device pointer to { a_clip_val, a_clip_valn } (unused for per-token; nothing is read on
 * the host, so the call can be captured in a HIP graph).
 * a_scale (fp32, device): per token [M] <- 1 / s_m;  otherwise [2] <- { 1 / s, zp }.
 * The dequantized activation of the reference is then (q [+ 128 + zp]) * a_scale * smooth[k].
 * A row of zeros (s_m = 127/0) is quantized to zeros with a_scale 0; the reference produces NaN.
 * x and smooth 16-byte aligned, K and ldx multiples of 8 elements.
 * Reference: quant_dequant_activ (fms_mo/aiu_addons/i8i8/i8i8_aiu_op.py:203-231).
 */
enum { FMSMO_MS_PER_TOKEN = 0, FMSMO_MS_SYMM = 1, FMSMO_MS_ASYMM = 2 };
int fmsmo_quant_act_i8_mulscale(const void* x, int x_dtype, int64_t ldx, const void* smooth,
                                const void* clip, int meta_dtype, int compute_dtype, int mode,
                                int8_t* q, int64_t ldq, float* a_scale, int64_t M, int64_t K,
                                fmsmo_stream_t stream);

/* Variants of the per-token FP8 (OCP e4m3fn) activation quantizer. */
enum {
  /* s_m = max(amax_m/448, 1e-12) in fp32; q = e4m3( clamp(f32(x)/s_m, -448, 448) ).
     Cast and clamp: _quantize_affine_float8_custom (fms_mo/aiu_addons/fp8/fp8_linear.py:54-72);
     scale: tests/aiu_addons/test_fp8_addon.py:65-79 (the dynamic-scale rule itself lives in
     torchao, outside the reference tree). */
  FMSMO_FP8_LINEAR = 0,
  /* s_m = max( rnd_T(amax_m/448), 1e-5 ) in x's dtype T; q = e4m3( rnd_T(x/s_m) ), no clamp.
     LinearFuncFPxFwdBwd.forward (fms_mo/modules/linear.py:1939-1948). */
  FMSMO_FP8_FPXACC = 1,
  /* as FMSMO_FP8_FPXACC, then |q| < 0.0087890625 flushed to zero (linear.py:1949-1953). */
  FMSMO_FP8_FPXACC_DL8 = 2
};
/* scale != NULL on input with static_scale != 0: use scale[0] for every row (per-tensor static
   activation scale, fp8_linear.py:150-161) instead of the dynamic per-token one. */
int fmsmo_quant_act_fp8_pertoken(const void* x, int x_dtype, int64_t ldx, int variant,
                                 int static_scale, uint8_t* q, int64_t ldq, float* scale,
                                 int64_t M, int64_t K, fmsmo_stream_t stream);
/*
 * The same quantizer with the rule of its dynamic scale spelled out by the caller:
 *   s = max( amax / 448, scale_floor )
 * formed in fp32 from the widened abs-max (scale_dtype = FMSMO_F32) or with the quotient and the
 * floor both rounded to x's dtype (scale_dtype = x_dtype: what torch computes when the division
 * runs on the 16-bit tensor and the clamp bound is a python scalar).  The quotients, the clamp
 * and the cast are the variant's.  per_tensor = 0: amax per row, scale [M] written.
 * per_tensor = 1: amax over the whole tensor, taken from col_amax (fp32 [K] on the device, the
 * per-column abs-max that fmsmo_absmax_cols left there), scale [1] written; nothing is read back
 * to the host, so both launches can be captured in a HIP graph.
 * FP8Linear's dynamic activation scale (fms_mo/aiu_addons/fp8/fp8_linear.py:163-194,236-251) is
 * computed inside torchao (to_affine_quantized_floatx), which is not part of the reference tree:
 * the floor and the dtype of the division are the two properties that code fixes and the
 * reference's own files do not, hence parameters here; (1e-12, FMSMO_F32) is the rule of the
 * reference's test helper (tests/aiu_addons/test_fp8_addon.py:65-79) and the default of
 * fmsmo_quant_act_fp8_pertoken.  LinearFuncFPxFwdBwd's per-tensor scales
 * (fms_mo/modules/linear.py:1939-1948) are (1e-5, x_dtype) with per_tensor = 1.
 * scale_floor must be positive and below 2^60, and must not round to zero in scale_dtype
 * (FMSMO_ERR_UNSUPPORTED otherwise: a zero row would be divided by a zero scale).
 */
int fmsmo_quant_act_fp8_dynamic(const void* x, int x_dtype, int64_t ldx, int variant,
                                int per_tensor, const float* col_amax, float scale_floor,
                                int scale_dtype, uint8_t* q, int64_t ldq, float* scale,
                                int64_t M, int64_t K, fmsmo_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * 2. W8A8 GEMMs on MFMA.   C[M,N] = A[M,K] . B[N,K]^T
 *    Requirements: K % 16 == 0, lda/ldb % 16 == 0, A and B 16-byte aligned.
 * ------------------------------------------------------------------------------------------ */

/*
 * int8 x int8 -> int32, exact (no saturation can occur for K < 2^17).
 * Reference: cutlass_mm.run (fms_mo/custom_ext_kernels/cutlass_i8i32gemm.cu:100-120, .cpp:34),
 * torch.ops.cutlass_gemm.i8i32nt (custom_ext_kernels/utils.py:336-364),
 * gemm_i8<int32_t,NT> / torch.ops.mygemm.gemm_nt_i8i32 (ext_kernel_cublas.cpp:103-195,
 * utils.py:186-206), torch.ops.fms_mo.imatmul (utils.py:690-720).
 */
int fmsmo_gemm_i8_i32(const int8_t* a, int64_t lda, const int8_t* b, int64_t ldb, int32_t* c,
                      int64_t ldc, int64_t M, int64_t N, int64_t K, fmsmo_stream_t stream);
/*
 * The same with an optional scratch buffer, as for fmsmo_gemm_i8_dq_ws below: shapes with few
 * output tiles and a long reduction run as K slices whose int32 partial sums are added in a fixed
 * order (exact, so the result is the single-pass one bit for bit); fmsmo_gemm_workspace_bytes
 * tells the bytes a shape can use, workspace == NULL or fewer bytes runs the single pass.
 * Up to 16 rows (and the batches of up to 64 rows that fmsmo_gemm_i8_dq sends there) run on the
 * weight-streaming kernels with either call.
 * Same reference interfaces as fmsmo_gemm_i8_i32; the workspace has no counterpart there.
 */
int fmsmo_gemm_i8_i32_ws(const int8_t* a, int64_t lda, const int8_t* b, int64_t ldb, int32_t* c,
                         int64_t ldc, int64_t M, int64_t N, int64_t K, void* workspace,
                         int64_t workspace_bytes, fmsmo_stream_t stream);

/*
 * int8 GEMM with the dequantizing epilogue fused:  y = acc * (a_scale x w_scale) + bias.
 * a_scale: fp32 [M] (a_scale_n == M) or one value (a_scale_n == 1); w_scale likewise [N] or 1;
 * bias: [N] of bias_dtype or NULL (nothing is added then: a zero product keeps its sign, as with
 * the -0.0 bias buffer the reference's module holds for a layer without bias, linear.py:897-911).
 * epilogue: FMSMO_EPI_REF_F16 | FMSMO_EPI_F32.
 * M <= 16 is routed to the weight-streaming (HBM-bound) kernel, and so are 17 <= M <= 64 when
 * K is 1024, 2048 or 4096 (5120 and 8192 up to M = 32).
 * Reference: QLinearINT8Deploy.iaddmm_int, plain branch (fms_mo/modules/linear.py:1177-1188),
 * torch.ops.fms_mo.iaddmm (custom_ext_kernels/utils.py:729-737).
 */
int fmsmo_gemm_i8_dq(const int8_t* a, int64_t lda, const int8_t* b, int64_t ldb,
                     const float* a_scale, int64_t a_scale_n, const float* w_scale,
                     int64_t w_scale_n, const void* bias, int bias_dtype, int epilogue, void* y,
                     int y_dtype, int64_t ldy, int64_t M, int64_t N, int64_t K,
                     fmsmo_stream_t stream);

/*
 * e4m3 x e4m3 -> fp32 accumulate, y = out( acc * a_scale[m] * w_scale[n] + bias[n] ).
 * Reference: the torch._scaled_mm call made through addmm_float8_unwrapped_inference in
 * FP8Linear.forward (fms_mo/aiu_addons/fp8/fp8_linear.py:275-283); CPU semantics
 * _scaled_mm_cpu_out (fms_mo/aiu_addons/fp8/fp8_spyre_op.py:35-60).
 */
int fmsmo_gemm_fp8_dq(const uint8_t* a, int64_t lda, const uint8_t* b, int64_t ldb,
                      const float* a_scale, int64_t a_scale_n, const float* w_scale,
                      int64_t w_scale_n, const void* bias, int bias_dtype, void* y, int y_dtype,
                      int64_t ldy, int64_t M, int64_t N, int64_t K, fmsmo_stream_t stream);

/*
 * The two *_dq GEMMs with a caller-provided workspace (the library allocates nothing).  When the
 * output has few tiles and the reduction is long (16 < M <= 1024, at most 128 tiles of 128 x 128,
 * K % 128 == 0: a batch of tens to hundreds of tokens through a projection with few output
 * columns) the reduction is split into slices that run side by side and a second kernel adds the
 * slices in a fixed order and applies the epilogue: 17 x 4096 x 14336 runs on 256 compute units
 * instead of 32.  int32 partial sums are exact, so the int8 result is bit-identical to
 * fmsmo_gemm_i8_dq's; the e4m3 result differs from fmsmo_gemm_fp8_dq's only by the order of the
 * fp32 additions.  From 384 rows and K >= 8192 the slices run on 256 x 128 tiles of the
 * register-staged kernel (more, shorter slices: more partial sums).  Shapes whose 128 x 64 tiles
 * fill half a round of the compute units or more with a short reduction (192-256 tiles and
 * K <= 8192, or M > 128, 96-191 tiles and K <= 4096), and a full round of 128 x 128 tiles, run in
 * one pass instead and ask for no workspace.  fmsmo_gemm_workspace_bytes
 * returns the bytes a shape can use at most (0: no split); with fewer bytes the call takes the
 * split that fits them (the 128 x 128 tiles' never needs more than 16 MiB), with none or
 * workspace == NULL it is fmsmo_gemm_*_dq.  workspace: 16-byte aligned
 * device memory, contents undefined before and after, private to the call while it runs.
 * No counterpart in the reference (its GEMMs are single launches of CUTLASS / cuBLASLt kernels).
 */
int64_t fmsmo_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K);

/*
 * Which kernel the *_dq GEMMs run for a shape, without launching anything (host-only; for tests,
 * tuning and capacity planning).  with_workspace = 1 describes the *_dq_ws calls given a
 * sufficient workspace, with_workspace = 2 what fmsmo_gemm_i8_dq_noalloc runs (the split that
 * fits its static scratch; FMSMO_ERR_SCRATCH where that call returns it).  tile_m / tile_n are 0 for the decode and generic kernels; splits is the
 * number of K slices (1 = single pass).  The choice weighs the measured efficiency of each tile
 * shape against how full the last round of tiles leaves the 256 compute units, e.g.
 * 4096 x 6144 runs 512 tiles of 256 x 192 (two full rounds) rather than 384 of 256 x 256.
 * 2048 x 4096 runs 256 tiles of 256 x 128 rather than 128 of 256 x 256.  When the last round of
 * 256 x 256 tiles would be nearly empty, the *_dq calls run its columns (at least 1024) as a second
 * GEMM behind the first: the plan describes the first, fmsmo_gemm_tail_columns tells the cut.
 * No counterpart in the reference (CUTLASS / cuBLASLt choose internally).
 */
enum fmsmo_plan_kernel {
  FMSMO_PLAN_DECODE = 0,                /* skinny-M weight-streaming kernels */
  FMSMO_PLAN_TILE_REGISTER_STAGED = 1,  /* MFMA tiles, 128-byte K slabs staged through registers */
  FMSMO_PLAN_TILE_LDS_DMA = 2,          /* MFMA tiles, 64-byte K stages loaded straight into LDS */
  FMSMO_PLAN_GENERIC = 3                /* K % 64 != 0: one thread per output element */
};
int fmsmo_gemm_plan(int64_t M, int64_t N, int64_t K, int with_workspace, int* kernel, int* tile_m,
                    int* tile_n, int* splits);
/* Columns that the single-pass *_dq GEMMs cut off the end of N and run as a second GEMM behind
   the first (0: the GEMM runs whole; fmsmo_gemm_plan describes the first, main part).  Host-only. */
int64_t fmsmo_gemm_tail_columns(int64_t M, int64_t N, int64_t K);
int fmsmo_gemm_i8_dq_ws(const int8_t* a, int64_t lda, const int8_t* b, int64_t ldb,
                        const float* a_scale, int64_t a_scale_n, const float* w_scale,
                        int64_t w_scale_n, const void* bias, int bias_dtype, int epilogue, void* y,
                        int y_dtype, int64_t ldy, int64_t M, int64_t N, int64_t K, void* workspace,
                        int64_t workspace_bytes, fmsmo_stream_t stream);
int fmsmo_gemm_fp8_dq_ws(const uint8_t* a, int64_t lda, const uint8_t* b, int64_t ldb,
                         const float* a_scale, int64_t a_scale_n, const float* w_scale,
                         int64_t w_scale_n, const void* bias, int bias_dtype, void* y, int y_dtype,
                         int64_t ldy, int64_t M, int64_t N, int64_t K, void* workspace,
                         int64_t workspace_bytes, fmsmo_stream_t stream);

/*
 * fmsmo_gemm_i8_dq_ws without a workspace argument and without any allocation: the split-K
 * partial sums live in a device array that is part of the library's code object
 * (FMSMO_STATIC_SCRATCH_BYTES, resident on every GPU the library is loaded on until the process
 * ends).  It has NO counterpart in the reference; it is for callers that cannot allocate: code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  The call makes
 * no hipMalloc / hipFree and uses no allocating library routine; the caller still passes inputs
 * and outputs.  Results are bit-identical to fmsmo_gemm_i8_dq_ws given a sufficient workspace
 * (and so to fmsmo_gemm_i8_dq).
 * The call takes the split that fits the array: where the preferred one (register-staged slices
 * of a long reduction) needs more, the 128 x 128 tiles' split, whose need never exceeds the array
 * under the current policy (16 < M <= 1024, at most 128 such tiles, up to 256 / tiles slices).
 * A shape none of whose splits would fit returns FMSMO_ERR_SCRATCH (fmsmo_last_error() says how
 * many bytes it needs): the check guards changes of that policy.  Shapes that take no split use
 * no scratch at all.
 * All calls on one GPU share that GPU's array: two calls that overlap in time on the same GPU
 * (different streams, different threads) race on it; calls on one stream are ordered and safe.
 * Nothing in the array has to be cleared between calls (every slice stores its whole block of
 * partial sums before the reduction reads it).  The device address of the array is looked up on
 * the first call on each device (hipGetSymbolAddress); make that first call outside a graph
 * capture.
 */
#define FMSMO_STATIC_SCRATCH_BYTES (16 << 20)
int fmsmo_gemm_i8_dq_noalloc(const int8_t* a, int64_t lda, const int8_t* b, int64_t ldb,
                             const float* a_scale, int64_t a_scale_n, const float* w_scale,
                             int64_t w_scale_n, const void* bias, int bias_dtype, int epilogue,
                             void* y, int y_dtype, int64_t ldy, int64_t M, int64_t N, int64_t K,
                             fmsmo_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * 3. Skinny-M (decode) variants, M <= 16: stream the weights once from HBM.
 *    Same arithmetic and arguments as the two *_dq GEMMs above.
 * ------------------------------------------------------------------------------------------ */
int fmsmo_gemv_i8_dq(const int8_t* a, int64_t lda, const int8_t* b, int64_t ldb,
                     const float* a_scale, int64_t a_scale_n, const float* w_scale,
                     int64_t w_scale_n, const void* bias, int bias_dtype, int epilogue, void* y,
                     int y_dtype, int64_t ldy, int64_t M, int64_t N, int64_t K,
                     fmsmo_stream_t stream);
int fmsmo_gemv_fp8_dq(const uint8_t* a, int64_t lda, const uint8_t* b, int64_t ldb,
                      const float* a_scale, int64_t a_scale_n, const float* w_scale,
                      int64_t w_scale_n, const void* bias, int bias_dtype, void* y, int y_dtype,
                      int64_t ldy, int64_t M, int64_t N, int64_t K, fmsmo_stream_t stream);

/*
 * Fused decode linear for a decode step of one to four tokens: y = dequant( quant(x) . W^T ) in
 * one launch.  Every block quantizes the (tiny) activation rows itself -- the arithmetic of
 * fmsmo_quant_act_i8_pertoken for a 16-bit compute dtype: x fp16 / bf16 [M,K], smooth of x's dtype
 * or NULL -- and then runs a weight-streaming kernel of fmsmo_gemv_i8_dq on the codes, so the
 * result is bit-identical to the two calls in sequence while a kernel launch and the round trip
 * of the codes through memory are saved in front of every linear layer of a single-stream decode
 * step.  a_scale_out (fp32 [M], may be NULL) receives the tokens' scales (the reference's
 * input_scale side effect).
 * fmsmo_decode_linear_ok(M, K) != 0 tells whether a shape is served: M == 1 and either K <= 8192
 * in one of the row kernel's sizes (1024, 2048, 4096, 8192 and what pads to them) or K = 14336 /
 * 12800 (the streaming kernel quantizes the rows while the head of its weight stream is in
 * flight); M <= 4 at K = 4096 and M <= 3 at K = 14336 / 12800 (the same kernel).  With more
 * tokens or other row lengths the quantization that every block repeats costs more than the
 * launch it saves, and the call returns FMSMO_ERR_UNSUPPORTED: use the two kernels.
 * smooth_dtype = FMSMO_F32 (x fp16 / bf16 with fp32 divisors: torch promotes the whole quantizer
 * to fp32, the arithmetic of fmsmo_quant_act_i8_pertoken with compute_dtype FMSMO_F32) is served
 * by the streaming kernel where fmsmo_decode_linear_f32s_ok(M, K) != 0: K = 4096 up to two tokens,
 * K = 14336 / 12800 one token; otherwise smooth_dtype must equal x_dtype.
 * x and smooth 16-byte aligned, ldx % 8 == 0, w as for fmsmo_gemv_i8_dq.
 * Reference: QLinearINT8Deploy.forward for a decode step -- qa_dynamic_max_qfunc followed by
 * iaddmm_int (fms_mo/modules/linear.py:1085-1100, 1177-1188, 1309-1338); no fused counterpart.
 */
int fmsmo_decode_linear_ok(int64_t M, int64_t K);
int fmsmo_decode_linear_f32s_ok(int64_t M, int64_t K);
int fmsmo_decode_linear_i8(const void* x, int x_dtype, int64_t ldx, const void* smooth,
                           int smooth_dtype, int saturate, const int8_t* w, int64_t ldw, const float* w_scale,
                           int64_t w_scale_n, const void* bias, int bias_dtype, int epilogue,
                           void* y, int y_dtype, int64_t ldy, float* a_scale_out, int64_t M,
                           int64_t N, int64_t K, fmsmo_stream_t stream);
/*
 * The same for e4m3 weights: the block quantizes the tokens with the dynamic per-token recipe of
 * fmsmo_quant_act_fp8_pertoken(FMSMO_FP8_LINEAR) and runs fmsmo_gemv_fp8_dq's kernel on them:
 * scales and codes are the quantizer's bit for bit, and so is the result wherever the two-call
 * path streams the weights in the same shape (one token: K <= 8192; K = 14336 with N <= 4096);
 * elsewhere the fp32 partial sums are added in another order.  Served shapes as told by
 * fmsmo_decode_linear_ok.
 * Reference: FP8Linear.forward with dynamic activation scales
 * (fms_mo/aiu_addons/fp8/fp8_linear.py:217-283) on one token.
 */
int fmsmo_decode_linear_fp8(const void* x, int x_dtype, int64_t ldx, const uint8_t* w, int64_t ldw,
                            const float* w_scale, int64_t w_scale_n, const void* bias,
                            int bias_dtype, void* y, int y_dtype, int64_t ldy, float* a_scale_out,
                            int64_t M, int64_t N, int64_t K, fmsmo_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * 4. Chunked reduced-precision accumulation ("chunk-truncate") matmuls.
 *    Per K-chunk of chunk_size: p = dot(a_chunk, b_chunk) in a fresh accumulator; p is
 *    range-clamped / LSB-rounded; acc += p (truncate_then_accumulate != 0) or the running
 *    accumulator itself is rounded after each chunk (== 0).  A K tail is zero-padded.
 * ------------------------------------------------------------------------------------------ */

/*
 * int8 -> int32.  p = clamp(p, -2^(b-1), 2^(b-1)-1) if b = max_acc_bits < 32;
 * p = ((p + 2^(t-1)) >> t) << t if t = chunk_trun_bits > 0 (arithmetic shift).
 * c_in (int32 [M,N], may be NULL, may alias d) is the initial accumulator.
 * chunk_size: a power of two >= 32.
 * Reference: imatmul_kernel (fms_mo/custom_ext_kernels/triton_kernels.py:211-302) as launched
 * by tl_matmul_chunk_truncate (:468-621); the PyTorch chunk loop of iaddmm_int
 * (fms_mo/modules/linear.py:1142-1175) gives the same values after its final 2^t scaling.
 */
int fmsmo_matmul_chunk_i8(const int8_t* a, int64_t lda, const int8_t* b, int64_t ldb,
                          const int32_t* c_in, int32_t* d, int64_t ldd, int64_t M, int64_t N,
                          int64_t K, int chunk_size, int chunk_trun_bits, int max_acc_bits,
                          int truncate_then_accumulate, fmsmo_stream_t stream);

/*
 * Floating point -> fp32.  op_dtype: FMSMO_OP_E4M3 (1-byte operands), FMSMO_OP_F16 or
 * FMSMO_OP_BF16 (2-byte operands), FMSMO_OP_F32 (4-byte operands).  lda / ldb / K count
 * ELEMENTS.  On the IEEE-754 word u of p:
 *   u = (u + (t ? 1<<(t-1) : 0)) & ~((1<<t)-1),  t = chunk_trun_bits in [0,22];
 * clamp_dl16 != 0 forces t = 14 and then p >= 8581545984 -> +inf, p <= -8581545984 -> -inf,
 * |p| < 4.665707820095122e-10 -> 0.   The order of the fp32 additions inside one chunk is the
 * MFMA unit's (the reference leaves it to tl.dot).  chunk_size: power of two >= 32 (e4m3) or
 * >= 16 (f16/bf16/f32).  c_in: optional fp32 initial accumulator (D = A.B + C).
 * Reference: matmul_kernel / matmul_kernel_DABC / round_and_trun
 * (fms_mo/custom_ext_kernels/triton_kernels.py:96-205,305-423,432-465).
 */
int fmsmo_matmul_chunk_fp(const void* a, int64_t lda, const void* b, int64_t ldb, int op_dtype,
                          const float* c_in, float* d, int64_t ldd, int64_t M, int64_t N,
                          int64_t K, int chunk_size, int chunk_trun_bits, int clamp_dl16,
                          int truncate_then_accumulate, fmsmo_stream_t stream);

/*
 * The two chunked matmuls with the dequantization fused into their epilogue (one launch instead of
 * the matmul and three or four elementwise passes over [M,N]):
 *   y[m,n] = epilogue( acc[m,n], a_scale[m or 0], w_scale[n or 0], bias[n] ),  epilogue one of
 *   FMSMO_EPI_*; acc is the chunked accumulator of fmsmo_matmul_chunk_i8 / _fp with c_in = NULL
 *   (for integers it still carries the factor 2^t of its cleared low bits; (2^t a) s = a (2^t s)
 *   exactly, so the reference's `trun_scale * input_scale` needs no separate multiply).
 * a_scale_n in {1, M}, w_scale_n in {1, N}; bias [N] of bias_dtype or NULL; y of y_dtype.
 * With nothing to round or clamp (int8, t = 0, 32 accumulator bits) the call is fmsmo_gemm_i8_dq.
 * Reference: the serial chunk loop of iaddmm_int and its final
 * `accumulator * (trun_scale * input_scale * w_scale) + bias` = FMSMO_EPI_F32_MULADD
 * (fms_mo/modules/linear.py:1142-1175); imatmul bound to tl_matmul_chunk_truncate followed by the
 * fp16-scale epilogue = FMSMO_EPI_REF_F16 (:1213-1251, 1177-1188); LinearFuncFPxFwdBwd.forward and
 * LinearFuncINT8FwdFP32Bwd.forward = FMSMO_EPI_SEQ_OUT (:1955-1975, 2180-2189).
 */
int fmsmo_matmul_chunk_i8_dq(const int8_t* a, int64_t lda, const int8_t* b, int64_t ldb,
                             const float* a_scale, int64_t a_scale_n, const float* w_scale,
                             int64_t w_scale_n, const void* bias, int bias_dtype, int epilogue,
                             void* y, int y_dtype, int64_t ldy, int64_t M, int64_t N, int64_t K,
                             int chunk_size, int chunk_trun_bits, int max_acc_bits,
                             int truncate_then_accumulate, fmsmo_stream_t stream);
int fmsmo_matmul_chunk_fp_dq(const void* a, int64_t lda, const void* b, int64_t ldb, int op_dtype,
                             const float* a_scale, int64_t a_scale_n, const float* w_scale,
                             int64_t w_scale_n, const void* bias, int bias_dtype, int epilogue,
                             void* y, int y_dtype, int64_t ldy, int64_t M, int64_t N, int64_t K,
                             int chunk_size, int chunk_trun_bits, int clamp_dl16,
                             int truncate_then_accumulate, fmsmo_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * 5. Grouped int8 GEMM for mixture-of-experts FFNs (uneven rows per expert, one launch).
 *    Rows of A are sorted by expert; expert e owns rows [offsets[e], offsets[e+1]).
 *    B is [E][N][K] (expert stride ldb_e elements), w_scale [E][N], bias [E][N] or NULL.
 *    offsets is a DEVICE array of E+1 int32; the row counts are never read back.  total_rows =
 *    offsets[E] must be given on the host (it sizes the output and bounds the grid; with whole
 *    128-byte reductions the launch is one persistent block per compute unit and the blocks
 *    count the tiles themselves).  Arithmetic per expert == fmsmo_gemm_i8_dq.
 *    The reference has no grouped type: every expert w1/w2/w3 is its own QLinearINT8Deploy
 *    (fms_mo/utils/dq_utils.py:86-106), so each expert's rows must equal that module's output.
 * ------------------------------------------------------------------------------------------ */
int fmsmo_grouped_gemm_i8_dq(const int8_t* a, int64_t lda, const int8_t* b, int64_t ldb,
                             int64_t ldb_e, const int32_t* offsets, int num_experts,
                             int64_t total_rows, const float* a_scale, const float* w_scale,
                             const void* bias, int bias_dtype, int epilogue, void* y,
                             int y_dtype, int64_t ldy, int64_t N, int64_t K,
                             fmsmo_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * 6. Offline weight path: float weights -> int8 rows (+ integer row sums), one pass over W.
 *      t_nk = rnd_T1( W_nk * smooth_k )                              (smooth may be NULL)
 *      FMSMO_WQ_MUL:  q_nk = rint( clamp( rnd_T2( coef_n * t_nk ), -127, 127 ) )
 *      FMSMO_WQ_DIV:  q_nk = clamp( rint( rnd_T2( t_nk / coef_n ) ), -127, 127 )
 *      row_sum_n = sum_k q_nk                                         (row_sum may be NULL)
 *    T1 = promote(w_dtype, smooth_dtype), T2 = promote(T1, coef_dtype), the dtypes torch uses.
 *    coef has N elements or 1.  W and smooth 16-byte aligned, K and ldw multiples of 8 elements.
 *    MUL with coef = 127 / clip_val: the AIU checkpoint writer, process_weight
 *    (fms_mo/utils/aiu_utils.py:237-279) after process_smoothquant (:87-122); row_sum is
 *    process_zero_shift (:282-333).  DIV with coef = w_scale: QLinearINT8Deploy.from_fms_mo
 *    (fms_mo/modules/linear.py:861-866).
 * ------------------------------------------------------------------------------------------ */
enum { FMSMO_WQ_MUL = 0, FMSMO_WQ_DIV = 1 };
int fmsmo_quant_weight_i8(const void* w, int w_dtype, int64_t ldw, const void* smooth,
                          int smooth_dtype, const void* coef, int coef_dtype, int64_t coef_n,
                          int mode, int8_t* q, int64_t ldq, int32_t* row_sum, int64_t N, int64_t K,
                          fmsmo_stream_t stream);

/*
 * Per-column running abs-max over the rows of x:  out[k] = max( out[k], max_m |x[m][k]| ), fp32.
 * The caller initialises out (zeros for a fresh statistic, the running value otherwise; values
 * must be >= 0).  Serves the SmoothQuant statistics: the activation scale collected by forward
 * hooks (fms_mo/quant/ptq.py:2586-2595: comming_max = x.view(-1, K).abs().max(dim=0), running
 * max) and the weight column maximum of get_smoothq_scale (fms_mo/modules/linear.py:345-368) and
 * process_smoothquant (fms_mo/utils/aiu_utils.py:105-107).  x 16-byte aligned, K and ldx
 * multiples of 8 elements.
 */
int fmsmo_absmax_cols(const void* x, int x_dtype, int64_t ldx, int64_t M, int64_t K, float* out,
                      fmsmo_stream_t stream);

/*
 * Bias with the zero-point correction of asymmetric per-tensor activations folded in, for use
 * as the bias of fmsmo_gemm_i8_dq when the activation codes are stored minus `offset`:
 *   out[n] = bias[n] + (offset + a_meta[1]) * (sum_k w[n,k]) * a_meta[0] * w_scale[n]
 * a_meta: device fp32 { 1 / activation scale, zero point }, as written by
 * fmsmo_quant_act_i8_mulscale(FMSMO_MS_ASYMM); bias may be NULL; out: fp32 [N].
 * w 16-byte aligned, K and ldw multiples of 16.
 * Reference: the (x_int + zp_x) / scale_x dequantization of quant_dequant_activ
 * (fms_mo/aiu_addons/i8i8/i8i8_aiu_op.py:219-223) multiplied out over the integer GEMM; the
 * integer row sums are the zero_shift of process_zero_shift (fms_mo/utils/aiu_utils.py:282-333).
 */
int fmsmo_zero_shift_bias(const int8_t* w, int64_t ldw, const float* w_scale, int64_t w_scale_n,
                          const float* a_meta, float offset, const void* bias, int bias_dtype,
                          float* out, int64_t N, int64_t K, fmsmo_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * 7. Batched matmuls of attention (quantized m1 . m2 per batch entry).
 * ------------------------------------------------------------------------------------------ */

/*
 * Static per-tensor int8 quantizer in the compute dtype T (torch's promotion of x's dtype and the
 * scale's), for both operands of a batched matmul:
 *   q = clamp( rint( rnd_T( rnd_T(x / scale) + offset ) ), -128, 127 )
 * x: [batch][R][C] (row stride ldx, batch stride stride_x, in elements).
 * transpose == 0: q [batch][R][ldq];  transpose != 0: q [batch][C][ldq] with q[c][r] = code of
 * x[r][c], which turns an operand stored as [k][n] into the [n][k] layout the MFMA kernels read.
 * Columns of q past the data are zero-filled (ldq pads the reduction dimension: a multiple of 8,
 * of 64 when transposing; use a multiple of 64 for fmsmo_bmm_i8_dq).  batch <= 65535.
 * Reference: QBmmINT8Deploy.qfunc_raw as called by its forward with offset = zero point - 128 for
 * m1 and 0 for m2 (fms_mo/modules/bmm.py:699-711, 735-737).
 */
int fmsmo_quant_i8_affine(const void* x, int x_dtype, int64_t ldx, int64_t stride_x, float scale,
                          float offset, int compute_dtype, int transpose, int8_t* q, int64_t ldq,
                          int64_t stride_q, int64_t batch, int64_t R, int64_t C,
                          fmsmo_stream_t stream);

/*
 * y[b] = ( a[b] . b[b]^T ) * (a_scale[0] * b_scale[0]) + bias[b][n]      for b in [0, batch)
 * a: [batch * M][K] (the batches stacked, row stride lda), b: [batch][N][K] (row stride ldb, batch
 * stride stride_b), y: [batch * M][N] (row stride ldy); a_scale, b_scale: device fp32 scalars;
 * bias: device fp32 [batch][N] or NULL (the zero-point correction of an asymmetric m1, see
 * fmsmo_zero_shift_bias, which accepts the stacked [batch * N][K] operand).  int32 (int8) or fp32
 * (e4m3) accumulation on MFMA, fp32 epilogue.  K % 64 == 0 (zero-pad the operands),
 * lda/ldb/stride_b % 16 == 0, 16-byte aligned operands, batch * M * lda < 2^31.
 * Reference: QBmmINT8Deploy.forward (fms_mo/modules/bmm.py:719-748; the reference still
 * simulates this product with an fp16 matmul) and spyre::scaled_bmm
 * (fms_mo/aiu_addons/fp8/fp8_spyre_op.py:102-140).
 */
int fmsmo_bmm_i8_dq(const int8_t* a, int64_t lda, const int8_t* b, int64_t ldb, int64_t stride_b,
                    const float* a_scale, const float* b_scale, const float* bias, void* y,
                    int y_dtype, int64_t ldy, int64_t batch, int64_t M, int64_t N, int64_t K,
                    fmsmo_stream_t stream);
int fmsmo_bmm_fp8_dq(const uint8_t* a, int64_t lda, const uint8_t* b, int64_t ldb,
                     int64_t stride_b, const float* a_scale, const float* b_scale,
                     const float* bias, void* y, int y_dtype, int64_t ldy, int64_t batch,
                     int64_t M, int64_t N, int64_t K, fmsmo_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* FMSMO_HIP_H_ */
