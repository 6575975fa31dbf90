/*
 * daxq -- C ABI of the MI355X (gfx950) W8A8 linear that replaces the DAX dynamic
 * quantized Linear (INT8 and FP8 OCP e4m3fn).
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless stated; the caller owns and
 *     allocates all buffers, the library never allocates, never synchronises the
 *     device and only uses the stream it is given (a hipStream_t passed as void*;
 *     NULL is the null stream);
 *   - matrices are row-major with an explicit leading dimension in ELEMENTS;
 *   - return value 0 on success, a negative DAXQ_ERR_* otherwise; the text of
 *     the last error on the calling thread is returned by daxq_last_error();
 *   - calls on different streams, and from different host threads, may run concurrently: the library keeps no
 *     mutable process state apart from a per-kernel record of the devices whose launch attributes it has set
 *     (atomic; filled by daxq_init or by a kernel's first launch on a device).
 *
 * Reference paths cited below are relative to the DAX checkout.
 */
#ifndef DAXQ_H
#define DAXQ_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DAXQ_ABI_VERSION 5

#define DAXQ_OK 0
#define DAXQ_ERR_ARG (-1)    /* null pointer, negative size, bad enum */
#define DAXQ_ERR_ALIGN (-2)  /* pointer / leading dimension / K not aligned as required */
#define DAXQ_ERR_DEVICE (-3) /* current device is not gfx950 */
#define DAXQ_ERR_LAUNCH (-4) /* the HIP runtime refused the launch */

/* K granularity of the GEMM entry points: operands whose logical K is not a
 * multiple of this are zero-padded by the producer: the quantisers below write
 * zeros into columns [k, roundup(k, DAXQ_K_ALIGN)) as far as the row reaches
 * (ld_q may be smaller); a row stride ld_q beyond that keeps rows apart, or makes
 * q a column slice of a wider buffer, and those bytes are not touched. */
#define DAXQ_K_ALIGN 128

/* quantised formats (one byte per element) */
#define DAXQ_FMT_I8 0   /* two's-complement int8 */
#define DAXQ_FMT_E4M3 1 /* OCP float8 e4m3fn */
#define DAXQ_FMT_E5M2 2 /* OCP float8 e5m2 */

/* floating-point element types of activations, outputs and bias */
#define DAXQ_BF16 0
#define DAXQ_F16 1
#define DAXQ_F32 2

/* how a dynamic activation scale, absmax / quant_max, is rounded before the floor (and the floor with it) */
#define DAXQ_SCALE_ROUND_NONE 0 /* kept in fp32: what is left of the chain when a code generator fuses it, as under the
                                   torch.compile decorator of the reference's forward (dax/quant/nn/dynamic/linear.py:143) */
#define DAXQ_SCALE_ROUND_X 1    /* to x's own element type: the eager dtype chain, dax/quant/nn/dynamic/functional.py:124-129 */

typedef void* daxq_stream_t;

int daxq_abi_version(void);
const char* daxq_last_error(void);

/* Fills in facts about `device` (CU count, max engine clock in kHz, LDS bytes per
 * workgroup, gcnArchName) and returns DAXQ_ERR_DEVICE when it is not a gfx950.
 * Replaces the CUDA-version guards of dax/quant/nn/dynamic/linear.py:44-57. */
int daxq_device_info(int device, int* cu_count, int* clock_khz, int* lds_bytes, char* arch, int arch_len);

/* Optional set-up for the current HIP device: raises the dynamic LDS limit of every GEMM kernel now instead of at a
 * kernel's first launch (a kernel attribute cannot be changed while a stream is being captured, so without this call
 * the first launch of each kernel has to happen outside a capture).  Idempotent, cheap after the first call, launches
 * nothing.  No counterpart in the reference, whose kernels come from torch. */
int daxq_init(void);

/*
 * Dynamic per-token symmetric activation quantisation, INT8.
 * Replaces dynamic_quantize_to_int8 / _dynamic_quantize_func / quantize_to_int8
 *   dax/quant/nn/dynamic/functional.py:181-206, :54-148
 *   dax/quant/nn/quantized/functional.py:17-20
 * x      bf16 [m, k], leading dimension ld_x
 * q      int8 [m, ld_q]; columns [k, min(ld_q, roundup(k, DAXQ_K_ALIGN))) are written as zeros
 * scale  fp32 [m]   = f32( max( bf16_rne( f32(rowamax) / 127 ), 2^-23 ) )
 * q[r,c] = clamp( rint( f32(x[r,c]) * (1.0f / scale[r]) ), -128, 127 )
 */
int daxq_act_quant_i8(const void* x, int64_t m, int64_t k, int64_t ld_x,
                      int8_t* q, int64_t ld_q, float* scale, daxq_stream_t stream);

/*
 * Dynamic per-token symmetric activation quantisation, FP8 OCP e4m3fn.
 * Replaces dynamic_quantize_to_fp8 / quantize_to_fp8
 *   dax/quant/nn/dynamic/functional.py:152-177, dax/quant/nn/quantized/functional.py:11-13
 * scale as above with 448; q = e4m3fn_rne( clamp( f32(x) / scale, -448, 448 ) ), one byte each.
 */
int daxq_act_quant_e4m3(const void* x, int64_t m, int64_t k, int64_t ld_x,
                        uint8_t* q, int64_t ld_q, float* scale, daxq_stream_t stream);

/*
 * The same for OCP e5m2 activations, the default activation dtype of the reference's FP8 qconfig
 *   dax/quant/quantization/qconfig.py:85-87;  scale with 57344, q = e5m2_rne( clamp( f32(x) / scale, -57344, 57344 ) ).
 */
int daxq_act_quant_e5m2(const void* x, int64_t m, int64_t k, int64_t ld_x,
                        uint8_t* q, int64_t ld_q, float* scale, daxq_stream_t stream);

/*
 * Producer fused with the per-token quantiser: LayerNorm + per-column multiply-add.
 *   y = bf16( layer_norm_f32(x, eps) * mul[g] + add[g] ),  g = row / rows_per_group,  then y is quantised as above.
 * This is the adaLN pattern of the DiT, whose operation order the reference spells out at
 *   dax/adapters/wan/transformer_adapter.py:151-153   (norm(x.float()) * (1 + scale) + shift).type_as(x)
 * (mul = 1 + scale, add = shift, one group per batch element), and a LayerNorm with its own weight and
 * bias (mul = weight, add = bias, one group).  Under the reference's torch.compile
 *   dax/adapters/wan/functional.py:33-36
 * Inductor fuses the quantiser's row reduction (dax/quant/nn/dynamic/functional.py:124-129) into this
 * producer; eagerly the bf16 tensor y makes a round trip through memory.
 * x bf16 [m, k]; mul, add fp32 [groups, k] or NULL (1 / 0); y bf16 [m, ld_y] or NULL when only the
 * quantised form is wanted; q, scale as for daxq_act_quant_*.  k % 8 == 0, k <= 8192, 16-byte aligned rows.
 * Statistics in fp32 (mean, biased variance, 1/sqrt(var + eps)); floating point: results match an fp32
 * LayerNorm to its rounding, not bit for bit.
 */
int daxq_layernorm_act_quant_i8(const void* x, int64_t m, int64_t k, int64_t ld_x, const float* mul, const float* add,
                                int64_t rows_per_group, float eps, void* y, int64_t ld_y,
                                int8_t* q, int64_t ld_q, float* scale, daxq_stream_t stream);
int daxq_layernorm_act_quant_e4m3(const void* x, int64_t m, int64_t k, int64_t ld_x, const float* mul, const float* add,
                                  int64_t rows_per_group, float eps, void* y, int64_t ld_y,
                                  uint8_t* q, int64_t ld_q, float* scale, daxq_stream_t stream);
int daxq_layernorm_act_quant_e5m2(const void* x, int64_t m, int64_t k, int64_t ld_x, const float* mul, const float* add,
                                  int64_t rows_per_group, float eps, void* y, int64_t ld_y,
                                  uint8_t* q, int64_t ld_q, float* scale, daxq_stream_t stream);

/*
 * Producer fused with the per-token quantiser: GELU in its tanh form, the activation between the two
 * FFN linears of the DiT (the second one, 13824 -> 5120, is where the unfused quantiser reads 3.1 GB).
 *   y = bf16( gelu(f32(x), approximate="tanh") ), then y is quantised as above.
 * Same fusion as above (dax/adapters/wan/functional.py:33-36 over dax/quant/nn/dynamic/functional.py:124-129).
 * x bf16 [m, k], k % 8 == 0, k <= 14336; y bf16 [m, ld_y] or NULL; q, scale as for daxq_act_quant_*.
 * Floating point: exp and reciprocal are the hardware approximations (1 ulp), results match torch's
 * gelu to bf16 rounding, not bit for bit.
 */
int daxq_gelu_tanh_act_quant_i8(const void* x, int64_t m, int64_t k, int64_t ld_x, void* y, int64_t ld_y,
                                int8_t* q, int64_t ld_q, float* scale, daxq_stream_t stream);
int daxq_gelu_tanh_act_quant_e4m3(const void* x, int64_t m, int64_t k, int64_t ld_x, void* y, int64_t ld_y,
                                  uint8_t* q, int64_t ld_q, float* scale, daxq_stream_t stream);
int daxq_gelu_tanh_act_quant_e5m2(const void* x, int64_t m, int64_t k, int64_t ld_x, void* y, int64_t ld_y,
                                  uint8_t* q, int64_t ld_q, float* scale, daxq_stream_t stream);

/*
 * Leaf quantisers with a caller-supplied per-row scale (used once per weight at conversion).
 * Replace quantize_to_int8 / quantize_to_fp8 with a [rows,1] scale
 *   dax/quant/nn/quantized/functional.py:11-20, called from dax/quant/nn/dynamic/linear.py:292-296
 * x bf16 [m, k]; scale fp32 [m]; q [m, ld_q] with columns [k, min(ld_q, roundup(k, DAXQ_K_ALIGN))) zero.
 */
int daxq_quantize_rows_i8(const void* x, int64_t m, int64_t k, int64_t ld_x, const float* scale,
                          int8_t* q, int64_t ld_q, daxq_stream_t stream);
int daxq_quantize_rows_e4m3(const void* x, int64_t m, int64_t k, int64_t ld_x, const float* scale,
                            uint8_t* q, int64_t ld_q, daxq_stream_t stream);
int daxq_quantize_rows_e5m2(const void* x, int64_t m, int64_t k, int64_t ld_x, const float* scale,
                            uint8_t* q, int64_t ld_q, daxq_stream_t stream);

/*
 * The quantisers above for any element type the reference accepts (fp32, fp16, bf16:
 *   dax/quant/nn/dynamic/functional.py:99-103) and any quantised format, selected by arguments:
 * x_dtype DAXQ_BF16 / DAXQ_F16 / DAXQ_F32, q_fmt DAXQ_FMT_I8 / _E4M3 / _E5M2.
 * daxq_act_quant_rows: per-row dynamic scale, computed and floored in x's own type before it is widened
 *   (the eager dtype chain of :124-129: fp16 rounds the quotient to fp16, fp32 does not round);
 * daxq_quantize_rows: leaf quantiser with the caller's per-row scale (dax/quant/nn/quantized/functional.py:11-20).
 * Last-dimension groups (block (1, ..., 1, G)) are rows of the [numel / G, G] view and use these two.
 */
int daxq_act_quant_rows(const void* x, int x_dtype, int q_fmt, int64_t m, int64_t k, int64_t ld_x,
                        void* q, int64_t ld_q, float* scale, daxq_stream_t stream);
/* daxq_act_quant_rows with the arguments _dynamic_quantize_func takes from its caller
 *   dax/quant/nn/dynamic/functional.py:54-61, :126-127
 * quant_max (> 0) instead of the format's own maximum, eps (>= 0) instead of 2^-23 as the floor of the scale, and
 * scale_round = DAXQ_SCALE_ROUND_X (what daxq_act_quant_rows does) or DAXQ_SCALE_ROUND_NONE:
 *   scale = max( round( f32(rowamax) / quant_max ), round( eps ) ),   round = to x's element type, or none.
 * The scale is fp32 and the leaf quantiser computes in fp32 (a scale of a 16-bit type changes that arithmetic:
 * daxq_block_quantize).  e4m3fn / e5m2 rows of bf16 elements divide element by element when the scale is not rounded. */
int daxq_act_quant_rows_ex(const void* x, int x_dtype, int q_fmt, int64_t m, int64_t k, int64_t ld_x,
                           void* q, int64_t ld_q, float* scale, float quant_max, float eps, int scale_round,
                           daxq_stream_t stream);
int daxq_quantize_rows(const void* x, int x_dtype, int q_fmt, int64_t m, int64_t k, int64_t ld_x, const float* scale,
                       void* q, int64_t ld_q, daxq_stream_t stream);

/*
 * Any other block shape of _dynamic_quantize_func (dax/quant/nn/dynamic/functional.py:54-148: per-channel
 * activations, 2-d tiles, blocks over leading dimensions).  The contiguous tensor x is seen through the view of
 * _get_reduction_params (:13-51): nd <= 8 dimensions view_shape[0..nd), reduced[d] != 0 for the dimensions a block
 * spans.  view_shape and reduced are HOST arrays, read before the call returns.
 * daxq_block_scale:    scale[b] = max( round( absmax(block b) / qmax ), round( eps ) ), b row-major over the kept
 *                      dimensions; round = to x's own type when round_to_x != 0 (dynamic rule), none otherwise.
 * daxq_block_quantize: q[i] = leaf quantiser of x[i] with its block's scale; q has x's shape, one byte per element.
 *                      scale_dtype: the element type of the scale the caller asked _dynamic_quantize_func for
 *                      (:128-129); the values are passed as fp32 either way (exact widening).  DAXQ_F32 (every wrapper
 *                      of the reference): fp32 arithmetic.  A 16-bit type: 1.0 / scale is rounded to it, and x * inv and
 *                      x / scale to what type promotion makes of x and the scale -- that 16-bit type when x has it too,
 *                      fp32 otherwise (dax/quant/nn/quantized/functional.py:11-20).
 */
int daxq_block_scale(const void* x, int x_dtype, int nd, const int64_t* view_shape, const int32_t* reduced, float qmax,
                     float eps, int round_to_x, float* scale, daxq_stream_t stream);
int daxq_block_quantize(const void* x, int x_dtype, int q_fmt, int nd, const int64_t* view_shape, const int32_t* reduced,
                        const float* scale, int scale_dtype, void* q, daxq_stream_t stream);

/*
 * Per-tensor schemes (the block of dax/quant/qscheme.py:10-26 is the whole tensor).  The GEMM and the leaf
 * quantisers above take a scale per row / per channel; a per-tensor scale is handed to them written out as a
 * vector, which gives the same arithmetic per element.  These entry points keep that on the device.
 *
 * daxq_tensor_scale: dynamic per-tensor scale from per-row statistics (daxq_row_minmax):
 *   a = max_i max(-row_min[i], row_max[i]);  scale1[0] = max( round(a / qmax), round(eps) ), round = RNE to bf16 when
 *   round_bf16 == 1, to fp16 when it is 2 (the activation rule for a tensor of that type,
 *   dax/quant/nn/dynamic/functional.py:124-129) or none when 0 (fp32 tensors, and the observer rule,
 *   dax/quant/quantization/observer.py:97-134); expand[0..n_expand) receives the same value.
 * daxq_tensor_minmax_update: running min / max of a calibration observer,
 *   dax/quant/quantization/observer.py:200-214:  min_inout[0] = min(min_inout[0], min_i row_min[i]), same for max.
 * daxq_broadcast_f32: dst[0..n) = src[0]; how dax/quant/nn/quantized/linear.py:98-100 expands its input scale.
 */
int daxq_tensor_scale(const float* row_min, const float* row_max, int64_t m, float qmax, float eps, int round_bf16,
                      float* scale1, float* expand, int64_t n_expand, daxq_stream_t stream);
int daxq_tensor_minmax_update(const float* row_min, const float* row_max, int64_t m,
                              float* min_inout, float* max_inout, daxq_stream_t stream);
int daxq_broadcast_f32(const float* src, float* dst, int64_t n, daxq_stream_t stream);

/*
 * Per-row min and max of a bf16 matrix, in fp32: the statistics of the per-channel weight observer.
 * Replaces PerChannelMinMaxObserver.forward   dax/quant/quantization/observer.py:284-312
 */
int daxq_row_minmax(const void* x, int64_t m, int64_t k, int64_t ld_x,
                    float* min_out, float* max_out, daxq_stream_t stream);
/* the same for x of element type x_dtype (DAXQ_BF16 / DAXQ_F16 / DAXQ_F32): weights of fp16 / fp32 modules */
int daxq_row_minmax_t(const void* x, int x_dtype, int64_t m, int64_t k, int64_t ld_x,
                      float* min_out, float* max_out, daxq_stream_t stream);

/*
 * scale[i] = max( max(-min[i], max[i]) / qmax, 2^-23 ) in fp32 (no bf16 rounding).
 * Replaces UniformQuantizationObserverBase._calculate_qparams   dax/quant/quantization/observer.py:97-134
 */
int daxq_scale_from_minmax(const float* min_in, const float* max_in, int64_t n, float qmax,
                           float* scale, daxq_stream_t stream);
/* the same with the observer's own floor instead of 2^-23 (its `eps` buffer, dax/quant/quantization/observer.py:19-35, :125) */
int daxq_scale_from_minmax_eps(const float* min_in, const float* max_in, int64_t n, float qmax, float eps,
                               float* scale, daxq_stream_t stream);

/*
 * INT8 GEMM on MFMA with the fused epilogue.
 * Replaces out_dtype(aten.mm, int32, Xq, Wq^T) and the scale / cast / bias tail
 *   dax/quant/nn/dynamic/linear.py:214-228
 * xq   int8 [m, k] (ld_xq), sx fp32 [m]; wq int8 [n, k] (ld_wq), sw fp32 [n];
 * bias bf16 [n] or NULL; out bf16 [m, n] (ld_out).
 * acc  optional int32 [m, n] (ld_acc) dump of the exact accumulators, or NULL.
 * k must be a multiple of DAXQ_K_ALIGN; xq, wq 16-byte aligned with ld % 16 == 0.
 *   acc[i,j] = sum_k xq[i,k] * wq[j,k]                         (exact)
 *   out[i,j] = bf16( f32( bf16( f32_rne(acc) * sx[i] * sw[j] ) ) + f32(bias[j]) )
 */
int daxq_linear_i8(const int8_t* xq, int64_t ld_xq, const float* sx,
                   const int8_t* wq, int64_t ld_wq, const float* sw,
                   const void* bias, void* out, int64_t ld_out,
                   int32_t* acc, int64_t ld_acc,
                   int64_t m, int64_t n, int64_t k, daxq_stream_t stream);

/*
 * FP8 e4m3fn GEMM on MFMA (fp32 accumulate) with the fused epilogue.
 * Replaces torch._scaled_mm(Xq, Wq^T, scale_a, scale_b, bias, out_dtype=bf16)
 *   dax/quant/nn/dynamic/linear.py:155-173
 *   out[i,j] = bf16( (sum_k f32(xq[i,k]) * f32(wq[j,k])) * sx[i] * sw[j] + f32(bias[j]) )
 * acc is an optional fp32 [m, n] dump of the raw accumulators, or NULL.
 */
int daxq_linear_e4m3(const uint8_t* xq, int64_t ld_xq, const float* sx,
                     const uint8_t* wq, int64_t ld_wq, const float* sw,
                     const void* bias, void* out, int64_t ld_out,
                     float* acc, int64_t ld_acc,
                     int64_t m, int64_t n, int64_t k, daxq_stream_t stream);

/* As daxq_linear_e4m3 with e5m2 activation bytes against e4m3fn weight bytes (mixed-format MFMA). */
int daxq_linear_e5m2_e4m3(const uint8_t* xq, int64_t ld_xq, const float* sx,
                          const uint8_t* wq, int64_t ld_wq, const float* sw,
                          const void* bias, void* out, int64_t ld_out,
                          float* acc, int64_t ld_acc,
                          int64_t m, int64_t n, int64_t k, daxq_stream_t stream);

/*
 * The general form of the three entry points above: any operand pairing the reference's constructor accepts
 *   dax/quant/nn/dynamic/linear.py:42-89   (int8 x int8; any of FP8_ALLOWED_DTYPES for activations and weights,
 *                                           dax/quant/nn/quantized/functional.py:4-7)
 * and any module dtype (out_dtype = the float weight's dtype, :263): out and bias are out_dtype elements
 * (DAXQ_BF16 / DAXQ_F16 / DAXQ_F32).
 *   int8: out = T( f32( T( f32_rne(acc) * sx[i] * sw[j] ) ) + f32(bias[j]) )   T = round to out_dtype   (:221-228)
 *   fp8:  out = T( acc * sx[i] * sw[j] + f32(bias[j]) )                        (torch._scaled_mm, :155-173)
 * acc: optional int32 (int8) / fp32 (fp8) dump of the raw accumulators.
 * kernel: 0 = the library's choice by shape.  Other values pick one implementation, for tests and comparisons: low 16
 * bits 2 / 5 = the generic kernel on 256x256 / 128x128 tiles (an implementation of its own, any shape), 8 / 11 / 14 =
 * the tiled kernel on 256x256 / 128x128 / 256x128 tiles (int8: 16x16x64 MFMAs; fp8: 16x16x128 MFMAs; needs m, n >= the
 * tile edge, 256 for the 256x128 tiles);
 * bits 16-23, when not zero, set the depth of the tile-order groups; bits 24-27 the tile order of the 256x256 kernels
 * (0 = by shape, 1 = groups of tile rows, 2 = banded patches of 8 x 4 tiles per XCD; every order computes every tile
 * once, the results are the same bits); bits 28-29 the treatment of the last, partial round of workgroups of a launch
 * of 256x256 tiles in row groups (0 = by shape: when the launch has one to eight whole rounds and the tiles left over
 * number at most a quarter of the CUs, they run as their 128x128 quadrants with a CU each, and when they
 * number at most half of the CUs, as their 256x128 halves with a CU each, in workgroups of the same grid behind
 * those of the whole tiles;
 * 1 = never; 2 = whenever they number at most a quarter / half of the CUs).
 * int8 results are the same bits for every choice.  fp8 results are the same bits for every choice of tile size, tile
 * order and cut of the tiled kernel (one sequence of MFMAs per output element), so an output row does not depend on
 * how many rows the launch has; the generic kernel (any fp8 launch with n < 128, or m < 128 rows) adds in another
 * order and agrees to fp32 rounding.  Every kernel writes bf16, fp16 and fp32; the accumulator dump of the tiled
 * kernels exists with bf16 outputs.  The choice is an argument of the call: the library keeps no process-wide
 * selection.
 */
int daxq_linear_w8a8(int x_fmt, int w_fmt, int out_dtype,
                     const void* xq, int64_t ld_xq, const float* sx,
                     const void* wq, int64_t ld_wq, const float* sw,
                     const void* bias, void* out, int64_t ld_out,
                     void* acc, int64_t ld_acc,
                     int64_t m, int64_t n, int64_t k, int kernel, daxq_stream_t stream);

/*
 * The whole forward of the dynamic W8A8 linear in one call: the per-token quantiser of x followed by the GEMM with the
 * fused epilogue, i.e. daxq_act_quant_rows + daxq_linear_w8a8 (or its split-K form) on the caller's stream.
 * Replaces Linear.forward
 *   dax/quant/nn/dynamic/linear.py:146-228   (FP8 branch :146-178, INT8 branch :181-228)
 * x     [m, k] of x_dtype elements (DAXQ_BF16 / DAXQ_F16 / DAXQ_F32), leading dimension ld_x
 * xq    scratch for the quantised activation, one byte per element, [rows_alloc, ld_xq], ld_xq >= roundup(k, DAXQ_K_ALIGN);
 *       16-byte aligned, ld_xq % 16 == 0; the call writes rows [0, m) (columns [k, roundup(k)) as zeros)
 * sx    scratch for the per-token scales, fp32 [rows_alloc]
 * wq    quantised weight [n, roundup(k, DAXQ_K_ALIGN)] (ld_wq), pad columns zero; sw fp32 [n]; bias [n] of out_dtype or NULL
 * out   [rows_alloc, n] of out_dtype elements (ld_out); rows [0, m) are the result
 * rows_alloc >= m: rows that xq, sx and out really hold.  With m < 128 <= rows_alloc (and n >= 128) the tiled kernels run
 *       on 128 rows of those buffers (twice as fast as the kernel that takes fewer rows); rows [m, 128) of out then hold
 *       unspecified values.  Pass rows_alloc = m to have nothing beyond row m touched.
 * workspace / workspace_bytes: optional split-K workspace as for daxq_linear_w8a8_splitk (counters zero), or NULL.
 *       INT8 launches with bf16 outputs and few tiles then cut K into ranges (same bits as the plain launch).
 * kernel: as for daxq_linear_w8a8 (0 = the library's choice).
 * act_scale_round: DAXQ_SCALE_ROUND_X, the reference's eager arithmetic, or DAXQ_SCALE_ROUND_NONE, the per-token scale
 *       kept in fp32 as under the torch.compile decorator of the reference's forward (:143).
 * Formats and output types as for daxq_linear_w8a8.  The caller owns every buffer; nothing is allocated.
 */
int daxq_dynamic_linear(int x_dtype, int x_fmt, int w_fmt, int out_dtype, int act_scale_round,
                        const void* x, int64_t ld_x,
                        void* xq, int64_t ld_xq, float* sx, int64_t rows_alloc,
                        const void* wq, int64_t ld_wq, const float* sw, const void* bias,
                        void* out, int64_t ld_out,
                        int64_t m, int64_t n, int64_t k,
                        void* workspace, int64_t workspace_bytes, int kernel, daxq_stream_t stream);
/* The three pairings of the bf16 DiT by name (bf16 x, bias and out; eager scale; rows_alloc = m; no workspace; the library's kernel):
 * int8 x int8 (dax/quant/nn/dynamic/linear.py:181-228), e4m3fn x e4m3fn and e5m2 x e4m3fn (:146-178). */
int daxq_dynamic_linear_i8(const void* x, int64_t ld_x, int8_t* xq, int64_t ld_xq, float* sx,
                           const int8_t* wq, int64_t ld_wq, const float* sw, const void* bias,
                           void* out, int64_t ld_out, int64_t m, int64_t n, int64_t k, daxq_stream_t stream);
int daxq_dynamic_linear_e4m3(const void* x, int64_t ld_x, uint8_t* xq, int64_t ld_xq, float* sx,
                             const uint8_t* wq, int64_t ld_wq, const float* sw, const void* bias,
                             void* out, int64_t ld_out, int64_t m, int64_t n, int64_t k, daxq_stream_t stream);
int daxq_dynamic_linear_e5m2_e4m3(const void* x, int64_t ld_x, uint8_t* xq, int64_t ld_xq, float* sx,
                                  const uint8_t* wq, int64_t ld_wq, const float* sw, const void* bias,
                                  void* out, int64_t ld_out, int64_t m, int64_t n, int64_t k, daxq_stream_t stream);

/* The tile order daxq_linear_w8a8 takes for a launch of 256x256 tiles when bits 24-27 of `kernel` are 0, as the value
 * of those bits: 1 = groups of tile rows, 2 = banded patches (large launches: K >= 2048, N >= 5120, M >= 7937 and no
 * XCD more than 5 % over its share of the tiles).  For tests and diagnostics; no
 * counterpart in the reference, whose matmul comes from a vendor library. */
int daxq_linear_tile_order_choice(int64_t m, int64_t n, int64_t k);

/*
 * Split-K form of daxq_linear_w8a8 for launches with too few output tiles to fill the CUs (a few hundred rows: the
 * text-token k / v projections of cross-attention, a single prompt): K is cut into `splits` equal ranges that run as
 * separate workgroups on 128x128 tiles, partial accumulators (int32 / fp32) go through `workspace`, and the workgroup
 * that finishes a tile last adds them in range order and applies the epilogue.  Results equal daxq_linear_w8a8's:
 * bit for bit for int8 (integer partial sums), to fp32 summation order for fp8.  bf16 outputs.  No counterpart in
 * the reference, whose matmul comes from a vendor library.
 *   splits     0 = daxq_linear_splitk_choice(m, n, k); 1 = the plain launch (workspace unused); else K / 128 must
 *              divide by it; needs m, n >= 128.
 *   workspace  device memory, 256-byte aligned, at least daxq_linear_splitk_workspace_bytes(m, n, splits) bytes.
 *              Its first 16 KiB are tile counters (at most 4096 output tiles of 128x128): they must be ZERO when
 *              the call is made and every call leaves them zero, so a workspace is cleared once (a hipMemset of those
 *              16 KiB, or a small clear kernel; not a hipMemsetAsync inside a captured graph) and then reused for any
 *              shapes.  Calls that share a workspace must not overlap in time.
 */
int daxq_linear_splitk_choice(int64_t m, int64_t n, int64_t k);
int64_t daxq_linear_splitk_workspace_bytes(int64_t m, int64_t n, int splits);
int daxq_linear_w8a8_splitk(int x_fmt, int w_fmt,
                            const void* xq, int64_t ld_xq, const float* sx,
                            const void* wq, int64_t ld_wq, const float* sw,
                            const void* bias, void* out, int64_t ld_out,
                            int64_t m, int64_t n, int64_t k,
                            int splits, void* workspace, int64_t workspace_bytes, daxq_stream_t stream);

/*
 * daxq_linear_w8a8_splitk without a workspace argument, for callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.
 * Counters and partial results live in a device array inside the library (16 KiB + 512 x 64 KiB = 33 570 816 bytes on
 * every GPU the library runs on, held until the process ends); the call allocates and frees nothing.
 *   limit   ceil(m / 128) * ceil(n / 128) * splits <= 512 (what daxq_linear_splitk_choice picks always fits);
 *           larger requests return DAXQ_ERR_ARG and launch nothing.
 *   sharing every call on a GPU uses that GPU's one array: calls that overlap in time on one GPU (two streams, two
 *           threads, two graphs replayed side by side) race.  Calls on one stream are ordered and safe.
 * Results equal daxq_linear_w8a8_splitk's for the same arguments, bit for bit (same kernels, same summation order).
 */
int daxq_linear_w8a8_splitk_static(int x_fmt, int w_fmt,
                                   const void* xq, int64_t ld_xq, const float* sx,
                                   const void* wq, int64_t ld_wq, const float* sw,
                                   const void* bias, void* out, int64_t ld_out,
                                   int64_t m, int64_t n, int64_t k,
                                   int splits, daxq_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* DAXQ_H */
