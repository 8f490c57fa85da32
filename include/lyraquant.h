/* lyraquant.h -- C ABI of the MI355X (gfx950) quantized-linear library `liblyraquant.so`.
 *
 * Every entry point enqueues HIP kernels on the caller's stream and returns immediately
 * (stream-ordered, no implicit synchronisation, no host-side allocation unless stated).
 * All pointers are DEVICE pointers unless the parameter name starts with `host_`.
 * Return value: LQ_OK (0) or a negative lq_status_t; lq_last_error() gives the message of the
 * last failure on the calling thread.  Nothing throws across this boundary.
 *
 * Each declaration cites the interface of the lyraDiff reference that it replaces
 * (paths relative to the reference's src/lyradiff/).  The reference's C++ templates on
 * T in {float, half, __nv_bfloat16} become an lq_dtype_t argument.
 *
 * Conventions: activations row-major [M,K]; weights row-major [N,K] before repacking; outputs
 * row-major [M,N].  "rows32 layout" = the byte matrix [N, Kb] re-ordered as
 * [N/32][Kb/16][32][16] (see lq_repack_rows32).
 */
#ifndef LYRAQUANT_H_
#define LYRAQUANT_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* lq_stream_t; /* a hipStream_t; NULL selects the null stream */

typedef enum { LQ_F32 = 0, LQ_F16 = 1, LQ_BF16 = 2, LQ_I32 = 3 } lq_dtype_t;

typedef enum {
    LQ_OK = 0,
    LQ_ERR_ARG = -1,         /* null pointer, bad enum */
    LQ_ERR_SHAPE = -2,       /* shape not supported by the kernels (message says which rule) */
    LQ_ERR_HIP = -3,         /* a HIP runtime call failed */
    LQ_ERR_UNSUPPORTED = -4  /* dtype combination not built */
} lq_status_t;

typedef enum { LQ_W_INT8 = 0, LQ_W_FP8 = 1, LQ_W_INT4 = 2 } lq_weight_kind_t;

/* Message of the last failing call on this thread ("" if none).  No reference counterpart:
 * the reference throws std::runtime_error / LyraException (utils/cuda_utils.h:128-147). */
const char* lq_last_error(void);

/* Library version, major*10000 + minor*100 + patch. */
int lq_version(void);

/* ---------------------------------------------------------------------------------------------
 * INT8 SmoothQuant activation quantisation
 * ------------------------------------------------------------------------------------------- */

/* q[r,k] = sat_s8(rne((f32(src[r,k]) * pre[k]) / s)), s = in_scale[0] or in_scale[r] when
 * per_token != 0.  pre may be NULL (treated as all ones).
 * Replaces invokeSqInputQuant<T> (kernels/quant_kernels/quant_kernels.h:8-17, kernels
 * sqInputQuant / sqPerTokenInputQuant quant_kernels.cu:51-115); rows = batch_size*seq_len.
 * Lifts the reference's limits (dim even; per-token only for dim <= 2048). */
int lq_sq_input_quant(int8_t* dst, const void* src, lq_dtype_t src_dtype, const float* pre_quant_scale,
                      const float* input_quant_scale, int per_token, size_t rows, size_t dim,
                      lq_stream_t stream);

/* Dynamic per-token variant: scale_out[r] = max_k|f32(src)*pre[k]| / 127 (1 when the row is all
 * zero) and q as above with that scale, in one pass.  The reference has only the consumer of a
 * per-token scale (quant_kernels.cu:93-115); the amax formula is that of its weight path
 * (quant_kernels.cu:207). */
int lq_sq_dynamic_quant(int8_t* dst, float* scale_out, const void* src, lq_dtype_t src_dtype,
                        const float* pre_quant_scale, size_t rows, size_t dim, lq_stream_t stream);

/* y[r,n] = T(f32(acc[r,n]) * s_in * s_w[n]).  Replaces invokeSqOutputDequant<T>
 * (quant_kernels.h:19-28, quant_kernels.cu:117-171). */
int lq_sq_output_dequant(void* dst, lq_dtype_t dst_dtype, const int32_t* src, const float* input_quant_scale,
                         const float* weight_quant_scale, int per_token, size_t rows, size_t dim,
                         lq_stream_t stream);

/* Per-output-channel weight quantisation on device: w' = w/pre[k], scale_out[n] = max_k|w'|/127,
 * q = sat_s8(rne(w'/scale)).  Replaces invokeGetINT8WeightScale<T> (quant_kernels.h:30-37,
 * quant_kernels.cu:173-223,270-312).  Output q is plain row-major [d_out, d_in]. */
int lq_int8_weight_quant(float* scale_out, int8_t* q_out, const void* weight, lq_dtype_t w_dtype,
                         const float* pre_quant_scale, size_t d_out, size_t d_in, lq_stream_t stream);

/* hidden [rows, 2*dim] -> q [rows, dim]:  h = x[:, :dim] + b[:dim]; g = gelu_tanh(x[:, dim:] + b[dim:]);
 * q = sat_s8(rne(f32(h*g) * pre[k] / in_scale[0])); adds and products rounded to T as the
 * reference does.  bias may be NULL.  Replaces invokeFusedAddBiasGegluInt8O<T>
 * (kernels/quant_kernels/ffn_kernels_int8.h:12-21, ffn_kernels_int8.cu:102-237); lifts its
 * dim in {1280,2560,5120} limit to any dim % 8 == 0.  T in {F16, BF16, F32}.
 * The first F16 / BF16 call on a device builds a constant lookup table on `stream` and waits for that
 * one kernel (later calls never block); under stream capture it records the table kernel instead. */
int lq_geglu_int8(int8_t* dst, const void* hidden, const void* bias, lq_dtype_t dtype,
                  const float* pre_quant_scale, const float* input_quant_scale, size_t rows, size_t dim,
                  lq_stream_t stream);

/* Same with the dynamic per-token scale of lq_sq_dynamic_quant (scale_out[rows]). */
int lq_geglu_int8_dynamic(int8_t* dst, float* scale_out, const void* hidden, const void* bias,
                          lq_dtype_t dtype, const float* pre_quant_scale, size_t rows, size_t dim,
                          lq_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * FP8 e4m3 (OCP e4m3fn) per-tensor quantisation
 * ------------------------------------------------------------------------------------------- */

/* *scale = max(*scale, max_i |f32(x_i)| / 448); the caller zero-initialises *scale, as the
 * reference's callers do (utils/common_macro_def.h:68).  Replaces invokeGetFP8WeightScale<T>
 * (kernels/lora/load_lora.h:30-31, load_lora.cu:16-23,48-54,108-112). */
int lq_fp8_amax_scale(float* scale, const void* x, lq_dtype_t dtype, size_t n, lq_stream_t stream);

/* dst[i] = e4m3_satfinite_rne(f32(src[i]) * (invert ? 1.0f/scale[0] : scale[0])).
 * Replaces invokeCudaD2DScaleCpyConvert<T_IN, __nv_fp8_e4m3> (utils/memory_utils.cu:431-446). */
int lq_fp8_scale_cast(uint8_t* dst, const void* src, lq_dtype_t dtype, const float* scale, int invert,
                      size_t n, lq_stream_t stream);

/* Dynamic per-tensor activation quant in one call: scale_out[0] = max|x|/448, then the cast
 * above with invert = 1.  No single reference counterpart (its activation scales are static,
 * layers/flux_attention_processor/FluxAttentionFP8Processor.cc:165-192); the two formulas are
 * those of the two functions above.  Overwrites scale_out (no zero-init needed). */
int lq_fp8_amax_cast(uint8_t* dst, float* scale_out, const void* src, lq_dtype_t dtype, size_t n,
                     lq_stream_t stream);
/* How lq_fp8_amax_cast runs: normally one launch (one 1024-thread workgroup per CU) whose workgroups exchange their
 * maxima through statically allocated device memory; each stream owns one of 16 exchange slots per device (work of
 * one stream runs in order), so calls on up to 16 streams may be in flight together.  Under stream capture, on the
 * per-thread default stream, on further streams and for unaligned buffers it runs three scratch-free kernels instead
 * (zero the scale, atomic-max pass, cast pass).  The exchange assumes the grid becomes resident; when kernels of OTHER
 * streams hold the device for longer than its bounded wait (~0.1 s), the workgroups that gave up cast with a NaN
 * scale, write NaN to scale_out and raise a flag:
 * lq_fp8_amax_cast_status() returns 0 if nothing went wrong on the current device since the last call, 1 if a
 * one-launch quantisation timed out (flag cleared; lq_last_error() explains), 2 if overlapping calls of
 * lq_fp8_amax_cast_static corrupted its ticket counters (stays until lq_fp8_amax_cast_static_reset), negative on a HIP
 * error.  It copies 8 bytes from the device and therefore waits for the null stream; call it after synchronising the
 * streams that quantised.  No reference counterpart. */
int lq_fp8_amax_cast_status(void);
/* The exchange slot (0..15) `stream` owns on the current device, assigned on first use; -1 when all 16 are taken (calls
 * on that stream then run the scratch-free kernels); negative status on a HIP error.  For diagnostics and tests. */
int lq_fp8_amax_cast_slot(lq_stream_t stream);
/* Gives the slot of `stream` back (call it when the stream is destroyed or done quantising, with none of its calls still
 * running): returns the freed slot, -1 if the stream owned none.  A process that creates and destroys streams without
 * it runs out of slots after 16 and silently takes the slower three-kernel route. */
int lq_fp8_amax_cast_release_slot(lq_stream_t stream);

/* lq_fp8_amax_cast for callers that cannot allocate or tolerate a kernel that waits: code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference.  Two launches, no barrier:
 * a partial-maximum pass whose workgroups leave their maxima and a ticket counter in a static device array
 * (the static block is 115 KiB per GPU, held until the process ends; its address is looked up once per device on first use) -- the
 * workgroup drawing the last ticket writes scale_out[0] = max|x| / 448 and re-arms the counter -- then the cast pass.
 * Same results as lq_fp8_amax_cast, bit for bit.  Calls no allocating routine.  n from 1 to
 * lq_fp8_amax_cast_static_max_elems() (2^28: 8192 partial maxima of 32768 elements), src and dst 16-byte aligned;
 * anything else is rejected with LQ_ERR_SHAPE / LQ_ERR_ARG.  All calls on one GPU share the one array: calls that
 * overlap in time (different streams, or a graph replay next to eager calls) race -- serialise them.  An overlap can leave
 * the ticket counters where no later call ever draws the last ticket (scale_out then stays unwritten while the call
 * returns LQ_OK): a ticket that one launch alone cannot issue raises a flag that lq_fp8_amax_cast_status() reports as 2,
 * and lq_fp8_amax_cast_static_reset (one tiny launch on `stream`, allocates nothing) puts counters and flag back to
 * zero -- run it once the overlapping calls have finished. */
int lq_fp8_amax_cast_static(uint8_t* dst, float* scale_out, const void* src, lq_dtype_t dtype, size_t n,
                            lq_stream_t stream);
/* Measurement aid, no counterpart in the reference: lq_fp8_amax_cast's one launch with four readings of the device's constant
 * 100 MHz clock per workgroup, stamps[4*w + 0..3] = workgroup w started, its partial maximum is formed (all its loads are back),
 * it is released from the grid-wide exchange, its stores are acknowledged.  stamps: device memory, 4 * 512 entries, zeroed by
 * the caller (entries of workgroups beyond the launch's grid stay zero).  LQ_ERR_UNSUPPORTED when the call would not take the
 * one-launch route (fewer than 4096 elements, unaligned buffers, no free exchange slot, stream capture). */
int lq_fp8_amax_cast_timeline(uint8_t* dst, float* scale_out, const void* src, lq_dtype_t dtype, size_t n,
                              unsigned long long* stamps, lq_stream_t stream);
size_t lq_fp8_amax_cast_static_max_elems(void);
int lq_fp8_amax_cast_static_reset(lq_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * W4A4 group-wise INT4 activation quantisation
 * ------------------------------------------------------------------------------------------- */

/* v = f32(x[m,k]) / smooth[k] (smooth may be NULL); scales[m,g] = max_{k in group g}|v| / 7;
 * q = clamp(rne(v / scales[m,g]), -8, 7); q_words[m, k/8] packs 8 values per uint32, element i
 * of the word in bits [4i, 4i+3].  scale_dtype F32 (as the reference stores) or F16 (scale is
 * rounded to fp16 first and the rounded value quantises).  group must be 64, k % 64 == 0.
 * Replaces the quantisation half of invokeFusedQuantizeAndLoraDownSimple
 * (kernels/w4a4_gemm/w4a4_gemm.h:6-16, w4a4_gemm.cu:206-214,769-954) without the LoRA-down
 * branch; lifts its m % 256 == 0 limit. */
int lq_w4a4_quantize(uint32_t* q_words, void* scales, lq_dtype_t scale_dtype, const void* x,
                     lq_dtype_t x_dtype, const float* smooth, int m, int k, int group, lq_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * Offline weight repack (MFMA-friendly tiled layout)
 * ------------------------------------------------------------------------------------------- */

/* Bytes per weight row: k for INT8/FP8, k/2 for INT4. */
size_t lq_weight_row_bytes(lq_weight_kind_t kind, size_t k);

/* dst = rows32 layout of the row-major byte matrix src [n, row_bytes]:
 *   dst[((nb*(row_bytes/16) + kc)*32 + r)*16 + b] = src[(nb*32 + r)*row_bytes + kc*16 + b].
 * A pure permutation (same byte count); n % 32 == 0, row_bytes % 16 == 0; dst != src.
 * Plays the role of preprocess_weights_for_mixed_gemm (kernels/cutlass_kernels/
 * cutlass_preprocessors.cpp:484-530): one-time re-ordering of a quantized weight for the
 * matrix-core operand layout -- here gfx950 MFMA instead of NVIDIA mma. */
int lq_repack_rows32(uint8_t* dst, const uint8_t* src, size_t n, size_t row_bytes, lq_stream_t stream);

/* Inverse permutation (for tests and for exporting a weight back to [N,K]). */
int lq_unpack_rows32(uint8_t* dst, const uint8_t* src, size_t n, size_t row_bytes, lq_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * Quantized GEMMs with fused dequant / bias / cast epilogue.  B is always the rows32 layout.
 * ------------------------------------------------------------------------------------------- */

/* C[m,n] = T( f32(sum_k A[m,k]*B[n,k]) * (alpha_col[n] * alpha_row[per_token ? m : 0]) [+ f32(bias[n])] )
 * with an exact int32 accumulator.  out_dtype F16/BF16/F32, or I32 (raw accumulator; scales and
 * bias ignored and may be NULL).  bias (nullable) has the output dtype.  n % 32 == 0, k % 64 == 0.
 * Replaces CutlassInt8GemmRunner<T>::gemm (kernels/cutlass_kernels/int8_gemm/int8_gemm.h:16-90,
 * int8_gemm_template.h:45-189,644-672) with EpilogueVisitorPerRowPerCol
 * (kernels/cutlass_extensions/include/cutlass_extensions/epilogue/threadblock/
 * epilogue_per_row_per_col_scale.h:239-305), as reached through cublasMMWrapper::runGemmInt8
 * (utils/cublasMMWrapper.h:368-385); the bias add replaces the separate bias kernels that
 * follow it (layers/basic_transformer/BasicTransformerInt8Block.cc:452,838). */
int lq_gemm_int8(void* C, lq_dtype_t out_dtype, const int8_t* A, const int8_t* B_rows32,
                 const float* alpha_col, const float* alpha_row, int per_token, const void* bias,
                 int m, int n, int k, lq_stream_t stream);

/* C[m,n] = T( act( (a_scale[0]*b_scale[0]) * sum_k A[m,k]*B[n,k] + f32(bias[n]) ) + beta*f32(residual[m,n]) )
 * on e4m3 operands with fp32 accumulation; act = tanh-GELU when gelu != 0.  bias and residual are
 * nullable and have the output dtype (F16/BF16/F32).  n % 32 == 0, k % 64 == 0.
 * Replaces the FP8 overload of cublasMMWrapper::GemmWithResidualAndBias
 * (utils/cublasMMWrapper.h:299-318, cublasMMWrapper.cc:1104-1274), whose (transa=T, weight as
 * "A", m/n swapped) column-major call is this row-major product. */
int lq_gemm_fp8(void* C, lq_dtype_t out_dtype, const uint8_t* A, const uint8_t* B_rows32,
                const float* a_scale, const float* b_scale, const void* bias, int gelu,
                const void* residual, float beta, int m, int n, int k, lq_stream_t stream);

/* C[m,n] = T( fold_{g=0..k/64-1} r = fmaf( f32(sum_{k in g} a*b) * sA[m,g], sB[n,g], r ) [+ f32(bias[n])] )
 * on nibble-packed int4 operands (A: uint32 words [m, k/8]; B: rows32 layout of the byte matrix
 * [n, k/2]), exact int32 group sums on the int8 MFMA.  Scales F32 or F16; out F16/BF16/F32.
 * n % 32 == 0, k % 128 == 0, group == 64.
 * Replaces the GEMM half of invokeFusedW4A4GemmAndLoraUp (kernels/w4a4_gemm/w4a4_gemm.h:18-30,
 * w4a4_gemm.cu:227-512,665-767) without the LoRA-up branch; the bias add replaces invokeAddBias
 * (layers/flux_attention_processor/FluxAttentionInt4Processor.cc:216-230). */
int lq_gemm_w4a4(void* C, lq_dtype_t out_dtype, const uint32_t* A_words, const uint8_t* B_rows32,
                 const void* sA, const void* sB, lq_dtype_t scale_dtype, const void* bias,
                 int m, int n, int k, int group, lq_stream_t stream);

/* lq_gemm_fp8 with the output's re-quantisation for the next FP8 linear prepared in the epilogue (no counterpart as
 * one call in the reference: its blocks run GemmWithResidualAndBias, then getFP8WeightScale-style amax or a calibrated
 * static scale, then invokeCudaD2DScaleCpyConvert as separate kernels, e.g.
 * layers/flux_single_transformer_block/FluxSingleTransformerFP8Block.cc:216-281):
 *   out_scale (optional): out_scale[0] = max(out_scale[0], max|C| / 448) over the T-rounded outputs -- exactly what
 *     lq_fp8_amax_scale(out_scale, C, ...) would add, without the pass over C; zero it before the call, then cast with
 *     lq_fp8_scale_cast(dst, C, dtype, out_scale, 1, m*n, stream).
 *   C_fp8 + C_fp8_scale (optional, static scale): C_fp8[m,n] = e4m3( f32(T(y)) * (1 / C_fp8_scale[0]) ), the codes
 *     lq_fp8_scale_cast would produce from C; C may then be NULL and the 16-bit output is never written.
 * Everything else as lq_gemm_fp8 (which is this call with the three extra pointers NULL). */
int lq_gemm_fp8_ex(void* C, lq_dtype_t out_dtype, const uint8_t* A, const uint8_t* B_rows32,
                   const float* a_scale, const float* b_scale, const void* bias, int gelu,
                   const void* residual, float beta, int m, int n, int k,
                   float* out_scale, uint8_t* C_fp8, const float* C_fp8_scale, lq_stream_t stream);

/* lq_gemm_fp8 without activation or residual that also joins the largest output into out_max[0]:
 *   out_max[0] = max( out_max[0], max_{m,n} f32(C[m,n]), 0 )      (the caller zeroes it; a float >= 0)
 * for lq_fp8_gelu_cast below, which derives the dynamic e4m3 scale of gelu(C) from it without a pass over C.  With 256-row
 * and 256-column multiples and k % 128 == 0 this runs the persistent one-wavefront-per-SIMD kernel (the maximum costs its
 * epilogue two instructions per four outputs, where an activation in the epilogue would cost it 13-18 us per tile). */
int lq_gemm_fp8_max(void* C, lq_dtype_t out_dtype, const uint8_t* A, const uint8_t* B_rows32, const float* a_scale,
                    const float* b_scale, const void* bias, int m, int n, int k, float* out_max, lq_stream_t stream);

/* Activation and dynamic FP8 quantisation of a stored GEMM output y [n elements] in one pass:
 *   h = T(gelu_tanh(y))   (invokeFusedBiasAndGelu on a stored T tensor, kernels/flux_single_transformer_block/
 *                          flux_single_transformer_kernels.cu:122-141, 194-201; the same arithmetic as gelu == 2 above)
 *   scale_out[0] = max|h| / 448,  dst = e4m3( h * (1 / scale_out[0]) ),  h_out (optional, T) = h
 * src_max[0] >= max(y, 0) exactly (lq_gemm_fp8_max leaves it): T(gelu(.)) is non-decreasing from 0 up, so max|h| =
 * h(src_max) whenever src_max >= 0.5 -- the result is then bit for bit that of lq_fp8_amax_cast on h.  A tensor without a
 * single value of 0.5 or more takes max(h(src_max), 0.171875) for max|h|: an upper bound (no |gelu| of a negative number
 * exceeds 0.17), not the exact maximum.
 * clear_max (optional, != src_max): set to 0 by this launch -- the slot the NEXT lq_gemm_fp8_max will accumulate into, so that a
 * chain that alternates two slots needs no fill launch between its steps. */
int lq_fp8_gelu_cast(uint8_t* dst, float* scale_out, void* h_out, const void* src, lq_dtype_t dtype, size_t n,
                     const float* src_max, float* clear_max, lq_stream_t stream);

/* ---- FP8 activations in k-panels -------------------------------------------------------------------------------------
 * A quantised activation [rows, k] stored as [k / 64][rows][64] instead of row-major: element (r, j) lies at byte
 * ((j / 64) * rows + r) * 64 + j % 64.  The 64 bytes a GEMM k-tile takes from each activation row are then contiguous over
 * the rows (256 rows = 16 KiB of whole 128-byte cache lines); from a row-major operand a 64-byte k-tile takes half a line
 * per row and every line is requested from L2 twice, one k-tile apart.  This is to the activation what rows32 is to the
 * weight: a layout made by the producer (here the quantiser, in the same pass) for the GEMM's transfers.  k % 64 == 0 and
 * rows * k < 2^32.  The reference has no counterpart (its FP8 activations are row-major, utils/memory_utils.cu:431-446);
 * codes, scale and GEMM outputs are bit for bit those of the row-major entry points.
 *   lq_fp8_amax_cast_panels   = lq_fp8_amax_cast (same one-launch form, same fall-back sequence) writing k-panels
 *   lq_fp8_scale_cast_panels  = lq_fp8_scale_cast (given scale: the reference's static _input_scale flow) writing k-panels
 *   lq_fp8_gelu_cast_panels   = lq_fp8_gelu_cast without h_out, writing k-panels
 *   lq_gemm_fp8_panels        = lq_gemm_fp8 without activation or residual on such an activation; with out_max also
 *                               lq_gemm_fp8_max (out_max may be NULL)
 * and for the static-scale sequences of the FLUX blocks (the row-major forms are documented further down):
 *   lq_layernorm_mod_fp8_panels, lq_layernorm_mod_fp8_dual_panels, lq_gate_residual_layernorm_mod_fp8_panels
 *                             = the LayerNorm + cast kernels writing their codes as k-panels [dim / 64][batch * rows][64]
 *   lq_gemm_fp8_codes_panels  = lq_gemm_fp8_codes reading its activation AND writing its codes as k-panels ([n / 64][m][64]; a
 *                               block of columns of a wider tensor of panels is the pointer C + (first column / 64) * m * 64)
 *   lq_gemm_fp8_gated_panels  = lq_gemm_fp8_gated reading its activation as k-panels */
/* The same layout for the INT8 path: lq_sq_dynamic_quant writing its codes as k-panels (scale_out as there; dim % 64 == 0,
 * dim <= 16384, 16-byte aligned buffers) and lq_gemm_int8 reading them.  Bit-identical codes, scales and outputs. */
int lq_sq_dynamic_quant_panels(int8_t* dst_panels, float* scale_out, const void* src, lq_dtype_t src_dtype,
                               const float* pre_quant_scale, size_t rows, size_t dim, lq_stream_t stream);
int lq_gemm_int8_panels(void* C, lq_dtype_t out_dtype, const int8_t* A_panels, const int8_t* B_rows32, const float* alpha_col,
                        const float* alpha_row, int per_token, const void* bias, int m, int n, int k, lq_stream_t stream);
int lq_fp8_amax_cast_panels(uint8_t* dst_panels, float* scale_out, const void* src, lq_dtype_t dtype, size_t rows, size_t k,
                            lq_stream_t stream);
int lq_fp8_scale_cast_panels(uint8_t* dst_panels, const void* src, lq_dtype_t dtype, const float* scale, int invert, size_t rows,
                             size_t k, lq_stream_t stream);
int lq_fp8_gelu_cast_panels(uint8_t* dst_panels, float* scale_out, const void* src, lq_dtype_t dtype, size_t rows, size_t k,
                            const float* src_max, float* clear_max, lq_stream_t stream);
int lq_gemm_fp8_panels(void* C, lq_dtype_t out_dtype, const uint8_t* A_panels, const uint8_t* B_rows32, const float* a_scale,
                       const float* b_scale, const void* bias, int m, int n, int k, float* out_max, lq_stream_t stream);
int lq_gemm_fp8_codes_panels(uint8_t* C_fp8_panels, const float* C_fp8_scale, lq_dtype_t round_dtype, const uint8_t* A_panels,
                             const uint8_t* B_rows32, const float* a_scale, const float* b_scale, const void* bias, int gelu, int m,
                             int n, int k, lq_stream_t stream);
int lq_gemm_fp8_gated_panels(void* C, lq_dtype_t out_dtype, const uint8_t* A_panels, const uint8_t* B_rows32, const float* a_scale,
                             const float* b_scale, const void* bias, const void* gate, size_t rows_per_gate, const void* residual,
                             int m, int n, int k, lq_stream_t stream);
int lq_layernorm_mod_fp8_panels(uint8_t* dst_panels, const void* src, const void* scale, const void* shift, lq_dtype_t dtype,
                                const float* input_scale, size_t batch, size_t rows_per_batch, size_t dim, float eps,
                                lq_stream_t stream);
int lq_layernorm_mod_fp8_dual_panels(uint8_t* dst_a_panels, const float* input_scale_a, uint8_t* dst_b_panels,
                                     const float* input_scale_b, const void* src, const void* scale, const void* shift,
                                     lq_dtype_t dtype, size_t batch, size_t rows_per_batch, size_t dim, float eps,
                                     lq_stream_t stream);
int lq_gate_residual_layernorm_mod_fp8_panels(uint8_t* dst_panels, void* hidden_out, const void* attn, const void* gate,
                                              const void* input, const void* scale, const void* shift, lq_dtype_t dtype,
                                              const float* input_scale, size_t batch, size_t rows_per_batch, size_t dim,
                                              float eps, lq_stream_t stream);

/* lq_gemm_fp8 (no activation) whose epilogue applies FLUX's gate and second residual:
 *   C[m,n] = T( T( T(y[m,n]) * gate[m / rows_per_gate, n] ) + residual[m,n] ),  y = (sa*sb)*acc + bias[n]
 * with every rounding of the reference's sequence "GEMM stores T, then multiply and add in T": it replaces
 * GemmWithResidualAndBias followed by invokeFusedGateAndResidual
 * (layers/flux_attn_post_processor/FluxAttnPostFP8Processor.cc:203-236,
 * layers/flux_single_transformer_block/FluxSingleTransformerFP8Block.cc:255-290,
 * kernels/flux_single_transformer_block/flux_single_transformer_kernels.cu:42-65,162-170).
 * gate [ceil(m / rows_per_gate), n] and residual [m, n] have the output dtype; C may alias residual. */
int lq_gemm_fp8_gated(void* C, lq_dtype_t out_dtype, const uint8_t* A, const uint8_t* B_rows32,
                      const float* a_scale, const float* b_scale, const void* bias, const void* gate,
                      size_t rows_per_gate, const void* residual, int m, int n, int k, lq_stream_t stream);

/* lq_gemm_fp8 that writes only e4m3 codes of its output, into a destination whose rows are `ldc` bytes apart:
 *   C_fp8[m*ldc + n] = e4m3( f32(T(act(y))) * (1 / C_fp8_scale[0]) ),  T = round_dtype (F16/BF16/F32)
 * gelu: 0 none; 1 tanh-GELU of the fp32 value (the GELU_BIAS epilogue, cublasMMWrapper.cc:1195-1199);
 * 2 tanh-GELU of T(y), the activation the reference applies to the stored GEMM output in invokeFusedCatAndGelu
 * (flux_single_transformer_kernels.cu:9-40).  With ldc = attn_dim + mlp_dim and C_fp8 offset by attn_dim this
 * fills the right-hand block of the single block's concatenated projection input directly
 * (FluxSingleTransformerFP8Block.cc:216-253) and the 16-bit intermediates are never written.
 * ldc >= n, ldc % 4 == 0, C_fp8 4-byte aligned. */
int lq_gemm_fp8_codes(uint8_t* C_fp8, size_t ldc, const float* C_fp8_scale, lq_dtype_t round_dtype,
                      const uint8_t* A, const uint8_t* B_rows32, const float* a_scale, const float* b_scale,
                      const void* bias, int gelu, int m, int n, int k, lq_stream_t stream);

/* lq_fp8_scale_cast on a matrix view: rows `src_ld` elements apart are cast into rows `dst_ld` bytes apart
 * (the left-hand, attention block of the concatenated tensor above).  cols % 16 == 0; every row of both views
 * 16-byte aligned. */
int lq_fp8_scale_cast_2d(uint8_t* dst, size_t dst_ld, const void* src, size_t src_ld, lq_dtype_t dtype,
                         const float* scale, int invert, size_t rows, size_t cols, lq_stream_t stream);

/* Weight-only quantized GEMM (W8A16 / W4A16 with per-output-channel scales):
 *   C[m,n] = T( f32(scale[n]) * sum_k A[m,k]*q[k,n] [+ f32(bias[n])] ),  fp32 accumulation
 * A, C, scale, bias of `dtype` (F16 or BF16); B_prepared from lq_repack_weight_only.  n % 32 == 0, k % 64 == 0.
 * Replaces CutlassFpAIntBGemmRunner<T, uint8_t | uint4b_t, PER_COLUMN_SCALE_ONLY>::gemm (A, B, weight_scales, [biases,]
 * C, m, n, k, ...) (kernels/cutlass_kernels/fpA_intB_gemm/fpA_intB_gemm.h:27-130).  The reference multiplies every
 * dequantised weight by the scale in T inside the main loop; here the scale is applied once per output.
 * Two tile configurations: 0 = 256x256 (eight wavefronts, three stages; chosen from 192 such tiles up), 1 = 256x128 (four
 * wavefronts, two stages); both walk k in the same order and give the same bits.  lq_gemm_set_thread_tactic(0 | 1) picks
 * one for the calling thread's next calls (the gemm_config argument of CutlassFpAIntBGemmRunner::gemm), -1 the built-in rule. */
int lq_gemm_weight_only(void* C, const void* A, lq_dtype_t dtype, const uint8_t* B_prepared, lq_weight_kind_t kind,
                        const void* scales, const void* bias, int m, int n, int k, lq_stream_t stream);

/* The same GEMM with group-wise ("fine-grained") scales and optional zero points along k:
 *   C[m,n] = T( sum_k A[m,k] * w[k,n] [+ f32(bias[n])] ),  w[k,n] the dequantised weight formed in T per element:
 *     F16:   w = T( T(q[k,n] * scale[k/g, n]) + zero[k/g, n] )      (multiply, then add: two roundings)
 *     BF16:  w = T( f32( q[k,n] * scale[k/g, n] + zero[k/g, n] ) )  (one fused multiply-add rounded to fp32, then to bf16; the
 *            reference's __hfma2 rounds the exact sum to bf16 once -- the two differ by one bf16 step where the fp32 value
 *            falls on a bf16 midpoint, measured on < 1e-3 of random weights)
 *   and w = T(q * scale) for both when `zeros` is NULL; q is the signed code (the +128 / +8 of the prepared layout removed).
 * scales and zeros are row-major [k / group_size, n] of `dtype`; group_size 64 or 128, k % group_size == 0.
 * Replaces CutlassFpAIntBGemmRunner<T, uint8_t | uint4b_t, FINEGRAINED_SCALE_ONLY | FINEGRAINED_SCALE_AND_ZEROS>::gemm(A, B,
 * weight_scales, weight_zero_points, biases, C, m, n, k, group_size, ...) (kernels/cutlass_kernels/fpA_intB_gemm/
 * fpA_intB_gemm.h:58-85); the per-element arithmetic is that of its MmaTensorOpDequantizer
 * (kernels/cutlass_extensions/include/cutlass_extensions/gemm/warp/mma_tensorop_dequantizer.h:150-222,370-390). */
int lq_gemm_weight_only_grouped(void* C, const void* A, lq_dtype_t dtype, const uint8_t* B_prepared, lq_weight_kind_t kind,
                                const void* scales, const void* zeros, const void* bias, int m, int n, int k, int group_size,
                                lq_stream_t stream);

/* One-time preparation of a weight-only weight: src_kn is the row-major [k, n] matrix of signed codes as
 * symmetric_quantize leaves it before preprocessing ("unprocessed_quantized_weight": int8, or for INT4 [k, n/2] bytes
 * with column 2j in the low nibble; kernels/cutlass_kernels/cutlass_preprocessors.cpp:532-631).  dst (k*n bytes for
 * INT8, k*n/2 for INT4) receives the layout lq_gemm_weight_only reads; the role of preprocess_weights_for_mixed_gemm
 * (cutlass_preprocessors.cpp:484-530), whose own layout is specific to NVIDIA's mma fragments. */
int lq_repack_weight_only(uint8_t* dst, const int8_t* src_kn, lq_weight_kind_t kind, size_t k, size_t n, lq_stream_t stream);

/* SmoothQuant smoothing vector, device side (calibration time).  The reference consumes a precomputed
 * pre_quant_scale from nvidia-modelopt (lyradiff/convert_model_scripts/convert_sd_quant_model.py:199,340); these two
 * calls produce it in the closed form its benchmark configuration states:
 *   lq_col_absmax:    out[k] = max(out[k], max_m |x[m,k]|)   -- zero `out` once, then call per calibration batch / weight
 *   lq_smooth_vector: s[k] = act_absmax[k]^alpha / weight_absmax[k]^(1-alpha);  pre_quant_scale[k] = 1/s[k];
 *                     smooth_out (optional) receives s, the factor the weight columns are multiplied by offline
 *                     (equivalently lq_int8_weight_quant divides by pre_quant_scale, quant_kernels.cu:197-199).
 * x [rows, dim] F16/BF16/F32, dim % 8 == 0. */
int lq_col_absmax(float* out, const void* x, lq_dtype_t dtype, size_t rows, size_t dim, lq_stream_t stream);
int lq_smooth_vector(float* pre_quant_scale, float* smooth_out, const float* act_absmax, const float* weight_absmax,
                     float alpha, size_t dim, lq_stream_t stream);

/* LayerNorm fused with the INT8 SmoothQuant quantisation that follows it: invokeLayerNormInt8O and, with a
 * residual, invokeFusedResidualBiasLayerNormInt8O (kernels/quant_kernels/layer_norm_int8.h:8-38):
 *   h = src [+ residual [+ bias]]   (T arithmetic; h is written to dst2 when a residual is given)
 *   y = T( gamma[k] * ((h - mean) * rstd) + beta[k] ),  mean/var over the row in fp32, rstd = 1/sqrt(var + eps)
 *   q = sat_s8(rne( f32(y) * pre[k] / s ))
 * s = input_quant_scale[0] (static, the reference's mode) or, when scale_out is given instead, the dynamic
 * per-token scale max_k|f32(y)*pre[k]| / 127 written to scale_out[rows] (amax <= 2^-24: s = 1).
 * src, residual, dst2 [rows, dim], bias, gamma, beta [dim] of `dtype` (F16 or BF16); pre_quant_scale fp32 [dim]
 * or NULL; dim % 8 == 0, dim <= 6144.  The statistics are fp32 sums in this library's own fixed order (the
 * reference runs Welford updates in T), so q agrees with the reference to within one step, not bit for bit. */
int lq_layernorm_int8(int8_t* dst, float* scale_out, void* dst2, const void* src, const void* residual,
                      const void* bias, const void* gamma, const void* beta, lq_dtype_t dtype,
                      const float* pre_quant_scale, const float* input_quant_scale, size_t rows, size_t dim,
                      float eps, lq_stream_t stream);

/* FLUX adaLN modulation fused with the FP8 cast that follows it: invokeLayerNormWithShiftAndScale
 * (kernels/norms/layer_norm.h:18-27, kernels/norms/layer_norm.cu:406-475) + invokeCudaD2DScaleCpyConvert
 * (layers/flux_attn_post_processor/FluxAttnPostFP8Processor.cc:125-140):
 *   y = T( T( T(scale[b,k] + 1) * T((x - mean) * rstd) ) + shift[b,k] ),  q = e4m3_rne_satfinite( f32(y) * (1/s) )
 * src [batch * rows_per_batch, dim], scale and shift [batch, dim] of `dtype` (F16 or BF16), s = input_scale[0]
 * (the reference's calibrated static scale).  Same remark on the statistics as above. */
int lq_layernorm_mod_fp8(uint8_t* dst, const void* src, const void* scale, const void* shift, lq_dtype_t dtype,
                         const float* input_scale, size_t batch, size_t rows_per_batch, size_t dim, float eps,
                         lq_stream_t stream);

/* lq_layernorm_mod_fp8 for a normalised tensor with two consumers, each with its own calibrated input scale (FLUX's
 * single block feeds norm_hidden to both to_qkv and proj_mlp: FluxSingleAttentionFP8Processor.cc:155-172,
 * FluxSingleTransformerFP8Block.cc:209-214): one read of src, two code tensors, no 16-bit tensor written. */
int lq_layernorm_mod_fp8_dual(uint8_t* dst_a, const float* input_scale_a, uint8_t* dst_b, const float* input_scale_b,
                              const void* src, const void* scale, const void* shift, lq_dtype_t dtype, size_t batch,
                              size_t rows_per_batch, size_t dim, float eps, lq_stream_t stream);

/* invokeFusedGateAndResidual + invokeLayerNormWithShiftAndScale + invokeCudaD2DScaleCpyConvert in one pass
 * (layers/flux_attn_post_processor/FluxAttnPostFP8Processor.cc:112-140):
 *   hidden_out = T( T(attn * gate[b,k]) + input ),  dst = lq_layernorm_mod_fp8(hidden_out, scale, shift, input_scale)
 * attn, input, hidden_out [batch * rows_per_batch, dim]; gate, scale, shift [batch, dim]; hidden_out may alias input. */
int lq_gate_residual_layernorm_mod_fp8(uint8_t* dst, void* hidden_out, const void* attn, const void* gate,
                                       const void* input, const void* scale, const void* shift, lq_dtype_t dtype,
                                       const float* input_scale, size_t batch, size_t rows_per_batch, size_t dim,
                                       float eps, lq_stream_t stream);

/* The same without a quantisation: dst = T( adaLN(hidden) ), for the W4A4 linears, which quantise per group of 64 and
 * also feed the 16-bit tensor to their low-rank branch (layers/flux_attn_post_processor/
 * FluxAttnPostInt4Processor.cc:118-150).  attn, gate and hidden_out are all NULL for a plain
 * invokeLayerNormWithShiftAndScale of `input` (kernels/norms/layer_norm.h:18-27). */
int lq_gate_residual_layernorm_mod(void* dst, void* hidden_out, const void* attn, const void* gate, const void* input,
                                   const void* scale, const void* shift, lq_dtype_t dtype, size_t batch,
                                   size_t rows_per_batch, size_t dim, float eps, lq_stream_t stream);

/* W4A4 GEMM with the SVDQuant low-rank branch of invokeFusedW4A4GemmAndLoraUp
 * (kernels/w4a4_gemm/w4a4_gemm.h:18-30; lora_up_gemm, kernels/w4a4_gemm/w4a4_gemm.cu:514-663):
 *   C = T( sum_g f32(p_g) * sA * sB  +  sum_r lora_act[m, r] * lora_up[n, r]  [+ bias[n]] ),
 * the second sum on the 16-bit float matrix instruction with fp32 accumulation, added to the same fp32
 * accumulator before the single rounding to T.  lora_act [m, lora_rank] and lora_up [n, lora_rank] are
 * row-major F16 or BF16 (lora_dtype), lora_rank a multiple of 16; both NULL disables the branch and the call
 * is then exactly lq_gemm_w4a4. */
int lq_gemm_w4a4_lora(void* C, lq_dtype_t out_dtype, const uint32_t* A_words, const uint8_t* B_rows32,
                      const void* sA, const void* sB, lq_dtype_t scale_dtype, const void* bias,
                      const void* lora_act, const void* lora_up, lq_dtype_t lora_dtype, int lora_rank,
                      int m, int n, int k, int group, lq_stream_t stream);

/* Epilogue options of lq_gemm_w4a4_ex, applied in this order to y = acc [+ low-rank] [+ bias] (fp32):
 *   gelu     0 none; 1 tanh-GELU of y; 2 tanh-GELU of T(y) (invokeFusedBiasAndGelu on a stored GEMM output,
 *            kernels/flux_single_transformer_block/flux_single_transformer_kernels.cu:122-141,194-201)
 *   addend   y = T( T(y) + addend[m,n] ): joins another linear's stored output (invokeFusedBiasAndResidual,
 *            flux_single_transformer_kernels.cu:67-93; FluxSingleTransformerInt4Block.cc:297-305)
 *   gate + residual   y = T( T( T(y) * gate[m / rows_per_gate, n] ) + residual[m,n] ) (invokeFusedGateAndResidual)
 *   C_fp8    e4m3( f32(T(y)) / C_fp8_scale[0] ) into rows ldc_fp8 bytes apart, next to or instead of C
 *            (invokeCudaD2DScaleCpyConvert in front of the FP8 ff_linear, FluxAttnPostInt4Processor.cc:167-173)
 * All pointers optional (NULL = step skipped); tensors have the output dtype. */
typedef struct lq_epilogue {
    int gelu;
    const void* addend;
    const void* gate;
    size_t rows_per_gate;
    const void* residual;
    uint8_t* C_fp8;
    size_t ldc_fp8;
    const float* C_fp8_scale;
} lq_epilogue_t;

/* lq_gemm_w4a4_lora with the epilogue options above (epi may be NULL; C may be NULL when epi->C_fp8 is given):
 * the W4A4 linears of the FLUX INT4 blocks followed by their bias/GELU, residual, gate and FP8 re-quantisation
 * kernels (layers/flux_attn_post_processor/FluxAttnPostInt4Processor.cc:155-205,
 * layers/flux_single_transformer_block/FluxSingleTransformerInt4Block.cc:260-316). */
int lq_gemm_w4a4_ex(void* C, lq_dtype_t out_dtype, const uint32_t* A_words, const uint8_t* B_rows32,
                    const void* sA, const void* sB, lq_dtype_t scale_dtype, const void* bias,
                    const void* lora_act, const void* lora_up, lq_dtype_t lora_dtype, int lora_rank,
                    int m, int n, int k, int group, const lq_epilogue_t* epi, lq_stream_t stream);

/* Down projection of the low-rank branch, the second half of invokeFusedQuantizeAndLoraDownSimple
 * (kernels/w4a4_gemm/w4a4_gemm.h:6-16; kernels/w4a4_gemm/w4a4_gemm.cu:931-953):
 *   out[m, r] = T_out( sum_k x[m, k] * lora_down[r, k] ),  x the UNsmoothed activations,
 * fp32 accumulation in a fixed order (the reference adds k-tiles with float atomics into a zeroed buffer).
 * x [m, k] and lora_down [rank, k] row-major F16 or BF16 (dtype), rank 32 or 64, k % 64 == 0;
 * out_dtype F32 (the reference's intermediate), F16 or BF16. */
int lq_lora_down(void* out, lq_dtype_t out_dtype, const void* x, const void* lora_down, lq_dtype_t dtype,
                 int m, int k, int rank, lq_stream_t stream);

/* Both halves of invokeFusedQuantizeAndLoraDownSimple (kernels/w4a4_gemm/w4a4_gemm.h:6-16; w4a4_gemm.cu:769-953) from ONE
 * read of x, as the reference has it: q_words/scales exactly as lq_w4a4_quantize writes them (the same bits), lora_act
 * [m, rank] = T_act( sum_k x[m,k] * lora_down[rank,k] ) as lq_lora_down defines it (fp32 accumulation in a fixed order; the
 * order differs from lq_lora_down's, so the two agree to fp32 rounding of the sum, not bit for bit).
 * One launch when x is F16/BF16, smooth is given, rank == 32, k % 128 == 0 and act_dtype is F32 or x_dtype; every other
 * combination that the two separate entry points accept runs them one after the other inside this call. */
int lq_w4a4_quantize_lora_down(uint32_t* q_words, void* scales, lq_dtype_t scale_dtype, void* lora_act,
                               lq_dtype_t act_dtype, const void* x, lq_dtype_t x_dtype, const float* smooth,
                               const void* lora_down, int m, int k, int rank, int group, lq_stream_t stream);

/* dst[i] = T(src[i]), the float -> T copy between the reference's two W4A4 kernels
 * (invokeCudaD2DcpyConvert<T, float>, utils/memory_utils.cu:398-402). */
int lq_cast_f32(void* dst, lq_dtype_t dst_dtype, const float* src, size_t n, lq_stream_t stream);

/* Between the QKV projections and the attention of a FLUX block: per-head RMSNorm of q and k, rotary embedding, and the
 * concatenation [text tokens, image tokens] -- invokeFusedRmsNormCatAndRope and (context_seq = 0) invokeFusedRmsNormAndRope
 * (kernels/rope/flux_apply_rope.h; kernels/rope/flux_apply_rope.cu:74-156,291-319; call sites
 * layers/flux_attention_processor/FluxAttentionFP8Processor.cc:232-245,
 * layers/flux_single_attention_processor/FluxSingleAttentionFP8Processor.cc:183-193).
 *   qkv [batch, seq, 3, heads, head_dim], context_qkv [batch, context_seq, 3, heads, head_dim] (or NULL with context_seq 0),
 *   out [batch, context_seq + seq, 3, heads, head_dim]: the flash-attention input of the reference (its nhidden_buffer),
 *   norm_qk / norm_added_qk [2 * head_dim]: the q weights then the k weights (qk_norm_weight, encoder_qk_norm_weight),
 *   rope [.., context_seq + seq, head_dim / 2, 2, 2] with rope_batch_stride elements between batches (0: one table for all).
 * q and k:  n = T(x * (1 / sqrt(mean(x^2) + eps))) * w  in T, then every pair (n0, n1) -> (T(T(n0*r00) + T(n1*r01)),
 * T(T(n0*r10) + T(n1*r11)));  v is copied.  dtype F16 or BF16 for every tensor; head_dim 64 or 128. */
int lq_rmsnorm_rope(void* out, const void* qkv, const void* context_qkv, const void* norm_qk, const void* norm_added_qk,
                    const void* rope, size_t rope_batch_stride, lq_dtype_t dtype, int batch, int seq, int context_seq,
                    int heads, int head_dim, float eps, lq_stream_t stream);

/* dst[i] = T( dst[i] + T( src[i] * T(alpha) ) ): merges a full-rank LoRA delta into a 16-bit (or fp32) weight
 * (invokeLoadLora, kernels/lora/load_lora.h + load_lora.cu:6-14,92-96).  An FP8 weight is re-quantised after the
 * merge the way FP8LoraWeight::load_lora / clear_lora do (interface/IFLoraWeight.h:79-128): restore the 16-bit
 * master copy, lq_load_lora, zero the scale, lq_fp8_amax_scale, lq_fp8_scale_cast, lq_repack_rows32. */
int lq_load_lora(void* dst, const void* src, lq_dtype_t dtype, size_t n, float alpha, lq_stream_t stream);

/* Forces the tile configuration ("tactic") used by the GEMM of `kind` (process-wide); -1 restores
 * the built-in static table.  Stands in for the CutlassGemmConfig argument of
 * CutlassInt8GemmRunner<T>::gemm and the tactic cache of GemmPluginProfiler
 * (kernels/cutlass_kernels/int8_gemm/int8_gemm.h:24-39, layers/gemm_utils/GemmProfiler.cc:78-143).
 * Unknown tactic numbers make the next GEMM call fail with LQ_ERR_ARG.  INT8 / FP8: 0-5 tile shapes with two wavefronts
 * per SIMD, 6 = 256x256 tiles with one wavefront per SIMD, 7 = the persistent form of 6 (one workgroup per CU walks its
 * tiles; full 256x256 tiles, k %% 128 == 0, scales and bias only, fp16 / bf16 output -- any other call runs as 6). */
int lq_gemm_set_tactic(lq_weight_kind_t kind, int tactic);

/* Tile configuration for the GEMM calls the CALLING THREAD makes from now on (any kind), ahead of every
 * other choice; -1 clears it.  This is how a per-call configuration argument is expressed
 * (the gemmConfig parameter of CutlassInt8GemmRunner<T>::gemm,
 * kernels/cutlass_kernels/int8_gemm/int8_gemm.h:24-36) without a process-wide side effect. */
int lq_gemm_set_thread_tactic(int tactic);

/* Number of tile configurations of the `kind` GEMM: valid tactic numbers are 0 .. count-1
 * (CutlassInt8GemmRunner<T>::getConfigs, kernels/cutlass_kernels/int8_gemm/int8_gemm.h:38-39). */
int lq_gemm_tactic_count(lq_weight_kind_t kind);

/* Per-shape tactic cache, the role of the reference's MNKProfileMap
 * (layers/gemm_utils/GemmProfiler.h:131-251).  A GEMM call picks, in this order: the process-wide
 * tactic of lq_gemm_set_tactic, the cache entry for its exact (m, n, k), the entry for (m rounded up
 * to a power of two, n, k) -- the bucket GemmPluginProfiler::getBestConfig uses
 * (layers/gemm_utils/GemmProfiler.cc:131-143) -- and last the built-in table.  tactic = -1 removes
 * an entry; lq_gemm_get_shape_tactic returns -1 when no entry applies.  Thread safe. */
int lq_gemm_set_shape_tactic(lq_weight_kind_t kind, int m, int n, int k, int tactic);
int lq_gemm_get_shape_tactic(lq_weight_kind_t kind, int m, int n, int k);

/* The per-shape tactic cache as a byte string, so that a process need not profile again what an earlier one measured
 * on the same part: the role of GemmPluginProfiler::serialize / deserialize / getSerializationSize
 * (layers/gemm_utils/GemmProfiler.cc:26-75; SmoothQuantGemmPlugin::serialize, layers/gemm_utils/SmoothQuantGemm.cc:177-194).
 * Format: the four bytes "LQT1", the entry count, then {kind, m, n, k, tactic} per entry, all little-endian int32.
 * lq_gemm_tactics_serialize writes lq_gemm_tactics_serialized_size() bytes (LQ_ERR_ARG when the buffer is smaller);
 * lq_gemm_tactics_deserialize checks the whole table (magic, length, kinds, tactic numbers against
 * lq_gemm_tactic_count) before it adds the entries to the cache, replacing entries of the same shape.  Host memory. */
size_t lq_gemm_tactics_serialized_size(void);
int lq_gemm_tactics_serialize(void* buffer, size_t buffer_bytes, size_t* written);
int lq_gemm_tactics_deserialize(const void* data, size_t bytes);

/* Set-up-time profiler, the role of GemmPluginProfiler::profileTactics
 * (layers/gemm_utils/GemmProfiler.cc:78-127,161-265): runs every tile configuration of the `kind`
 * GEMM on shape (m, n, k) with synthetic operands placed in `workspace` (caller-owned device memory
 * of at least lq_gemm_profile_workspace(kind, m, n, k) bytes, 256-byte aligned), times each between
 * two events on `stream`, stores the fastest in the per-shape cache and reports it.  Blocks the host
 * until the timed runs have finished; not for use under stream capture. */
size_t lq_gemm_profile_workspace(lq_weight_kind_t kind, int m, int n, int k);
int lq_gemm_profile(lq_weight_kind_t kind, int m, int n, int k, void* workspace, size_t workspace_bytes,
                    int* best_tactic, float* best_us, lq_stream_t stream);

/* Measurement aid (no reference counterpart): `probes` one-wavefront workgroups each record, into
 * out_ticks[2*i] and out_ticks[2*i+1], how far the shader clock counter and the constant 100 MHz counter advanced
 * while they idled for `microseconds`.  100 MHz * out[2i] / out[2i+1] is the clock the compute units ran at during that
 * window; launched on a second stream next to a kernel it tells the clock that kernel was given (the matrix kernels
 * are power-limited on random operands).  Enqueued on `stream`, returns immediately; 1 <= probes <= 1024. */
int lq_shader_clock_probe(uint64_t* out_ticks, int probes, unsigned microseconds, lq_stream_t stream);

/* Measurement aid (no reference counterpart): one 256-thread workgroup per CU; every wavefront issues `iters` times 16
 * independent v_mfma_f32_32x32x64_f8f6f4 (a 128x128 wavefront tile) on register operands drawn from `operand_codes` (e4m3
 * codes, n_codes >= 4096, 4-byte aligned; NULL = all-zero operands), two sets of fragments alternating, with no memory or
 * LDS traffic and no instruction that depends on an MFMA in flight: 2*32*32*64 * 16 * iters * 4 * *workgroups FLOP per launch.  Timed by the caller, it gives what the matrix pipes
 * alone sustain on this part -- on real codes they are power limited well below the published peak, on zeros they are not.
 * `sink` (4 bytes of device memory) is practically never written; *workgroups (optional) receives the grid size. */
int lq_mfma_fp8_probe(float* sink, const uint8_t* operand_codes, size_t n_codes, int iters, int* workgroups, lq_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* LYRAQUANT_H_ */
