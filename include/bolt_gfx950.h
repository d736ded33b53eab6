/*
 * C-ABI of libbolt_gfx950.so -- the MI355X (gfx950) implementation of Bolt's quantized
 * matrix-product path. Plain pointers, sizes and Bolt's own POD records only.
 *
 * Every function that replaces a Bolt function keeps that function's argument list and
 * meaning, with the `_gfx950` suffix Bolt's per-architecture back ends use (`_x86`, `_arm`);
 * the comment above each declaration names the interface it replaces. `arch` selects the
 * pointer convention:
 *   AMD_GFX950         all data pointers are HOST pointers; the call stages operands to the
 *                      GPU, runs, copies results back and returns when they are in place.
 *   AMD_GFX950_DEVICE  all data pointers (matrices, vectors, tmp, results) are DEVICE pointers,
 *                      4-byte aligned; work is enqueued on the library stream and the call
 *                      returns without waiting. TensorDesc and `scale` arguments stay on the host:
 *                      a call that computes a scale and returns it through such a pointer (dynamic
 *                      quantisation, u8 results with a dynamic output scale) returns as soon as that
 *                      scale has reached the host; its tensors follow in stream order.
 * Errors come back as Bolt's EE codes; nothing here calls exit().
 *
 * Threads: like the reference, every function is re-entrant on disjoint buffers. Each calling thread has its own
 * context (stream, scratch words, staging buffers, last-error text): bolt_gfx950_set_stream, _synchronize, _last_error,
 * _timer_* and the "quantize_fused_spin" option act on the calling thread's context; the other options are process-wide.
 */
#ifndef BOLT_GFX950_H
#define BOLT_GFX950_H

/* Inside Bolt, whose own headers already define TensorDesc, EE, Arch ..., define
 * BOLT_GFX950_NO_TYPES before including this file so only the prototypes are taken. */
#ifndef BOLT_GFX950_NO_TYPES
#include "bolt_types.h"
#endif
#include <stdbool.h>
#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- runtime ------------------------------------------------------------------------- */
/* No counterpart in the reference (a CPU library needs no device context). */
EE bolt_gfx950_init(void);
/* stream: a hipStream_t (NULL = the default stream) for the calling thread's calls. The library never creates
 * streams. Changing the stream first waits for the work this thread enqueued on the previous one (the thread's
 * scratch words are shared by its calls). */
EE bolt_gfx950_set_stream(void *stream);
EE bolt_gfx950_synchronize(void);
const char *bolt_gfx950_last_error(void);
/* Tuning / test knobs. "gemm_tile": -1 shape heuristic (default), 0 general kernel, 2 the
 * register-staged 128x128 tiled kernel (needs K % 16 == 0), 7 / 10 / 11 the LDS-DMA
 * kernels (256x256 fragment-prefetch, 128x128 fragment-prefetch, 256x256 ping-pong; need
 * K % 64 == 0), 12 the 256x256 ping-pong kernel that requests A in whole 128-byte lines (needs
 * K % 128 == 0, else it runs as 11), 13 the same with the B fragments loaded straight into registers instead of
 * through LDS (K % 128 == 0, else 11), 14 the few-rows kernel, 15 the 128x128 fragment-prefetch kernel with the
 * program order of a K step written out (K % 64 == 0), 16 the same run by two groups of four waves on alternate
 * K tiles (K % 128 == 0, else 15); a variant whose shape requirement fails falls back to the general kernel. "conv_panel": which kernel a convolution with up to 64 output channels and
 * K <= 1024 uses: 4 (default) / 2 the filter-panel-in-LDS kernel with 64 / 32 pixels per wave, 0 the
 * shared-pipeline kernel. "conv_direct": whether that filter-panel kernel gathers from the caller's
 * u8 tensor in place when the channel count is a multiple of 16: 1 (default) for int32 and fp32
 * results, 2 for u8 results as well, 0 never (the input is first re-laid as a padded s8 image).
 * "quantize_fused": 1 (default) runs a dynamic quantisation (fp32 or int32 input, scale taken from
 * the tensor's maximum) as one launch that reads the tensor once and keeps it in registers
 * across a grid-wide barrier, for tensors of up to 512 K elements that are 16-byte aligned (less
 * latency per call; larger tensors are faster in two passes); 0 always takes the two-pass form.
 * "bnn_mfma": how the 1-bit convolution runs: 2 (default) on the matrix cores
 * with its operands expanded to E2M1 pairs (v_mfma_scale_f32_16x16x128_f8f6f4) where the shape has
 * that kernel (256+ output channels, 128+ tiles of 256 pixels) and as 1 otherwise; 1 on the int8
 * matrix cores with one byte per value; 0 on the vector ALU (xor + popcount).
 * "lstm_gemm_rows" (>= 1, default 4): the LSTM cell sends calls with at least this many batch rows through the
 * matrix cores when its weight carries the GEMM packing (rnn_transform_filter_gfx950). Every variant
 * returns the same bytes. "conv_onepass" (default 1): a u8 convolution through the filter-panel kernel runs once, its
 * workgroups agreeing on the tensor-wide maximum with the accumulators in registers, where all of them fit the device
 * at once; 0 = two passes (maximum only, then the stores). "encoder_fused" (default 1): the encoder layer's
 * FullyConnected in front of the GELU also applies the GELU and quantises, in one launch; 0 = separate kernels, which
 * keep the fp32 intermediate. "quantize_fused_spin" (calling thread only): polling rounds of the bounded grid-wide wait (one-launch quantiser,
 * one-pass convolution, fused encoder FullyConnected) before a workgroup gives up and the call falls back to two passes (0 = default, about a second; tests use 1). */
EE bolt_gfx950_set_option(const char *name, int value);
/* Event counters for tests and monitoring: "quantize_fused_fallbacks" = dynamic quantisations whose one-launch form
 * gave up waiting for its grid (the CUs were held by other work) and were redone in two passes. NOT_FOUND otherwise. */
EE bolt_gfx950_get_counter(const char *name, unsigned long long *value);
void *bolt_gfx950_malloc(size_t bytes);
void bolt_gfx950_free(void *dptr);
EE bolt_gfx950_memcpy_h2d(void *dst, const void *src, size_t bytes);
EE bolt_gfx950_memcpy_d2h(void *dst, const void *src, size_t bytes);
EE bolt_gfx950_memcpy_d2d(void *dst, const void *src, size_t bytes);  /* enqueued on the library's stream, does not wait */
/* Event pair on the library stream; stop returns the elapsed milliseconds after waiting. */
EE bolt_gfx950_timer_start(void);
EE bolt_gfx950_timer_stop(float *ms);

/* ---- blas_enhance: axpby -------------------------------------------------------------- */
/* compute/blas_enhance/include/blas_enhance.h:25-26  vector_vector_axpby: y = a * x + b * y. DT_F32 only, as in the
 * x86 build (compute/blas_enhance/src/cpu/x86/axpby.cpp); every element is fma(a, x, y * b) like the reference's
 * 8-wide body (cpu/x86/fp32/axpby.cpp:23-29). */
EE vector_vector_axpby_gfx950(F32 a, TensorDesc xDesc, const void *x, F32 b, TensorDesc yDesc, void *y, Arch arch);

/* ---- blas_enhance: int8 GEMM --------------------------------------------------------- */
/* compute/blas_enhance/include/blas_enhance.h:36-37  matrix_matrix_multiply_tmp_bytes */
EE matrix_matrix_multiply_tmp_bytes_gfx950(TensorDesc matrixADesc, TensorDesc matrixBDesc, U32 *bytes, Arch arch);
/* blas_enhance.h:39-48  matrix_matrix_multiply
 * C = C_in + offsetC + A(u8) x B(s8); the first N int32 of `tmp` are offsetC (+ folded bias);
 * scale: NULL -> int32, scale[0] > 0 -> fp32 * (1/scale[0]), scale[0] < 0 -> u8 with scale[1]. */
EE matrix_matrix_multiply_gfx950(TensorDesc matrixADesc, const void *matrixA, TensorDesc matrixBDesc,
    const void *matrixB, U32 bytes, void *tmp, TensorDesc matrixCDesc, void *matrixC, const F32 *scale, Arch arch);
/* blas_enhance.h:67  matrix_matrix_multiply_rhs_format */
DataFormat matrix_matrix_multiply_rhs_format_gfx950(DataType dt);
/* blas_enhance.h:70  matrix_matrix_multiply_transform_rhs_bytes */
EE matrix_matrix_multiply_transform_rhs_bytes_gfx950(TensorDesc desc, U32 *bytes, U32 *rhsBytes, Arch arch);
/* blas_enhance.h:73-74  matrix_matrix_multiply_transform_rhs */
EE matrix_matrix_multiply_transform_rhs_gfx950(TensorDesc desc, const void *src, TensorDesc *descTran, void *dst,
    Arch arch);

/* ---- blas_enhance: int8 GEMV --------------------------------------------------------- */
/* blas_enhance.h:55  matrix_vector_multiply_tmp_bytes */
EE matrix_vector_multiply_tmp_bytes_gfx950(TensorDesc matrixDesc, TensorDesc vectorDesc, U32 *bytes, Arch arch);
/* blas_enhance.h:57-66  matrix_vector_multiply */
EE matrix_vector_multiply_gfx950(TensorDesc matrixDesc, const void *matrix, TensorDesc vectorDesc, const void *vector,
    U32 bytes, void *tmp, TensorDesc resultDesc, void *result, const F32 *scale, Arch arch);
/* blas_enhance.h:77  matrix_vector_multiply_weight_format */
DataFormat matrix_vector_multiply_weight_format_gfx950(DataType dt);
/* blas_enhance.h:79  matrix_vector_multiply_transform_weight_bytes */
EE matrix_vector_multiply_transform_weight_bytes_gfx950(TensorDesc desc, U32 *bytes, Arch arch);
/* blas_enhance.h:82-83  matrix_vector_multiply_transform_weight */
EE matrix_vector_multiply_transform_weight_gfx950(TensorDesc desc, const void *src, TensorDesc *descTran, void *dst,
    Arch arch);

/* ---- tensor_computing: quantize / dequantize / requantize ---------------------------- */
/* compute/tensor/src/cpu/x86/quantize.cpp:19  quantize_x86 (reached from quantize(),
 * compute/tensor/src/quantize.cpp:19-34). F32 -> {I8, U8_Q}, U8_Q -> I8, I32 -> {I8, U8_Q}.
 * `scale` is a host pointer, read and written as the reference does. */
EE quantize_gfx950(TensorDesc dDesc, const void *data, TensorDesc *qDesc, void *qData, F32 *scale, int mode,
    Arch arch);
/* compute/tensor/src/cpu/x86/dequantize.cpp:19  dequantize_x86 (bias ignored, as on x86). */
EE dequantize_gfx950(TensorDesc qDesc, void *qData, const F32 *scale, TensorDesc bDesc, void *bData,
    TensorDesc dDesc, void *dData, Arch arch);
/* compute/tensor/src/cpu/x86/quantize.cpp:64  quantize_bias_offsetC */
EE quantize_bias_offsetC_gfx950(const void *bias, TensorDesc biasDesc, DataType qType, const void *filter,
    TensorDesc filterDesc, const F32 *scale, void *offsetCBias, Arch arch);
/* compute/tensor/src/cpu/requantize.cpp:20  requantize_cpu */
EE requantize_gfx950(TensorDesc inputDesc, INT8 *input, F32 inputScale, TensorDesc outputDesc, INT8 *output,
    F32 outputScale, Arch arch);

/* ---- tensor_computing: int8 FullyConnected ------------------------------------------- */
/* compute/tensor/src/fully_connected.cpp:107-159  fully_connected_infer_forward_tmp_bytes */
EE fully_connected_infer_forward_tmp_bytes_gfx950(TensorDesc inputDesc, TensorDesc filterDesc, TensorDesc outputDesc,
    U32 *bytes, Arch arch);
/* compute/tensor/src/fully_connected.cpp:307-498  fully_connected, x86 int8 branch (:372-495), with
 * the Tensor arguments unwrapped as get_ptr_from_tensor / get_scale do (tensor_auxiliary.h:26-37):
 * input is DT_U8_Q [M, K] with scale inputScale; filter is the DT_I8 output of
 * matrix_matrix_multiply_transform_rhs (M > 1) or matrix_vector_multiply_transform_weight (M == 1)
 * with scale filterScale; bias is fp32 [N] or NULL. Output DT_F32: dequantised with
 * inputScale * filterScale; DT_U8_Q with *outputScale > 0: requantised in the product's epilogue;
 * DT_U8_Q with *outputScale <= 0: int32 result, then dynamic requantisation, new scale written to
 * *outputScale (host); DT_I32: raw accumulators. tmp needs the bytes the query above returns. */
EE fully_connected_gfx950(TensorDesc inputDesc, const void *input, F32 inputScale, TensorDesc filterDesc,
    const void *filter, F32 filterScale, TensorDesc biasDesc, const void *bias, U32 tmpBytes, void *tmp,
    TensorDesc outputDesc, void *output, F32 *outputScale, Arch arch);

/* ---- tensor_computing: int8 matmul ---------------------------------------------------- */
/* compute/tensor/src/matmul.cpp:203-300 (matmul_infer_forward_tmp_bytes) and :302-576 (matmul), the
 * x86 int8 branch with the Tensor arguments unwrapped: fp32 operands are quantised as whole tensors
 * (A -> U8_Q, B -> I8, the caller's scale as a floor; pass 0 or less for none), operands that
 * already have those types come with their scale; every 2-D slice [.., M, K] x [.., K, N] then goes
 * through matrix_matrix_multiply with B packed per slice, and C = cvt(acc) * (1 / (scaleA * scaleB))
 * (DT_F32) or the raw accumulators (DT_I32). Leading dimensions of A and B must equal C's or be
 * absent (a 2-D operand is shared by all slices). The bias copy of the reference is not part of the
 * int8 branch's result and is left out. For a vector result (M == 1 or N == 1) the reference swaps
 * the operand types (A -> I8, B -> U8_Q, :374-382) and goes through matrix_vector_multiply per
 * slice (:531-548): u8 matrix B x s8 row vector A when M == 1, s8 matrix A (packed into tmp) x u8
 * column vector B otherwise; operands handed over already quantised must then be I8 / U8_Q. */
EE matmul_infer_forward_tmp_bytes_gfx950(TensorDesc matrixADesc, bool transposeA, TensorDesc matrixBDesc, bool transposeB,
    TensorDesc matrixCDesc, U32 *bytes, Arch arch);
EE matmul_gfx950(TensorDesc matrixADesc, bool transposeA, const void *matrixA, F32 scaleA, TensorDesc matrixBDesc,
    bool transposeB, const void *matrixB, F32 scaleB, U32 tmpBytes, void *tmp, TensorDesc matrixCDesc, void *matrixC,
    Arch arch);

/* ---- tensor_computing: int8 convolution ---------------------------------------------- */
/* The inner (TensorDesc + pointer) forms the reference's convolution*() reach on x86:
 *   convolution_transform_filter_bytes_x86   compute/tensor/src/cpu/x86/convolution.cpp:105-170
 *   convolution_transform_filter_int8        compute/tensor/src/cpu/x86/int8/convolution_transform.cpp:192-238
 *   convolution_infer_forward_tmp_bytes_int8 compute/tensor/src/cpu/x86/int8/convolution.cpp:17-95
 *   convolution_int8                         compute/tensor/src/cpu/x86/int8/convolution.cpp:97-150
 * Sizes are this back end's own (a back end answers its own size queries); callers allocate what
 * the queries return, exactly as ConvolutionCPU does (convolution_cpu.hpp:454-523).
 * Filter: DT_I8 DF_NCHW [oc, ic, fh, fw] -> blob tagged DF_NCHWC2NxC4 = [offsetC oc*4 | packed].
 * Input: DT_U8_Q in DF_NCHWC8 or DF_NCHWC16. Output DF_NCHWC16 (what the reference produces; a
 * trailing block is 8 wide when oc % 16 == 8) or DF_NCHWC8; DT_F32 (optionally + eltwiseInput, laid
 * out like the output), DT_I32, or DT_U8_Q with the tensor-wide dynamic output scale.
 * scale[3] = {input scale, output scale (written), filter scale}, host memory. group must be 1. */
/* convolution_infer_output_size_cpu (compute/tensor/src/convolution.cpp:28-109) as the AVX-512 build answers it:
 * oh / ow from the padding, dilation, stride and round mode; DF_NCHWC16 for a DT_U8_Q target with fn != 8, else
 * DF_NCHWC8; NOT_SUPPORTED when fn % 8 != 0. convolution_infer_forward_algorithm_x86 (cpu/x86/convolution.cpp:23-103)
 * for a quantised target: POINTWISE for 1x1 filters, DIRECT otherwise; an algorithm already chosen is kept. */
EE convolution_infer_output_size_gfx950(TensorDesc inputDesc, TensorDesc filterDesc, ConvolutionParamSpec convParamSpec,
    TensorDesc *outputDesc, DataType targetDataType, Arch arch);
EE convolution_infer_forward_algorithm_gfx950(TensorDesc inputDesc, TensorDesc filterDesc, TensorDesc outputDesc,
    ConvolutionParamSpec convParamSpec, ConvolutionPolicy policy, ConvolutionForwardAlgorithm *algorithm,
    DataType targetDataType, ActivationParamSpec activationDesc, Arch arch);
/* Filter blob bytes: fn * 4 + ALIGN(fn, 16) * ALIGN(fh * fw * ALIGN(fc, 16), 64) + 32. That equals the reference's
 * fn * ALIGN(fc, 16) * fh * fw + fn * 4 + 32 whenever fn % 16 == 0 and fh * fw * ALIGN(fc, 16) % 64 == 0 (every
 * BASELINE shape) and is larger otherwise, so allocate from THIS query. ftmDesc = the filter's desc with
 * df = DF_NCHWC2NxC4 and the channel dim rounded up to 16, as convolution_transform_filter_int8 returns it. */
EE convolution_transform_filter_bytes_gfx950(TensorDesc filterDesc, ConvolutionParamSpec convParamSpec,
    ConvolutionForwardAlgorithm algorithm, U32 *bytes, Arch arch);
EE convolution_transform_filter_gfx950(TensorDesc filterDesc, const void *filter, ConvolutionParamSpec convParamSpec,
    ConvolutionForwardAlgorithm algorithm, TensorDesc *ftmDesc, void *filterTransformed, Arch arch);
EE convolution_infer_forward_tmp_bytes_gfx950(TensorDesc inputDesc, TensorDesc filterDesc, TensorDesc outputDesc,
    ConvolutionParamSpec convParamSpec, ConvolutionForwardAlgorithm algorithm, U32 *bytes, Arch arch);
EE convolution_gfx950(TensorDesc inputDesc, const void *input, const void *eltwiseInput, TensorDesc filterDesc,
    const void *filter, ConvolutionParamSpec convParamSpec, ConvolutionForwardAlgorithm algorithm, TensorDesc biasDesc,
    const void *bias, U32 tmpBytes, void *tmp, TensorDesc outputDesc, void *output, F32 *scale,
    ActivationParamSpec activationDesc, Arch arch);

/* Int8 convolution with one filter scale per OUTPUT CHANNEL. No counterpart in the reference, whose int8 kernels
 * carry one scale for the whole filter (compute/tensor/src/cpu/x86/int8/avx512/convolution_direct.cpp:2406-2422,
 * 2687-2692); this is the convolution a channel-wise quantised filter needs. Same descs, filter blob, tmp size and
 * layouts as convolution_gfx950; scaleW = oc fp32 scales (device memory with AMD_GFX950_DEVICE, host memory with
 * AMD_GFX950), bias = oc fp32 values or NULL.
 *   f = cvt(acc) * (1.0f / (scale[0] * scaleW[oc]))      single fp32 operations, the reciprocal first
 *   f = f + bias[oc]; f = f + eltwise (DT_F32 result only); f = max(f, 0) with ACTIVATION_RELU
 *   DT_F32  : f is the result; scale[1] is left alone.
 *   DT_U8_Q : one output scale for the tensor. scale[1] > 0 on entry: static, q = quantise(f, scale[1]); otherwise
 *             dynamic, s = 127 / max|f| over the tensor (1 when that is 0), q = quantise(f, s), scale[1] = s on return
 *             (quantise = the fp32 -> u8 arithmetic of quantize_gfx950: rne(f * s + 128.0f) clamped to [1, 255]).
 * With every scaleW[oc] equal, bias NULL or all zero and a DT_F32 result this is convolution_gfx950 (the reference) bit
 * for bit; the u8 result equals quantize_gfx950 applied to the DT_F32 result. scale = host {input, output}. */
EE bolt_gfx950_convolution_int8_perchannel(TensorDesc inputDesc, const void *input, const void *eltwiseInput,
    TensorDesc filterDesc, const void *filter, ConvolutionParamSpec convParamSpec, const F32 *scaleW, TensorDesc biasDesc,
    const void *bias, U32 tmpBytes, void *tmp, TensorDesc outputDesc, void *output, F32 *scale,
    ActivationParamSpec activationDesc, Arch arch);
/* convolution_gfx950 / bolt_gfx950_convolution_int8_perchannel for chains of quantised operators that must not wait
 * for the host (no counterpart in the reference, which returns the new output scale through the host pointer
 * scale[1]): device pointers only, the input scale is READ from device memory (*dscaleI, e.g. what the producing
 * call left there) and the output scale is LEFT in device memory (*dscaleO); the call only enqueues.
 *   scaleW == NULL: one filter scale filterScale; DT_F32 / DT_I32 / DT_U8_Q results and every byte as convolution_gfx950
 *                   gives them for scale = {*dscaleI, -, filterScale}; *dscaleO = what that call leaves in scale[1]
 *                   (dscaleO may be NULL for DT_F32 / DT_I32). bias is required, as there.
 *   scaleW != NULL: the per-channel form above; DT_U8_Q with staticOutputScale > 0 quantises with that scale, otherwise
 *                   dynamically; *dscaleO = the scale used (untouched for DT_F32).
 * tmp: at least convolution_infer_forward_tmp_bytes_gfx950. A dynamic u8 result then runs the convolution twice
 * (maximum, then store). With the bolt_gfx950_convolution_async_tmp_bytes it runs ONCE where the shape allows (at most
 * 64 output channels, a reduction of at most 1024, channels a multiple of 16, every workgroup resident at once): the
 * workgroups agree on the tensor-wide maximum with their values in registers. The extra 4 bytes per output element are
 * only written if that agreement is abandoned (other work held the CUs; bounded wait, bolt_gfx950_set_option
 * "quantize_fused_spin"): the workgroups then park their values there and the last one to finish quantises the
 * tensor alone -- slow, correct, and still without the host. */
EE bolt_gfx950_convolution_async_tmp_bytes(TensorDesc inputDesc, TensorDesc filterDesc, TensorDesc outputDesc,
    ConvolutionParamSpec convParamSpec, U32 *bytes);
EE bolt_gfx950_convolution_async(TensorDesc inputDesc, const void *input, const void *eltwiseInput, TensorDesc filterDesc,
    const void *filter, ConvolutionParamSpec convParamSpec, TensorDesc biasDesc, const void *bias, U32 tmpBytes, void *tmp,
    TensorDesc outputDesc, void *output, const float *dscaleI, F32 filterScale, const F32 *scaleW, float *dscaleO,
    F32 staticOutputScale, ActivationParamSpec activationDesc);

/* ---- tensor_computing: int8 deconvolution (transposed convolution) ------------------------ */
/* The (TensorDesc + pointer) forms behind the reference's deconvolution*() on x86:
 *   deconvolution_infer_output_size_cpu        compute/tensor/src/deconvolution.cpp:23-65
 *   deconvolution_infer_forward_algorithm_cpu  compute/tensor/src/cpu/deconvolution.cpp:23-55
 *   deconvolution_transform_filter_bytes_cpu   compute/tensor/src/cpu/deconvolution.cpp:128-156
 *   deconvolution_transform_filter_cpu         compute/tensor/src/cpu/deconvolution.cpp:158-186
 *   deconvolution_infer_forward_tmp_bytes_cpu  compute/tensor/src/cpu/deconvolution.cpp:188-250
 *   deconvolution_cpu                          compute/tensor/src/cpu/deconvolution.cpp:487-538
 * Input DT_U8_Q: DF_NCHW runs the reference's IM2COL_GEMM route (deconvolution_gemm, :252-365), DF_NCHWC16 its
 * POINTWISE route (deconvolution_pointwise_x86, cpu/x86/deconvolution.cpp:130-257); both multiply every input pixel
 * with the [ic] x [fh * fw * oc] filter matrix and add the columns onto the output pixels they land on, and differ in
 * where bias, ReLU and the change of type sit -- each is reproduced bit for bit, including what the call leaves in
 * the caller's scale array: scale[3] = {input, output (in / out), filter}, host memory;
 *   IM2COL_GEMM: DT_F32 leaves it alone; DT_U8_Q sets scale[2] = scale[0] * scale[2] and, when scale[1] <= 0 on entry,
 *                scale[1] = the dynamic output scale (scale[1] > 0: quantised with that scale);
 *   POINTWISE:   scale[1] = the output scale (DT_U8_Q; always dynamic), or what the inner convolution left there
 *                (DT_F32: input * filter scale; with kernel == stride the scale of its u8 columns); DT_U8_Q with
 *                overlapping taps also sets scale[2] = scale[0] * scale[2].
 * Filter: DT_I8 DF_NCHW [ic, oc, fh, fw] -> blob of deconvolution_transform_filter_bytes_gfx950 bytes; ftmDesc is what
 * the reference returns for the algorithm (DF_NKNxKx 2-D for IM2COL_GEMM, DF_NCHWC2NxC4 for POINTWISE).
 * Output: DF_NCHWC16, DT_U8_Q or DT_F32. ic % 8 == 0 (DF_NCHWC16 input: ic % 16 == 0), oc % 16 == 0, group 1, no
 * dilation; ACTIVATION_NULL or ACTIVATION_RELU. GROUP_DECONV (depthwise) and DF_NCHWC8 inputs return NOT_SUPPORTED:
 * for the latter the reference lays its bias rows out in blocks of 8 under a 16-channel output. */
EE deconvolution_infer_output_size_gfx950(TensorDesc inputDesc, TensorDesc filterDesc, ConvolutionParamSpec convParamSpec,
    TensorDesc *outputDesc, DataType targetDataType, Arch arch);
EE deconvolution_infer_forward_algorithm_gfx950(TensorDesc inputDesc, TensorDesc filterDesc, TensorDesc outputDesc,
    ConvolutionParamSpec convParamSpec, ConvolutionPolicy policy, ConvolutionForwardAlgorithm *algorithm,
    DataType targetDataType, Arch arch);
EE deconvolution_transform_filter_bytes_gfx950(TensorDesc filterDesc, ConvolutionParamSpec convParamSpec,
    ConvolutionForwardAlgorithm algorithm, U32 *bytes, Arch arch);
EE deconvolution_transform_filter_gfx950(TensorDesc filterDesc, const void *filter, ConvolutionParamSpec convParamSpec,
    ConvolutionForwardAlgorithm algorithm, TensorDesc *ftmDesc, void *filterTransformed, Arch arch);
EE deconvolution_infer_forward_tmp_bytes_gfx950(TensorDesc inputDesc, TensorDesc filterDesc, TensorDesc outputDesc,
    ConvolutionParamSpec convParamSpec, ConvolutionForwardAlgorithm algorithm, U32 *bytes, Arch arch);
EE deconvolution_gfx950(TensorDesc inputDesc, void *input, TensorDesc filterDesc, const void *filter,
    ConvolutionParamSpec convParamSpec, ConvolutionForwardAlgorithm algorithm, TensorDesc scaleDesc, void *scale,
    TensorDesc biasDesc, const void *bias, U32 tmpBytes, void *tmp, TensorDesc outputDesc, void *output,
    ActivationParamSpec activationDesc, Arch arch);

/* ---- tensor_computing: int8 depthwise convolution ------------------------------------------ */
/* depthwise_convolution_transform_filter_int8 (compute/tensor/src/cpu/x86/int8/depthwise_convolution_transform.cpp:17-69,
 * bytes: compute/tensor/src/depthwise_pointwise_convolution.cpp:197-205) and depthwise_pointwise_convolution_int8
 * (compute/tensor/src/cpu/x86/int8/avx512/depthwise_convolution_direct.cpp:441-599), each + Arch.
 * The filter blob is byte for byte the reference's: [offsetC c*4 | per 16 channels: [tap / 4][channel][tap % 4]],
 * tagged DF_NCHWN8HW4 as the reference tags it. The convolution reproduces the one result that function defines:
 * DT_I32 output (DF_NCHWC16) of the depthwise stage alone, from a DT_U8_Q DF_NCHWC16 input, ReLU or no activation,
 * acc = offsetC + round(bias * sI * sF) + sum in_u8 * w, scale[1] = sI * sF on return. Paddings and dilation must be
 * 0 / 1 (the reference's gather ignores them), c % 16 == 0; a pointwise filter, an eltwise input and DT_F32 / DT_U8_Q
 * outputs return NOT_SUPPORTED (the reference's fp32 epilogue converts the wrong register, its quantised result never
 * reaches the output tensor, its pointwise stage is not run). tmp is not used. */
EE depthwise_convolution_transform_filter_bytes_int8_gfx950(TensorDesc filterDesc, U32 *bytes, Arch arch);
EE depthwise_convolution_transform_filter_int8_gfx950(TensorDesc filterDesc, const INT8 *filter, TensorDesc *ftmDesc,
    INT8 *filterTransformed, Arch arch);
EE depthwise_pointwise_convolution_int8_gfx950(TensorDesc inputDesc, UINT8 *inArray, F32 *eltwiseInput,
    TensorDesc dwFilterDesc, const INT8 *dwFilterArray, TensorDesc pwFilterDesc, const INT8 *pwFilterArray,
    ConvolutionParamSpec convParamSpec, TensorDesc dwBiasDesc, const F32 *dwBiasArray, TensorDesc pwBiasDesc,
    const F32 *pwBiasArray, U32 tmpBytes, void *tmp, TensorDesc outputDesc, void *outArray, F32 *scale,
    ActivationParamSpec depthwiseActivationParamSpec, ActivationParamSpec pointwiseActivationParamSpec, Arch arch);

/* ---- offline quantisation: weight storage, load-time expansion, stored scales -------------------- */
/* The data-parallel part of the post-training quantisation tool (model_tools/tools/quantization/
 * post_training_quantization.cpp -> ms_datatype_converter): the three weight-storage converters of
 * model_tools/src/model_data_type_converter.cpp:22-103, same arguments + Arch, EE instead of void / F32:
 *   ws_datatype_converter_int8  q = rne(w * scale), scale = max(127.0 / max|w|, *scale) (in: floor, out: used)
 *   ws_datatype_converter_int4  two values per byte, nibble = rne(w * 7.0 / max|w|) + 7, low nibble first;
 *                               scale = max(7.0 / max|w|, *scale). paramNum must be even (the reference misplaces
 *                               an odd trailing element, :99-101).
 *   ws_datatype_converter_bnn   one bit per weight (w > 0), first weight in the top bit; *scale = the first positive
 *                               weight (the reference returns it). paramNum % 8 == 0.
 * and the expansion a model loader applies to such weights (common/model_spec/src/model_deserialize.cpp:162-222):
 *   dequantize_int8_weight / dequantize_int4_weight  d = (1 / scale) * value (the DT_F32 instantiations)
 *   dequantize_int4_int8 / dequantize_int4_u8_q      value = nibble - 7 as s8, or + 128 as u8
 * originalPtr / q are fp32 / packed inputs, targetPtr / d outputs; host or device pointers by Arch. */
EE ws_datatype_converter_int8_gfx950(U8 *originalPtr, U8 *targetPtr, int paramNum, F32 *scale, Arch arch);
EE ws_datatype_converter_int4_gfx950(U8 *originalPtr, U8 *targetPtr, int paramNum, F32 *scale, Arch arch);
EE ws_datatype_converter_bnn_gfx950(U8 *originalPtr, U8 *targetPtr, int paramNum, F32 *scale, Arch arch);
EE dequantize_int8_weight_gfx950(int num, F32 scale, INT8 *q, F32 *d, Arch arch);
EE dequantize_int4_weight_gfx950(int num, F32 scale, INT8 *q, F32 *d, Arch arch);
EE dequantize_int4_int8_gfx950(int num, INT8 *q, INT8 *d, Arch arch);
EE dequantize_int4_u8_q_gfx950(int num, INT8 *q, UINT8 *d, Arch arch);
/* The rules by which the engine's int8 operators turn the QuantSpec records a .bolt model stores for them
 * (OperatorSpec::feature_scale, common/uni/include/parameter_spec.h:753-756; copied by Operator::init_feature_scale,
 * inference/engine/include/operator.hpp:139-150) into scales[3] = {input, output, filter}. The three operator
 * classes differ, and operatorKind selects whose rule is applied:
 *   BOLT_GFX950_OP_CONVOLUTION      (convolution_cpu.hpp:143-157) input: the first record, if positive and the input is
 *       not yet I8 / U8_Q, else the tensor's own scale; output: the last record, -2 there or no record -> -1 (dynamic),
 *       whatever the output type.
 *   BOLT_GFX950_OP_FULLY_CONNECTED  (fully_connected_cpu.hpp:92-103) input: as above but only with MORE than one record;
 *       output: only for an I8 / U8_Q output type, the last record unchanged (-2 stays -2), no record -> -1; for
 *       any other output type the operator leaves the tensor's scale alone and scales[1] is returned as -1.
 *   BOLT_GFX950_OP_DECONVOLUTION    (deconvolution_cpu.hpp:65-84) as FullyConnected; for a non-quantised output type
 *       scales[1] is the 0 that `F32 scales[3] = {-1}` leaves there.
 * MatMul has two inputs and three records (matmul_cpu.hpp:46-56) and is not covered.
 * *labelledNoQuant (optional) = 1 when the first record is 0 (operator.hpp:164-169).
 * Pure host logic: no GPU is touched, no Arch. A clip value c from the tool's scale table is stored as 127 / c. */
#define BOLT_GFX950_OP_CONVOLUTION 0
#define BOLT_GFX950_OP_FULLY_CONNECTED 1
#define BOLT_GFX950_OP_DECONVOLUTION 2
EE bolt_gfx950_operator_scales(int operatorKind, const QuantSpec *featureScale, U32 numQuantFeature, DataType inputDataType,
    DataType outputDataType, F32 inputTensorScale, F32 filterScale, F32 scales[3], int *labelledNoQuant);

/* ---- 1-bit (XNOR / DoReFa) convolution ---------------------------------------------- */
/* compute/tensor/src/cpu/arm/bnn/convolution.cpp:16-72 (convolution_bnn), filter transform
 * compute/tensor/src/cpu/arm/bnn/convolution_transform_bnn.h:32-86, tmp bytes
 * compute/tensor/src/cpu/arm/convolution.cpp:413-455, naive semantics
 * compute/tensor/src/cpu/general/convolution.cpp:141-178. The reference reaches these through the
 * same convolution_* dispatchers when filterDesc.dt is DT_BIN01 / DT_BIN11; here they are separate
 * symbols with convolution_bnn's own argument list (+ Arch).
 *   filter : DT_BIN11 (bit 1 = +1, bit 0 = -1) or DT_BIN01 (bit = value), [oc, ic, fh, fw], MSB first;
 *            DF_NCHW bit string or the reference's DF_NCHWN16C8 bytes -> blob tagged DF_NCHWN16C8
 *            of the size convolution_transform_filter_bytes_bnn_gfx950 returns: the bit-packed filter
 *            (oc*ic*fh*fw/8 bytes, the reference's size, rounded up to 256; byte order this library's)
 *            followed by the same filter as int8 values and as E2M1 pairs in the GEMM's packed
 *            layout, which is what the matrix-core routes multiply with.
 *   input  : DF_NCHWC8, DT_F32 (binarised on the fly: x >= 0 for BIN11, x >= 0.5 for BIN01, the
 *            thresholds of the reference's fp16 packing) or already packed bits of the filter's type,
 *            [n][ic/8][ih][iw] bytes, MSB = first channel of each 8.
 *   output : DF_NCHWC8, DT_F32 = fma(S, scale[oc], bias[oc]) or DT_I32 = S, the integer sum
 *            (XNOR: fh*fw*ic - 2*popcount(x ^ w) with padding counted as -1; DoReFa: popcount(x & w)).
 *   fp32 stands where the reference's ARM kernels use fp16. ic and oc must be multiples of 32,
 *   group 1, no dilation. scale / bias: fp32 [oc], same pointer convention as the other buffers. */
EE convolution_transform_filter_bytes_bnn_gfx950(TensorDesc filterDesc, U32 *bytes, Arch arch);
EE convolution_transform_filter_bnn_gfx950(TensorDesc filterDesc, const void *filter, TensorDesc *ftmDesc,
    void *filterTransformed, Arch arch);
EE convolution_infer_forward_tmp_bytes_bnn_gfx950(TensorDesc inputDesc, ConvolutionParamSpec convParamSpec, U32 *bytes,
    Arch arch);
EE convolution_bnn_gfx950(TensorDesc inputDesc, const void *input, TensorDesc filterDesc, const void *filter,
    ConvolutionParamSpec convParamSpec, TensorDesc scaleDesc, const void *scale, TensorDesc biasDesc, const void *bias,
    U32 tmpBytes, void *tmp, TensorDesc outputDesc, void *output, ActivationParamSpec activationDesc, Arch arch);

/* ---- quantised pooling and concatenation --------------------------------------------- */
/* pooling_x86 with DT_U8_Q data (compute/tensor/src/cpu/x86/pooling.cpp:22-61 ->
 * pooling_uint8, compute/tensor/src/cpu/x86/int8/avx512/pooling_int8.cpp:316-429). Input and output
 * DT_U8_Q in DF_NCHWC16, channels a multiple of 16, pad_top < kernel_h and pad_left < kernel_w as
 * in the reference; outputDesc carries the output height and width (pooling_infer_output_size is
 * the caller's, compute/tensor/src/pooling.cpp). Windows are clipped to the image. POOLING_MAX:
 * byte maximum. POOLING_MEAN: the reference's fixed-point form -- (sum of (u8 - 128)) * (65536 /
 * taps) >> 16 with a logical shift, + 128, unsigned saturation; taps = the clipped window, or
 * kernel_h * kernel_w with count_include_pad. scale: F32[2] in host memory, scale[0] = input scale
 * (read), scale[1] = output scale (written): scale[0] for max, scale[0] * (65536 / (kh*kw)) *
 * (kh*kw) / 65536 for mean. idx is unused for u8 data (as in the reference). Every window must
 * overlap the image, otherwise NOT_SUPPORTED. */
EE pooling_gfx950(TensorDesc inputDesc, const void *input, PoolingParamSpec poolingParamSpec, void *scale,
    TensorDesc outputDesc, void *output, void *idx, Arch arch);

/* concat_cpu (compute/tensor/src/cpu/concat.cpp:164-189): num inputs joined along
 * p.axis (counted from the outermost dimension, negative from the innermost, as in the reference).
 * With outputDesc.dt == DT_I8 and both scale pointers set, *outputScale = min(inputScale[0..num))
 * and every input is rescaled to it with requantize_cpu's arithmetic (compute/tensor/src/cpu/
 * requantize.cpp:20-50) while it is copied; the reference rescales its inputs in place first and
 * then copies, this entry point leaves the inputs untouched. Without scales it is a plain
 * concatenation of any element type. inputDesc / input / inputScale are host arrays of num entries;
 * inputScale and outputScale point to host memory; null or empty inputs are skipped (their scales
 * still take part in the minimum, as in the reference). All inputs must already be in the output's
 * data format (the reference's transformFormat step is not provided): DF_NCHWC8 / DF_NCHWC16
 * tensors join along the channel axis in whole channel blocks. tmp is unused. */
EE concat_infer_forward_tmp_bytes_gfx950(U32 num, const TensorDesc *inputDesc, TensorDesc outputDesc, U32 *bytes,
    Arch arch);
EE concat_gfx950(U32 num, const TensorDesc *inputDesc, void *const *input, const F32 *inputScale, ConcatParamSpec p,
    void *tmp, TensorDesc outputDesc, void *output, F32 *outputScale, Arch arch);

/* ---- int8 LSTM cell -------------------------------------------------------------------- */
/* rnncell_int8 -> lstmcell_int8 (compute/tensor/src/cpu/x86/int8/rnn.cpp:16-44, lstm.cpp:20-179), the
 * caller of the int8 matrix-vector product in recurrent models (compute/tensor/src/cpu/rnn.cpp:467-504).
 * Per batch row m: [x_m | h_m] is quantised to u8 with its own scale (scale[0] if positive, else
 * 127 / max|.|), multiplied with the int8 weight, dequantised with scale[1] as the weight scale, the
 * row's bias is added, then i, g, f, o gates (sigmoid, tanh, sigmoid(f + forget_bias), sigmoid), cell and
 * hidden state update with the reference's zoneout arithmetic.
 *   xDesc        DT_F32 [batch, xDim]; row m of currentX starts at currentX + m * batchStrideX floats
 *   filterDesc[0] DT_I8 [4 * num_outputs, xDim + num_outputs], tagged DF_NKN32 as the reference does;
 *   filter[0]    the output of matrix_vector_multiply_transform_weight_gfx950 for that matrix (packed
 *                rows followed by the compensation vector, which is where the reference reads offsetC),
 *                or, tagged DF_NKNx_NKN32, the output of rnn_transform_filter_gfx950 below
 *   bias[0]      DT_F32; row m reads 4 * num_outputs floats at bias[0] + m * steps * 4 * num_outputs with
 *                steps = batchStrideH / num_outputs / (bi_direction + 1), exactly as the reference
 *   scale        host F32[2] = {activation scale or <= 0 for dynamic, weight scale}; not written
 *   state        DT_F32 [batch][num_outputs (C) | num_outputs (H)], updated in place
 *   output       row m at output + m * batchStrideH floats, num_outputs floats
 *   tmp          rnncell_infer_forward_tmp_bytes_gfx950 bytes
 * Integer accumulators are exact; the gates use expf / tanhf where the reference's vector loop uses its
 * polynomial exp and its scalar tail uses double-precision libm: results agree to about 1e-6.
 * With num_projection > 0 (lstm.cpp:60-62, 128, 165-178) the gates produce num_projection values per row:
 * filterDesc[0] is [4 * num_projection, xDim + num_outputs], the bias row 4 * num_projection floats, the state row
 * [num_projection (C) | num_outputs (H)], and filter[1] is the fp32 projection matrix in the DF_NKN32 layout the
 * reference reads, [num_outputs / 32][num_projection][32] (num_outputs % 32 == 0); the hidden state and the output are
 * that matrix times the gates' values, every element one chain of fused multiply-adds over k ascending from 0
 * (mvm_nkn32_with_bias, cpu/x86/fp32/mvm_nkn32.h:19-140).
 * Modes other than RNN_LSTM and activation types other than ACTIVATION_TANH return NOT_SUPPORTED. */
EE rnncell_infer_forward_tmp_bytes_gfx950(TensorDesc inputDesc, TensorDesc filterDesc, TensorDesc outputDesc,
    RNNParamSpec rnnParamSpec, U32 *bytes, Arch arch);
/* rnn_transform_filter_bytes / rnn_transform_filter (compute/tensor/src/rnn.cpp:33-141) for the int8 LSTM weight:
 * s8 [4 * num_outputs][xDim + num_outputs] row-major (DF_NORMAL) -> a blob tagged DF_NKNx_NKN32 that holds the
 * matrix-vector blob above followed by the same matrix in the GEMM's packed layout. Given such a blob,
 * rnncell_gfx950 sends a call with at least `lstm_gemm_rows` batch rows (option, default 4) through the matrix
 * cores as ONE product that reads the weight once, instead of once per row; results are bit for bit those of
 * the matrix-vector route (exact int32 sums, the same dequantisation arithmetic). */
EE rnn_transform_filter_bytes_gfx950(TensorDesc filterDesc, RNNParamSpec rnnParamSpec, U32 *bytes, Arch arch);
EE rnn_transform_filter_gfx950(TensorDesc filterDesc, const void *filter, RNNParamSpec rnnParamSpec,
    TensorDesc *ftmDesc, void *filterTransformed, Arch arch);
EE rnncell_gfx950(TensorDesc xDesc, const void *currentX, const TensorDesc *filterDesc, const void **filter,
    const TensorDesc *biasDesc, const void **bias, F32 *scale, void *state, U32 tmpBytes, void *tmp,
    RNNParamSpec rnnParamSpec, U32 batchStrideX, U32 batchStrideH, TensorDesc hDesc, void *output, Arch arch);

/* ---- BERT-style int8 encoder layer (device pointers only, asynchronous) ------------- */
/* One post-LayerNorm transformer encoder layer as Bolt runs it for an int8 BERT model: the four
 * FullyConnected operators (QKV merged into one, as model_tools' FC+FC merge does for BERT,
 * model_tools/include/OPOptimizers/FCFCOptimizer.hpp) are int8 GEMMs on activations quantised
 * per tensor, dynamically (scale 127 / max|x|, quantize_x86 F32 -> U8_Q), with per-output-channel
 * weight scales; attention scores / softmax / context, residual adds, LayerNorm
 * (compute/tensor/src/cpu/x86/fp32/layer_norm.cpp:21-67, eps 1e-6) and tanh-GELU
 * (x86_functions_fp32.h:127-149) are fp32. Head size 64; no attention mask.
 *   hidden, out : fp32 [batch * seq, hidden]
 *   w*          : outputs of matrix_matrix_multiply_transform_rhs_gfx950 for [K, N] =
 *                 [hidden, 3*hidden] (Q | K | V columns), [hidden, hidden], [hidden, ffn], [ffn, hidden]
 *   s*          : fp32 [N] weight scales, Bolt convention (quantised = real * scale)
 *   b*          : fp32 [N] biases or NULL;  ln*: fp32 [hidden]
 * All pointers are device pointers except `layer` itself; the call enqueues 11 kernels on the
 * library stream and returns. workspace: 256-byte aligned, size from the query. */
typedef struct {
    U32 batch, seq, hidden, heads, ffn;
    const void *wqkv, *wo, *w1, *w2;
    const float *sqkv, *so, *s1, *s2;
    const float *bqkv, *bo, *b1, *b2;
    const float *ln1_gamma, *ln1_beta, *ln2_gamma, *ln2_beta;
} BoltEncoderLayerInt8;
EE bolt_gfx950_encoder_layer_int8_workspace_bytes(const BoltEncoderLayerInt8 *layer, size_t *bytes);
EE bolt_gfx950_encoder_layer_int8(const BoltEncoderLayerInt8 *layer, const float *hidden, float *out, void *workspace,
    size_t workspaceBytes);
/* Inspection hook: byte offsets inside `workspace` of the fp32 intermediates a call leaves behind, in
 * this order: qkv [T, 3*hidden], attention context [T, hidden], attention output projection
 * [T, hidden], first LayerNorm output [T, hidden], first FFN product before GELU [T, ffn] (the activated
 * values are never stored: the quantiser ahead of the second FFN product applies GELU to what it
 * reads), FFN output [T, hidden]. */
EE bolt_gfx950_encoder_layer_int8_workspace_layout(const BoltEncoderLayerInt8 *layer, size_t *offsets);
/* numLayers such layers back to back (a BERT encoder is twelve): layer i + 1 reads what layer i wrote. The result is,
 * bit for bit, that of numLayers calls of bolt_gfx950_encoder_layer_int8; what the stack saves is the abs-max pass over
 * every layer's input but the first -- the LayerNorm that closes a layer folds max|out| into the scratch slots, which
 * is exactly the maximum the next layer's input quantiser wants. All layers share batch, seq and hidden (else
 * NOT_MATCH); the workspace (size from the query) holds one layer's intermediates and two [T, hidden] fp32 buffers
 * that carry the activations from layer to layer. hidden and out may be the same buffer only for numLayers > 1. */
EE bolt_gfx950_encoder_stack_int8_workspace_bytes(const BoltEncoderLayerInt8 *layers, U32 numLayers, size_t *bytes);
EE bolt_gfx950_encoder_stack_int8(const BoltEncoderLayerInt8 *layers, U32 numLayers, const float *hidden, float *out,
    void *workspace, size_t workspaceBytes);

/* The layer's fp32 pieces on their own (device pointers, asynchronous):
 *   attention: qkv rows [Q | K | V] of 3*hidden floats -> ctx = softmax(Q K^T / 8) V per head of 64
 *   add_layernorm: out = LayerNorm(a + b) (b may be NULL), hidden % 4 == 0, hidden <= 2048
 *   gelu: in place, n % 4 == 0 */
EE bolt_gfx950_attention_f32(const float *qkv, U32 batch, U32 seq, U32 hidden, U32 heads, float *ctx);
EE bolt_gfx950_add_layernorm_f32(const float *a, const float *b, const float *gamma, const float *beta, U32 rows,
    U32 hidden, float *out);
EE bolt_gfx950_gelu_f32(float *x, size_t n);

/* ---- asynchronous forms with device-resident scales (AMD_GFX950_DEVICE only) -------- */
/* No counterpart in the reference: Bolt keeps a tensor's scale in host memory
 * (common/memory/include/tensor.hpp:83-96). These keep it on the GPU so that
 * quantize -> GEMM -> dequantize chains never wait for the host.
 *   quantize: *dscale (device, in/out) plays the role of `scale` in quantize_gfx950.
 *   GEMM/GEMV: fp32 out[m][n] = cvt(acc) * (1.0f / (*dscaleI * scaleW[n])) + bias[n], with
 *   per-output-channel weight scales scaleW[N] and optional fp32 bias[N] (both device);
 *   reduces to the per-tensor reference epilogue when every scaleW[n] is equal and bias is NULL. */
EE bolt_gfx950_quantize_f32_async(const float *data, U32 n, DataType qdt, void *q, float *dscale, int mode);

/* No counterpart in the reference. bolt_gfx950_quantize_f32_async for callers that cannot allocate device memory
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc): same arguments, same bytes
 * and same scale, but the partial-maximum slots its kernels need live in a static device array of 4 KiB that each
 * GPU holds until the process ends, and the call runs no hipMalloc / hipFree or any allocating routine (nor does
 * it initialise the rest of the library). At most BOLT_GFX950_NOALLOC_MAX_ELEMENTS elements (NOT_SUPPORTED beyond,
 * with the reason in bolt_gfx950_last_error()). Enqueued on the library's stream (bolt_gfx950_set_stream; the
 * default stream if none was set). All calls on one GPU share that array: calls that overlap on one GPU (two
 * streams, two threads) race. The array's device address is looked up once per GPU -- by bolt_gfx950_init(), or else
 * by the first call on that GPU, and that lookup (a module load and a symbol query) is neither capture-safe nor free of
 * allocation inside the runtime: call bolt_gfx950_init() or make one warm-up call on the GPU before using this entry
 * point under graph capture or inside a region that forbids allocation. */
#define BOLT_GFX950_NOALLOC_MAX_ELEMENTS (1u << 30)
EE bolt_gfx950_quantize_f32_noalloc(const float *data, U32 n, DataType qdt, void *q, float *dscale, int mode);
EE bolt_gfx950_mmm_int8_perchannel(U32 M, U32 N, U32 K, const void *A, const void *packedB, const I32 *offsetC,
    float *C, const float *dscaleI, const float *scaleW, const float *bias);
/* The same product with a u8 result for the next quantised operator: the fp32 value above put through the fp32 -> u8
 * quantiser (quantize_gfx950's arithmetic, avx512/quantize.cpp:150-155: rne(f * s + 128.0f) clamped to [1, 255]) with
 * the static output scale outputScale > 0. No counterpart in the reference, whose u8 epilogue has one scale for all
 * columns (blas_common_int8.h:565-590). C: [M][N] u8, device. */
EE bolt_gfx950_mmm_int8_perchannel_u8(U32 M, U32 N, U32 K, const void *A, const void *packedB, const I32 *offsetC,
    void *C, const float *dscaleI, const float *scaleW, const float *bias, F32 outputScale);
EE bolt_gfx950_mvm_int8_perchannel(U32 N, U32 K, const void *packedW, const void *x, const I32 *offsetC, float *y,
    const float *dscaleI, const float *scaleW, const float *bias);
/* `batch` independent matrix_vector_multiply products in ONE launch (decode serving: many
 * requests, one step each): product b multiplies weight blob number b % weightCopies (blobs are
 * weightStride bytes apart, each a complete transform_weight output) with activation vector
 * x + b*K, writes y + b*N, and uses dscaleI[b] as its input scale. offsetC is each blob's own
 * compensation vector (no folded bias); bias, if given, is the fp32 bias of the per-channel
 * epilogue. No counterpart in the reference, whose GEMV is one call per vector
 * (mvm_avx512_vnni.cpp:703-759). */
EE bolt_gfx950_mvm_int8_strided_batch(U32 batch, U32 N, U32 K, const void *packedW, size_t weightStride,
    U32 weightCopies, const void *x, float *y, const float *dscaleI, const float *scaleW, const float *bias);

#ifdef __cplusplus
}
#endif
#endif
