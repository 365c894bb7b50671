/*
 * mxq.h - C ABI of libmxq_hip.so: MI355X (gfx950) kernels for MXNet's INT8
 * quantized-inference operators.
 *
 * This is the launcher the C++ FCompute<gpu> host functions call in place of
 * mshadow's Kernel<OP,gpu>::Launch, broadcast::RTCReduce, cublasGemmEx and
 * cudnnConvolutionForward.  Every entry point
 *   - takes plain device pointers, sizes and a raw hipStream_t (as void*; NULL
 *     is the default stream),
 *   - only enqueues work on that stream: no allocation, no free, no device or
 *     stream synchronisation, no retained state (the library has no mutable
 *     process-wide variables; the entry points are re-entrant and may be called
 *     concurrently from different threads on different streams, provided that
 *     calls in flight at the same time do not share a workspace),
 *   - returns 0 on success and -1 on failure with the message available from
 *     mxq_last_error() on the calling thread (the convention of
 *     include/mxnet/c_api_error.h:39-58 in the reference).
 * All pointers named min / max are DEVICE pointers to one float32, exactly as the
 * reference's min/max TBlobs of shape (1,).
 *
 * Reference paths are relative to the apache/mxnet tree.
 */
#ifndef MXQ_H_
#define MXQ_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MXQ_ABI_VERSION 3

/* element type codes = mshadow::TypeFlag (3rdparty/mshadow/mshadow/base.h:351-364) */
#define MXQ_FLOAT32 0
#define MXQ_FLOAT64 1
#define MXQ_UINT8 3
#define MXQ_INT32 4
#define MXQ_INT8 5
#define MXQ_INT64 6

/* Last error message of the calling thread ("" if none). */
const char* mxq_last_error(void);
int mxq_abi_version(void);

/* ---- _contrib_quantize_v2 ------------------------------------------------
 * Replaces QuantizeV2Operator<gpu>::Forward for fp32 input
 * (src/operator/quantization/quantize_v2-inl.h:218-305): the
 * Kernel<quantize_v2_zero_centered|quantize_v2_unsigned,gpu>::Launch calls and,
 * when uncalibrated, the two broadcast::RTCReduce passes (min, max) in front
 * of them.  out_type is MXQ_INT8 or MXQ_UINT8 (the reference's GPU build
 * refuses uint8, :198-201; here it follows the CPU kernel :66-95 and
 * saturates where the reference is undefined).  calibrated != 0 uses
 * (min_calib, max_calib); otherwise the range is reduced on the device in
 * `workspace` (>= mxq_quantize_v2_workspace(n) bytes, 16-byte aligned) and
 * never crosses the host. */
size_t mxq_quantize_v2_workspace(size_t n);
int mxq_quantize_v2(void* stream, const float* in, void* out, float* omin, float* omax,
                    size_t n, int out_type, int calibrated, float min_calib, float max_calib,
                    void* workspace, size_t workspace_bytes);

/* mxq_quantize_v2 for callers that cannot allocate (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc) and bring no workspace: the reduction
 * partials of the uncalibrated path live in a 16 KiB array inside the library's device
 * image (one copy per GPU, held until the process ends).  It has no counterpart in the
 * reference, whose operator always draws its temp space from the framework's resource
 * pool.  Same arguments and results as mxq_quantize_v2 without the workspace; n is
 * limited to 2^31 elements (a larger n is refused with an error).  The call allocates and
 * frees nothing.  All calls on one GPU share that GPU's array: calls that overlap in time
 * on one GPU (different streams) race on it and must be serialised by the caller; calls
 * on one stream, or on different GPUs, are safe.  The first uncalibrated call on a GPU
 * looks the array's address up (hipGetDevice, hipGetSymbolAddress: host runtime calls that
 * may load the code object); make that first call outside any stream capture, every later
 * call on that GPU only launches kernels and may be captured. */
int mxq_quantize_v2_noalloc(void* stream, const float* in, void* out, float* omin, float* omax,
                            size_t n, int out_type, int calibrated, float min_calib,
                            float max_calib);

/* ---- _contrib_quantize (v1) ---------------------------------------------
 * Replaces QuantizeCompute<gpu> (src/operator/quantization/quantize-inl.h:90-131):
 * same kernels, the range arrives as two device scalars. */
int mxq_quantize(void* stream, const float* in, const float* imin, const float* imax, void* out,
                 float* omin, float* omax, size_t n, int out_type);

/* Identity pass for int8/uint8 input of quantize_v2 (quantize_v2-inl.h:203-216):
 * copies n bytes and writes the constant ranges. */
int mxq_quantize_v2_passthrough(void* stream, const void* in, void* out, float* omin,
                                float* omax, size_t n, int in_type, int calibrated,
                                float min_calib, float max_calib);

/* ---- _contrib_requantize -------------------------------------------------
 * Replaces RequantizeForward<gpu> (src/operator/quantization/requantize-inl.h:127-240):
 * int32 -> int8 with the input range (imin, imax) read from the device;
 * calibrated uses MaxAbs(min_calib, max_calib), uncalibrated reduces the int32
 * min and max on the device first (workspace as above). */
size_t mxq_requantize_workspace(size_t n);
int mxq_requantize(void* stream, const int32_t* in, const float* imin, const float* imax,
                   int8_t* out, float* omin, float* omax, size_t n, int calibrated,
                   float min_calib, float max_calib, void* workspace, size_t workspace_bytes);

/* ---- _contrib_dequantize -------------------------------------------------
 * Replaces DequantizeOperator<gpu>::Forward
 * (src/operator/quantization/dequantize-inl.h:115-144); in_type MXQ_INT8 or
 * MXQ_UINT8. */
int mxq_dequantize(void* stream, const void* in, int in_type, const float* imin,
                   const float* imax, float* out, size_t n);

/* ---- _contrib_quantized_act (relu) -----------------------------------------
 * int8 max(x, 0); the range passes through unchanged
 * (src/operator/quantization/quantized_activation.cc:84-120, CPU-only in the
 * reference through dnnl/dnnl_quantized_act.cc:33-45). */
int mxq_quantized_relu(void* stream, const int8_t* in, const float* imin, const float* imax,
                       int8_t* out, float* omin, float* omax, size_t n);

/* ---- _contrib_quantized_pooling ---------------------------------------------
 * Replaces QuantizedCuDNNPoolingOp::Forward
 * (src/operator/quantization/quantized_pooling.cu:33-128): cudnnPoolingForward on
 * the NCHW int8 tensor plus the two range copies.  OH / OW are the extents
 * QuantizedPoolingShape computed (quantized_pooling.cc:82-121; global pooling is
 * kernel = (H, W), stride 1, OH = OW = 1).  Windows and the divisor of avg follow
 * the reference's own pooling loops (src/operator/nn/pool.h:476-522):
 * count_include_pad != 0 is cuDNN's COUNT_INCLUDE_PADDING, the mode the reference
 * selects.  max ignores padding; avg returns nearest-even(sum / divisor): that
 * rounding lives inside cuDNN / oneDNN in the reference and is not pinned by its
 * sources (its test accepts +-2).  in_type MXQ_INT8 or MXQ_UINT8 (the reference's
 * GPU build takes int8 only). */
#define MXQ_POOL_MAX 0
#define MXQ_POOL_AVG 1
int mxq_quantized_pooling_nchw(void* stream, const void* in, int in_type, int N, int C, int H,
                               int W, int kernel_h, int kernel_w, int stride_h, int stride_w,
                               int pad_h, int pad_w, int OH, int OW, int pool_type,
                               int count_include_pad, const float* imin, const float* imax,
                               void* out, float* omin, float* omax);

/* ---- _contrib_quantized_flatten ----------------------------------------------
 * Replaces QuantizedFlattenCompute (src/operator/quantization/quantized_flatten-inl.h:39-94;
 * registered for cpu only in the reference, quantized_flatten.cc:35): copies n_bytes
 * of int8/uint8 data and the two range scalars; in == out (the operator's in-place
 * option, quantized_flatten.cc:52-56) copies nothing. */
int mxq_quantized_flatten(void* stream, const void* in, const float* imin, const float* imax,
                          void* out, float* omin, float* omax, size_t n_bytes);

/* ---- _contrib_quantized_elemwise_add ---------------------------------------------
 * Replaces DNNLQuantizedElemwiseAddForward
 * (src/operator/quantization/dnnl/dnnl_quantized_elemwise_add.cc:134-257; the operator is
 * cpu-only in the reference, quantized_elemwise_add.cc:80-87) for operands of one shape:
 * out = saturate(nearest-even(lhs * s0 + rhs * s1)) in binary32, s = output scale / input
 * scale with the reference's ranges (127.5 int8, 255.5 uint8, 2^31 - 1 int32).
 * Uncalibrated: out is int32 over (-(|A|+|B|), |A|+|B|).  Calibrated: out has the inputs'
 * type (int8 when they differ) over (min_calib, max_calib).  A uint8 operand beside an
 * int8 one is first halved to int8, as the reference does.  The rounding itself lives
 * inside oneDNN in the reference and is not pinned by its sources (its test accepts a
 * dequantized error of 2). */
int mxq_quantized_elemwise_add(void* stream, const void* lhs, int lhs_type, const void* rhs,
                               int rhs_type, const float* lhs_min, const float* lhs_max,
                               const float* rhs_min, const float* rhs_max, void* out, int out_type,
                               float* omin, float* omax, size_t n, int calibrated,
                               float min_calib, float max_calib);

/* _contrib_quantized_npi_add (src/operator/quantization/quantized_elemwise_add.cc:141-178,
 * dnnl/dnnl_quantized_elemwise_add.cc:134-257; cpu only in the reference): the quantized sum
 * of two contiguous operands under numpy broadcasting (shapes aligned at the last axis, an
 * extent of 1 stretches).  Equal shapes are forwarded to mxq_quantized_elemwise_add; for
 * different shapes a uint8 operand next to an int8 one is taken at its own scale, as the
 * reference's binary primitive does.  out_type as for mxq_quantized_elemwise_add; the output
 * has fewer than 2^32 elements. */
int mxq_quantized_broadcast_add(void* stream, const void* lhs, int lhs_type, int lhs_ndim,
                                const int64_t* lhs_shape, const void* rhs, int rhs_type,
                                int rhs_ndim, const int64_t* rhs_shape, const float* lhs_min,
                                const float* lhs_max, const float* rhs_min, const float* rhs_max,
                                void* out, int out_type, float* omin, float* omax,
                                int calibrated, float min_calib, float max_calib);

/* ---- _contrib_quantized_elemwise_mul ---------------------------------------------
 * Replaces QuantizedElemwiseMulOpForward
 * (src/operator/quantization/quantized_elemwise_mul.cc:114-206; registered for cpu only,
 * :232) for int8 operands of one shape: out[i] = (out_type)(lhs[i] * rhs[i] * out_scale),
 * the int product converted to binary32, multiplied, truncated.
 *   out_type MXQ_INT32 (uncalibrated): out_scale = 1, range from
 *     QuantizationRangeForMultiplication<int8,int8,int32> (quantization_utils.h:141-170);
 *   out_type MXQ_INT8 (calibrated): out_scale = (127.5 / MaxAbs(calib)) / lhs_scale /
 *     rhs_scale with scale = 127.5 / MaxAbs(range), range (min_calib, max_calib);
 *   out_type MXQ_FLOAT32 (enable_float_output): out_scale = 1 / lhs_scale / rhs_scale in
 *     binary64, rounded once; omin / omax are not written and may be NULL.
 * A calibrated product whose truncated value does not fit int8 is undefined in the
 * reference; the low byte of the truncated int32 is stored (what its x86 build does). */
int mxq_quantized_elemwise_mul(void* stream, const int8_t* lhs, const int8_t* rhs,
                               const float* lhs_min, const float* lhs_max, const float* rhs_min,
                               const float* rhs_max, void* out, int out_type, float* omin,
                               float* omax, size_t n, int calibrated, float min_calib,
                               float max_calib);

/* ---- _contrib_quantized_embedding --------------------------------------------------
 * Replaces QuantizedEmbeddingOpForward
 * (src/operator/quantization/quantized_indexing_op.cc:103-122; cpu only, :146) and the
 * TakeZeroAxisCPU<clip> kernel it launches (src/operator/tensor/indexing_op.cc:30-61):
 * out[i, :] = weight[clip(int64(indices[i]), 0, input_dim - 1), :], int8 rows of output_dim
 * bytes; the weight's range is passed through.  index_type is the mshadow type flag of
 * `indices` (float32, float64, uint8, int32, int8 or int64). */
int mxq_quantized_embedding(void* stream, const void* indices, int index_type,
                            const int8_t* weight, const float* min_weight,
                            const float* max_weight, int8_t* out, float* omin, float* omax,
                            size_t n_indices, int64_t input_dim, int64_t output_dim);

/* ---- _contrib_quantized_transpose --------------------------------------------------
 * Replaces DNNLQuantizedTransposeForward
 * (src/operator/quantization/dnnl/dnnl_quantized_transpose.cc; shapes and types
 * quantized_transpose.cc:31-66; cpu only in the reference): out = in permuted so that out
 * axis d is in axis axes[d] (axes == NULL reverses the axes, TransposeParam's default),
 * one byte per element (int8 or uint8), ndim <= 8; the range is passed through.
 * _contrib_quantized_reshape (quantized_reshape.cc:31-46) needs no entry point of its own:
 * it is mxq_quantized_flatten's copy. */
int mxq_quantized_transpose(void* stream, const void* in, const float* imin, const float* imax,
                            void* out, float* omin, float* omax, int ndim,
                            const int64_t* in_shape, const int* axes);

/* ---- _contrib_quantize_asym ----------------------------------------------------------
 * Replaces QuantizeAsymOp<gpu>::Forward
 * (src/operator/quantization/quantize_asym-inl.h:78-160): float32 -> uint8 with
 * scale = 255 / (max - min), shift = 255 - max * scale,
 * out = (uint8)(in * scale + shift + 0.5) (the 0.5 in binary64), over (min_calib,
 * max_calib) or, uncalibrated, the data's own min and max (workspace of
 * mxq_quantize_asym_workspace(n) bytes, 16-byte aligned).  int8 input: out = in + 128,
 * scale 1, shift 128; uint8 input: copied, scale 1, shift 0.  A value outside [0, 256) is
 * undefined in the reference; the low byte of the truncated int32 is stored. */
size_t mxq_quantize_asym_workspace(size_t n);
int mxq_quantize_asym(void* stream, const void* in, int in_type, uint8_t* out, float* oscale,
                      float* oshift, size_t n, int calibrated, float min_calib, float max_calib,
                      void* workspace, size_t workspace_bytes);

/* ---- _contrib_quantized_batch_norm, _contrib_quantized_batch_norm_relu ----------------
 * Replaces DNNLQuantizedBatchNormForward
 * (src/operator/quantization/dnnl/dnnl_quantized_batch_norm.cc:34-130; cpu-only in the
 * reference): data [outer][channels][inner] int8 (uint8 is first scaled to int8 by
 * 127.5 / 255.5), inference statistics.  Per channel
 *   invstd = float(1.0 / sqrt(double(var) + eps)),
 *   w = gamma * invstd * MaxAbs(data range) / MaxAbs(calib range),
 *   b = (beta - mean * gamma * invstd) * 127.5 / MaxAbs(calib range),
 * out = saturate(nearest-even((w / sqrt(1 + eps)) * x + b)), with max(0, .) before the
 * rounding for the relu form; the output range is (min_calib, max_calib), which the
 * operator requires.  The factor and offset follow the reference's own file; the
 * normalisation itself (the second division by sqrt(1 + eps), the order of multiply and
 * add, the rounding) runs inside oneDNN there and is not pinned by its sources (its test
 * accepts rtol 0.1, atol 8).  workspace: mxq_quantized_batch_norm_workspace(channels)
 * bytes, 4-byte aligned. */
size_t mxq_quantized_batch_norm_workspace(int64_t channels);
int mxq_quantized_batch_norm(void* stream, const void* data, int data_type, const float* gamma,
                             const float* beta, const float* moving_mean,
                             const float* moving_var, const float* min_data,
                             const float* max_data, int8_t* out, float* omin, float* omax,
                             int64_t outer, int64_t channels, int64_t inner, double eps,
                             float min_calib, float max_calib, int relu, void* workspace,
                             size_t workspace_bytes);

/* ---- _contrib_quantized_concat -----------------------------------------------------
 * Replaces DNNLQuantizedConcatForward
 * (src/operator/quantization/dnnl/dnnl_quantized_concat.cc:41-115; cpu-only in the
 * reference).  Input i is [outer, in_axis[i], inner] contiguous, the output
 * [outer, sum in_axis, inner].  Output range = hull of the input ranges and 0; out_type is
 * int8 as soon as one input is (quantized_concat.cc:83-103).  An input whose scale equals
 * the output's is copied, any other is rescaled: saturate(nearest-even(x * out_scale /
 * in_scale)) in binary32 (oneDNN's reorder; same caveat as above).  in, in_type, in_min,
 * in_max, in_axis are host arrays of num_args entries; the data and range pointers in
 * them are device pointers. */
int mxq_quantized_concat(void* stream, int num_args, const void* const* in, const int* in_type,
                         const float* const* in_min, const float* const* in_max,
                         const int64_t* in_axis, int64_t outer, int64_t inner, void* out,
                         int out_type, float* omin, float* omax);

/* ---- _contrib_quantized_fully_connected ----------------------------------
 * Replaces QuantizedFullyConnectedForwardGPU
 * (src/operator/quantization/quantized_fully_connected.cu:58-138): cublasGemmEx
 * (s8 x s8 -> s32, data [M,K] row-major, weight [N,K] row-major), the
 * QuantizationRangeForS8S8MultiplicationStruct launch and QuantizedBiasAddKernel.
 * The bias is added exactly, as the CPU operator does
 * (quantized_fully_connected.cc:149-174: the int8 bias is rescaled to int32 once
 * and summed in integers), not through the GPU kernel's float round trip.
 *   bias        int8 [N] or NULL (then min_bias/max_bias are ignored)
 *   out32       int32 [M,N] or NULL
 *   omin, omax  output range (always written)
 *   out8        int8 [M,N] or NULL: fused _contrib_requantize of the
 *               accumulator with the calibrated range (min_calib, max_calib),
 *               bit-identical to mxq_requantize on out32; relu != 0 clamps the
 *               int8 at zero; rmin/rmax receive the requantized range.
 * At least one of out32 / out8 must be given.
 *   workspace   device scratch (16-byte aligned) or NULL.  Shapes with few output tiles and
 *               a long K are split along K over several work-groups per tile, which leave
 *               their int32 partial sums in the workspace (integer addition is
 *               associative: the result is the unsplit one bit for bit); this is the
 *               operator's kTempSpace (quantized_fully_connected.cc:369-372).
 *               mxq_quantized_fc_workspace() returns the bytes with which the call takes
 *               its fastest route (0 when it would not split; fused_int8_only != 0 says
 *               that only out8 will be given); with less, or NULL, nothing is split. */
size_t mxq_quantized_fc_workspace(int M, int N, int K, int fused_int8_only);
int mxq_quantized_fc(void* stream, const int8_t* data, const int8_t* weight, const int8_t* bias,
                     int M, int N, int K, const float* min_data, const float* max_data,
                     const float* min_weight, const float* max_weight, const float* min_bias,
                     const float* max_bias, int32_t* out32, float* omin, float* omax,
                     int8_t* out8, float* rmin, float* rmax, int relu, float min_calib,
                     float max_calib, void* workspace, size_t workspace_bytes);

/* _contrib_quantized_fully_connected -> _contrib_requantize -> _contrib_dequantize in one
 * launch: the three operators a quantized graph runs where a float consumer follows the
 * layer (quantized_fully_connected.cu:58-138, requantize-inl.h:89-125 with a calibrated
 * range, dequantize-inl.h:64-75).  out_f32 [M,N] receives float(q) * (R / 127) with q the
 * requantized int8 value and R = max(|min_calib|, |max_calib|): bit-identical to
 * mxq_dequantize(mxq_requantize(out32)) element by element; relu != 0 clamps q at zero
 * first.  omin/omax and rmin/rmax are written as by mxq_quantized_fc.  The int8 tensor
 * between the operators is never stored.  Workspace as for mxq_quantized_fc (size it with
 * fused_int8_only = 0). */
int mxq_quantized_fc_f32(void* stream, const int8_t* data, const int8_t* weight,
                         const int8_t* bias, int M, int N, int K, const float* min_data,
                         const float* max_data, const float* min_weight, const float* max_weight,
                         const float* min_bias, const float* max_bias, float* out_f32,
                         float* omin, float* omax, float* rmin, float* rmax, int relu,
                         float min_calib, float max_calib, void* workspace,
                         size_t workspace_bytes);

/* _contrib_quantized_fully_connected -> _contrib_requantize -> _contrib_quantized_elemwise_add
 * (-> _contrib_quantized_act) in one launch: a layer whose requantized int8 output is added
 * to a second int8 tensor of the same shape, the residual sum of a bottleneck block
 * (quantized_fully_connected.cu:58-138, requantize-inl.h:89-125,
 * quantized_elemwise_add.cc:30-134 / dnnl/dnnl_quantized_elemwise_add.cc:134-257 with a
 * calibrated int8 output, quantized_activation.cc:84-120).  In NHWC a 1x1 unit-stride
 * unpadded convolution is this call on the flattened pixels (M = N*H*W, K = C, N = O).
 *   residual       int8 [M,N], range (min_residual, max_residual)
 *   min/max_calib  the layer's own requantization range, as for mxq_quantized_fc
 *   sum_*_calib    the sum's calibrated range; rmin / rmax receive it
 *   sum_relu != 0  clamps the sum at zero
 * out8 is bit-identical to mxq_quantized_elemwise_add(out8 of mxq_quantized_fc, residual)
 * followed by mxq_quantized_relu; neither intermediate tensor is stored.  (The element
 * rounding of the sum is this library's own choice: in the reference it happens inside
 * oneDNN and its parity is unpinned, as for mxq_quantized_elemwise_add.)  out8 may be the
 * residual's own buffer (the shortcut updated in place).  Workspace as for
 * mxq_quantized_fc with fused_int8_only = 1. */
int mxq_quantized_fc_sum(void* stream, const int8_t* data, const int8_t* weight,
                         const int8_t* bias, int M, int N, int K, const float* min_data,
                         const float* max_data, const float* min_weight, const float* max_weight,
                         const float* min_bias, const float* max_bias, const int8_t* residual,
                         const float* min_residual, const float* max_residual, int8_t* out8,
                         float* omin, float* omax, float* rmin, float* rmax, float min_calib,
                         float max_calib, float sum_min_calib, float sum_max_calib, int sum_relu,
                         void* workspace, size_t workspace_bytes);

/* ---- _contrib_quantized_conv ----------------------------------------------
 * Replaces QuantizedCuDNNConvOp::Forward
 * (src/operator/quantization/quantized_conv.cu:101-219): the NHWC int8
 * cudnnConvolutionForward, the float->int32 cast, the range kernel and the bias
 * kernel.  Operands are NHWC here (data [N,H,W,C], weight [O,KH,KW,C], output
 * [N,OH,OW,O]); the layout adapters below replace the three TransposeImpl calls
 * (:147-148,183) for callers holding the operator's NCHW tensors.  Epilogue
 * and workspace arguments as for mxq_quantized_fc (the reference passes cuDNN its own
 * workspace out of the operator's temp space, quantized_conv.cu:121-177). */
size_t mxq_quantized_conv_workspace(int N, int H, int W, int C, int O, int KH, int KW,
                                    int stride_h, int stride_w, int pad_h, int pad_w,
                                    int dilate_h, int dilate_w, int fused_int8_only);
int mxq_quantized_conv_nhwc(void* stream, const int8_t* data, const int8_t* weight,
                            const int8_t* bias, int N, int H, int W, int C, int O, int KH,
                            int KW, int stride_h, int stride_w, int pad_h, int pad_w,
                            int dilate_h, int dilate_w, const float* min_data,
                            const float* max_data, const float* min_weight,
                            const float* max_weight, const float* min_bias,
                            const float* max_bias, int32_t* out32, float* omin, float* omax,
                            int8_t* out8, float* rmin, float* rmax, int relu, float min_calib,
                            float max_calib, void* workspace, size_t workspace_bytes);
/* The same convolution with the int32 output written as the operator's own layout,
 * [N,O,OH,OW]: the kernel's epilogue stores channel planes directly, which replaces the
 * third TransposeImpl (quantized_conv.cu:183) and the NHWC int32 buffer it reads. */
int mxq_quantized_conv_nhwc_out_nchw(void* stream, const int8_t* data, const int8_t* weight,
                                     const int8_t* bias, int N, int H, int W, int C, int O,
                                     int KH, int KW, int stride_h, int stride_w, int pad_h,
                                     int pad_w, int dilate_h, int dilate_w,
                                     const float* min_data, const float* max_data,
                                     const float* min_weight, const float* max_weight,
                                     const float* min_bias, const float* max_bias,
                                     int32_t* out32_nchw, float* omin, float* omax,
                                     void* workspace, size_t workspace_bytes);

/* _contrib_quantized_conv on the operator's own tensors: data int8 [N,C,H,W], weight int8
 * [O,C,KH,KW], bias int8 [O] or NULL, out32 int32 [N,O,OH,OW] -- everything
 * QuantizedCuDNNConvOp::Forward does between its inputs and its outputs
 * (src/operator/quantization/quantized_conv.cu:101-219, layout rule quantized_conv.cc:38-45),
 * the three TransposeImpl calls included (:145-148,183).  Unpadded 1 x 1 convolutions over
 * 16 | C channels never leave the channel-plane layout (strided ones and planes that are
 * no multiple of 16 bytes through a gathering loader in the same kernel or, where that
 * would fetch single bytes, after the pixels they read were gathered into the workspace);
 * every other geometry goes through the layout adapters and
 * mxq_quantized_conv_nhwc_out_nchw inside this call.
 * `workspace` (16-byte aligned) must hold mxq_quantized_conv_nchw_workspace() bytes: the
 * operator's kTempSpace (quantized_conv.cu:121-160 asks for three tensor copies plus
 * cuDNN's workspace there; 0 here for most unpadded 1 x 1 layers).  operands_aligned16 != 0
 * says that data and weight both start on 16-byte marks, as a framework's allocations do;
 * with 0 the query returns enough for the adapter route as well, which every geometry and
 * alignment can take. */
size_t mxq_quantized_conv_nchw_workspace(int N, int C, int H, int W, int O, int KH, int KW,
                                         int stride_h, int stride_w, int pad_h, int pad_w,
                                         int dilate_h, int dilate_w, int operands_aligned16);
int mxq_quantized_conv_nchw(void* stream, const int8_t* data, const int8_t* weight,
                            const int8_t* bias, int N, int C, int H, int W, int O, int KH, int KW,
                            int stride_h, int stride_w, int pad_h, int pad_w, int dilate_h,
                            int dilate_w, const float* min_data, const float* max_data,
                            const float* min_weight, const float* max_weight,
                            const float* min_bias, const float* max_bias, int32_t* out32,
                            float* omin, float* omax, void* workspace, size_t workspace_bytes);

/* [N,C,H,W] int8 -> [N,H,W,C] int8 (also OIHW -> OHWI for the weight). */
int mxq_nchw_to_nhwc_i8(void* stream, const int8_t* in, int8_t* out, int N, int C, int H, int W);
/* The same with the channel extent of the output padded to C_padded >= C with zeros
 * ([N,H,W,C_padded]): zero channels add nothing to a convolution, and a channel count
 * that is a multiple of 16 takes mxq_quantized_conv_nhwc's fast path. */
int mxq_nchw_to_nhwc_pad_i8(void* stream, const int8_t* in, int8_t* out, int N, int C, int H,
                            int W, int C_padded);
/* Space-to-depth by 2 on the way: [N,C,H,W] -> [N,H2,W2,C_padded] with
 * out[n][h2][w2][(dh*2+dw)*C + c] = in[n][c][2*h2 - off_h + dh][2*w2 - off_w + dw] (zero
 * outside the image; channels 4*C..C_padded-1 zero), H2 = (H + off_h + 1) / 2, likewise W2,
 * off in {0,1}.  A KxK stride-2 convolution with padding p over C channels equals the
 * ceil(K/2) x ceil(K/2) unit-stride convolution with padding (p - off) / 2 over this tensor
 * (off = p mod 2) and the weight transformed the same way with off = 0, whenever both
 * give the same output extent; few-channel stride-2 stems run that way. */
int mxq_nchw_to_s2d_nhwc_i8(void* stream, const int8_t* in, int8_t* out, int N, int C, int H,
                            int W, int off_h, int off_w, int C_padded);
/* [N,H,W,C] -> [N,C,H,W]; elem_bytes 1 (int8) or 4 (int32). */
int mxq_nhwc_to_nchw(void* stream, const void* in, void* out, int N, int C, int H, int W,
                     int elem_bytes);

#ifdef __cplusplus
}
#endif
#endif /* MXQ_H_ */
