/*
 * CPU oracle for MXNet's INT8 quantized-inference operator path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing shipped links or calls this file: it is
 * the checker that the HIP kernels are compared against, and the timed CPU
 * baseline of the benchmark.  It restates, operation by operation, the native
 * (mshadow) CPU arithmetic of the reference; every function cites the
 * reference lines it follows (paths relative to the apache/mxnet tree).
 *
 * Build: gcc -O2 -ffp-contract=off -fopenmp -shared -fPIC (no -mfma, no
 * -ffast-math): every written float operation is one correctly rounded
 * IEEE-754 binary32 operation, as in the reference's CPU build
 * (CMakeLists.txt:244-256 uses -O3 -msse3, no FMA).
 *
 * How each function is pinned (tests/test_oracle_*.py):
 *   - qref_quantize_int8 / qref_requantize / qref_dequantize_*: hand-derived
 *     known answers, the numpy baselines of the reference's own tests
 *     (tests/python/quantization/test_quantization.py:66-235), odd symmetry,
 *     monotonicity, saturation, an exact rational (fractions.Fraction)
 *     evaluation of every rounding step on small inputs.
 *   - qref_quantize_uint8: exact rational evaluation + known answers.
 *   - qref_minmax_*: numpy min/max (order independent), NaN propagation.
 *   - qref_range_for_multiplication / qref_bias_i8_to_i32: known answers and
 *     exact rational evaluation.
 *   - qref_fc / qref_conv_nchw: numpy int64 matmul, torch int conv on the
 *     same operands, the reference test's integer-valued fp32 Dense/Conv
 *     construction, identity / single-tap special cases.
 *   - qref_pool_nchw: max pooling is exact integer work, pinned against torch
 *     max_pool2d on integer-valued floats and brute force.  For avg pooling the
 *     window and divisor follow the reference's own fp32 pooling loop, but the
 *     ROUNDING of the quotient to int8 lives in cuDNN / oneDNN (third-party,
 *     absent): PARITY UNPINNED for that one step.  Here: nearest, ties to even,
 *     of the exact quotient; checked against an exact rational evaluation and
 *     against the reference test's own bound (|int8 - fp32 pooling| <= 2,
 *     tests/python/quantization/test_quantization.py:634-639).
 *   - qref_elemwise_add / qref_concat_rescale: the scale derivation follows the
 *     reference's own files, but the arithmetic that applies the scales runs inside
 *     oneDNN (dnnl::sum, dnnl::reorder; third-party, absent): PARITY UNPINNED for
 *     the rounding of each element.  Here: saturate(nearest-even(sum of the scaled
 *     operands)) with every binary32 operation rounded on its own; checked against
 *     an exact rational evaluation of that rule, against the reference test's own
 *     bound (|dequantized - fp32 sum| <= 2,
 *     tests/python/quantization/test_quantization.py:375-433) and through the
 *     special cases the scales make exact (equal ranges, concat of equal scales is a
 *     byte copy).
 *   - qref_elemwise_mul / qref_quantize_asym: native CPU loops of the reference, every
 *     step a written C++ operation: exact rational evaluation of each rounding step,
 *     hand-derived known answers, the reference test's own bound for the product
 *     (tests/python/quantization/test_quantization.py:436-497), closed forms (the
 *     int32 product is exact; asymmetric quantization maps min -> 0 and max -> 255).
 *     Results outside the output type are undefined in the reference: the low byte of
 *     the truncated int32 is kept, as gcc's x86 code for that conversion does.
 *   - qref_batch_norm: the per-channel factor and offset follow the reference's own file
 *     (dnnl_quantized_batch_norm.cc:66-112) and are pinned by exact rational evaluation;
 *     the normalisation that applies them runs inside oneDNN (third-party, absent):
 *     PARITY UNPINNED for the second division by sqrt(1 + eps), the order of multiply and
 *     add and the rounding of each element.  Here: saturate(nearest-even(w' * x + b)),
 *     every binary32 operation rounded on its own; checked against an exact rational
 *     evaluation of that rule and the reference test's own bound against the float batch
 *     norm (tests/python/quantization/test_quantization.py:990-1054).
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

/* ---- quantization_utils.h:41-81 ---------------------------------------- */

/* Sign: (val > 0) - (val < 0); quantization_utils.h:41-44 */
static inline int q_sign(float v) { return (v > 0.0f) - (v < 0.0f); }
/* std::max / std::min argument order semantics; quantization_utils.h:55-71 */
static inline float q_max(float a, float b) { return (a < b) ? b : a; }
static inline float q_min(float a, float b) { return (b < a) ? b : a; }
/* MaxAbs / MinAbs cast to float first; quantization_utils.h:73-81 */
static inline float q_maxabs(float a, float b) { return q_max(fabsf(a), fabsf(b)); }

#define Q_I8_RANGE 127.0f          /* MinAbs(MaxValue<int8>(), MinValue<int8>()) */
#define Q_I32_RANGE 2147483648.0f  /* MinAbs(float(INT32_MIN), float(INT32_MAX)) = 2^31 */

/* FloatToQuantized<int8_t>; quantization_utils.h:83-89 */
static inline int8_t q_float_to_i8(float x, float scale) {
  float t = fabsf(x) * scale;
  float u = t + 0.5f;
  float v = q_min(u, Q_I8_RANGE);
  return (int8_t)((float)q_sign(x) * v);
}

/* QuantizedToFloat<int32_t>; quantization_utils.h:91-97 */
static inline float q_i32_to_float(int32_t q, float min_range, float max_range) {
  float real_range = q_maxabs(min_range, max_range);
  float scale = real_range / Q_I32_RANGE;
  return (float)q * scale;
}

int qref_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* ---- quantize_v2 -------------------------------------------------------- */

/* quantize_v2_zero_centered::Map, quantize_v2-inl.h:98-114 (and the v1 twin
 * quantize_zero_centered, quantize-inl.h:71-88).  Launched over all elements by
 * Kernel<OP,cpu>::Launch (src/operator/mxnet_op.h:1013-1032). */
void qref_quantize_int8(const float* in, size_t n, float imin, float imax, int8_t* out,
                        float* omin, float* omax) {
  float real_range = q_maxabs(imin, imax);
  float scale = Q_I8_RANGE / real_range;
#pragma omp parallel for schedule(static)
  for (ptrdiff_t i = 0; i < (ptrdiff_t)n; ++i) out[i] = q_float_to_i8(in[i], scale);
  *omin = -real_range;
  *omax = real_range;
}

/* quantize_v2_unsigned::Map, quantize_v2-inl.h:66-81: the scale is a double
 * division narrowed to float, the product is a float, the +0.5 is a double
 * add, the cast truncates.  The reference has no clamp: out-of-range input is
 * undefined there; this restatement clamps to [0,255] so it is total. */
void qref_quantize_uint8(const float* in, size_t n, float imin, float imax, uint8_t* out,
                         float* omin, float* omax) {
  const double min_limit = 0.0, max_limit = 255.0;
  const float scale = (float)((max_limit - min_limit) / (double)(imax - imin));
#pragma omp parallel for schedule(static)
  for (ptrdiff_t i = 0; i < (ptrdiff_t)n; ++i) {
    float t = (in[i] - imin) * scale;
    double u = (double)t + 0.5;
    if (!(u > 0.0)) u = 0.0;
    if (u > 255.0) u = 255.0;
    out[i] = (uint8_t)u;
  }
  *omin = imin;
  *omax = imax;
}

/* red::minimum / red::maximum over the whole tensor (NaN-propagating),
 * 3rdparty/mshadow/mshadow/base.h:1054-1115, called from
 * quantize_v2-inl.h:258-263. */
void qref_minmax_f32(const float* in, size_t n, float* omin, float* omax) {
  float mn = INFINITY, mx = -INFINITY;
  int has_nan = 0;
#pragma omp parallel for schedule(static) reduction(min : mn) reduction(max : mx) \
    reduction(| : has_nan)
  for (ptrdiff_t i = 0; i < (ptrdiff_t)n; ++i) {
    float x = in[i];
    if (x != x) has_nan = 1;
    if (x < mn) mn = x;
    if (x > mx) mx = x;
  }
  if (has_nan) mn = mx = NAN;
  *omin = mn;
  *omax = mx;
}

/* int32 min/max for the uncalibrated requantize, requantize-inl.h:177-191. */
void qref_minmax_i32(const int32_t* in, size_t n, int32_t* omin, int32_t* omax) {
  int32_t mn = INT32_MAX, mx = INT32_MIN;
#pragma omp parallel for schedule(static) reduction(min : mn) reduction(max : mx)
  for (ptrdiff_t i = 0; i < (ptrdiff_t)n; ++i) {
    int32_t x = in[i];
    if (x < mn) mn = x;
    if (x > mx) mx = x;
  }
  *omin = mn;
  *omax = mx;
}

/* ---- requantize --------------------------------------------------------- */

/* RequantizeKernel::Map, requantize-inl.h:89-125; real_range is
 * MaxAbs(min_calib, max_calib) (requantize-inl.h:144-154) or, uncalibrated,
 * MaxAbs of the float images of the int32 min and max (:155-238). */
void qref_requantize(const int32_t* in, size_t n, float imin, float imax, float real_range,
                     int8_t* out, float* omin, float* omax) {
  float in_range = q_maxabs(imin, imax);
  float in_scale = in_range / Q_I32_RANGE;
  /* FloatToQuantized(x, -real_range, real_range): MaxAbs(-r, r) = |r| */
  float rr = q_maxabs(-real_range, real_range);
  float scale = Q_I8_RANGE / rr;
#pragma omp parallel for schedule(static)
  for (ptrdiff_t i = 0; i < (ptrdiff_t)n; ++i) {
    float f = (float)in[i] * in_scale;
    out[i] = q_float_to_i8(f, scale);
  }
  *omin = -real_range;
  *omax = real_range;
}

/* The range the uncalibrated requantize derives from the data,
 * requantize-inl.h:177-227 (QuantizedToFloatStruct on the int32 min and max,
 * then MaxAbs in RequantizeKernel::Map :107-124). */
float qref_requantize_actual_range(const int32_t* in, size_t n, float imin, float imax) {
  int32_t mn, mx;
  qref_minmax_i32(in, n, &mn, &mx);
  return q_maxabs(q_i32_to_float(mn, imin, imax), q_i32_to_float(mx, imin, imax));
}

/* ---- dequantize --------------------------------------------------------- */

/* dequantize_zero_centered::Map, dequantize-inl.h:64-75 */
void qref_dequantize_int8(const int8_t* in, size_t n, float imin, float imax, float* out) {
  float real_range = q_maxabs(imax, imin);
  float scale = real_range / Q_I8_RANGE;
#pragma omp parallel for schedule(static)
  for (ptrdiff_t i = 0; i < (ptrdiff_t)n; ++i) out[i] = (float)in[i] * scale;
}

/* dequantize_unsigned::Map, dequantize-inl.h:49-61 (limits 0 and 255) */
void qref_dequantize_uint8(const uint8_t* in, size_t n, float imin, float imax, float* out) {
  float scale = (imax - imin) / (255.0f - 0.0f);
#pragma omp parallel for schedule(static)
  for (ptrdiff_t i = 0; i < (ptrdiff_t)n; ++i) {
    float p = (float)in[i] * scale;
    out[i] = p + imin;
  }
}

/* ---- quantized FC / conv ------------------------------------------------ */

/* QuantizationRangeForMultiplication<int8,int8,int32>(all_sign=true),
 * quantization_utils.h:134-157 */
void qref_range_for_multiplication(float min_a, float max_a, float min_b, float max_b,
                                   float* min_c, float* max_c) {
  float a_one = q_maxabs(min_a, max_a) / Q_I8_RANGE;
  float b_one = q_maxabs(min_b, max_b) / Q_I8_RANGE;
  float c_one = a_one * b_one;
  *max_c = c_one * Q_I32_RANGE;
  *min_c = -*max_c;
}

/* QuantizedSumInitKernelWithBias::Map, quantized_fully_connected.cc:149-174 */
void qref_bias_i8_to_i32(const int8_t* bias, size_t n, float min_out, float max_out,
                         float min_bias, float max_bias, int32_t* bias32) {
  float one_out = (float)((double)q_maxabs(min_out, max_out) / (double)INT32_MAX);
  float one_bias = (float)((double)q_maxabs(min_bias, max_bias) / (double)INT8_MAX);
  for (size_t i = 0; i < n; ++i) {
    if (one_out != 0.0f) {
      float p = (float)bias[i] * one_bias;
      bias32[i] = (int32_t)(p / one_out);
    } else {
      bias32[i] = 0;
    }
  }
}

/* Net effect of QuantizedFullyConnectedForwardCPU,
 * quantized_fully_connected.cc:218-297: the +128 shift of the data, the
 * -128*sum_k w[n,k] correction and cblas_gemm_s8u8s32 with beta=1 cancel to
 *   out[m,n] = bias32[n] + sum_k data[m,k] * weight[n,k]
 * in wrap-around int32.  data [M,K] row-major, weight [N,K] row-major. */
void qref_fc(const int8_t* data, const int8_t* weight, const int32_t* bias32, int M, int N,
             int K, int32_t* out) {
#pragma omp parallel for schedule(static) collapse(2)
  for (int m = 0; m < M; ++m) {
    for (int n = 0; n < N; ++n) {
      const int8_t* a = data + (size_t)m * K;
      const int8_t* b = weight + (size_t)n * K;
      int32_t acc = 0;
      for (int k = 0; k < K; ++k) acc += (int32_t)a[k] * (int32_t)b[k];
      out[(size_t)m * N + n] = (int32_t)((uint32_t)acc + (uint32_t)(bias32 ? bias32[n] : 0));
    }
  }
}

/* Exact int32 cross-correlation with the shapes of QuantizedConvShape,
 * quantized_conv.cc:30-131: data [N,C,H,W], weight [O,C,KH,KW], out
 * [N,O,OH,OW], OH = (H + 2*pad - dilate*(KH-1) - 1)/stride + 1, num_group 1.
 * bias32 (nullable) is added per output channel as in the FC. */
void qref_conv_nchw(const int8_t* data, const int8_t* weight, const int32_t* bias32, int N,
                    int C, int H, int W, int O, int KH, int KW, int stride_h, int stride_w,
                    int pad_h, int pad_w, int dil_h, int dil_w, int32_t* out) {
  const int OH = (H + 2 * pad_h - (dil_h * (KH - 1) + 1)) / stride_h + 1;
  const int OW = (W + 2 * pad_w - (dil_w * (KW - 1) + 1)) / stride_w + 1;
#pragma omp parallel for schedule(static) collapse(2)
  for (int n = 0; n < N; ++n) {
    for (int o = 0; o < O; ++o) {
      for (int oh = 0; oh < OH; ++oh) {
        for (int ow = 0; ow < OW; ++ow) {
          int32_t acc = 0;
          for (int c = 0; c < C; ++c) {
            for (int kh = 0; kh < KH; ++kh) {
              int ih = oh * stride_h - pad_h + kh * dil_h;
              if (ih < 0 || ih >= H) continue;
              for (int kw = 0; kw < KW; ++kw) {
                int iw = ow * stride_w - pad_w + kw * dil_w;
                if (iw < 0 || iw >= W) continue;
                acc += (int32_t)data[(((size_t)n * C + c) * H + ih) * W + iw] *
                       (int32_t)weight[(((size_t)o * C + c) * KH + kh) * KW + kw];
              }
            }
          }
          out[(((size_t)n * O + o) * OH + oh) * OW + ow] =
              (int32_t)((uint32_t)acc + (uint32_t)(bias32 ? bias32[o] : 0));
        }
      }
    }
  }
}

/* quantized ReLU on int8 is max(x, 0); the min/max ranges pass through
 * (dnnl/dnnl_quantized_act.cc:33-45).  Applied to the requantized int8. */
void qref_relu_i8(const int8_t* in, size_t n, int8_t* out) {
#pragma omp parallel for schedule(static)
  for (ptrdiff_t i = 0; i < (ptrdiff_t)n; ++i) out[i] = in[i] > 0 ? in[i] : 0;
}

/* ---- _contrib_quantized_pooling ------------------------------------------
 * 2-D pooling of an NCHW int8 (is_unsigned = 0) or uint8 tensor; min/max pass
 * through (quantized_pooling.cu:76-98).  Output extents are the caller's
 * (QuantizedPoolingShape, quantized_pooling.cc:32-133).  The window of output
 * (oh, ow) and the divisor follow pool_sum_2d_nchw_cpu / pool_max_2d_nchw_cpu
 * (src/operator/nn/pool.h:476-522): hstart = oh*sh - ph, hend = min(hstart+kh,
 * H+ph), divisor = (hend-hstart)*(wend-wstart) before clipping to the image when
 * padding counts (cuDNN's COUNT_INCLUDE_PADDING, quantized_pooling.cu:46-50),
 * after clipping otherwise.  max: padding never wins (cudnn NOT_PROPAGATE_NAN
 * max over valid taps); an empty window yields the type's minimum.
 * avg: q = nearest-even(sum / divisor), saturated - see the header. */
void qref_pool_nchw(const void* in_, int is_unsigned, int N, int C, int H, int W, int KH,
                    int KW, int sh, int sw, int ph, int pw, int OH, int OW, int is_avg,
                    int count_include_pad, void* out_) {
  const int8_t* in_s = (const int8_t*)in_;
  const uint8_t* in_u = (const uint8_t*)in_;
  int8_t* out_s = (int8_t*)out_;
  uint8_t* out_u = (uint8_t*)out_;
  const int lo = is_unsigned ? 0 : -128, hi = is_unsigned ? 255 : 127;
#pragma omp parallel for schedule(static)
  for (ptrdiff_t nc = 0; nc < (ptrdiff_t)N * C; ++nc) {
    const size_t ibase = (size_t)nc * H * W, obase = (size_t)nc * OH * OW;
    for (int oh = 0; oh < OH; ++oh) {
      for (int ow = 0; ow < OW; ++ow) {
        int hstart = oh * sh - ph, wstart = ow * sw - pw;
        int hend = hstart + KH < H + ph ? hstart + KH : H + ph;
        int wend = wstart + KW < W + pw ? wstart + KW : W + pw;
        int pool_size = (hend - hstart) * (wend - wstart);
        if (hstart < 0) hstart = 0;
        if (wstart < 0) wstart = 0;
        if (hend > H) hend = H;
        if (wend > W) wend = W;
        if (!count_include_pad) pool_size = (hend - hstart) * (wend - wstart);
        int32_t acc = is_avg ? 0 : lo;
        for (int h = hstart; h < hend; ++h)
          for (int w = wstart; w < wend; ++w) {
            const size_t i = ibase + (size_t)h * W + w;
            const int v = is_unsigned ? (int)in_u[i] : (int)in_s[i];
            if (is_avg)
              acc += v;
            else if (v > acc)
              acc = v;
          }
        int q = acc;
        if (is_avg) {
          /* float(sum)/float(divisor) is exact whenever the quotient is a tie (k + 0.5
           * is representable) and cannot be rounded onto one otherwise, so rintf of
           * it is nearest-even of the exact quotient */
          const float avg = pool_size > 0 ? (float)acc / (float)pool_size : 0.0f;
          q = (int)rintf(avg);
          if (q < lo) q = lo;
          if (q > hi) q = hi;
        }
        if (is_unsigned)
          out_u[obase + (size_t)oh * OW + ow] = (uint8_t)q;
        else
          out_s[obase + (size_t)oh * OW + ow] = (int8_t)q;
      }
    }
  }
}

/* ---- _contrib_quantized_elemwise_add / _contrib_quantized_concat ---------------
 * The DNNL operators' ranges: 127.5 for int8, 255.5 for uint8, 2^31 - 1 for int32
 * (quantization_utils.h:37-39). */
static inline float q_type_range(int is_unsigned) { return is_unsigned ? 255.5f : 127.5f; }

/* saturate to [lo, hi], then nearest-even; NaN converts to 0 */
static inline int32_t q_round_sat(float f, float lo, float hi) {
  if (f != f) return 0;
  if (f < lo) f = lo;
  if (f > hi) f = hi;
  return (int32_t)rintf(f);
}

/* dnnl_quantized_elemwise_add.cc:134-257 for operands of one shape.
 * out_kind: 0 int32 (uncalibrated), 1 int8, 2 uint8 (calibrated).  Scales:
 * A_scale = range(A) / MaxAbs(A_min, A_max) (:152-157); output scale =
 * double(range(out)) / MaxAbs(calib) or / (|A| + |B|), rounded to float (:169-178);
 * scales[i] = output_scale / scale_i (:180-182).  A uint8 operand next to an int8 one
 * is first reordered to int8 with scale 0.5 and its scale doubled (:189-210).
 * The sum itself is dnnl::sum: dst = saturate(round(s0 * a + s1 * b)). */
static void elemwise_add_impl(const void* lhs_, int lhs_unsigned, const void* rhs_,
                              int rhs_unsigned, size_t n, float lhs_min, float lhs_max,
                              float rhs_min, float rhs_max, int out_kind, int calibrated,
                              float min_calib, float max_calib, int halve_mixed, void* out_,
                              float* omin, float* omax) {
  const float a_absmax = q_maxabs(lhs_min, lhs_max), b_absmax = q_maxabs(rhs_min, rhs_max);
  const float a_scale = q_type_range(lhs_unsigned) / a_absmax;
  const float b_scale = q_type_range(rhs_unsigned) / b_absmax;
  const double out_range = out_kind == 0 ? 2147483647.0 : (out_kind == 1 ? 127.5 : 255.5);
  float output_min, output_max, output_scale;
  if (calibrated) {
    output_min = min_calib;
    output_max = max_calib;
    output_scale = (float)(out_range / (double)q_maxabs(output_min, output_max));
  } else {
    output_max = a_absmax + b_absmax;
    output_min = -output_max;
    output_scale = (float)(out_range / (double)output_max);
  }
  float s0 = output_scale / a_scale, s1 = output_scale / b_scale;
  const int halve_a = halve_mixed && lhs_unsigned && !rhs_unsigned;
  const int halve_b = halve_mixed && rhs_unsigned && !lhs_unsigned;
  if (halve_a) s0 = (float)((double)s0 * (1.0 / 0.5));
  if (halve_b) s1 = (float)((double)s1 * (1.0 / 0.5));
  const float lo = out_kind == 0 ? -2147483648.0f : (out_kind == 1 ? -128.0f : 0.0f);
  /* the largest binary32 below 2^31: what oneDNN saturates int32 to */
  const float hi = out_kind == 0 ? 2147483520.0f : (out_kind == 1 ? 127.0f : 255.0f);
#pragma omp parallel for schedule(static)
  for (ptrdiff_t i = 0; i < (ptrdiff_t)n; ++i) {
    int a = lhs_unsigned ? (int)((const uint8_t*)lhs_)[i] : (int)((const int8_t*)lhs_)[i];
    int b = rhs_unsigned ? (int)((const uint8_t*)rhs_)[i] : (int)((const int8_t*)rhs_)[i];
    if (halve_a) a = q_round_sat((float)a * 0.5f, -128.0f, 127.0f);
    if (halve_b) b = q_round_sat((float)b * 0.5f, -128.0f, 127.0f);
    const float x = (float)a * s0;
    const float y = (float)b * s1;
    const int32_t q = q_round_sat(x + y, lo, hi);
    if (out_kind == 0)
      ((int32_t*)out_)[i] = q;
    else if (out_kind == 1)
      ((int8_t*)out_)[i] = (int8_t)q;
    else
      ((uint8_t*)out_)[i] = (uint8_t)q;
  }
  *omin = output_min;
  *omax = output_max;
}

void qref_elemwise_add(const void* lhs_, int lhs_unsigned, const void* rhs_, int rhs_unsigned,
                       size_t n, float lhs_min, float lhs_max, float rhs_min, float rhs_max,
                       int out_kind, int calibrated, float min_calib, float max_calib,
                       void* out_, float* omin, float* omax) {
  elemwise_add_impl(lhs_, lhs_unsigned, rhs_, rhs_unsigned, n, lhs_min, lhs_max, rhs_min, rhs_max,
                    out_kind, calibrated, min_calib, max_calib, 1, out_, omin, omax);
}

/* The same sum for operands the caller has already stretched to one shape, as
 * _contrib_quantized_npi_add computes it when the shapes differ: dnnl::binary with the two
 * scales, and no reorder of a uint8 operand to int8 (that is only made on the same-shape
 * route, dnnl_quantized_elemwise_add.cc:183-210).  PARITY UNPINNED like qref_elemwise_add. */
void qref_broadcast_add(const void* lhs_, int lhs_unsigned, const void* rhs_, int rhs_unsigned,
                        size_t n, float lhs_min, float lhs_max, float rhs_min, float rhs_max,
                        int out_kind, int calibrated, float min_calib, float max_calib,
                        void* out_, float* omin, float* omax) {
  elemwise_add_impl(lhs_, lhs_unsigned, rhs_, rhs_unsigned, n, lhs_min, lhs_max, rhs_min, rhs_max,
                    out_kind, calibrated, min_calib, max_calib, 0, out_, omin, omax);
}

/* One input of dnnl_quantized_concat.cc:68-98 brought to the output's scale:
 * scale_x = range(type x) / MaxAbs(min_x, max_x) (GetScale, :35-38); equal scales (and
 * types) copy, otherwise a reorder with scale out_scale / in_scale. */
void qref_concat_rescale(const void* in_, int in_unsigned, size_t n, float imin, float imax,
                         float omin, float omax, int out_unsigned, void* out_) {
  const float out_scale = q_type_range(out_unsigned) / q_maxabs(omin, omax);
  const float in_scale = q_type_range(in_unsigned) / q_maxabs(imin, imax);
  if (in_scale == out_scale && in_unsigned == out_unsigned) {
    memcpy(out_, in_, n);
    return;
  }
  const float scale = out_scale / in_scale;
  const float lo = out_unsigned ? 0.0f : -128.0f, hi = out_unsigned ? 255.0f : 127.0f;
#pragma omp parallel for schedule(static)
  for (ptrdiff_t i = 0; i < (ptrdiff_t)n; ++i) {
    const int v = in_unsigned ? (int)((const uint8_t*)in_)[i] : (int)((const int8_t*)in_)[i];
    const int32_t q = q_round_sat((float)v * scale, lo, hi);
    if (out_unsigned)
      ((uint8_t*)out_)[i] = (uint8_t)q;
    else
      ((int8_t*)out_)[i] = (int8_t)q;
  }
}

/* QuantizedElemwiseMulOpForward, quantized_elemwise_mul.cc:114-206.  out_kind: 0 int32
 * (uncalibrated, out_scale = 1, range from QuantizationRangeForMultiplication), 1 int8
 * (calibrated), 2 float32 (enable_float_output; omin / omax untouched).
 * kInt8Range is the float 127.5 (quantization_utils.h:38); output_data_range is a double. */
void qref_elemwise_mul(const int8_t* lhs, const int8_t* rhs, size_t n, float lhs_min,
                       float lhs_max, float rhs_min, float rhs_max, int out_kind,
                       float min_calib, float max_calib, void* out_, float* omin, float* omax) {
  const float k_int8_range = 127.5f;
  float out_scale = 1.0f;
  if (out_kind == 1) {
    const double output_data_range = (double)k_int8_range;
    const float out_data_scale =
        (float)(output_data_range / (double)q_maxabs(min_calib, max_calib));
    const float lhs_scale = k_int8_range / q_maxabs(lhs_min, lhs_max);
    const float rhs_scale = k_int8_range / q_maxabs(rhs_min, rhs_max);
    out_scale = out_data_scale / lhs_scale / rhs_scale;
    *omin = min_calib;
    *omax = max_calib;
  } else if (out_kind == 0) {
    qref_range_for_multiplication(lhs_min, lhs_max, rhs_min, rhs_max, omin, omax);
  } else {
    const float lhs_scale = k_int8_range / q_maxabs(lhs_min, lhs_max);
    const float rhs_scale = k_int8_range / q_maxabs(rhs_min, rhs_max);
    out_scale = (float)(1.0 / (double)lhs_scale / (double)rhs_scale);
  }
#pragma omp parallel for schedule(static)
  for (ptrdiff_t i = 0; i < (ptrdiff_t)n; ++i) {
    const int8_t a = lhs[i], b = rhs[i];
    const float f = (float)(a * b) * out_scale;
    if (out_kind == 0)
      ((int32_t*)out_)[i] = (int32_t)f;
    else if (out_kind == 1)
      ((int8_t*)out_)[i] = (int8_t)(int32_t)f;
    else
      ((float*)out_)[i] = f;
  }
}

/* quantize_asymmetric::Map and QuantizeAsymOp::Forward for float input,
 * quantize_asym-inl.h:62-76,103-152: scale = 255 / (max - min), shift = 255 - max * scale,
 * out = (uint8)(x * scale + shift + 0.5), the last addition in double. */
void qref_quantize_asym(const float* in, size_t n, float min_range, float max_range,
                        uint8_t* out, float* oscale, float* oshift) {
  const float scale = 255.0f / (max_range - min_range);
  const float shift = 255.0f - max_range * scale;
#pragma omp parallel for schedule(static)
  for (ptrdiff_t i = 0; i < (ptrdiff_t)n; ++i) {
    const float t = in[i] * scale + shift;
    out[i] = (uint8_t)(int32_t)((double)t + 0.5);
  }
  *oscale = scale;
  *oshift = shift;
}

/* DNNLQuantizedBatchNormForward, dnnl_quantized_batch_norm.cc:34-130, on data laid out
 * [outer][channels][inner]; the reference's dnnl::batch_normalization_forward over mean 0
 * and variance 1 is restated as dst = saturate(round((w / sqrtf(1 + eps)) * src + b)). */
void qref_batch_norm(const void* data_, int data_unsigned, size_t outer, size_t channels,
                     size_t inner, const float* gamma, const float* beta, const float* mean,
                     const float* var, float min_data, float max_data, double eps,
                     float min_calib, float max_calib, int relu, int8_t* out, float* omin,
                     float* omax) {
  const float max_abs_data = q_maxabs(min_data, max_data);
  const float max_abs_output = q_maxabs(min_calib, max_calib);
  const float unit_std = sqrtf(1.0f + (float)eps);
  *omin = min_calib;
  *omax = max_calib;
#pragma omp parallel for schedule(static) collapse(2)
  for (ptrdiff_t o = 0; o < (ptrdiff_t)outer; ++o) {
    for (ptrdiff_t c = 0; c < (ptrdiff_t)channels; ++c) {
      const float invstd = (float)(1.0 / sqrt((double)var[c] + eps));
      const float w = gamma[c] * invstd * max_abs_data / max_abs_output;
      const float b = (beta[c] - mean[c] * gamma[c] * invstd) * 127.5f / max_abs_output;
      const float wn = w / unit_std;
      const size_t base = ((size_t)o * channels + (size_t)c) * inner;
      for (size_t i = 0; i < inner; ++i) {
        int x = data_unsigned ? (int)((const uint8_t*)data_)[base + i]
                              : (int)((const int8_t*)data_)[base + i];
        if (data_unsigned) x = q_round_sat((float)x * (127.5f / 255.5f), -128.0f, 127.0f);
        float f = (float)x * wn + b;
        if (relu && f < 0.0f) f = 0.0f;
        out[base + i] = (int8_t)q_round_sat(f, -128.0f, 127.0f);
      }
    }
  }
}
