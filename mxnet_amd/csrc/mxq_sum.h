// The residual sum as an epilogue step: int8 + int8 -> int8 over a calibrated range,
// optionally followed by the int8 relu of _contrib_quantized_act
// (quantized_activation.cc:84-120).  It mirrors add_kernel in mxq_eltwise.hip and the CPU
// oracle bit for bit.  The scales come from the reference's own files
// (src/operator/quantization/quantized_elemwise_add.cc:30-134,
// dnnl/dnnl_quantized_elemwise_add.cc:134-257); the element arithmetic itself (two float
// products, one sum, nearest-even, saturation, NaN -> 0) happens inside oneDNN in the
// reference and is not pinned by anything in its tree: parity unpinned, as for add_kernel.  A kernel that holds the
// left operand in registers applies it to 16-byte pieces on their way out.
#ifndef MXQ_SUM_H_
#define MXQ_SUM_H_

#include <hip/hip_runtime.h>

#include <cstdint>

namespace mxq {

struct SumRule {
  float s0, s1;  // output levels per level of the left / right operand
  int fast;      // neither product can overflow: no NaN, the one-instruction clamp applies
};

// dnnl_quantized_elemwise_add.cc:143-210 for two int8 operands and a calibrated int8 output:
// every scale is the type's range (127.5) over the tensor's largest magnitude.
__device__ __forceinline__ SumRule sum_rule(float a_absmax, float b_absmax, float min_calib,
                                            float max_calib) {
  SumRule r;
  const float a_scale = 127.5f / a_absmax;
  const float b_scale = 127.5f / b_absmax;
  const float x = fabsf(min_calib), y = fabsf(max_calib);
  const float out_scale = static_cast<float>(127.5 / static_cast<double>((x < y) ? y : x));
  r.s0 = out_scale / a_scale;
  r.s1 = out_scale / b_scale;
  r.fast = fabsf(r.s0) < 1e30f && fabsf(r.s1) < 1e30f;  // false for NaN as well
  return r;
}

// One element: saturate, round to nearest even, NaN -> 0; with RELU the negative results
// become 0 (clamping at 0 before the rounding gives the same integer).
template <bool RELU, bool FAST>
__device__ __forceinline__ uint32_t sum_one(int a, int b, const SumRule& r) {
  const float p = static_cast<float>(a) * r.s0;
  const float q = static_cast<float>(b) * r.s1;
  float f = p + q;
  constexpr float lo = RELU ? 0.0f : -128.0f;
  if (FAST)  // nearest-even(f) in the low mantissa byte of f + 1.5 * 2^23
    return __float_as_uint(__builtin_amdgcn_fmed3f(f, lo, 127.0f) + 12582912.0f);
  if (f != f) return 0u;
  f = f < lo ? lo : f;
  f = f > 127.0f ? 127.0f : f;
  return static_cast<uint32_t>(static_cast<int>(rintf(f)));
}

// Four int8 pairs (x: left operand, y: right operand, byte k of each) -> four int8 results.
template <bool RELU, bool FAST>
__device__ __forceinline__ uint32_t sum4(uint32_t x, uint32_t y, const SumRule& r) {
  if (RELU && FAST) {
    // results in [0, 127]: v_cvt_pk_u8_f32 rounds to nearest even, saturates and places the
    // byte in one instruction (instead of the 1.5 * 2^23 add and three quarters of a pack)
    uint32_t w = 0;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int a = static_cast<int>(static_cast<int8_t>((x >> (8 * k)) & 0xffu));
      const int b = static_cast<int>(static_cast<int8_t>((y >> (8 * k)) & 0xffu));
      const float p = static_cast<float>(a) * r.s0;
      const float q = static_cast<float>(b) * r.s1;
      w = __builtin_amdgcn_cvt_pk_u8_f32(__builtin_amdgcn_fmed3f(p + q, 0.0f, 127.0f), k, w);
    }
    return w;
  }
  uint32_t q[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int a = static_cast<int>(static_cast<int8_t>((x >> (8 * k)) & 0xffu));
    const int b = static_cast<int>(static_cast<int8_t>((y >> (8 * k)) & 0xffu));
    q[k] = sum_one<RELU, FAST>(a, b, r);
  }
  const uint32_t lo = __builtin_amdgcn_perm(q[1], q[0], 0x0c0c0400u);
  const uint32_t hi = __builtin_amdgcn_perm(q[3], q[2], 0x04000c0cu);
  return lo | hi;
}

}  // namespace mxq
#endif  // MXQ_SUM_H_
