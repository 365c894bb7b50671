// Quantized element-wise add and concat for gfx950: the two operators that join
// branches of a quantized CNN (residual sums, inception-style concatenations).
//   _contrib_quantized_elemwise_add  src/operator/quantization/quantized_elemwise_add.cc:30-134
//                                    dnnl/dnnl_quantized_elemwise_add.cc:134-257
//   _contrib_quantized_concat        src/operator/quantization/quantized_concat.cc:31-141
//                                    dnnl/dnnl_quantized_concat.cc:41-115
// Both exist for cpu only in the reference and hand their arithmetic to oneDNN
// (dnnl::sum / dnnl::reorder with scales).  What is restated here is the scale
// derivation of the reference's own files plus the primitives' documented rule
// dst = saturate(round_nearest_even(sum_i scale_i * src_i)), evaluated in binary32 with
// every operation rounded on its own.
//
// Both are byte streams bound by HBM: 16 elements per lane per segment where the
// output is a byte type, 4 where it is int32 (so that every lane stores 16 bytes).
#include <hip/hip_runtime.h>

#include <type_traits>
#include <vector>

#include <cstdint>

#include "../../include/mxq.h"
#include "mxq_common.h"

namespace mxq {


namespace {

constexpr int kThreads = 256;
constexpr int kMaxConcatPerLaunch = 16;

typedef uint32_t u4 __attribute__((ext_vector_type(4)));
typedef int i4 __attribute__((ext_vector_type(4)));
typedef float f4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float maxabs(float a, float b) {
  float x = fabsf(a), y = fabsf(b);
  return (x < y) ? y : x;
}

// quantization_utils.h:37-39
__device__ __forceinline__ float type_range(int type) {
  return type == MXQ_INT8 ? 127.5f : 255.5f;
}
__device__ __forceinline__ double type_range_wide(int type) {
  return type == MXQ_INT32 ? 2147483647.0 : (type == MXQ_INT8 ? 127.5 : 255.5);
}

// saturate, then round to nearest even, into the output type; NaN converts to 0
template <int OUT>
__device__ __forceinline__ int narrow(float f) {
  constexpr float lo = OUT == MXQ_INT32 ? -2147483648.f : (OUT == MXQ_INT8 ? -128.f : 0.f);
  constexpr float hi = OUT == MXQ_INT32 ? 2147483520.f : (OUT == MXQ_INT8 ? 127.f : 255.f);
  if (f != f) return 0;
  f = f < lo ? lo : f;
  f = f > hi ? hi : f;
  return static_cast<int>(rintf(f));
}

// The same for a value known not to be NaN, as the low byte of the returned word: one
// clamp, then an add of 1.5 * 2^23, which leaves nearest-even(f) in the low mantissa bits
// (|f| <= 255, the sum's unit in the last place is 1 and 1.5 * 2^23 is even).
template <int OUT>
__device__ __forceinline__ uint32_t narrow_byte(float f) {
  constexpr float lo = OUT == MXQ_INT8 ? -128.f : 0.f;
  constexpr float hi = OUT == MXQ_INT8 ? 127.f : 255.f;
  return __float_as_uint(__builtin_amdgcn_fmed3f(f, lo, hi) + 12582912.f);
}
// 16 bytes written through the XCD's L2 (device-scope store) instead of lingering there as
// a dirty line: keeps the HBM write stream of a narrowing kernel sequential.  A store of
// more than 8 bytes reads its data registers over the two wait states after it issues and
// no VALU instruction may overwrite them before; the compiler pads its own stores but
// cannot see into this one, hence the s_nop.
__device__ __forceinline__ void stream_store16(u4 v, u4* p) {
  asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" ::"v"(p), "v"(v) : "memory");
}
// the low bytes of four words in one word
__device__ __forceinline__ uint32_t pack_low_bytes(uint32_t b0, uint32_t b1, uint32_t b2,
                                                   uint32_t b3) {
  const uint32_t lo = __builtin_amdgcn_perm(b1, b0, 0x0c0c0400u);  // {b0.0, b1.0, 0, 0}
  const uint32_t hi = __builtin_amdgcn_perm(b3, b2, 0x04000c0cu);  // {0, 0, b2.0, b3.0}
  return lo | hi;
}

template <bool UNSIGNED>
__device__ __forceinline__ int byte_of(uint32_t w, int k) {
  const uint32_t b = (w >> (8 * k)) & 0xffu;
  return UNSIGNED ? static_cast<int>(b) : static_cast<int>(static_cast<int8_t>(b));
}

// uint8 -> int8 at half scale, as the reference's reorder with scale 0.5 does before a
// mixed-type sum (dnnl_quantized_elemwise_add.cc:189-210)
__device__ __forceinline__ int halve_u8(int v) {
  return narrow<MXQ_INT8>(static_cast<float>(v) * 0.5f);
}

struct AddArgs {
  const uint8_t* lhs;
  const uint8_t* rhs;
  void* out;
  size_t n;
  const float* lhs_min;
  const float* lhs_max;
  const float* rhs_min;
  const float* rhs_max;
  float* omin;
  float* omax;
  float min_calib, max_calib;
  int calibrated, vec_ok;
};

// LU / RU: the operand is uint8.  FAST: both scales are small enough that neither
// product overflows, so no NaN can arise and the one-instruction clamp applies.
// HALVE: a uint8 operand next to an int8 one is first brought to int8 at half scale (the
// same-shape sum); without it both operands keep their own scale (the broadcasting sum).
template <int OUT, bool LU, bool RU, bool HALVE = true>
struct AddRule {
  float s0, s1, omin, omax;
  static constexpr bool kHalveL = HALVE && LU && !RU, kHalveR = HALVE && RU && !LU;
  __device__ __forceinline__ float sum(int a, int b) const {
    if (kHalveL) a = halve_u8(a);
    if (kHalveR) b = halve_u8(b);
    const float x = static_cast<float>(a) * s0;
    const float y = static_cast<float>(b) * s1;
    return x + y;
  }
  __device__ __forceinline__ int apply(int a, int b) const { return narrow<OUT>(sum(a, b)); }
  template <bool FAST>
  __device__ __forceinline__ uint32_t apply4(uint32_t x, uint32_t y) const {
    uint32_t q[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const float f = sum(byte_of<LU>(x, k), byte_of<RU>(y, k));
      q[k] = FAST ? narrow_byte<OUT>(f) : static_cast<uint32_t>(narrow<OUT>(f));
    }
    return pack_low_bytes(q[0], q[1], q[2], q[3]);
  }
  __device__ __forceinline__ bool fast() const {
    return fabsf(s0) < 1e30f && fabsf(s1) < 1e30f;  // false for NaN as well
  }
};

// dnnl_quantized_elemwise_add.cc:143-210
template <int OUT, bool LU, bool RU, bool HALVE = true>
__device__ __forceinline__ AddRule<OUT, LU, RU, HALVE> add_rule(const AddArgs& a) {
  AddRule<OUT, LU, RU, HALVE> r;
  const float a_absmax = maxabs(*a.lhs_min, *a.lhs_max);
  const float b_absmax = maxabs(*a.rhs_min, *a.rhs_max);
  const float a_scale = type_range(LU ? MXQ_UINT8 : MXQ_INT8) / a_absmax;
  const float b_scale = type_range(RU ? MXQ_UINT8 : MXQ_INT8) / b_absmax;
  const double out_range = type_range_wide(OUT);
  float out_scale;
  if (a.calibrated) {
    r.omin = a.min_calib;
    r.omax = a.max_calib;
    out_scale = static_cast<float>(out_range / static_cast<double>(maxabs(r.omin, r.omax)));
  } else {
    r.omax = a_absmax + b_absmax;
    r.omin = -r.omax;
    out_scale = static_cast<float>(out_range / static_cast<double>(r.omax));
  }
  r.s0 = out_scale / a_scale;
  r.s1 = out_scale / b_scale;
  if (r.kHalveL) r.s0 = static_cast<float>(static_cast<double>(r.s0) * (1.0 / 0.5));
  if (r.kHalveR) r.s1 = static_cast<float>(static_cast<double>(r.s1) * (1.0 / 0.5));
  return r;
}

// 16 elements per lane and segment: 16 bytes of each operand in, 16 bytes out
template <int OUT, bool LU, bool RU, bool FAST>
__device__ __forceinline__ void add_bytes(const AddArgs& a, const AddRule<OUT, LU, RU>& r,
                                          size_t t0, size_t stride) {
  const size_t nv = a.n >> 4;
  const u4* l16 = reinterpret_cast<const u4*>(a.lhs);
  const u4* r16 = reinterpret_cast<const u4*>(a.rhs);
  u4* o16 = reinterpret_cast<u4*>(a.out);
  size_t q = t0;
  for (; q + stride < nv; q += 2 * stride) {
    u4 x[2], y[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      x[j] = __builtin_nontemporal_load(l16 + q + j * stride);
      y[j] = __builtin_nontemporal_load(r16 + q + j * stride);
    }
    // both results before the first store: the stores are opaque to the compiler's count of
    // outstanding memory operations, a wait placed behind one would wait for it too
    u4 v[2];
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int w = 0; w < 4; ++w) v[j][w] = r.template apply4<FAST>(x[j][w], y[j][w]);
#pragma unroll
    for (int j = 0; j < 2; ++j) stream_store16(v[j], o16 + q + j * stride);
  }
  for (; q < nv; q += stride) {
    const u4 x = l16[q], y = r16[q];
    u4 v;
#pragma unroll
    for (int w = 0; w < 4; ++w) v[w] = r.template apply4<FAST>(x[w], y[w]);
    stream_store16(v, o16 + q);
  }
}

// The int32 sum of large tensors: one contiguous chunk per work-group, no loop.  Every lane
// requests its two dwords of each operand (512 lanes, a lane's dwords 2 KiB apart), then adds
// and writes the chunk's 16 KiB of output with two 16-byte stores.  As for the widening cast,
// this is the fastest pattern measured for a write-dominated stream (64 M elements: 62.8 us
// against 69.0 us for 4 KiB runs per wave of a grid-stride kernel; one, four or eight dwords
// per lane: 67.2 / 68.4 / 67.4 us).
constexpr int kAddChunkThreads = 512;
constexpr int kAddChunkPieces = 2;
constexpr size_t kAddChunkMinElements = size_t(1) << 24;

template <bool LU, bool RU>
__global__ __launch_bounds__(kAddChunkThreads) void add32_chunk_kernel(AddArgs a) {
  const AddRule<MXQ_INT32, LU, RU> r = add_rule<MXQ_INT32, LU, RU>(a);
  const size_t nq = a.n >> 2;
  const size_t base = size_t(blockIdx.x) * (kAddChunkPieces * kAddChunkThreads);
  const uint32_t* l4 = reinterpret_cast<const uint32_t*>(a.lhs);
  const uint32_t* r4 = reinterpret_cast<const uint32_t*>(a.rhs);
  uint32_t x[kAddChunkPieces], y[kAddChunkPieces];
#pragma unroll
  for (int j = 0; j < kAddChunkPieces; ++j) {
    const size_t q = base + size_t(j) * kAddChunkThreads + threadIdx.x;
    x[j] = q < nq ? __builtin_nontemporal_load(l4 + q) : 0u;
    y[j] = q < nq ? __builtin_nontemporal_load(r4 + q) : 0u;
  }
  // the descriptor ends with the tensor: pieces past the last whole quad are dropped
  const size_t left = nq > base ? nq - base : 0;
  const uint32_t bytes = left >= size_t(kAddChunkPieces) * kAddChunkThreads
                             ? kAddChunkPieces * kAddChunkThreads * 16
                             : static_cast<uint32_t>(left * 16);
  const __amdgpu_buffer_rsrc_t dst = __builtin_amdgcn_make_buffer_rsrc(
      reinterpret_cast<i4*>(a.out) + base, 0, bytes, 0x00020000);
#pragma unroll
  for (int j = 0; j < kAddChunkPieces; ++j) {
    i4 v;
#pragma unroll
    for (int k = 0; k < 4; ++k) v[k] = r.apply(byte_of<LU>(x[j], k), byte_of<RU>(y[j], k));
    __builtin_amdgcn_raw_buffer_store_b128(v, dst, (j * kAddChunkThreads + threadIdx.x) * 16, 0,
                                           18 /* sc1 + nt */);
  }
  if (blockIdx.x == 0) {
    // the ragged tail (< 4 elements) and the range
    const size_t i = (nq << 2) + threadIdx.x;
    if (i < a.n) {
      const int xv = LU ? static_cast<int>(a.lhs[i]) : static_cast<int>(static_cast<int8_t>(a.lhs[i]));
      const int yv = RU ? static_cast<int>(a.rhs[i]) : static_cast<int>(static_cast<int8_t>(a.rhs[i]));
      static_cast<int32_t*>(a.out)[i] = r.apply(xv, yv);
    }
    if (threadIdx.x == 0) {
      *a.omin = r.omin;
      *a.omax = r.omax;
    }
  }
}

template <int OUT, bool LU, bool RU>
__global__ __launch_bounds__(kThreads) void add_kernel(AddArgs a) {
  const AddRule<OUT, LU, RU> r = add_rule<OUT, LU, RU>(a);
  const size_t stride = size_t(gridDim.x) * kThreads;
  const size_t t0 = size_t(blockIdx.x) * kThreads + threadIdx.x;
  size_t done = 0;
  if (a.vec_ok) {
    if (OUT == MXQ_INT32) {
      // Write-dominated (2 bytes in, 4 out): as in the dequantize kernel a wave owns whole
      // 4 KiB runs of the output; lane l takes the dwords l, l + 64, l + 128, l + 192 of
      // each operand's 1 KiB and issues four device-scope 16-byte stores back to back,
      // each instruction writing 1 KiB of consecutive addresses (69.6 -> 66.9 us at 64 M
      // elements against 16-byte segments a grid-stride apart).
      const size_t nq = a.n >> 2;
      const uint32_t* l4 = reinterpret_cast<const uint32_t*>(a.lhs);
      const uint32_t* r4 = reinterpret_cast<const uint32_t*>(a.rhs);
      i4* o4 = reinterpret_cast<i4*>(a.out);
      constexpr int kRun = 256, kPer = kRun / 64, kWaves = kThreads / 64;
      const size_t runs = nq / kRun;
      const int lane = threadIdx.x & 63;
      const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
      for (size_t run = size_t(blockIdx.x) * kWaves + wave; run < runs;
           run += size_t(gridDim.x) * kWaves) {
        uint32_t x[kPer], y[kPer];
#pragma unroll
        for (int j = 0; j < kPer; ++j) {
          x[j] = __builtin_nontemporal_load(l4 + run * kRun + j * 64 + lane);
          y[j] = __builtin_nontemporal_load(r4 + run * kRun + j * 64 + lane);
        }
        const __amdgpu_buffer_rsrc_t dst =
            __builtin_amdgcn_make_buffer_rsrc(o4 + run * kRun, 0, kRun * 16, 0x00020000);
#pragma unroll
        for (int j = 0; j < kPer; ++j) {
          i4 v;
#pragma unroll
          for (int k = 0; k < 4; ++k) v[k] = r.apply(byte_of<LU>(x[j], k), byte_of<RU>(y[j], k));
          __builtin_amdgcn_raw_buffer_store_b128(v, dst, (j * 64 + lane) * 16, 0, 18 /* sc1 + nt */);
        }
      }
      for (size_t q = runs * kRun + t0; q < nq; q += stride) {
        const uint32_t x = l4[q], y = r4[q];
        i4 v;
#pragma unroll
        for (int k = 0; k < 4; ++k) v[k] = r.apply(byte_of<LU>(x, k), byte_of<RU>(y, k));
        __builtin_nontemporal_store(v, o4 + q);
      }
      done = nq << 2;
    } else {
      if (r.fast())
        add_bytes<OUT, LU, RU, true>(a, r, t0, stride);
      else
        add_bytes<OUT, LU, RU, false>(a, r, t0, stride);
      done = (a.n >> 4) << 4;
    }
  }
  for (size_t i = done + t0; i < a.n; i += stride) {
    const int x = LU ? static_cast<int>(a.lhs[i]) : static_cast<int>(static_cast<int8_t>(a.lhs[i]));
    const int y = RU ? static_cast<int>(a.rhs[i]) : static_cast<int>(static_cast<int8_t>(a.rhs[i]));
    const int s = r.apply(x, y);
    if (OUT == MXQ_INT32)
      static_cast<int32_t*>(a.out)[i] = s;
    else
      static_cast<uint8_t*>(a.out)[i] = static_cast<uint8_t>(s);
  }
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    *a.omin = r.omin;
    *a.omax = r.omax;
  }
}

// ---- broadcasting add ---------------------------------------------------------------

constexpr int kMaxBroadcastDims = 6;

struct BroadcastAddArgs {
  AddArgs add;  // operands, ranges, calibration; n = number of output elements (< 2^32)
  int nd;       // merged axes, innermost last
  uint32_t dim[kMaxBroadcastDims];
  uint32_t lstride[kMaxBroadcastDims], rstride[kMaxBroadcastDims];  // 0 on a broadcast axis
  int lhs_unsigned, rhs_unsigned;
};

// dnnl_quantized_elemwise_add.cc:143-182 for operands of different shapes: the scales as for
// the plain sum, but a uint8 operand next to an int8 one is taken as it is (the reorder to
// int8 at half scale is only made on the same-shape route, :185-210)
template <int OUT, bool LU, bool RU>
using BroadcastRule = AddRule<OUT, LU, RU, false>;

// 16 results from 16 bytes of each operand, stored as OUT
template <int OUT, bool LU, bool RU, bool FAST>
__device__ __forceinline__ void broadcast_store16(const BroadcastRule<OUT, LU, RU>& r, u4 x, u4 y,
                                                  void* out, size_t piece) {
  if (OUT == MXQ_INT32) {
    i4* o = static_cast<i4*>(out) + piece * 4;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      i4 v;
#pragma unroll
      for (int k = 0; k < 4; ++k) v[k] = r.apply(byte_of<LU>(x[w], k), byte_of<RU>(y[w], k));
      o[w] = v;  // a lane's 64 bytes: left to the cache to merge into whole lines
    }
  } else {
    u4 v;
#pragma unroll
    for (int w = 0; w < 4; ++w) v[w] = r.template apply4<FAST>(x[w], y[w]);
    stream_store16(v, static_cast<u4*>(out) + piece);
  }
}

// Innermost runs of at least 1 KiB in 16-byte pieces: one wave per 4 KiB of a run, so the
// run's position in both operands is wave-uniform (scalar divisions, once per 4 KiB) and an
// operand that is stretched along the run is one scalar byte.
template <int OUT, bool LU, bool RU>
__global__ __launch_bounds__(kThreads) void broadcast_add_rows_kernel(BroadcastAddArgs p) {
  const AddArgs& a = p.add;
  const BroadcastRule<OUT, LU, RU> r = add_rule<OUT, LU, RU, false>(a);
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    *a.omin = r.omin;
    *a.omax = r.omax;
  }
  const int last = p.nd - 1;
  const uint32_t inner16 = p.dim[last] >> 4;
  const uint32_t chunks = (inner16 + 255u) >> 8;
  const uint32_t rows = static_cast<uint32_t>(a.n) / p.dim[last];
  const uint32_t items = rows * chunks;
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t wave =
      __builtin_amdgcn_readfirstlane(blockIdx.x * (kThreads / 64) + (threadIdx.x >> 6));
  const uint32_t nwaves = gridDim.x * (kThreads / 64);
  const bool fast = r.fast();
  for (uint32_t item = wave; item < items; item += nwaves) {
    const uint32_t row = item / chunks, k = item - row * chunks;
    uint32_t rest = row, lo = 0, ro = 0;
    for (int d = last - 1; d >= 0; --d) {
      const uint32_t up = rest / p.dim[d], c = rest - up * p.dim[d];
      lo += c * p.lstride[d];
      ro += c * p.rstride[d];
      rest = up;
    }
    // Loads are unconditional and branch-free (indices clamped to the run, a stretched
    // operand reads the other operand's bytes and discards them: at most one is stretched
    // along the run): with loads inside branches the compiler drains the memory counter,
    // stores included, before every batch.
    const bool lrun = p.lstride[last] != 0, rrun = p.rstride[last] != 0;
    const uint32_t lsplat = lrun ? 0u : a.lhs[lo] * 0x01010101u;
    const uint32_t rsplat = rrun ? 0u : a.rhs[ro] * 0x01010101u;
    const uint8_t* lbase = lrun ? a.lhs + lo : a.rhs + ro;
    const uint8_t* rbase = rrun ? a.rhs + ro : a.lhs + lo;
    if (OUT == MXQ_INT32) {
      // a dword of each operand per lane and step: every store instruction writes 1 KiB of
      // consecutive output
      const uint32_t e0 = k << 12;  // first element of this piece within the run
      const uint32_t left4 = (p.dim[last] - e0) >> 2;
      const uint32_t* l4 = reinterpret_cast<const uint32_t*>(lbase + e0);
      const uint32_t* r4 = reinterpret_cast<const uint32_t*>(rbase + e0);
      i4* o4 = static_cast<i4*>(a.out) + ((size_t(row) * p.dim[last] + e0) >> 2);
      for (int jj = 0; jj < 16 && static_cast<uint32_t>(jj) * 64u < left4; jj += 4) {
        uint32_t xs[4], ys[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint32_t g = (jj + j) * 64 + lane;
          const uint32_t gc = g < left4 ? g : left4 - 1u;
          const uint32_t xv = __builtin_nontemporal_load(l4 + gc);
          const uint32_t yv = __builtin_nontemporal_load(r4 + gc);
          xs[j] = lrun ? xv : lsplat;
          ys[j] = rrun ? yv : rsplat;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint32_t g = (jj + j) * 64 + lane;
          i4 v;
#pragma unroll
          for (int b = 0; b < 4; ++b) v[b] = r.apply(byte_of<LU>(xs[j], b), byte_of<RU>(ys[j], b));
          if (g < left4) __builtin_nontemporal_store(v, o4 + g);
        }
      }
      continue;
    }
    const uint32_t left = inner16 - (k << 8);
    const uint32_t c0 = k << 8;
    const u4* l16 = reinterpret_cast<const u4*>(lbase) + c0;
    const u4* r16 = reinterpret_cast<const u4*>(rbase) + c0;
    const size_t piece0 = size_t(row) * inner16 + c0 + lane;
    // NB steps of 64 lanes x 16 bytes, all loads first, all results before the first store
    // (the stores are opaque to the compiler's count of outstanding operations)
    auto steps = [&](auto nb) {
      constexpr int NB = decltype(nb)::value;
      u4 x[NB], y[NB], v[NB];
#pragma unroll
      for (int j = 0; j < NB; ++j) {
        const uint32_t t = lane + 64u * j < left ? lane + 64u * j : left - 1u;
        const u4 xv = __builtin_nontemporal_load(l16 + t);
        const u4 yv = __builtin_nontemporal_load(r16 + t);
        x[j] = lrun ? xv : u4{lsplat, lsplat, lsplat, lsplat};
        y[j] = rrun ? yv : u4{rsplat, rsplat, rsplat, rsplat};
      }
      if (fast) {
#pragma unroll
        for (int j = 0; j < NB; ++j)
#pragma unroll
          for (int w = 0; w < 4; ++w) v[j][w] = r.template apply4<true>(x[j][w], y[j][w]);
      } else {
#pragma unroll
        for (int j = 0; j < NB; ++j)
#pragma unroll
          for (int w = 0; w < 4; ++w) v[j][w] = r.template apply4<false>(x[j][w], y[j][w]);
      }
#pragma unroll
      for (int j = 0; j < NB; ++j)
        if (lane + 64u * j < left) stream_store16(v[j], static_cast<u4*>(a.out) + piece0 + 64 * j);
    };
    if (OUT != MXQ_INT32) {
      if (left > 128u)
        steps(std::integral_constant<int, 4>());
      else if (left > 64u)
        steps(std::integral_constant<int, 2>());
      else
        steps(std::integral_constant<int, 1>());
    }
  }
}

// Any other layout: 16 outputs of one innermost run per lane where runs are whole 16-byte
// pieces, else one output per lane; positions by division.
template <int OUT, bool LU, bool RU>
__global__ __launch_bounds__(kThreads) void broadcast_add_kernel(BroadcastAddArgs p) {
  const AddArgs& a = p.add;
  const BroadcastRule<OUT, LU, RU> r = add_rule<OUT, LU, RU, false>(a);
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    *a.omin = r.omin;
    *a.omax = r.omax;
  }
  const uint32_t n = static_cast<uint32_t>(a.n);
  const uint32_t stride = gridDim.x * kThreads;
  const int last = p.nd - 1;
  if (a.vec_ok) {
    const uint32_t inner16 = p.dim[last] >> 4;
    const bool fast = r.fast();
    for (uint32_t q = blockIdx.x * kThreads + threadIdx.x; q < (n >> 4); q += stride) {
      uint32_t rest = q / inner16;
      const uint32_t c = (q - rest * inner16) << 4;
      uint32_t lo = c * p.lstride[last], ro = c * p.rstride[last];
      for (int d = last - 1; d >= 0; --d) {
        const uint32_t up = rest / p.dim[d], k = rest - up * p.dim[d];
        lo += k * p.lstride[d];
        ro += k * p.rstride[d];
        rest = up;
      }
      u4 x, y;
      if (p.lstride[last]) {
        x = *reinterpret_cast<const u4*>(a.lhs + lo);
      } else {
        const uint32_t b = a.lhs[lo] * 0x01010101u;
        x = u4{b, b, b, b};
      }
      if (p.rstride[last]) {
        y = *reinterpret_cast<const u4*>(a.rhs + ro);
      } else {
        const uint32_t b = a.rhs[ro] * 0x01010101u;
        y = u4{b, b, b, b};
      }
      if (fast)
        broadcast_store16<OUT, LU, RU, true>(r, x, y, a.out, q);
      else
        broadcast_store16<OUT, LU, RU, false>(r, x, y, a.out, q);
    }
    return;
  }
  for (uint32_t i = blockIdx.x * kThreads + threadIdx.x; i < n; i += stride) {
    uint32_t rest = i, lo = 0, ro = 0;
    for (int d = last; d >= 0; --d) {
      const uint32_t up = rest / p.dim[d], k = rest - up * p.dim[d];
      lo += k * p.lstride[d];
      ro += k * p.rstride[d];
      rest = up;
    }
    const int x = LU ? static_cast<int>(a.lhs[lo]) : static_cast<int>(static_cast<int8_t>(a.lhs[lo]));
    const int y = RU ? static_cast<int>(a.rhs[ro]) : static_cast<int>(static_cast<int8_t>(a.rhs[ro]));
    const int v = r.apply(x, y);
    if (OUT == MXQ_INT32)
      static_cast<int32_t*>(a.out)[i] = v;
    else
      static_cast<uint8_t*>(a.out)[i] = static_cast<uint8_t>(v);
  }
}

// ---- concat -----------------------------------------------------------------------

struct ConcatRanges {
  const float* mn[kMaxConcatPerLaunch];
  const float* mx[kMaxConcatPerLaunch];
  int count, first;
};

// dnnl_quantized_concat.cc:53-67: the output range is the hull of the input ranges and 0
__device__ __forceinline__ void range_hull(const float* const* mn, const float* const* mx,
                                           int count, float& lo, float& hi) {
  for (int i = 0; i < count; ++i) {
    const float a = *mn[i], b = *mx[i];
    if (a < lo) lo = a;
    if (b > hi) hi = b;
  }
}

// Only for more inputs than one launch carries: folds their ranges into omin / omax.
__global__ void concat_range_kernel(ConcatRanges r, float* omin, float* omax) {
  float lo = r.first ? 0.f : *omin;
  float hi = r.first ? 0.f : *omax;
  range_hull(r.mn, r.mx, r.count, lo, hi);
  *omin = lo;
  *omax = hi;
}

// Up to kMaxConcatPerLaunch inputs in one launch; input i owns the work-groups
// [block_end[i-1], block_end[i]).
struct ConcatArgs {
  const uint8_t* in[kMaxConcatPerLaunch];
  const float* mn[kMaxConcatPerLaunch];
  const float* mx[kMaxConcatPerLaunch];
  size_t row_bytes[kMaxConcatPerLaunch];  // extent along the axis x the trailing dimensions
  size_t out_off[kMaxConcatPerLaunch];    // first output byte of the input's slab
  int block_end[kMaxConcatPerLaunch];
  int in_type[kMaxConcatPerLaunch];
  int vec_ok[kMaxConcatPerLaunch];
  uint8_t* out;
  size_t rows;       // product of the dimensions before the axis
  size_t out_pitch;  // the output's extent along the axis x the trailing dimensions
  float* omin;
  float* omax;
  int count, out_type;
  int given_range;   // omin / omax already hold the hull of all inputs (more than one launch)
};

// MODE 0: byte copy, 1: rescale of finite scale (one-instruction clamp), 2: rescale, general
template <int MODE, bool IN_U, bool OUT_U>
__device__ __forceinline__ uint32_t concat_word(uint32_t w, float scale) {
  if (MODE == 0) return w;
  uint32_t q[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const float f = static_cast<float>(byte_of<IN_U>(w, k)) * scale;
    constexpr int OUT = OUT_U ? MXQ_UINT8 : MXQ_INT8;
    q[k] = MODE == 1 ? narrow_byte<OUT>(f) : static_cast<uint32_t>(narrow<OUT>(f));
  }
  return pack_low_bytes(q[0], q[1], q[2], q[3]);
}

// 16-byte pieces one work-group of the chunked form moves: kConcatChunkPieces per lane, all
// loads issued before the first store
constexpr int kConcatChunkPieces = 4;
constexpr size_t kConcatChunkMinBytes = size_t(1) << 24;

template <int MODE, bool IN_U, bool OUT_U, bool CHUNK>
__device__ __forceinline__ void concat_slab(const uint8_t* __restrict__ in,
                                            uint8_t* __restrict__ out, size_t rows,
                                            size_t row_bytes, size_t out_pitch, float scale,
                                            bool vec_ok, size_t t0, size_t stride) {
  if constexpr (CHUNK) {
    // t0 is the lane's first piece of the work-group's chunk, stride the work-group's width
    const size_t per_row = row_bytes >> 4;
    const size_t total = rows * per_row;
    const bool one_row = rows == 1;
    const bool narrow_index = total < (1ull << 32);
    u4 v[kConcatChunkPieces];
#pragma unroll
    for (int j = 0; j < kConcatChunkPieces; ++j) {
      const size_t q = t0 + size_t(j) * stride;
      v[j] = q < total ? __builtin_nontemporal_load(reinterpret_cast<const u4*>(in) + q)
                       : u4{0, 0, 0, 0};
    }
#pragma unroll
    for (int j = 0; j < kConcatChunkPieces; ++j) {
      const size_t q = t0 + size_t(j) * stride;
      size_t row = 0, col = q;
      if (!one_row) {
        if (narrow_index) {
          const uint32_t r32 = static_cast<uint32_t>(q) / static_cast<uint32_t>(per_row);
          row = r32;
          col = static_cast<uint32_t>(q) - r32 * static_cast<uint32_t>(per_row);
        } else {
          row = q / per_row;
          col = q - row * per_row;
        }
      }
#pragma unroll
      for (int w = 0; w < 4; ++w) v[j][w] = concat_word<MODE, IN_U, OUT_U>(v[j][w], scale);
      if (q < total) stream_store16(v[j], reinterpret_cast<u4*>(out + row * out_pitch) + col);
    }
  } else if (vec_ok) {
    const size_t per_row = row_bytes >> 4;
    const size_t total = rows * per_row;
    const bool one_row = rows == 1;
    const bool narrow_index = total < (1ull << 32);
    for (size_t q = t0; q < total; q += stride) {
      size_t row = 0, col = q;
      if (!one_row) {
        if (narrow_index) {
          const uint32_t r32 = static_cast<uint32_t>(q) / static_cast<uint32_t>(per_row);
          row = r32;
          col = static_cast<uint32_t>(q) - r32 * static_cast<uint32_t>(per_row);
        } else {
          row = q / per_row;
          col = q - row * per_row;
        }
      }
      u4 v = __builtin_nontemporal_load(reinterpret_cast<const u4*>(in + row * row_bytes) + col);
#pragma unroll
      for (int w = 0; w < 4; ++w) v[w] = concat_word<MODE, IN_U, OUT_U>(v[w], scale);
      stream_store16(v, reinterpret_cast<u4*>(out + row * out_pitch) + col);
    }
  } else {
    const size_t total = rows * row_bytes;
    for (size_t i = t0; i < total; i += stride) {
      const size_t row = i / row_bytes, col = i - row * row_bytes;
      uint8_t o = in[i];
      if (MODE != 0) {
        const int v = IN_U ? static_cast<int>(o) : static_cast<int>(static_cast<int8_t>(o));
        constexpr int OUT = OUT_U ? MXQ_UINT8 : MXQ_INT8;
        o = static_cast<uint8_t>(narrow<OUT>(static_cast<float>(v) * scale));
      }
      out[row * out_pitch + col] = o;
    }
  }
}

// dnnl_quantized_concat.cc:68-98: an input whose scale equals the output's is copied,
// any other goes through a reorder with scale out_scale / in_scale.
template <bool CHUNK>
__global__ __launch_bounds__(kThreads) void concat_kernel(ConcatArgs a) {
  float lo = 0.f, hi = 0.f;
  if (a.given_range) {
    lo = *a.omin;
    hi = *a.omax;
  } else {
    range_hull(a.mn, a.mx, a.count, lo, hi);
  }
  int part = 0;
  while (part + 1 < a.count && static_cast<int>(blockIdx.x) >= a.block_end[part]) ++part;
  const int first_block = part == 0 ? 0 : a.block_end[part - 1];
  // grid-stride form: the input's work-groups sweep it together; chunked form: each takes
  // kConcatChunkPieces x kThreads consecutive pieces
  const size_t stride = CHUNK ? size_t(kThreads) : size_t(a.block_end[part] - first_block) * kThreads;
  const size_t t0 = size_t(blockIdx.x - first_block) * kThreads * (CHUNK ? kConcatChunkPieces : 1) +
                    threadIdx.x;
  const int in_type = a.in_type[part];
  const float out_scale = type_range(a.out_type) / maxabs(lo, hi);
  const float in_scale = type_range(in_type) / maxabs(*a.mn[part], *a.mx[part]);
  const float scale = out_scale / in_scale;
  const bool copy = (in_scale == out_scale) && in_type == a.out_type;
  const bool finite = fabsf(scale) < 1e30f;  // false for NaN as well
  const uint8_t* in = a.in[part];
  uint8_t* out = a.out + a.out_off[part];
  const size_t rb = a.row_bytes[part];
  const bool v = a.vec_ok[part] != 0;
#define MXQ_SLAB(M, I, O) \
  concat_slab<M, I, O, CHUNK>(in, out, a.rows, rb, a.out_pitch, scale, v, t0, stride)
  const bool in_u = in_type == MXQ_UINT8, out_u = a.out_type == MXQ_UINT8;
  if (copy) {
    MXQ_SLAB(0, false, false);
  } else if (finite) {
    if (out_u) MXQ_SLAB(1, true, true);  // a uint8 output has uint8 inputs only
    else if (in_u) MXQ_SLAB(1, true, false);
    else MXQ_SLAB(1, false, false);
  } else {
    if (out_u) MXQ_SLAB(2, true, true);
    else if (in_u) MXQ_SLAB(2, true, false);
    else MXQ_SLAB(2, false, false);
  }
#undef MXQ_SLAB
  if (!a.given_range && blockIdx.x == 0 && threadIdx.x == 0) {
    *a.omin = lo;
    *a.omax = hi;
  }
}

// ---- elemwise_mul ---------------------------------------------------------------------

struct MulArgs {
  const uint8_t* lhs;
  const uint8_t* rhs;
  void* out;
  size_t n;
  const float* lhs_min;
  const float* lhs_max;
  const float* rhs_min;
  const float* rhs_max;
  float* omin;
  float* omax;
  float min_calib, max_calib;
  int vec_ok;
};

// quantized_elemwise_mul.cc:114-155: the factor applied to the integer product and the
// output range, for the three forms of the output
template <int OUT>
__device__ __forceinline__ float mul_scale(const MulArgs& a, float& omin, float& omax) {
  const float la = maxabs(*a.lhs_min, *a.lhs_max), lb = maxabs(*a.rhs_min, *a.rhs_max);
  if (OUT == MXQ_INT32) {
    // QuantizationRangeForMultiplication<int8, int8, int32>, all_sign
    omax = (la / 127.0f) * (lb / 127.0f) * 2147483648.0f;
    omin = -omax;
    return 1.0f;
  }
  const float lhs_scale = 127.5f / la, rhs_scale = 127.5f / lb;
  if (OUT == MXQ_FLOAT32)
    return static_cast<float>(1.0 / static_cast<double>(lhs_scale) / static_cast<double>(rhs_scale));
  omin = a.min_calib;
  omax = a.max_calib;
  const float out_data_scale =
      static_cast<float>(127.5 / static_cast<double>(maxabs(a.min_calib, a.max_calib)));
  return out_data_scale / lhs_scale / rhs_scale;
}

__device__ __forceinline__ int sbyte(uint32_t w, int k) {
  return static_cast<int>(static_cast<int8_t>((w >> (8 * k)) & 0xffu));
}

// static_cast<out_type>(a * b * out_scale) (quantized_elemwise_mul.cc:163-199): the int
// product as a float, times the factor, truncated.  Where the truncated value does not
// fit int8 the reference's conversion is undefined; this takes the low byte of the
// truncated int32, which is what the x86 build of the reference's loop produces.
template <int OUT>
__global__ __launch_bounds__(kThreads) void mul_kernel(MulArgs a) {
  float omin = 0.f, omax = 0.f;
  const float scale = mul_scale<OUT>(a, omin, omax);
  const size_t stride = size_t(gridDim.x) * kThreads;
  const size_t t0 = size_t(blockIdx.x) * kThreads + threadIdx.x;
  size_t done = 0;
  if (a.vec_ok) {
    if (OUT == MXQ_INT8) {
      const size_t nv = a.n >> 4;
      const u4* l16 = reinterpret_cast<const u4*>(a.lhs);
      const u4* r16 = reinterpret_cast<const u4*>(a.rhs);
      u4* o16 = reinterpret_cast<u4*>(a.out);
      auto product16 = [&](const u4& x, const u4& y) {
        u4 v;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          uint32_t b[4];
#pragma unroll
          for (int k = 0; k < 4; ++k)
            b[k] = static_cast<uint32_t>(
                static_cast<int>(static_cast<float>(sbyte(x[w], k) * sbyte(y[w], k)) * scale));
          v[w] = pack_low_bytes(b[0], b[1], b[2], b[3]);
        }
        return v;
      };
      size_t q = t0;
      for (; q + stride < nv; q += 2 * stride) {
        u4 x[2], y[2];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          x[j] = __builtin_nontemporal_load(l16 + q + j * stride);
          y[j] = __builtin_nontemporal_load(r16 + q + j * stride);
        }
#pragma unroll
        for (int j = 0; j < 2; ++j) stream_store16(product16(x[j], y[j]), o16 + q + j * stride);
      }
      for (; q < nv; q += stride) stream_store16(product16(l16[q], r16[q]), o16 + q);
      done = nv << 4;
    } else {
      const size_t nq = a.n >> 2;
      const uint32_t* l4 = reinterpret_cast<const uint32_t*>(a.lhs);
      const uint32_t* r4 = reinterpret_cast<const uint32_t*>(a.rhs);
      size_t q = t0;
      for (; q + stride < nq; q += 2 * stride) {
        uint32_t x[2], y[2];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          x[j] = __builtin_nontemporal_load(l4 + q + j * stride);
          y[j] = __builtin_nontemporal_load(r4 + q + j * stride);
        }
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          if (OUT == MXQ_INT32) {
            i4 v;
#pragma unroll
            for (int k = 0; k < 4; ++k) v[k] = sbyte(x[j], k) * sbyte(y[j], k);
            __builtin_nontemporal_store(v, reinterpret_cast<i4*>(a.out) + q + j * stride);
          } else {
            f4 v;
#pragma unroll
            for (int k = 0; k < 4; ++k)
              v[k] = static_cast<float>(sbyte(x[j], k) * sbyte(y[j], k)) * scale;
            __builtin_nontemporal_store(v, reinterpret_cast<f4*>(a.out) + q + j * stride);
          }
        }
      }
      for (; q < nq; q += stride) {
        const uint32_t x = l4[q], y = r4[q];
        if (OUT == MXQ_INT32) {
          i4 v;
#pragma unroll
          for (int k = 0; k < 4; ++k) v[k] = sbyte(x, k) * sbyte(y, k);
          reinterpret_cast<i4*>(a.out)[q] = v;
        } else {
          f4 v;
#pragma unroll
          for (int k = 0; k < 4; ++k) v[k] = static_cast<float>(sbyte(x, k) * sbyte(y, k)) * scale;
          reinterpret_cast<f4*>(a.out)[q] = v;
        }
      }
      done = nq << 2;
    }
  }
  for (size_t i = done + t0; i < a.n; i += stride) {
    const int p = static_cast<int>(static_cast<int8_t>(a.lhs[i])) *
                  static_cast<int>(static_cast<int8_t>(a.rhs[i]));
    const float f = static_cast<float>(p) * scale;
    if (OUT == MXQ_INT32)
      static_cast<int32_t*>(a.out)[i] = p;
    else if (OUT == MXQ_FLOAT32)
      static_cast<float*>(a.out)[i] = f;
    else
      static_cast<uint8_t*>(a.out)[i] = static_cast<uint8_t>(static_cast<int>(f));
  }
  if (OUT != MXQ_FLOAT32 && blockIdx.x == 0 && threadIdx.x == 0) {
    *a.omin = omin;
    *a.omax = omax;
  }
}

// ---- batch norm ---------------------------------------------------------------------------

struct BnArgs {
  const uint8_t* in;
  uint8_t* out;
  const float* gamma;
  const float* beta;
  const float* mean;
  const float* var;
  const float* min_data;
  const float* max_data;
  float* omin;
  float* omax;
  float* table;  // [2][C]: per-channel factor and offset in int8 units
  size_t n;
  uint32_t channels, inner;
  double eps;
  float min_calib, max_calib;
  int relu, vec_ok;
};

// dnnl_quantized_batch_norm.cc:66-112: gamma, beta and the moving statistics folded into
// one factor and one offset per channel in the units of the int8 input and output; then the
// library's own normalisation over mean 0 and variance 1, which divides the factor by
// sqrt(1 + eps) once more.
__device__ __forceinline__ void bn_channel(const BnArgs& a, uint32_t c, float max_abs_data,
                                           float max_abs_output, float unit_std, float& factor,
                                           float& offset) {
  const float invstd = static_cast<float>(1.0 / sqrt(static_cast<double>(a.var[c]) + a.eps));
  const float w = a.gamma[c] * invstd * max_abs_data / max_abs_output;
  offset = (a.beta[c] - a.mean[c] * a.gamma[c] * invstd) * 127.5f / max_abs_output;
  factor = w / unit_std;
}

__global__ __launch_bounds__(kThreads) void bn_table_kernel(BnArgs a) {
  const float max_abs_data = maxabs(*a.min_data, *a.max_data);
  const float max_abs_output = maxabs(a.min_calib, a.max_calib);
  const float unit_std = sqrtf(1.0f + static_cast<float>(a.eps));
  for (uint32_t c = blockIdx.x * kThreads + threadIdx.x; c < a.channels;
       c += gridDim.x * kThreads) {
    float w, b;
    bn_channel(a, c, max_abs_data, max_abs_output, unit_std, w, b);
    a.table[c] = w;
    a.table[a.channels + c] = b;
  }
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    *a.omin = a.min_calib;
    *a.omax = a.max_calib;
  }
}

// uint8 data is first brought to int8 at 127.5 / 255.5 of its value
// (dnnl_quantized_batch_norm.cc:47-65); at most 127.25, so no clamp is needed
template <bool IN_U>
__device__ __forceinline__ float bn_input(uint32_t word, int k) {
  if (!IN_U) return static_cast<float>(byte_of<false>(word, k));
  return rintf(static_cast<float>(byte_of<true>(word, k)) * (127.5f / 255.5f));
}

// relu before the rounding is a lower clamp at 0 instead of -128
template <bool IN_U, bool FAST>
__device__ __forceinline__ uint32_t bn_word(uint32_t x, float w, float b, float lo) {
  uint32_t r[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const float f = bn_input<IN_U>(x, j) * w + b;
    if (FAST) {
      r[j] = __float_as_uint(__builtin_amdgcn_fmed3f(f, lo, 127.f) + 12582912.f);
    } else {
      r[j] = static_cast<uint32_t>(narrow<MXQ_INT8>(f < lo ? lo : f));
    }
  }
  return pack_low_bytes(r[0], r[1], r[2], r[3]);
}

template <bool IN_U>
__device__ __forceinline__ u4 bn_sixteen(u4 x, float w, float b, float lo) {
  u4 v;
  // a finite factor and offset of this size keep every x * w + b finite: one-instruction
  // clamp; anything else (NaN, infinities from a zero range) takes the guarded conversion
  if (fabsf(w) < 1e30f && fabsf(b) < 1e30f) {
#pragma unroll
    for (int k = 0; k < 4; ++k) v[k] = bn_word<IN_U, true>(x[k], w, b, lo);
  } else {
#pragma unroll
    for (int k = 0; k < 4; ++k) v[k] = bn_word<IN_U, false>(x[k], w, b, lo);
  }
  return v;
}

template <bool IN_U>
__global__ __launch_bounds__(kThreads) void bn_kernel(BnArgs a) {
  const size_t stride = size_t(gridDim.x) * kThreads;
  const size_t t0 = size_t(blockIdx.x) * kThreads + threadIdx.x;
  const float* tw = a.table;
  const float* tb = a.table + a.channels;
  const float lo = a.relu != 0 ? 0.f : -128.f;
  if (a.vec_ok) {
    // 16 bytes of one channel per lane (inner % 16 == 0, fewer than 2^32 elements), two
    // loads in flight
    const uint32_t nv = static_cast<uint32_t>(a.n >> 4), inner16 = a.inner >> 4;
    const uint32_t step = static_cast<uint32_t>(stride);
    const u4* i16 = reinterpret_cast<const u4*>(a.in);
    u4* o16 = reinterpret_cast<u4*>(a.out);
    uint32_t q = static_cast<uint32_t>(t0);
    if (t0 >= nv) return;
    for (; nv - q > step; q += 2 * step) {
      const uint32_t q1 = q + step;
      const u4 x0 = __builtin_nontemporal_load(i16 + q);
      const u4 x1 = __builtin_nontemporal_load(i16 + q1);
      const uint32_t c0 = (q / inner16) % a.channels, c1 = (q1 / inner16) % a.channels;
      const float w0 = tw[c0], b0 = tb[c0], w1 = tw[c1], b1 = tb[c1];
      // both results before the first store: the stores are opaque to the compiler's count
      // of outstanding memory operations, a wait placed behind one would wait for it too
      const u4 v0 = bn_sixteen<IN_U>(x0, w0, b0, lo);
      const u4 v1 = bn_sixteen<IN_U>(x1, w1, b1, lo);
      stream_store16(v0, o16 + q);
      stream_store16(v1, o16 + q1);
      if (nv - q1 <= step) return;
    }
    const uint32_t c = (q / inner16) % a.channels;
    stream_store16(bn_sixteen<IN_U>(__builtin_nontemporal_load(i16 + q), tw[c], tb[c], lo),
                   o16 + q);
    return;
  }
  for (size_t i = t0; i < a.n; i += stride) {
    const uint32_t c = static_cast<uint32_t>((i / a.inner) % a.channels);
    const float f = bn_input<IN_U>(a.in[i], 0) * tw[c] + tb[c];
    a.out[i] = static_cast<uint8_t>(narrow<MXQ_INT8>(f < lo ? lo : f));
  }
}

constexpr int64_t kBnRowsMin = 2048;

// Rows of at least kBnRowsMin bytes (inner % 16 == 0): one wave per 4 KiB piece of a row, so
// the channel, its factor and offset are wave-uniform (no per-lane division) and a lane keeps
// four 16-byte loads in flight.
// No table kernel runs in front of this one: every wave folds its channel's four parameters
// itself (the function the table kernel calls, so the same factor and offset; one
// double-precision 1/sqrt per piece of up to 4 KiB) and the first thread passes the range on.
template <bool IN_U>
__global__ __launch_bounds__(kThreads) void bn_rows_kernel(BnArgs a) {
  const float max_abs_data = maxabs(*a.min_data, *a.max_data);
  const float max_abs_output = maxabs(a.min_calib, a.max_calib);
  const float unit_std = sqrtf(1.0f + static_cast<float>(a.eps));
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    *a.omin = a.min_calib;
    *a.omax = a.max_calib;
  }
  const uint32_t inner16 = a.inner >> 4;
  const uint32_t chunks = (inner16 + 255u) >> 8;
  const uint32_t rows = static_cast<uint32_t>(a.n / a.inner);
  const uint32_t items = rows * chunks;  // n < 2^32
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t wave =
      __builtin_amdgcn_readfirstlane(blockIdx.x * (kThreads / 64) + (threadIdx.x >> 6));
  const uint32_t nwaves = gridDim.x * (kThreads / 64);
  const float lo = a.relu != 0 ? 0.f : -128.f;
  const u4* i16 = reinterpret_cast<const u4*>(a.in);
  u4* o16 = reinterpret_cast<u4*>(a.out);
  for (uint32_t item = wave; item < items; item += nwaves) {
    const uint32_t row = item / chunks, k = item - row * chunks;
    const uint32_t c = row % a.channels;
    float w, b;
    bn_channel(a, c, max_abs_data, max_abs_output, unit_std, w, b);
    const uint32_t left = inner16 - (k << 8);
    const size_t base = size_t(row) * inner16 + (k << 8) + lane;
    u4 x[4] = {};
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (lane + 64u * j < left) x[j] = __builtin_nontemporal_load(i16 + base + 64 * j);
    u4 v[4];
    if (fabsf(w) < 1e30f && fabsf(b) < 1e30f) {
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) v[j][q] = bn_word<IN_U, true>(x[j][q], w, b, lo);
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) v[j][q] = bn_word<IN_U, false>(x[j][q], w, b, lo);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (lane + 64u * j < left) stream_store16(v[j], o16 + base + 64 * j);
  }
}

int grid_for(size_t work_items) {
  size_t want = (work_items + kThreads - 1) / kThreads;
  const size_t cap = size_t(num_cus()) * size_t(kCastBlocksPerCu);
  if (want < 1) want = 1;
  return static_cast<int>(want < cap ? want : cap);
}

bool byte_type(int t) { return t == MXQ_INT8 || t == MXQ_UINT8; }

}  // namespace
}  // namespace mxq

using namespace mxq;

extern "C" {

int mxq_quantized_elemwise_add(void* stream, const void* lhs, int lhs_type, const void* rhs,
                               int rhs_type, const float* lhs_min, const float* lhs_max,
                               const float* rhs_min, const float* rhs_max, void* out, int out_type,
                               float* omin, float* omax, size_t n, int calibrated,
                               float min_calib, float max_calib) {
  MXQ_API_BEGIN();
  MXQ_CHECK(byte_type(lhs_type) && byte_type(rhs_type),
            "quantized_elemwise_add takes int8 or uint8 inputs, got " << lhs_type << " and "
                                                                      << rhs_type);
  // ElemwiseAddType (quantized_elemwise_add.cc:50-78)
  const int want = !calibrated ? MXQ_INT32 : (lhs_type == rhs_type ? lhs_type : MXQ_INT8);
  MXQ_CHECK(out_type == want, "output type must be " << want << " for these inputs"
                                                     << (calibrated ? " (calibrated)" : "")
                                                     << ", got " << out_type);
  MXQ_CHECK(lhs_min != nullptr && lhs_max != nullptr && rhs_min != nullptr && rhs_max != nullptr &&
                omin != nullptr && omax != nullptr,
            "null range pointer");
  MXQ_CHECK(n == 0 || (lhs != nullptr && rhs != nullptr && out != nullptr), "null data pointer");
  AddArgs a;
  a.lhs = static_cast<const uint8_t*>(lhs);
  a.rhs = static_cast<const uint8_t*>(rhs);
  a.out = out;
  a.n = n;
  a.lhs_min = lhs_min; a.lhs_max = lhs_max; a.rhs_min = rhs_min; a.rhs_max = rhs_max;
  a.omin = omin; a.omax = omax;
  a.min_calib = min_calib; a.max_calib = max_calib;
  a.calibrated = calibrated != 0;
  const bool in_ok = out_type == MXQ_INT32
                         ? ((reinterpret_cast<uintptr_t>(lhs) | reinterpret_cast<uintptr_t>(rhs)) & 3u) == 0
                         : (aligned16(lhs) && aligned16(rhs));
  a.vec_ok = (in_ok && aligned16(out)) ? 1 : 0;
  const size_t per_lane = out_type == MXQ_INT32 ? 4 : 16;
  const int grid = grid_for(a.vec_ok ? (n + per_lane - 1) / per_lane : n);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool lu = lhs_type == MXQ_UINT8, ru = rhs_type == MXQ_UINT8;
#define MXQ_ADD(O, L, R) \
  hipLaunchKernelGGL((add_kernel<O, L, R>), dim3(grid), dim3(kThreads), 0, s, a)
  if (out_type == MXQ_INT32 && a.vec_ok && n >= kAddChunkMinElements) {
    const size_t per = size_t(kAddChunkPieces) * kAddChunkThreads;
    const size_t chunks = ((n >> 2) + per - 1) / per;
    MXQ_CHECK(chunks < (size_t(1) << 31), "tensor too large for one launch");
    const dim3 cg(static_cast<unsigned>(chunks)), cb(kAddChunkThreads);
    if (lu) {
      if (ru) hipLaunchKernelGGL((add32_chunk_kernel<true, true>), cg, cb, 0, s, a);
      else hipLaunchKernelGGL((add32_chunk_kernel<true, false>), cg, cb, 0, s, a);
    } else {
      if (ru) hipLaunchKernelGGL((add32_chunk_kernel<false, true>), cg, cb, 0, s, a);
      else hipLaunchKernelGGL((add32_chunk_kernel<false, false>), cg, cb, 0, s, a);
    }
  } else if (out_type == MXQ_INT32) {
    if (lu) { if (ru) MXQ_ADD(MXQ_INT32, true, true); else MXQ_ADD(MXQ_INT32, true, false); }
    else    { if (ru) MXQ_ADD(MXQ_INT32, false, true); else MXQ_ADD(MXQ_INT32, false, false); }
  } else if (out_type == MXQ_UINT8) {
    MXQ_ADD(MXQ_UINT8, true, true);
  } else {
    if (lu) MXQ_ADD(MXQ_INT8, true, false);
    else if (ru) MXQ_ADD(MXQ_INT8, false, true);
    else MXQ_ADD(MXQ_INT8, false, false);
  }
#undef MXQ_ADD
  MXQ_LAUNCH_CHECK();
  MXQ_API_END();
}

int mxq_quantized_broadcast_add(void* stream, const void* lhs, int lhs_type, int lhs_ndim,
                                const int64_t* lhs_shape, const void* rhs, int rhs_type,
                                int rhs_ndim, const int64_t* rhs_shape, const float* lhs_min,
                                const float* lhs_max, const float* rhs_min, const float* rhs_max,
                                void* out, int out_type, float* omin, float* omax,
                                int calibrated, float min_calib, float max_calib) {
  MXQ_API_BEGIN();
  MXQ_CHECK(lhs_ndim >= 0 && rhs_ndim >= 0 && (lhs_ndim == 0 || lhs_shape != nullptr) &&
                (rhs_ndim == 0 || rhs_shape != nullptr),
            "null shape pointer");
  // numpy broadcasting: shapes aligned at the last axis, an extent of 1 stretches
  const int nd = lhs_ndim > rhs_ndim ? lhs_ndim : rhs_ndim;
  std::vector<int64_t> ls(nd, 1), rs(nd, 1), os(nd, 1);
  for (int i = 0; i < lhs_ndim; ++i) ls[nd - lhs_ndim + i] = lhs_shape[i];
  for (int i = 0; i < rhs_ndim; ++i) rs[nd - rhs_ndim + i] = rhs_shape[i];
  bool same = lhs_ndim == rhs_ndim;
  size_t n = 1;
  for (int i = 0; i < nd; ++i) {
    MXQ_CHECK(ls[i] >= 0 && rs[i] >= 0, "negative extent");
    MXQ_CHECK(ls[i] == rs[i] || ls[i] == 1 || rs[i] == 1,
              "operands could not be broadcast together: axis " << i << " has " << ls[i]
                                                                << " and " << rs[i]);
    os[i] = ls[i] == 1 ? rs[i] : ls[i];
    same = same && ls[i] == rs[i];
    n *= static_cast<size_t>(os[i]);
  }
  // equal shapes take the plain sum, as the reference does
  if (same)
    return mxq_quantized_elemwise_add(stream, lhs, lhs_type, rhs, rhs_type, lhs_min, lhs_max,
                                      rhs_min, rhs_max, out, out_type, omin, omax, n, calibrated,
                                      min_calib, max_calib);
  MXQ_CHECK(byte_type(lhs_type) && byte_type(rhs_type),
            "quantized_npi_add takes int8 or uint8 inputs, got " << lhs_type << " and "
                                                                 << rhs_type);
  const int want = !calibrated ? MXQ_INT32 : (lhs_type == rhs_type ? lhs_type : MXQ_INT8);
  MXQ_CHECK(out_type == want, "output type must be " << want << " for these inputs"
                                                     << (calibrated ? " (calibrated)" : "")
                                                     << ", got " << out_type);
  MXQ_CHECK(lhs_min != nullptr && lhs_max != nullptr && rhs_min != nullptr && rhs_max != nullptr &&
                omin != nullptr && omax != nullptr,
            "null range pointer");
  MXQ_CHECK(n < (size_t(1) << 32), "broadcast output of " << n << " elements: at most 2^32 - 1");
  MXQ_CHECK(n == 0 || (lhs != nullptr && rhs != nullptr && out != nullptr), "null data pointer");
  BroadcastAddArgs p;
  AddArgs& a = p.add;
  a.lhs = static_cast<const uint8_t*>(lhs);
  a.rhs = static_cast<const uint8_t*>(rhs);
  a.out = out;
  a.n = n;
  a.lhs_min = lhs_min; a.lhs_max = lhs_max; a.rhs_min = rhs_min; a.rhs_max = rhs_max;
  a.omin = omin; a.omax = omax;
  a.min_calib = min_calib; a.max_calib = max_calib;
  a.calibrated = calibrated != 0;
  p.lhs_unsigned = lhs_type == MXQ_UINT8;
  p.rhs_unsigned = rhs_type == MXQ_UINT8;
  // element strides of the contiguous operands (0 where the operand is stretched), then
  // neighbouring axes with the same stretch pattern merged and unit axes dropped
  std::vector<int64_t> lst(nd, 0), rst(nd, 0);
  int64_t lacc = 1, racc = 1;
  for (int i = nd - 1; i >= 0; --i) {
    lst[i] = ls[i] == 1 ? 0 : lacc;
    rst[i] = rs[i] == 1 ? 0 : racc;
    lacc *= ls[i];
    racc *= rs[i];
  }
  std::vector<int64_t> md, ml, mr;
  for (int i = 0; i < nd; ++i) {
    if (os[i] == 1) continue;
    if (!md.empty() && ml.back() == lst[i] * os[i] && mr.back() == rst[i] * os[i]) {
      md.back() *= os[i];
      ml.back() = lst[i];
      mr.back() = rst[i];
    } else {
      md.push_back(os[i]);
      ml.push_back(lst[i]);
      mr.push_back(rst[i]);
    }
  }
  if (md.empty()) { md.push_back(1); ml.push_back(0); mr.push_back(0); }
  MXQ_CHECK(static_cast<int>(md.size()) <= kMaxBroadcastDims,
            "more than " << kMaxBroadcastDims << " axes after merging");
  p.nd = static_cast<int>(md.size());
  for (int i = 0; i < kMaxBroadcastDims; ++i) {
    p.dim[i] = i < p.nd ? static_cast<uint32_t>(md[i]) : 1;
    p.lstride[i] = i < p.nd ? static_cast<uint32_t>(ml[i]) : 0;
    p.rstride[i] = i < p.nd ? static_cast<uint32_t>(mr[i]) : 0;
  }
  // 16 outputs per lane when innermost runs are whole 16-byte pieces: every run of an
  // operand that is not stretched there then starts on a multiple of 16 elements
  a.vec_ok = (md.back() % 16 == 0 && aligned16(out) &&
              (ml.back() == 0 || aligned16(lhs)) && (mr.back() == 0 || aligned16(rhs)))
                 ? 1 : 0;
  if (n == 0) {
    // ranges only
    a.vec_ok = 0;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool lu = p.lhs_unsigned != 0, ru = p.rhs_unsigned != 0;
  const bool rows = a.vec_ok && md.back() >= 1024;
  const int grid = rows ? 2 * grid_for((n / static_cast<size_t>(md.back())) *
                                       ((static_cast<size_t>(md.back()) / 16 + 255) / 256) * 64)
                        : grid_for(a.vec_ok ? (n + 15) / 16 : (n ? n : 1));
#define MXQ_BCAST(O, L, R)                                                                   \
  do {                                                                                       \
    if (rows)                                                                                \
      hipLaunchKernelGGL((broadcast_add_rows_kernel<O, L, R>), dim3(grid), dim3(kThreads), 0, \
                         s, p);                                                              \
    else                                                                                     \
      hipLaunchKernelGGL((broadcast_add_kernel<O, L, R>), dim3(grid), dim3(kThreads), 0, s,  \
                         p);                                                                 \
  } while (0)
  if (out_type == MXQ_INT32) {
    if (lu) { if (ru) MXQ_BCAST(MXQ_INT32, true, true); else MXQ_BCAST(MXQ_INT32, true, false); }
    else    { if (ru) MXQ_BCAST(MXQ_INT32, false, true); else MXQ_BCAST(MXQ_INT32, false, false); }
  } else if (out_type == MXQ_UINT8) {
    MXQ_BCAST(MXQ_UINT8, true, true);
  } else {
    if (lu) MXQ_BCAST(MXQ_INT8, true, false);
    else if (ru) MXQ_BCAST(MXQ_INT8, false, true);
    else MXQ_BCAST(MXQ_INT8, false, false);
  }
#undef MXQ_BCAST
  MXQ_LAUNCH_CHECK();
  MXQ_API_END();
}

int mxq_quantized_elemwise_mul(void* stream, const int8_t* lhs, const int8_t* rhs,
                               const float* lhs_min, const float* lhs_max, const float* rhs_min,
                               const float* rhs_max, void* out, int out_type, float* omin,
                               float* omax, size_t n, int calibrated, float min_calib,
                               float max_calib) {
  MXQ_API_BEGIN();
  // QuantizedElemwiseMulOpType (quantized_elemwise_mul.cc:62-89)
  MXQ_CHECK(out_type == MXQ_FLOAT32 || out_type == (calibrated ? MXQ_INT8 : MXQ_INT32),
            "output type must be float32, or " << (calibrated ? "int8 (calibrated)" : "int32")
                                               << ", got " << out_type);
  MXQ_CHECK(lhs_min != nullptr && lhs_max != nullptr && rhs_min != nullptr && rhs_max != nullptr,
            "null range pointer");
  MXQ_CHECK(out_type == MXQ_FLOAT32 || (omin != nullptr && omax != nullptr),
            "null output range pointer");
  MXQ_CHECK(n == 0 || (lhs != nullptr && rhs != nullptr && out != nullptr), "null data pointer");
  MulArgs a;
  a.lhs = reinterpret_cast<const uint8_t*>(lhs);
  a.rhs = reinterpret_cast<const uint8_t*>(rhs);
  a.out = out;
  a.n = n;
  a.lhs_min = lhs_min; a.lhs_max = lhs_max; a.rhs_min = rhs_min; a.rhs_max = rhs_max;
  a.omin = omin; a.omax = omax;
  a.min_calib = min_calib; a.max_calib = max_calib;
  const bool in_ok = out_type == MXQ_INT8
                         ? (aligned16(lhs) && aligned16(rhs))
                         : ((reinterpret_cast<uintptr_t>(lhs) | reinterpret_cast<uintptr_t>(rhs)) & 3u) == 0;
  a.vec_ok = (in_ok && aligned16(out)) ? 1 : 0;
  const size_t per_lane = out_type == MXQ_INT8 ? 16 : 4;
  const int grid = grid_for(a.vec_ok ? (n + per_lane - 1) / per_lane : n);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (out_type == MXQ_INT8)
    hipLaunchKernelGGL((mul_kernel<MXQ_INT8>), dim3(grid), dim3(kThreads), 0, s, a);
  else if (out_type == MXQ_INT32)
    hipLaunchKernelGGL((mul_kernel<MXQ_INT32>), dim3(grid), dim3(kThreads), 0, s, a);
  else
    hipLaunchKernelGGL((mul_kernel<MXQ_FLOAT32>), dim3(grid), dim3(kThreads), 0, s, a);
  MXQ_LAUNCH_CHECK();
  MXQ_API_END();
}

size_t mxq_quantized_batch_norm_workspace(int64_t channels) {
  return channels > 0 ? static_cast<size_t>(channels) * 2 * sizeof(float) : 0;
}

int mxq_quantized_batch_norm(void* stream, const void* data, int data_type, const float* gamma,
                             const float* beta, const float* moving_mean,
                             const float* moving_var, const float* min_data,
                             const float* max_data, int8_t* out, float* omin, float* omax,
                             int64_t outer, int64_t channels, int64_t inner, double eps,
                             float min_calib, float max_calib, int relu, void* workspace,
                             size_t workspace_bytes) {
  MXQ_API_BEGIN();
  MXQ_CHECK(byte_type(data_type),
            "QuantizedBatchNorm only supports int8/uint8 input, while " << data_type
                                                                          << " is given.");
  MXQ_CHECK(outer >= 0 && channels > 0 && inner >= 0, "bad shape");
  MXQ_CHECK(channels < (int64_t(1) << 31) && inner < (int64_t(1) << 31), "extent too large");
  MXQ_CHECK(gamma != nullptr && beta != nullptr && moving_mean != nullptr && moving_var != nullptr,
            "null parameter pointer");
  MXQ_CHECK(min_data != nullptr && max_data != nullptr && omin != nullptr && omax != nullptr,
            "null range pointer");
  MXQ_CHECK(workspace != nullptr && workspace_bytes >= mxq_quantized_batch_norm_workspace(channels),
            "workspace too small: " << workspace_bytes << " < "
                                    << mxq_quantized_batch_norm_workspace(channels));
  MXQ_CHECK((reinterpret_cast<uintptr_t>(workspace) & 3u) == 0, "workspace must be 4-byte aligned");
  BnArgs a;
  a.in = static_cast<const uint8_t*>(data);
  a.out = reinterpret_cast<uint8_t*>(out);
  a.gamma = gamma; a.beta = beta; a.mean = moving_mean; a.var = moving_var;
  a.min_data = min_data; a.max_data = max_data; a.omin = omin; a.omax = omax;
  a.table = static_cast<float*>(workspace);
  a.n = static_cast<size_t>(outer) * static_cast<size_t>(channels) * static_cast<size_t>(inner);
  a.channels = static_cast<uint32_t>(channels);
  a.inner = static_cast<uint32_t>(inner);
  a.eps = eps;
  a.min_calib = min_calib; a.max_calib = max_calib;
  a.relu = relu;
  MXQ_CHECK(a.n == 0 || (data != nullptr && out != nullptr), "null data pointer");
  a.vec_ok = (inner % 16 == 0 && a.n < (size_t(1) << 32) && aligned16(data) && aligned16(out)) ? 1 : 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  // Rows of kBnRowsMin bytes and more: ONE launch, a wave per piece of a row of up to 4 KiB,
  // the waves fold their channel's parameters themselves.  Twice the work-groups per CU of
  // the narrowing kernels, as for concat (measured fastest); from 64 M elements one piece per
  // wave and no loop.  Shorter rows fill too little of a wave's four 1 KiB pieces (64 x 512
  // x 1024: 28.6 us that way, 18.4 us with 16 bytes per lane and the channel by division).
  if (a.n != 0 && a.vec_ok && inner >= kBnRowsMin) {
    const size_t waves = (a.n / a.inner) * ((a.inner / 16 + 255) / 256);
    int grid = 2 * grid_for(waves * 64);
    if (a.n >= (size_t(1) << 26))
      grid = static_cast<int>((waves + kThreads / 64 - 1) / (kThreads / 64));
    if (data_type == MXQ_UINT8)
      hipLaunchKernelGGL((bn_rows_kernel<true>), dim3(grid), dim3(kThreads), 0, s, a);
    else
      hipLaunchKernelGGL((bn_rows_kernel<false>), dim3(grid), dim3(kThreads), 0, s, a);
    MXQ_LAUNCH_CHECK();
    return 0;
  }
  hipLaunchKernelGGL(bn_table_kernel, dim3((a.channels + kThreads - 1) / kThreads < 64
                                               ? (a.channels + kThreads - 1) / kThreads
                                               : 64),
                     dim3(kThreads), 0, s, a);
  MXQ_LAUNCH_CHECK();
  if (a.n == 0) return 0;
  {
    const int grid = 2 * grid_for(a.vec_ok ? (a.n + 15) / 16 : a.n);
    if (data_type == MXQ_UINT8)
      hipLaunchKernelGGL((bn_kernel<true>), dim3(grid), dim3(kThreads), 0, s, a);
    else
      hipLaunchKernelGGL((bn_kernel<false>), dim3(grid), dim3(kThreads), 0, s, a);
  }
  MXQ_LAUNCH_CHECK();
  MXQ_API_END();
}

int mxq_quantized_concat(void* stream, int num_args, const void* const* in, const int* in_type,
                         const float* const* in_min, const float* const* in_max,
                         const int64_t* in_axis, int64_t outer, int64_t inner, void* out,
                         int out_type, float* omin, float* omax) {
  MXQ_API_BEGIN();
  MXQ_CHECK(num_args >= 1, "concat needs at least one input");
  MXQ_CHECK(in != nullptr && in_type != nullptr && in_min != nullptr && in_max != nullptr &&
                in_axis != nullptr,
            "null argument table");
  MXQ_CHECK(omin != nullptr && omax != nullptr, "null range pointer");
  MXQ_CHECK(outer >= 0 && inner >= 0, "negative extent");
  // QuantizedConcatType (quantized_concat.cc:83-103): int8 as soon as one input is
  int want = MXQ_UINT8;
  int64_t axis_total = 0;
  for (int i = 0; i < num_args; ++i) {
    MXQ_CHECK(byte_type(in_type[i]), "quantized_concat takes int8 or uint8 inputs, input "
                                         << i << " has type " << in_type[i]);
    if (in_type[i] == MXQ_INT8) want = MXQ_INT8;
    MXQ_CHECK(in_axis[i] >= 0, "negative extent of input " << i);
    MXQ_CHECK(in_min[i] != nullptr && in_max[i] != nullptr, "null range pointer of input " << i);
    axis_total += in_axis[i];
  }
  MXQ_CHECK(out_type == want, "output type must be " << want << ", got " << out_type);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool several = num_args > kMaxConcatPerLaunch;
  if (several) {
    for (int first = 0; first < num_args; first += kMaxConcatPerLaunch) {
      ConcatRanges r;
      r.count = num_args - first < kMaxConcatPerLaunch ? num_args - first : kMaxConcatPerLaunch;
      r.first = first == 0;
      for (int i = 0; i < kMaxConcatPerLaunch; ++i) {
        r.mn[i] = i < r.count ? in_min[first + i] : nullptr;
        r.mx[i] = i < r.count ? in_max[first + i] : nullptr;
      }
      hipLaunchKernelGGL(concat_range_kernel, dim3(1), dim3(1), 0, s, r, omin, omax);
      MXQ_LAUNCH_CHECK();
    }
  }
  const size_t pitch = static_cast<size_t>(axis_total) * static_cast<size_t>(inner);
  size_t offset = 0;
  for (int first = 0; first < num_args; first += kMaxConcatPerLaunch) {
    ConcatArgs a;
    a.count = num_args - first < kMaxConcatPerLaunch ? num_args - first : kMaxConcatPerLaunch;
    a.out = static_cast<uint8_t*>(out);
    a.rows = static_cast<size_t>(outer);
    a.out_pitch = pitch;
    a.omin = omin;
    a.omax = omax;
    a.out_type = out_type;
    a.given_range = several ? 1 : 0;
    size_t launch_bytes = 0;
    for (int i = 0; i < a.count; ++i)
      launch_bytes += a.rows * static_cast<size_t>(in_axis[first + i]) * static_cast<size_t>(inner);
    size_t part_bytes[kMaxConcatPerLaunch];
    bool all_vec = true;
    for (int i = 0; i < kMaxConcatPerLaunch; ++i) {
      const int k = first + (i < a.count ? i : 0);  // unused slots repeat a valid entry
      a.in[i] = static_cast<const uint8_t*>(in[k]);
      a.mn[i] = in_min[k];
      a.mx[i] = in_max[k];
      a.in_type[i] = in_type[k];
      a.row_bytes[i] = static_cast<size_t>(in_axis[k]) * static_cast<size_t>(inner);
      a.out_off[i] = offset;
      a.vec_ok[i] = 0;
      part_bytes[i] = 0;
      if (i < a.count) {
        part_bytes[i] = a.rows * a.row_bytes[i];
        MXQ_CHECK(part_bytes[i] == 0 || (in[k] != nullptr && out != nullptr), "null data pointer");
        const uint8_t* dst = a.out + offset;
        a.vec_ok[i] = (aligned16(a.in[i]) && aligned16(dst) && a.row_bytes[i] % 16 == 0 &&
                       (a.rows == 1 || pitch % 16 == 0)) ? 1 : 0;
        all_vec = all_vec && (a.vec_ok[i] != 0 || part_bytes[i] == 0);
        offset += a.row_bytes[i];
      }
    }
    // Large launches of 16-byte-aligned inputs: one chunk per work-group, no loop (measured
    // faster from 16 MiB: 32 MiB 15.3 -> 14.7 us, 64 x (256 + 64) x 56 x 56 31.1 -> 28.8 us inside a
    // graph; 8 MiB unchanged).  Otherwise twice the work-groups per CU of the narrowing kernels,
    // shared out in proportion to the bytes (at least one each, so that the block table
    // stays monotonic): the inputs of one launch finish together.
    const bool chunked = all_vec && launch_bytes >= kConcatChunkMinBytes;
    const size_t chunk_bytes = size_t(kConcatChunkPieces) * kThreads * 16;
    const int budget = 2 * grid_for(launch_bytes);
    size_t blocks64 = 0;
    for (int i = 0; i < kMaxConcatPerLaunch; ++i) {
      if (i < a.count) {
        const size_t bytes = part_bytes[i];
        if (chunked) {
          blocks64 += (bytes + chunk_bytes - 1) / chunk_bytes;
        } else {
          const size_t share = launch_bytes == 0 ? 1 : (size_t(budget) * bytes) / launch_bytes;
          const int fit = grid_for(a.vec_ok[i] ? bytes / 16 : bytes);
          blocks64 += share < 1 ? 1 : (share < size_t(fit) ? share : size_t(fit));
        }
      }
      MXQ_CHECK(blocks64 < (size_t(1) << 31), "tensors too large for one launch");
      a.block_end[i] = static_cast<int>(blocks64);
    }
    const int blocks = static_cast<int>(blocks64);
    if (chunked)
      hipLaunchKernelGGL(concat_kernel<true>, dim3(blocks), dim3(kThreads), 0, s, a);
    else
      hipLaunchKernelGGL(concat_kernel<false>, dim3(blocks), dim3(kThreads), 0, s, a);
    MXQ_LAUNCH_CHECK();
  }
  MXQ_API_END();
}

}  // extern "C"
