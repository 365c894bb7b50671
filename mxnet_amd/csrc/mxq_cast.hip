// Bandwidth-bound kernels of the INT8 path for gfx950: quantize (v1/v2),
// requantize, dequantize, and the single-pass min/max grid reduction the
// uncalibrated variants need.
//
// Arithmetic contract (bit-exact with the reference's native CPU kernels):
// every float operation below is one correctly rounded binary32 operation in
// the order the reference writes it; this file is compiled with
// -ffp-contract=off so no multiply-add is fused, and divisions are IEEE.
//   int8 :  R = max(|lo|,|hi|); s = 127.f / R; q = trunc(sign(x) * min(|x|*s + 0.5f, 127.f))
//           (quantization_utils.h:83-89, quantize_v2-inl.h:98-114)
//   uint8:  s = float(255.0 / double(hi - lo)); q = trunc(double((x - lo) * s) + 0.5)
//           (quantize_v2-inl.h:66-81; saturated to [0,255] where the reference is undefined)
//   requantize: f = float(q32) * (max(|imin|,|imax|) / 2^31), then the int8 rule
//           (quantization_utils.h:91-97, requantize-inl.h:89-125)
//   dequantize: int8 y = float(q) * (max(|hi|,|lo|) / 127.f)
//               uint8 y = float(q) * ((hi - lo) / 255.f) + lo   (dequantize-inl.h:49-75)
//
// Memory access pattern: a wave reads 1 KiB contiguous per load instruction
// (lane i owns bytes 16i..16i+15), UNROLL such segments are in flight per
// lane, loads are non-temporal (the tensors are streamed once), 2 work-groups of
// 256 threads per CU (more resident waves lower the achieved HBM bandwidth).
#include <hip/hip_runtime.h>

#include <atomic>
#include <cmath>
#include <cstdint>
#include <cstring>

#include "../../include/mxq.h"
#include "mxq_common.h"

namespace mxq {

namespace {

typedef float f4 __attribute__((ext_vector_type(4)));
typedef int i4 __attribute__((ext_vector_type(4)));

constexpr int kThreads = 256;
constexpr int kUnroll = 4;             // 16-byte segments in flight per lane
// Reduction workspace: one 16-byte partial {min, max, nan flag, -} per block of the
// reduce kernel, written with plain stores (nothing has to be initialised, no
// atomics, no fences); the consuming kernel of the same stream folds the partials
// in its prologue.  The reduce grid is capped so the workspace stays small.
constexpr int kMaxParts = 1024;
constexpr int kPartWords = 4;
constexpr size_t kWsBytes = size_t(kMaxParts) * kPartWords * 4;

// The reduction partials of mxq_quantize_v2_noalloc: library-owned device memory for callers
// that can neither allocate nor bring a workspace.  Every GPU the library runs on holds its
// own copy of this array at its own address until the process ends.  In host code the
// name below is only a handle for hipGetSymbolAddress; kernels are given the address that
// call returns (cached per device in g_noalloc_ptr).
static __device__ __align__(256) uint32_t scratch[kMaxParts * kPartWords];
constexpr int kMaxDevices = 64;
std::atomic<uint32_t*> g_noalloc_ptr[kMaxDevices];
constexpr size_t kNoAllocMaxElements = size_t(1) << 31;

__device__ __forceinline__ float maxabs(float a, float b) {
  float x = fabsf(a), y = fabsf(b);
  return (x < y) ? y : x;
}

template <typename T>
__device__ __forceinline__ T nt_load(const T* p) {
  return __builtin_nontemporal_load(p);
}
template <typename T>
__device__ __forceinline__ void nt_store(T v, T* p) {
  __builtin_nontemporal_store(v, p);
}
// Packed-byte output stream of the narrowing kernels: a device-scope store
// (global_store_dword ... sc1) is written through the XCD's L2 instead of lingering
// there as a dirty line, which keeps the HBM write stream sequential; measured 6.9
// against 6.3 TB/s for the fp32 -> int8 pattern with plain or non-temporal stores.
__device__ __forceinline__ void stream_store(uint32_t v, uint32_t* p) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// ---- per-element rules -------------------------------------------------------

// trunc(sign(x) * min(|x| * s + 0.5f, 127.f)); v >= 0.5 so the sign can be
// applied after the truncation.
__device__ __forceinline__ int quant_i8(float x, float s) {
  float t = fabsf(x) * s;
  float u = t + 0.5f;
  float v = (127.0f < u) ? 127.0f : u;
  int iv = static_cast<int>(v);
  return (x < 0.0f) ? -iv : ((x > 0.0f) ? iv : 0);
}

__device__ __forceinline__ int quant_u8(float x, float lo, float s) {
  float t = (x - lo) * s;
  double u = static_cast<double>(t) + 0.5;
  u = (u > 0.0) ? u : 0.0;
  u = (u > 255.0) ? 255.0 : u;
  return static_cast<int>(u);
}

__device__ __forceinline__ uint32_t pack4(int a, int b, int c, int d) {
  return (uint32_t(a) & 0xffu) | ((uint32_t(b) & 0xffu) << 8) | ((uint32_t(c) & 0xffu) << 16) |
         (uint32_t(d) << 24);
}

struct QuantI8 {
  float s;
  __device__ __forceinline__ int operator()(float x) const { return quant_i8(x, s); }
};
struct QuantU8 {
  float lo, s;
  __device__ __forceinline__ int operator()(float x) const { return quant_u8(x, lo, s); }
};

// static_cast<uint8_t>(x * scale + shift + 0.5) with the 0.5 a double
// (quantize_asym-inl.h:62-76).  Outside [0, 256) that conversion is undefined in the
// reference; here the low byte of the truncated int32 is kept, as its x86 build does.
struct QuantAsym {
  float scale, shift;
  __device__ __forceinline__ int operator()(float x) const {
    const float t = x * scale + shift;
    return static_cast<int>(static_cast<double>(t) + 0.5);
  }
};

__device__ __forceinline__ float to_float(float x) { return x; }
__device__ __forceinline__ float to_float(int32_t x) { return static_cast<float>(x); }

// ---- 4-byte source -> 1-byte destination streaming body ---------------------
// SrcT is float (quantize) or int32_t (requantize; pre scales the converted
// value).  Each lane converts 4 consecutive elements per segment and stores one
// dword; a wave reads 1 KiB and writes 256 B contiguous per segment.
template <typename SrcT, typename Rule, bool PRE>
__device__ __forceinline__ void narrow_stream(const SrcT* __restrict__ in,
                                              uint8_t* __restrict__ out, size_t n, Rule rule,
                                              float pre, bool rev = false) {
  typedef SrcT Vec4 __attribute__((ext_vector_type(4)));
  const size_t nquad = n >> 2;  // groups of 4 elements
  const Vec4* in4 = reinterpret_cast<const Vec4*>(in);
  uint32_t* out4 = reinterpret_cast<uint32_t*>(out);
  if (rev) {
    // back to front: the tail of the tensor, which the range reduction read last, is what
    // the memory-side cache still holds (measured: 3 % off the two-launch time at 256 MB)
    in4 += nquad - 1;
    out4 += nquad - 1;
  }
  const ptrdiff_t dir = rev ? -1 : 1;
  const size_t stride = size_t(gridDim.x) * kThreads;
  size_t q = size_t(blockIdx.x) * kThreads + threadIdx.x;
  // main loop: kUnroll segments, each `stride` quads apart
  for (; q + size_t(kUnroll - 1) * stride < nquad; q += size_t(kUnroll) * stride) {
    Vec4 x[kUnroll];
#pragma unroll
    for (int j = 0; j < kUnroll; ++j)
      x[j] = nt_load(in4 + dir * static_cast<ptrdiff_t>(q + size_t(j) * stride));
#pragma unroll
    for (int j = 0; j < kUnroll; ++j) {
      float f0 = to_float(x[j].x), f1 = to_float(x[j].y), f2 = to_float(x[j].z),
            f3 = to_float(x[j].w);
      if (PRE) {
        f0 = f0 * pre;
        f1 = f1 * pre;
        f2 = f2 * pre;
        f3 = f3 * pre;
      }
      stream_store(pack4(rule(f0), rule(f1), rule(f2), rule(f3)),
                   out4 + dir * static_cast<ptrdiff_t>(q + size_t(j) * stride));
    }
  }
  for (; q < nquad; q += stride) {
    Vec4 x = nt_load(in4 + dir * static_cast<ptrdiff_t>(q));
    float f0 = to_float(x.x), f1 = to_float(x.y), f2 = to_float(x.z), f3 = to_float(x.w);
    if (PRE) {
      f0 = f0 * pre;
      f1 = f1 * pre;
      f2 = f2 * pre;
      f3 = f3 * pre;
    }
    stream_store(pack4(rule(f0), rule(f1), rule(f2), rule(f3)),
                 out4 + dir * static_cast<ptrdiff_t>(q));
  }
  // ragged tail (< 4 elements)
  if (blockIdx.x == 0) {
    size_t i = (nquad << 2) + threadIdx.x;
    if (i < n) {
      float f = to_float(in[i]);
      if (PRE) f = f * pre;
      out[i] = static_cast<uint8_t>(rule(f));
    }
  }
}

// Scalar fallback for pointers that are not 16-byte (source) / 4-byte
// (destination) aligned.
template <typename SrcT, typename Rule, bool PRE>
__device__ __forceinline__ void narrow_scalar(const SrcT* __restrict__ in,
                                              uint8_t* __restrict__ out, size_t n, Rule rule,
                                              float pre) {
  const size_t stride = size_t(gridDim.x) * kThreads;
  for (size_t i = size_t(blockIdx.x) * kThreads + threadIdx.x; i < n; i += stride) {
    float f = to_float(in[i]);
    if (PRE) f = f * pre;
    out[i] = static_cast<uint8_t>(rule(f));
  }
}

// ---- reduced-range partials -------------------------------------------------------
// (the fold helpers need wave_reduce, defined with the reduction kernels below)
template <typename T, typename Op>
__device__ __forceinline__ T wave_reduce(T v, Op op);

struct MinU {
  __device__ __forceinline__ uint32_t operator()(uint32_t a, uint32_t b) const {
    return a < b ? a : b;
  }
};
struct MaxU {
  __device__ __forceinline__ uint32_t operator()(uint32_t a, uint32_t b) const {
    return a > b ? a : b;
  }
};

// Order-preserving map float -> uint32 (so unsigned min/max order floats) and back.
__device__ __forceinline__ uint32_t f2ord(float f) {
  uint32_t u = __builtin_bit_cast(uint32_t, f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float ord2f(uint32_t o) {
  uint32_t u = (o & 0x80000000u) ? (o & 0x7fffffffu) : ~o;
  return __builtin_bit_cast(float, u);
}

// Block-cooperative fold of `nparts` partials {min, max, flag} held as unsigned
// words whose unsigned order is the value order (floats through f2ord, int32
// with the sign bit flipped).  Every thread returns the global result.
__device__ __forceinline__ void fold_parts(const uint32_t* __restrict__ parts, int nparts,
                                           uint32_t& mn, uint32_t& mx, uint32_t& flag) {
  __shared__ uint32_t s_mn[kThreads / 64], s_mx[kThreads / 64], s_fl[kThreads / 64];
  mn = 0xffffffffu;
  mx = 0u;
  flag = 0u;
  for (int i = threadIdx.x; i < nparts; i += kThreads) {
    const uint32_t a = parts[i * kPartWords + 0], b = parts[i * kPartWords + 1];
    mn = a < mn ? a : mn;
    mx = b > mx ? b : mx;
    flag |= parts[i * kPartWords + 2];
  }
  mn = wave_reduce(mn, MinU());
  mx = wave_reduce(mx, MaxU());
  flag = wave_reduce(flag, MaxU());
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) {
    s_mn[wave] = mn;
    s_mx[wave] = mx;
    s_fl[wave] = flag;
  }
  __syncthreads();
#pragma unroll
  for (int w = 0; w < kThreads / 64; ++w) {
    mn = s_mn[w] < mn ? s_mn[w] : mn;
    mx = s_mx[w] > mx ? s_mx[w] : mx;
    flag |= s_fl[w];
  }
}

// Range left by the fp32 reduction, NaN-propagating like mshadow's red::minimum /
// red::maximum (3rdparty/mshadow/mshadow/base.h:1054-1115): any NaN makes both NaN.
__device__ __forceinline__ void load_range_f32(const uint32_t* parts, int nparts, float& lo,
                                               float& hi) {
  uint32_t mn, mx, nan;
  fold_parts(parts, nparts, mn, mx, nan);
  lo = ord2f(mn);
  hi = ord2f(mx);
  if (nan) lo = hi = NAN;
}

// Range left by the int32 reduction, converted to the float images
// QuantizedToFloat(min), QuantizedToFloat(max) (requantize-inl.h:192-227).
__device__ __forceinline__ void load_range_i32(const uint32_t* parts, int nparts, float in_scale,
                                               float& lo, float& hi) {
  uint32_t mn, mx, unused;
  fold_parts(parts, nparts, mn, mx, unused);
  lo = static_cast<float>(static_cast<int>(mn ^ 0x80000000u)) * in_scale;
  hi = static_cast<float>(static_cast<int>(mx ^ 0x80000000u)) * in_scale;
}

// ---- quantize kernels ----------------------------------------------------------
// The range is (lo, hi) by value, two device scalars when dlo != NULL (v1 operator
// inputs), or the reduction partials when parts != NULL (uncalibrated v2).
template <bool UNSIGNED, bool VEC>
__global__ __launch_bounds__(kThreads) void quantize_kernel(const float* __restrict__ in,
                                                            uint8_t* __restrict__ out,
                                                            float* __restrict__ omin,
                                                            float* __restrict__ omax, size_t n,
                                                            float lo, float hi,
                                                            const float* __restrict__ dlo,
                                                            const float* __restrict__ dhi,
                                                            const uint32_t* __restrict__ parts,
                                                            int nparts, int rev) {
  if (dlo != nullptr) {
    lo = *dlo;
    hi = *dhi;
  } else if (parts != nullptr) {
    load_range_f32(parts, nparts, lo, hi);
  }
  if (UNSIGNED) {
    QuantU8 rule;
    rule.lo = lo;
    rule.s = static_cast<float>((255.0 - 0.0) / static_cast<double>(hi - lo));
    if (VEC)
      narrow_stream<float, QuantU8, false>(in, out, n, rule, 0.f, rev != 0);
    else
      narrow_scalar<float, QuantU8, false>(in, out, n, rule, 0.f);
    if (blockIdx.x == 0 && threadIdx.x == 0) {
      *omin = lo;
      *omax = hi;
    }
  } else {
    const float r = maxabs(lo, hi);
    QuantI8 rule;
    rule.s = 127.0f / r;
    if (VEC)
      narrow_stream<float, QuantI8, false>(in, out, n, rule, 0.f, rev != 0);
    else
      narrow_scalar<float, QuantI8, false>(in, out, n, rule, 0.f);
    if (blockIdx.x == 0 && threadIdx.x == 0) {
      *omin = -r;
      *omax = r;
    }
  }
}

// ---- asymmetric quantize (float -> uint8 over [min, max]) ---------------------------
// scale = 255 / (max - min), shift = 255 - max * scale (quantize_asym-inl.h:103-152); the
// range is (lo, hi) by value or the reduction partials.
template <bool VEC>
__global__ __launch_bounds__(kThreads) void quantize_asym_kernel(
    const float* __restrict__ in, uint8_t* __restrict__ out, float* __restrict__ oscale,
    float* __restrict__ oshift, size_t n, float lo, float hi, const uint32_t* __restrict__ parts,
    int nparts, int rev) {
  if (parts != nullptr) load_range_f32(parts, nparts, lo, hi);
  QuantAsym rule;
  rule.scale = 255.0f / (hi - lo);
  rule.shift = 255.0f - hi * rule.scale;
  if (VEC)
    narrow_stream<float, QuantAsym, false>(in, out, n, rule, 0.f, rev != 0);
  else
    narrow_scalar<float, QuantAsym, false>(in, out, n, rule, 0.f);
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    *oscale = rule.scale;
    *oshift = rule.shift;
  }
}

// int8 -> uint8 with scale 1 and shift 128 (the sign bit flipped), or the uint8 identity
// with scale 1 and shift 0 (quantize_asym-inl.h:85-101)
template <bool FLIP>
__global__ __launch_bounds__(kThreads) void asym_bytes_kernel(const uint8_t* __restrict__ in,
                                                              uint8_t* __restrict__ out,
                                                              float* __restrict__ oscale,
                                                              float* __restrict__ oshift,
                                                              size_t n, int vec) {
  const size_t stride = size_t(gridDim.x) * kThreads;
  const size_t t0 = size_t(blockIdx.x) * kThreads + threadIdx.x;
  size_t done = 0;
  if (vec) {
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    const size_t nv = n >> 4;
    const u4* i16 = reinterpret_cast<const u4*>(in);
    u4* o16 = reinterpret_cast<u4*>(out);
    for (size_t q = t0; q < nv; q += stride) {
      u4 v = nt_load(i16 + q);
      if (FLIP) v ^= 0x80808080u;
      nt_store(v, o16 + q);
    }
    done = nv << 4;
  }
  for (size_t i = done + t0; i < n; i += stride) out[i] = FLIP ? (in[i] ^ 0x80u) : in[i];
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    *oscale = 1.0f;
    *oshift = FLIP ? 128.0f : 0.0f;
  }
}

// ---- requantize kernel -------------------------------------------------------
// real range: by value (calibrated), or MaxAbs of the float images of the int32
// min and max left in the reduction partials.
template <bool VEC>
__global__ __launch_bounds__(kThreads) void requantize_kernel(
    const int32_t* __restrict__ in, uint8_t* __restrict__ out, float* __restrict__ omin,
    float* __restrict__ omax, size_t n, const float* __restrict__ imin,
    const float* __restrict__ imax, float real_range, const uint32_t* __restrict__ parts,
    int nparts, int rev) {
  const float in_scale = maxabs(*imin, *imax) / 2147483648.0f;
  if (parts != nullptr) {
    float lo, hi;
    load_range_i32(parts, nparts, in_scale, lo, hi);
    real_range = maxabs(lo, hi);
  }
  QuantI8 rule;
  rule.s = 127.0f / maxabs(-real_range, real_range);
  if (VEC)
    narrow_stream<int32_t, QuantI8, true>(in, out, n, rule, in_scale, rev != 0);
  else
    narrow_scalar<int32_t, QuantI8, true>(in, out, n, rule, in_scale);
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    *omin = -real_range;
    *omax = real_range;
  }
}

// ---- dequantize kernel ---------------------------------------------------------
// Write-dominated (1 byte in, 4 out).  A wave owns whole 4 KiB runs of the output: lane l
// reads the dwords l, l + 64, l + 128, l + 192 of the run's 1 KiB of input and issues four
// 16-byte stores back to back, each instruction writing 1 KiB of consecutive addresses.
// Stores are device-scope (written through past the XCD's L2).  Measured at 64 M elements
// against lanes that take 16-byte segments a grid-stride apart (the pattern of the
// narrowing kernels): 56.2 against 58.5 us; a run of 8 or 16 KiB per wave, requesting the
// next run's input ahead of the stores, 32 contiguous bytes per lane or work-group spans
// of 16 - 64 KiB are all slower.
constexpr int kDeqRunQuads = 256;   // 16-byte pieces of one wave's output run (4 KiB)
// cache policy of the buffer stores: sc1 (bit 4) + nt (bit 1), written through and not kept
// (dequantize at 2^26 elements: 56.3 us; sc1 alone 56.8, nt alone 58.2, neither 59.7)
constexpr int kStreamOut = 18;
constexpr int kRsrcFlags = 0x00020000;

// One contiguous chunk per work-group, no loop: every lane requests its two dwords of the
// chunk's 4 KiB of input (512 lanes, a lane's dwords 2 KiB apart), then converts and writes
// the chunk's 16 KiB of output with two 16-byte stores.  From 16 M elements on this is the
// fastest pattern measured for the widening cast (64 M: 50.3 us against 56.3 us for 4 KiB
// runs per wave of a grid-stride kernel; 256 M: 196 against 237 us); exactly two pieces per
// lane matter (one: 60.7 us, three: 57.5, four: 58.9 at 64 M), the thread count little (128 /
// 256 / 512 / 1024 threads: 51.6 / 51.5 / 50.3 / 54.3 us).
constexpr int kDeqChunkThreads = 512;
constexpr int kDeqChunkPieces = 2;
constexpr size_t kDeqChunkMinElements = size_t(1) << 24;

template <bool UNSIGNED>
__global__ __launch_bounds__(kDeqChunkThreads) void dequantize_chunk_kernel(
    const uint8_t* __restrict__ in, float* __restrict__ out, size_t n,
    const float* __restrict__ imin, const float* __restrict__ imax) {
  const float lo = *imin, hi = *imax;
  const float scale = UNSIGNED ? (hi - lo) / (255.0f - 0.0f) : maxabs(hi, lo) / 127.0f;
  auto conv = [&](uint32_t byte) -> float {
    if (UNSIGNED) {
      float p = static_cast<float>(byte) * scale;
      return p + lo;
    } else {
      return static_cast<float>(static_cast<int>(static_cast<int8_t>(byte))) * scale;
    }
  };
  const size_t nquad = n >> 2;
  const size_t base = size_t(blockIdx.x) * (kDeqChunkPieces * kDeqChunkThreads);
  const uint32_t* in4 = reinterpret_cast<const uint32_t*>(in);
  uint32_t w[kDeqChunkPieces];
#pragma unroll
  for (int j = 0; j < kDeqChunkPieces; ++j) {
    const size_t q = base + size_t(j) * kDeqChunkThreads + threadIdx.x;
    w[j] = q < nquad ? nt_load(in4 + q) : 0u;
  }
  // the descriptor ends with the tensor: pieces past the last whole quad are dropped
  const size_t left = nquad > base ? nquad - base : 0;
  const uint32_t bytes = left >= size_t(kDeqChunkPieces) * kDeqChunkThreads
                             ? kDeqChunkPieces * kDeqChunkThreads * 16
                             : static_cast<uint32_t>(left * 16);
  const __amdgpu_buffer_rsrc_t dst = __builtin_amdgcn_make_buffer_rsrc(
      reinterpret_cast<f4*>(out) + base, 0, bytes, kRsrcFlags);
#pragma unroll
  for (int j = 0; j < kDeqChunkPieces; ++j) {
    f4 y;
    y.x = conv(w[j] & 0xffu);
    y.y = conv((w[j] >> 8) & 0xffu);
    y.z = conv((w[j] >> 16) & 0xffu);
    y.w = conv(w[j] >> 24);
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(i4, y), dst,
                                           (j * kDeqChunkThreads + threadIdx.x) * 16, 0,
                                           kStreamOut);
  }
  // the ragged tail (< 4 elements)
  if (blockIdx.x == 0) {
    const size_t i = (nquad << 2) + threadIdx.x;
    if (i < n) out[i] = conv(in[i]);
  }
}

template <bool UNSIGNED, bool VEC>
__global__ __launch_bounds__(kThreads) void dequantize_kernel(const uint8_t* __restrict__ in,
                                                              float* __restrict__ out, size_t n,
                                                              const float* __restrict__ imin,
                                                              const float* __restrict__ imax) {
  const float lo = *imin, hi = *imax;
  const float scale = UNSIGNED ? (hi - lo) / (255.0f - 0.0f) : maxabs(hi, lo) / 127.0f;
  auto conv = [&](uint32_t byte) -> float {
    if (UNSIGNED) {
      float p = static_cast<float>(byte) * scale;
      return p + lo;
    } else {
      return static_cast<float>(static_cast<int>(static_cast<int8_t>(byte))) * scale;
    }
  };
  auto conv4 = [&](uint32_t w) -> f4 {
    f4 y;
    y.x = conv(w & 0xffu);
    y.y = conv((w >> 8) & 0xffu);
    y.z = conv((w >> 16) & 0xffu);
    y.w = conv(w >> 24);
    return y;
  };
  const size_t stride = size_t(gridDim.x) * kThreads;
  if (VEC) {
    const size_t nquad = n >> 2;
    const uint32_t* in4 = reinterpret_cast<const uint32_t*>(in);
    f4* out4 = reinterpret_cast<f4*>(out);
    constexpr int kWaves = kThreads / 64, kPer = kDeqRunQuads / 64;
    const size_t runs = nquad / kDeqRunQuads;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    for (size_t r = size_t(blockIdx.x) * kWaves + wave; r < runs;
         r += size_t(gridDim.x) * kWaves) {
      const uint32_t* src = in4 + r * kDeqRunQuads;
      uint32_t w[kPer];
#pragma unroll
      for (int j = 0; j < kPer; ++j) w[j] = nt_load(src + j * 64 + lane);
      // one descriptor per run: the run's start is wave-uniform, the lane offset 32-bit
      const __amdgpu_buffer_rsrc_t dst = __builtin_amdgcn_make_buffer_rsrc(
          out4 + r * kDeqRunQuads, 0, kDeqRunQuads * 16, kRsrcFlags);
#pragma unroll
      for (int j = 0; j < kPer; ++j) {
        const f4 y = conv4(w[j]);
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(i4, y), dst,
                                               (j * 64 + lane) * 16, 0, kStreamOut);
      }
    }
    // what is left of the last, partial run, then the ragged tail (< 4 elements)
    for (size_t q = runs * kDeqRunQuads + size_t(blockIdx.x) * kThreads + threadIdx.x; q < nquad;
         q += stride)
      nt_store(conv4(nt_load(in4 + q)), out4 + q);
    if (blockIdx.x == 0) {
      size_t i = (nquad << 2) + threadIdx.x;
      if (i < n) out[i] = conv(in[i]);
    }
  } else {
    for (size_t i = size_t(blockIdx.x) * kThreads + threadIdx.x; i < n; i += stride)
      out[i] = conv(in[i]);
  }
}

// ---- single-pass min/max grid reduction -----------------------------------------
// Wave64 reduction: DPP within each row of 16 lanes, then two cross-row
// exchanges.  Afterwards every lane holds the wave's result.
template <typename T, typename Op>
__device__ __forceinline__ T wave_reduce(T v, Op op) {
  static_assert(sizeof(T) == 4, "32-bit payload");
  auto dpp = [](T x, auto ctrl) -> T {
    int xi = __builtin_bit_cast(int, x);
    int r = __builtin_amdgcn_update_dpp(xi, xi, decltype(ctrl)::value, 0xf, 0xf, false);
    return __builtin_bit_cast(T, r);
  };
  v = op(v, dpp(v, std::integral_constant<int, 0xB1>{}));   // quad_perm [1,0,3,2]
  v = op(v, dpp(v, std::integral_constant<int, 0x4E>{}));   // quad_perm [2,3,0,1]
  v = op(v, dpp(v, std::integral_constant<int, 0x141>{}));  // row_half_mirror
  v = op(v, dpp(v, std::integral_constant<int, 0x140>{}));  // row_mirror
  v = op(v, __shfl_xor(v, 16, 64));
  v = op(v, __shfl_xor(v, 32, 64));
  return v;
}

struct MinF {
  __device__ __forceinline__ float operator()(float a, float b) const { return fminf(a, b); }
};
struct MaxF {
  __device__ __forceinline__ float operator()(float a, float b) const { return fmaxf(a, b); }
};
struct MinI {
  __device__ __forceinline__ int operator()(int a, int b) const { return a < b ? a : b; }
};
struct MaxI {
  __device__ __forceinline__ int operator()(int a, int b) const { return a > b ? a : b; }
};
// Block-level fold; thread 0 returns the block's (mn, mx).
template <typename T, typename MinOp, typename MaxOp>
__device__ __forceinline__ void block_fold(T& mn, T& mx) {
  __shared__ T s_min[kThreads / 64], s_max[kThreads / 64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  mn = wave_reduce(mn, MinOp());
  mx = wave_reduce(mx, MaxOp());
  if (lane == 0) {
    s_min[wave] = mn;
    s_max[wave] = mx;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < kThreads / 64; ++w) {
      mn = MinOp()(mn, s_min[w]);
      mx = MaxOp()(mx, s_max[w]);
    }
  }
}

// fp32 min / max of the whole tensor in one pass; each block leaves one partial.
// NaN is detected through the largest |x| bit pattern (> 0x7f800000).
template <bool VEC>
__global__ __launch_bounds__(kThreads) void minmax_f32_kernel(const float* __restrict__ in,
                                                              size_t n, uint32_t* parts) {
  float mn = INFINITY, mx = -INFINITY;
  uint32_t amax = 0;
  auto fold = [&](float x) {
    mn = fminf(mn, x);
    mx = fmaxf(mx, x);
    uint32_t a = __builtin_bit_cast(uint32_t, x) & 0x7fffffffu;
    amax = a > amax ? a : amax;
  };
  const size_t stride = size_t(gridDim.x) * kThreads;
  if (VEC) {
    const size_t nquad = n >> 2;
    const f4* in4 = reinterpret_cast<const f4*>(in);
    size_t q = size_t(blockIdx.x) * kThreads + threadIdx.x;
    for (; q + size_t(kUnroll - 1) * stride < nquad; q += size_t(kUnroll) * stride) {
      f4 x[kUnroll];
#pragma unroll
      for (int j = 0; j < kUnroll; ++j) x[j] = nt_load(in4 + q + size_t(j) * stride);
#pragma unroll
      for (int j = 0; j < kUnroll; ++j) {
        fold(x[j].x);
        fold(x[j].y);
        fold(x[j].z);
        fold(x[j].w);
      }
    }
    for (; q < nquad; q += stride) {
      f4 x = nt_load(in4 + q);
      fold(x.x);
      fold(x.y);
      fold(x.z);
      fold(x.w);
    }
    if (blockIdx.x == 0) {
      size_t i = (nquad << 2) + threadIdx.x;
      if (i < n) fold(in[i]);
    }
  } else {
    for (size_t i = size_t(blockIdx.x) * kThreads + threadIdx.x; i < n; i += stride) fold(in[i]);
  }
  amax = wave_reduce(amax, MaxU());
  __shared__ uint32_t s_amax[kThreads / 64];
  if ((threadIdx.x & 63) == 0) s_amax[threadIdx.x >> 6] = amax;
  block_fold<float, MinF, MaxF>(mn, mx);  // contains the barrier that publishes s_amax
  if (threadIdx.x == 0) {
    for (int w = 1; w < kThreads / 64; ++w) amax = s_amax[w] > amax ? s_amax[w] : amax;
    uint32_t* part = parts + blockIdx.x * kPartWords;
    part[0] = f2ord(mn);
    part[1] = f2ord(mx);
    part[2] = amax > 0x7f800000u ? 1u : 0u;
  }
}

// int32 min / max of the whole tensor in one pass.
template <bool VEC>
__global__ __launch_bounds__(kThreads) void minmax_i32_kernel(const int32_t* __restrict__ in,
                                                              size_t n, uint32_t* parts) {
  int mn = INT32_MAX, mx = INT32_MIN;
  auto fold = [&](int x) {
    mn = x < mn ? x : mn;
    mx = x > mx ? x : mx;
  };
  const size_t stride = size_t(gridDim.x) * kThreads;
  if (VEC) {
    const size_t nquad = n >> 2;
    const i4* in4 = reinterpret_cast<const i4*>(in);
    size_t q = size_t(blockIdx.x) * kThreads + threadIdx.x;
    for (; q + size_t(kUnroll - 1) * stride < nquad; q += size_t(kUnroll) * stride) {
      i4 x[kUnroll];
#pragma unroll
      for (int j = 0; j < kUnroll; ++j) x[j] = nt_load(in4 + q + size_t(j) * stride);
#pragma unroll
      for (int j = 0; j < kUnroll; ++j) {
        fold(x[j].x);
        fold(x[j].y);
        fold(x[j].z);
        fold(x[j].w);
      }
    }
    for (; q < nquad; q += stride) {
      i4 x = nt_load(in4 + q);
      fold(x.x);
      fold(x.y);
      fold(x.z);
      fold(x.w);
    }
    if (blockIdx.x == 0) {
      size_t i = (nquad << 2) + threadIdx.x;
      if (i < n) fold(in[i]);
    }
  } else {
    for (size_t i = size_t(blockIdx.x) * kThreads + threadIdx.x; i < n; i += stride) fold(in[i]);
  }
  block_fold<int, MinI, MaxI>(mn, mx);
  if (threadIdx.x == 0) {
    // sign bit flipped: unsigned order == signed order
    uint32_t* part = parts + blockIdx.x * kPartWords;
    part[0] = static_cast<uint32_t>(mn) ^ 0x80000000u;
    part[1] = static_cast<uint32_t>(mx) ^ 0x80000000u;
    part[2] = 0u;
  }
}

// int8 relu on packed bytes: 16 values per lane per segment.
__global__ __launch_bounds__(kThreads) void relu_i8_kernel(const int8_t* __restrict__ in,
                                                           int8_t* __restrict__ out, size_t n,
                                                           const float* __restrict__ imin,
                                                           const float* __restrict__ imax,
                                                           float* __restrict__ omin,
                                                           float* __restrict__ omax, bool vec) {
  const size_t stride = size_t(gridDim.x) * kThreads;
  const size_t t0 = size_t(blockIdx.x) * kThreads + threadIdx.x;
  auto relu4 = [](uint32_t w) -> uint32_t {
    // a byte is negative iff its top bit is set: build a per-byte keep mask
    uint32_t neg = (w >> 7) & 0x01010101u;
    uint32_t mask = (neg * 0xffu) ^ 0xffffffffu;
    return w & mask;
  };
  if (vec) {
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    const size_t n16 = n >> 4;
    const u4* in16 = reinterpret_cast<const u4*>(in);
    u4* out16 = reinterpret_cast<u4*>(out);
    // four 16-byte pieces a grid stride apart in flight per lane
    size_t q = t0;
    for (; q + 3 * stride < n16; q += 4 * stride) {
      u4 w[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) w[j] = nt_load(in16 + q + j * stride);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        u4 r = {relu4(w[j].x), relu4(w[j].y), relu4(w[j].z), relu4(w[j].w)};
        nt_store(r, out16 + q + j * stride);
      }
    }
    for (; q < n16; q += stride) {
      u4 w = nt_load(in16 + q);
      u4 r = {relu4(w.x), relu4(w.y), relu4(w.z), relu4(w.w)};
      nt_store(r, out16 + q);
    }
    for (size_t i = (n16 << 4) + t0; i < n; i += stride) out[i] = in[i] > 0 ? in[i] : 0;
  } else {
    for (size_t i = t0; i < n; i += stride) out[i] = in[i] > 0 ? in[i] : 0;
  }
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    *omin = *imin;
    *omax = *imax;
  }
}

// The relu of large tensors: one contiguous 32 KiB chunk per work-group, no loop; every lane
// requests its eight 16-byte pieces (4 KiB apart), then clamps and stores them.  64 M
// elements: 23.2 -> 21.6 us against the grid-stride kernel (two builds, one box); 16 or 64 KiB
// chunks and 64 ... 1024 lanes stay at 22.6-25.9 us.  At 51 M elements the gain is 3 % alone
// and nothing inside the chained ResNet-50 body, below that the grid-stride kernel with its
// size-dependent grid is level or ahead: taken from 64 M elements on.
constexpr int kReluChunkPieces = 8;
constexpr size_t kReluChunkMinElements = size_t(1) << 26;

__global__ __launch_bounds__(kThreads) void relu_chunk_kernel(const int8_t* __restrict__ in,
                                                              int8_t* __restrict__ out, size_t n,
                                                              const float* __restrict__ imin,
                                                              const float* __restrict__ imax,
                                                              float* __restrict__ omin,
                                                              float* __restrict__ omax) {
  typedef uint32_t u4 __attribute__((ext_vector_type(4)));
  auto relu4 = [](uint32_t w) -> uint32_t {
    uint32_t neg = (w >> 7) & 0x01010101u;
    return w & ((neg * 0xffu) ^ 0xffffffffu);
  };
  const size_t n16 = n >> 4;
  const size_t base = size_t(blockIdx.x) * (kReluChunkPieces * kThreads);
  const u4* in16 = reinterpret_cast<const u4*>(in);
  u4* out16 = reinterpret_cast<u4*>(out);
  u4 w[kReluChunkPieces];
#pragma unroll
  for (int j = 0; j < kReluChunkPieces; ++j) {
    const size_t q = base + size_t(j) * kThreads + threadIdx.x;
    w[j] = q < n16 ? nt_load(in16 + q) : u4{0, 0, 0, 0};
  }
#pragma unroll
  for (int j = 0; j < kReluChunkPieces; ++j) {
    const size_t q = base + size_t(j) * kThreads + threadIdx.x;
    const u4 r = {relu4(w[j].x), relu4(w[j].y), relu4(w[j].z), relu4(w[j].w)};
    if (q < n16) nt_store(r, out16 + q);
  }
  if (blockIdx.x == 0) {
    const size_t i = (n16 << 4) + threadIdx.x;
    if (i < n) out[i] = in[i] > 0 ? in[i] : 0;
    if (threadIdx.x == 0) {
      *omin = *imin;
      *omax = *imax;
    }
  }
}

__global__ void passthrough_range_kernel(float* omin, float* omax, float lo, float hi) {
  *omin = lo;
  *omax = hi;
}

// Work-groups for `work_items` lane items.  Large tensors stream best with few resident
// waves (kCastBlocksPerCu); tensors of a few MB (the activations of one layer: their time is
// launch ramp and latency, not bandwidth) finish sooner with more of them.  Measured on
// [4096,768] / [4096,2304] / [4096,3072] fp32 -> int8: 4.8 / 9.9 / 11.7 us at 2 per CU
// against 3.9 / 9.1 / 11.5 with the caps below; dequantize 9.2 -> 8.3 and 11.1 -> 10.6 us.
int stream_grid(size_t work_items, size_t elements = 0, bool widening = false) {
  size_t want = (work_items + kThreads - 1) / kThreads;
  int per_cu = kCastBlocksPerCu;
  if (elements != 0 && elements <= (size_t(4) << 20))
    per_cu = 8;
  else if (elements != 0 && elements <= (size_t(16) << 20))
    per_cu = widening ? 12 : 3;
  size_t cap = size_t(num_cus()) * size_t(per_cu);
  if (want < 1) want = 1;
  return static_cast<int>(want < cap ? want : cap);
}

int reduce_grid(size_t n) {
  const int g = stream_grid((n + 3) / 4);
  return g < kMaxParts ? g : kMaxParts;
}

// Address of `scratch` on the calling thread's current device; looked up once per device.
uint32_t* noalloc_scratch() {
  int dev = 0;
  MXQ_HIP(hipGetDevice(&dev));
  MXQ_CHECK(dev >= 0 && dev < kMaxDevices, "device index " << dev << " out of range");
  uint32_t* p = g_noalloc_ptr[dev].load(std::memory_order_acquire);
  if (p == nullptr) {
    void* addr = nullptr;
    MXQ_HIP(hipGetSymbolAddress(&addr, HIP_SYMBOL(scratch)));
    MXQ_CHECK(addr != nullptr, "no device address for the scratch array");
    p = static_cast<uint32_t*>(addr);
    g_noalloc_ptr[dev].store(p, std::memory_order_release);
  }
  return p;
}

uint32_t* carve(void* workspace, size_t bytes) {
  MXQ_CHECK(workspace != nullptr, "the uncalibrated path needs a workspace");
  MXQ_CHECK(bytes >= kWsBytes, "workspace too small: " << bytes << " < " << kWsBytes);
  MXQ_CHECK(aligned16(workspace), "workspace must be 16-byte aligned");
  return static_cast<uint32_t*>(workspace);
}

void launch_quantize(hipStream_t s, const float* in, void* out, float* omin, float* omax,
                     size_t n, int out_type, float lo, float hi, const float* dlo,
                     const float* dhi, const uint32_t* parts, int nparts) {
  const bool vec = aligned16(in) && ((reinterpret_cast<uintptr_t>(out) & 3u) == 0);
  const int grid = stream_grid(vec ? (n + 3) / 4 : n, n);
  uint8_t* o = static_cast<uint8_t*>(out);
#define MXQ_Q(U, V) \
  hipLaunchKernelGGL((quantize_kernel<U, V>), dim3(grid), dim3(kThreads), 0, s, in, o, omin, \
                     omax, n, lo, hi, dlo, dhi, parts, nparts,                           \
                     parts != nullptr ? 1 : 0)
  if (out_type == MXQ_UINT8) {
    if (vec) MXQ_Q(true, true); else MXQ_Q(true, false);
  } else {
    if (vec) MXQ_Q(false, true); else MXQ_Q(false, false);
  }
#undef MXQ_Q
  MXQ_LAUNCH_CHECK();
}

}  // namespace
}  // namespace mxq

using namespace mxq;

extern "C" {

size_t mxq_quantize_v2_workspace(size_t) { return kWsBytes; }
size_t mxq_requantize_workspace(size_t) { return kWsBytes; }

int mxq_quantize_v2(void* stream, const float* in, void* out, float* omin, float* omax,
                    size_t n, int out_type, int calibrated, float min_calib, float max_calib,
                    void* workspace, size_t workspace_bytes) {
  MXQ_API_BEGIN();
  MXQ_CHECK(out_type == MXQ_INT8 || out_type == MXQ_UINT8,
            "quantize op only supports int8 and uint8 as output type, got " << out_type);
  MXQ_CHECK(omin != nullptr && omax != nullptr, "null range output");
  MXQ_CHECK(n == 0 || (in != nullptr && out != nullptr), "null data pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (calibrated) {
    if (n == 0) {
      // Kernel<gpu>::Launch is a no-op for N == 0 (mxnet_op.h:1179): ranges untouched
      return 0;
    }
    launch_quantize(s, in, out, omin, omax, n, out_type, min_calib, max_calib, nullptr, nullptr,
                    nullptr, 0);
  } else {
    if (n == 0) return 0;
    uint32_t* parts = carve(workspace, workspace_bytes);
    const int grid = reduce_grid(n);
    if (aligned16(in))
      hipLaunchKernelGGL((minmax_f32_kernel<true>), dim3(grid), dim3(kThreads), 0, s, in, n,
                         parts);
    else
      hipLaunchKernelGGL((minmax_f32_kernel<false>), dim3(grid), dim3(kThreads), 0, s, in, n,
                         parts);
    MXQ_LAUNCH_CHECK();
    launch_quantize(s, in, out, omin, omax, n, out_type, 0.f, 0.f, nullptr, nullptr, parts,
                    grid);
  }
  MXQ_API_END();
}

int mxq_quantize_v2_noalloc(void* stream, const float* in, void* out, float* omin, float* omax,
                            size_t n, int out_type, int calibrated, float min_calib,
                            float max_calib) {
  MXQ_API_BEGIN();
  MXQ_CHECK(n <= kNoAllocMaxElements,
            "mxq_quantize_v2_noalloc takes at most " << kNoAllocMaxElements << " elements, got "
                                                     << n);
  uint32_t* parts = calibrated ? nullptr : noalloc_scratch();
  const int rc = mxq_quantize_v2(stream, in, out, omin, omax, n, out_type, calibrated, min_calib,
                                 max_calib, parts, parts != nullptr ? kWsBytes : 0);
  if (rc != 0) return rc;
  MXQ_API_END();
}

int mxq_quantize(void* stream, const float* in, const float* imin, const float* imax, void* out,
                 float* omin, float* omax, size_t n, int out_type) {
  MXQ_API_BEGIN();
  MXQ_CHECK(out_type == MXQ_INT8 || out_type == MXQ_UINT8,
            "quantize op only supports int8 and uint8 as output type, got " << out_type);
  MXQ_CHECK(imin != nullptr && imax != nullptr && omin != nullptr && omax != nullptr,
            "null range pointer");
  MXQ_CHECK(n == 0 || (in != nullptr && out != nullptr), "null data pointer");
  if (n == 0) return 0;
  launch_quantize(static_cast<hipStream_t>(stream), in, out, omin, omax, n, out_type, 0.f, 0.f,
                  imin, imax, nullptr, 0);
  MXQ_API_END();
}

size_t mxq_quantize_asym_workspace(size_t) { return kWsBytes; }

int mxq_quantize_asym(void* stream, const void* in, int in_type, uint8_t* out, float* oscale,
                      float* oshift, size_t n, int calibrated, float min_calib, float max_calib,
                      void* workspace, size_t workspace_bytes) {
  MXQ_API_BEGIN();
  MXQ_CHECK(in_type == MXQ_FLOAT32 || in_type == MXQ_INT8 || in_type == MXQ_UINT8,
            "Asymmetric quantizaiton only supports int8, uint8 and float inputs, got "
                << in_type);
  MXQ_CHECK(oscale != nullptr && oshift != nullptr, "null scale / shift output");
  MXQ_CHECK(n == 0 || (in != nullptr && out != nullptr), "null data pointer");
  if (n == 0) return 0;  // Kernel<gpu>::Launch is a no-op for N == 0
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (in_type != MXQ_FLOAT32) {
    const int vec = (aligned16(in) && aligned16(out)) ? 1 : 0;
    const int grid = stream_grid(vec ? (n + 15) / 16 : n);
    const uint8_t* i8 = static_cast<const uint8_t*>(in);
    if (in_type == MXQ_INT8)
      hipLaunchKernelGGL((asym_bytes_kernel<true>), dim3(grid), dim3(kThreads), 0, s, i8, out,
                         oscale, oshift, n, vec);
    else
      hipLaunchKernelGGL((asym_bytes_kernel<false>), dim3(grid), dim3(kThreads), 0, s, i8, out,
                         oscale, oshift, n, vec);
    MXQ_LAUNCH_CHECK();
    return 0;
  }
  const float* f = static_cast<const float*>(in);
  const uint32_t* parts = nullptr;
  int nparts = 0;
  if (!calibrated) {
    uint32_t* ws = carve(workspace, workspace_bytes);
    nparts = reduce_grid(n);
    if (aligned16(in))
      hipLaunchKernelGGL((minmax_f32_kernel<true>), dim3(nparts), dim3(kThreads), 0, s, f, n, ws);
    else
      hipLaunchKernelGGL((minmax_f32_kernel<false>), dim3(nparts), dim3(kThreads), 0, s, f, n, ws);
    MXQ_LAUNCH_CHECK();
    parts = ws;
  }
  const bool vec = aligned16(in) && ((reinterpret_cast<uintptr_t>(out) & 3u) == 0);
  const int grid = stream_grid(vec ? (n + 3) / 4 : n);
  if (vec)
    hipLaunchKernelGGL((quantize_asym_kernel<true>), dim3(grid), dim3(kThreads), 0, s, f, out,
                       oscale, oshift, n, min_calib, max_calib, parts, nparts,
                       parts != nullptr ? 1 : 0);
  else
    hipLaunchKernelGGL((quantize_asym_kernel<false>), dim3(grid), dim3(kThreads), 0, s, f, out,
                       oscale, oshift, n, min_calib, max_calib, parts, nparts,
                       parts != nullptr ? 1 : 0);
  MXQ_LAUNCH_CHECK();
  MXQ_API_END();
}

int mxq_quantize_v2_passthrough(void* stream, const void* in, void* out, float* omin,
                                float* omax, size_t n, int in_type, int calibrated,
                                float min_calib, float max_calib) {
  MXQ_API_BEGIN();
  MXQ_CHECK(in_type == MXQ_INT8 || in_type == MXQ_UINT8, "pass-through needs int8/uint8 input");
  MXQ_CHECK(omin != nullptr && omax != nullptr, "null range output");
  MXQ_CHECK(n == 0 || (in != nullptr && out != nullptr), "null data pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  float lo, hi;
  if (calibrated) {
    lo = min_calib;
    hi = max_calib;
  } else if (in_type == MXQ_UINT8) {
    lo = 0.f;
    hi = 255.f;
  } else {
    lo = -127.f;
    hi = 127.f;
  }
  hipLaunchKernelGGL(passthrough_range_kernel, dim3(1), dim3(1), 0, s, omin, omax, lo, hi);
  MXQ_LAUNCH_CHECK();
  if (n != 0 && in != out) MXQ_HIP(hipMemcpyAsync(out, in, n, hipMemcpyDeviceToDevice, s));
  MXQ_API_END();
}

int mxq_requantize(void* stream, const int32_t* in, const float* imin, const float* imax,
                   int8_t* out, float* omin, float* omax, size_t n, int calibrated,
                   float min_calib, float max_calib, void* workspace, size_t workspace_bytes) {
  MXQ_API_BEGIN();
  MXQ_CHECK(imin != nullptr && imax != nullptr && omin != nullptr && omax != nullptr,
            "null range pointer");
  MXQ_CHECK(n == 0 || (in != nullptr && out != nullptr), "null data pointer");
  if (n == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool vec = aligned16(in) && ((reinterpret_cast<uintptr_t>(out) & 3u) == 0);
  const int grid = stream_grid(vec ? (n + 3) / 4 : n, n);
  uint8_t* o = reinterpret_cast<uint8_t*>(out);
  float real_range = 0.f;
  const uint32_t* parts = nullptr;
  int nparts = 0;
  if (calibrated) {
    float a = fabsf(min_calib), b = fabsf(max_calib);
    real_range = (a < b) ? b : a;
  } else {
    uint32_t* ws = carve(workspace, workspace_bytes);
    nparts = reduce_grid(n);
    if (aligned16(in))
      hipLaunchKernelGGL((minmax_i32_kernel<true>), dim3(nparts), dim3(kThreads), 0, s, in, n,
                         ws);
    else
      hipLaunchKernelGGL((minmax_i32_kernel<false>), dim3(nparts), dim3(kThreads), 0, s, in, n,
                         ws);
    MXQ_LAUNCH_CHECK();
    parts = ws;
  }
  if (vec)
    hipLaunchKernelGGL((requantize_kernel<true>), dim3(grid), dim3(kThreads), 0, s, in, o, omin,
                       omax, n, imin, imax, real_range, parts, nparts,
                       parts != nullptr ? 1 : 0);
  else
    hipLaunchKernelGGL((requantize_kernel<false>), dim3(grid), dim3(kThreads), 0, s, in, o,
                       omin, omax, n, imin, imax, real_range, parts, nparts,
                       parts != nullptr ? 1 : 0);
  MXQ_LAUNCH_CHECK();
  MXQ_API_END();
}

int mxq_quantized_relu(void* stream, const int8_t* in, const float* imin, const float* imax,
                       int8_t* out, float* omin, float* omax, size_t n) {
  MXQ_API_BEGIN();
  MXQ_CHECK(imin != nullptr && imax != nullptr && omin != nullptr && omax != nullptr,
            "null range pointer");
  MXQ_CHECK(n == 0 || (in != nullptr && out != nullptr), "null data pointer");
  const bool vec = aligned16(in) && aligned16(out);
  if (vec && n >= kReluChunkMinElements) {
    const size_t per = size_t(kReluChunkPieces) * kThreads;
    const size_t chunks = ((n >> 4) + per - 1) / per;
    MXQ_CHECK(chunks < (size_t(1) << 31), "tensor too large for one launch");
    hipLaunchKernelGGL(relu_chunk_kernel, dim3(static_cast<unsigned>(chunks)), dim3(kThreads), 0,
                       static_cast<hipStream_t>(stream), in, out, n, imin, imax, omin, omax);
    MXQ_LAUNCH_CHECK();
    return 0;
  }
  const int grid = stream_grid(n == 0 ? 1 : (vec ? (n + 15) / 16 : n), n);
  hipLaunchKernelGGL(relu_i8_kernel, dim3(grid), dim3(kThreads), 0,
                     static_cast<hipStream_t>(stream), in, out, n, imin, imax, omin, omax, vec);
  MXQ_LAUNCH_CHECK();
  MXQ_API_END();
}

int mxq_dequantize(void* stream, const void* in, int in_type, const float* imin,
                   const float* imax, float* out, size_t n) {
  MXQ_API_BEGIN();
  MXQ_CHECK(in_type == MXQ_INT8 || in_type == MXQ_UINT8,
            "dequantize op only supports input type int8 or uint8, got " << in_type);
  MXQ_CHECK(imin != nullptr && imax != nullptr, "null range pointer");
  MXQ_CHECK(n == 0 || (in != nullptr && out != nullptr), "null data pointer");
  if (n == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool vec = aligned16(out) && ((reinterpret_cast<uintptr_t>(in) & 3u) == 0);
  const int grid = stream_grid(vec ? (n + 3) / 4 : n, n, true);
  const uint8_t* i8 = static_cast<const uint8_t*>(in);
  if (vec && n >= kDeqChunkMinElements) {
    const size_t per = size_t(kDeqChunkPieces) * kDeqChunkThreads;
    const size_t chunks = ((n >> 2) + per - 1) / per;
    MXQ_CHECK(chunks < (size_t(1) << 31), "tensor too large for one launch");
    if (in_type == MXQ_UINT8)
      hipLaunchKernelGGL(dequantize_chunk_kernel<true>, dim3(static_cast<unsigned>(chunks)),
                         dim3(kDeqChunkThreads), 0, s, i8, out, n, imin, imax);
    else
      hipLaunchKernelGGL(dequantize_chunk_kernel<false>, dim3(static_cast<unsigned>(chunks)),
                         dim3(kDeqChunkThreads), 0, s, i8, out, n, imin, imax);
    MXQ_LAUNCH_CHECK();
    return 0;
  }
#define MXQ_D(U, V) \
  hipLaunchKernelGGL((dequantize_kernel<U, V>), dim3(grid), dim3(kThreads), 0, s, i8, out, n, \
                     imin, imax)
  if (in_type == MXQ_UINT8) {
    if (vec) MXQ_D(true, true); else MXQ_D(true, false);
  } else {
    if (vec) MXQ_D(false, true); else MXQ_D(false, false);
  }
#undef MXQ_D
  MXQ_LAUNCH_CHECK();
  MXQ_API_END();
}

}  // extern "C"
