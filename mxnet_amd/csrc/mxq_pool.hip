// Quantized pooling and flatten for gfx950: the operators that sit between the
// quantized convolutions and the quantized fully-connected layer of a CNN.
//   _contrib_quantized_pooling  src/operator/quantization/quantized_pooling.cu:33-128
//   _contrib_quantized_flatten  src/operator/quantization/quantized_flatten-inl.h:39-110
//
// Pooling is byte work bound by HBM: a work-group copies the contiguous run of input
// rows its outputs need (one band of a large plane, or several whole small planes)
// into LDS with 16-byte loads, then every thread folds its windows out of LDS.  The
// input is read from memory once even where windows overlap (3x3 / stride 2).
#include <hip/hip_runtime.h>

#include <cstdint>

#include "../../include/mxq.h"
#include "mxq_common.h"
#include "mxq_gemm.h"

namespace mxq {
namespace {

constexpr int kPoolThreads = 256;
constexpr int kPoolLdsBytes = 16384;  // input bytes staged per work-group (measured: 8 KiB and 32 KiB are both slower)

struct PoolArgs {
  const uint8_t* in;
  uint8_t* out;
  size_t total_in;  // bytes of the whole input tensor
  int planes, H, W, OH, OW, KH, KW, sh, sw, ph, pw;
  int is_avg, count_pad, is_unsigned;
  int ppb;    // planes per work-group (> 1 only when band == OH)
  int band;   // output rows per work-group
  int bands;  // bands per plane
  int vec_ok; // the tensor base is 16-byte aligned
  // floor(n / d) = umulhi(n, magic) for n * d < 2^32 (magic = 2^32 / d + 1; 0 stands for d = 1)
  const float* imin;  // the range passes through: written by the first thread of the grid
  const float* imax;
  float* omin;
  float* omax;
  uint32_t magic_per_row;    // d = items per output row
  uint32_t magic_per_plane;  // d = items per plane, used when ppb > 1
};

__device__ __forceinline__ int fast_div(int n, uint32_t magic) {
  return magic == 0 ? n : static_cast<int>(__umulhi(static_cast<uint32_t>(n), magic));
}

// One window out of a byte image (LDS or global): rows of `W` bytes starting at
// `img`, whose first row is image row `row0`.
template <bool UNSIGNED, typename Ptr>
__device__ __forceinline__ int pool_window(Ptr img, int row0, const PoolArgs& a, int oh, int ow) {
  int hstart = oh * a.sh - a.ph, wstart = ow * a.sw - a.pw;
  int hend = min(hstart + a.KH, a.H + a.ph), wend = min(wstart + a.KW, a.W + a.pw);
  int pool_size = (hend - hstart) * (wend - wstart);
  hstart = max(hstart, 0);
  wstart = max(wstart, 0);
  hend = min(hend, a.H);
  wend = min(wend, a.W);
  if (!a.count_pad) pool_size = (hend - hstart) * (wend - wstart);
  constexpr int lo = UNSIGNED ? 0 : -128, hi = UNSIGNED ? 255 : 127;
  int acc = a.is_avg ? 0 : lo;
  for (int h = hstart; h < hend; ++h) {
    const int base = (h - row0) * a.W;
    for (int w = wstart; w < wend; ++w) {
      const uint8_t b = img[base + w];
      const int v = UNSIGNED ? static_cast<int>(b) : static_cast<int>(static_cast<int8_t>(b));
      acc = a.is_avg ? acc + v : max(acc, v);
    }
  }
  if (!a.is_avg) return acc;
  // nearest, ties to even, of sum / divisor (exact: the binary32 quotient is exact on
  // ties and cannot round onto one)
  const float avg = pool_size > 0 ? static_cast<float>(acc) / static_cast<float>(pool_size) : 0.f;
  int q = static_cast<int>(rintf(avg));
  return min(max(q, lo), hi);
}

constexpr int kPoolItem = 8;  // horizontally adjacent outputs one thread computes at a time

// kPoolItem adjacent outputs of one row for a compile-time K x K window and horizontal
// stride.  Per window row the (kPoolItem-1)*SW + K wide strip is read from LDS as aligned
// dwords (indexing the shared array directly, so the reads stay LDS reads), realigned with
// the byte funnel shift and folded into the outputs that cover each byte.  Nothing branches
// on position: columns outside the image are replaced through a byte mask, rows outside it
// read a clamped row and are masked as a whole (the staged bytes have 16 bytes of slack in
// front and 64 behind), so border items cost what interior items cost.
// `base` is the byte offset, inside the shared array, of row `row0` of the item's plane.
template <bool UNSIGNED, bool AVG, int K, int SW>
__device__ __forceinline__ void pool_strip(const uint8_t* lds, int base, int row0, int row1,
                                           const PoolArgs& a, int oh, int ow0,
                                           int (&q)[kPoolItem]) {
  constexpr int lo = UNSIGNED ? 0 : -128, hi = UNSIGNED ? 255 : 127;
  constexpr int SPAN = (kPoolItem - 1) * SW + K;
  constexpr int NW = (SPAN + 3 + 3) / 4;  // aligned dwords covering the strip at any offset
  constexpr int neutral = AVG ? 0 : lo;
  constexpr uint32_t fill = (static_cast<uint32_t>(neutral) & 0xffu) * 0x01010101u;
  const uint32_t* words = reinterpret_cast<const uint32_t*>(lds);
  const int h0 = oh * a.sh - a.ph;
  const int w0 = ow0 * SW - a.pw;
  uint32_t keep[NW];
#pragma unroll
  for (int w = 0; w < NW; ++w) keep[w] = 0u;
#pragma unroll
  for (int j = 0; j < SPAN; ++j)
    if (static_cast<unsigned>(w0 + j) < static_cast<unsigned>(a.W))
      keep[j / 4] |= 0xffu << (8 * (j % 4));
  int acc[kPoolItem];
#pragma unroll
  for (int i = 0; i < kPoolItem; ++i) acc[i] = neutral;
  int rows_inside = 0;
#pragma unroll
  for (int r = 0; r < K; ++r) {
    const int h = h0 + r;
    const bool inside = static_cast<unsigned>(h) < static_cast<unsigned>(a.H);
    rows_inside += inside;
    const int hh = min(max(h, row0), row1 - 1);  // a staged row, whatever h is
    const int off = base + (hh - row0) * a.W + w0;
    const int wi = off >> 2;
    const uint32_t sft = static_cast<uint32_t>(off & 3);
    uint32_t d[NW + 1];
#pragma unroll
    for (int w = 0; w < NW; ++w) d[w] = words[wi + w];
    d[NW] = 0u;
    uint32_t x[NW];
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      const uint32_t k = inside ? keep[w] : 0u;
      x[w] = (__builtin_amdgcn_alignbyte(d[w + 1], d[w], sft) & k) | (fill & ~k);
    }
    int v[SPAN];
#pragma unroll
    for (int j = 0; j < SPAN; ++j) {
      const uint32_t byte = (x[j / 4] >> (8 * (j % 4))) & 0xffu;
      v[j] = UNSIGNED ? static_cast<int>(byte) : static_cast<int>(static_cast<int8_t>(byte));
    }
#pragma unroll
    for (int i = 0; i < kPoolItem; ++i)
#pragma unroll
      for (int k = 0; k < K; ++k)
        acc[i] = AVG ? acc[i] + v[i * SW + k] : max(acc[i], v[i * SW + k]);
  }
  if (!AVG) {
#pragma unroll
    for (int i = 0; i < kPoolItem; ++i) q[i] = acc[i];
    return;
  }
  const int padded_rows = min(h0 + K, a.H + a.ph) - h0;
#pragma unroll
  for (int i = 0; i < kPoolItem; ++i) {
    const int wstart = w0 + i * SW;
    const int wend = min(wstart + K, a.W + a.pw);
    const int pool_size = a.count_pad ? padded_rows * (wend - wstart)
                                      : rows_inside * (min(wend, a.W) - max(wstart, 0));
    const float avg =
        pool_size > 0 ? static_cast<float>(acc[i]) / static_cast<float>(pool_size) : 0.f;
    q[i] = min(max(static_cast<int>(rintf(avg)), lo), hi);
  }
}

// Max over K x K windows at horizontal stride 2 without touching single bytes: the strip's
// dwords are split into their even and odd bytes as two 16-bit lanes each (two ANDs), and
// rows, then neighbouring columns, are folded with the packed 16-bit max.  Signed bytes are
// first biased by 0x80 so that unsigned order is their order (0 is then the lowest value,
// which is also what masked-out positions become).  Per eight outputs: 4 instructions per
// strip dword and window row, 4 per dword to fold the rows, 4 per output pair to fold the
// columns, 2 to pack; the byte-at-a-time form above needs about twice as many.
typedef unsigned short us2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pk_max_u16(uint32_t x, uint32_t y) {
  return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(us2, x),
                                                                __builtin_bit_cast(us2, y)));
}

template <bool UNSIGNED, int K>
__device__ __forceinline__ void pool_strip_max2(const uint8_t* lds, int base, int row0, int row1,
                                                const PoolArgs& a, int oh, int ow0,
                                                uint32_t (&packed)[kPoolItem / 4]) {
  static_assert(K == 2 || K == 3, "window");
  constexpr int SPAN = (kPoolItem - 1) * 2 + K;
  constexpr int NW = (SPAN + 3 + 3) / 4;
  constexpr uint32_t bias = UNSIGNED ? 0u : 0x80808080u;
  const uint32_t* words = reinterpret_cast<const uint32_t*>(lds);
  const int h0 = oh * a.sh - a.ph;
  const int w0 = ow0 * 2 - a.pw;
  // Columns outside the image are masked to 0, the lowest biased value: one bit per strip
  // byte, then each dword's four bits spread to byte masks (bit k of the nibble times
  // 0x00204081 lands on bit 8k without carries).
  const int first = max(-w0, 0), last = max(min(a.W - w0, SPAN), first);
  const uint32_t valid = __builtin_amdgcn_ubfe(0xffffffffu, 0, last - first) << first;
  uint32_t keep_even[NW], keep_odd[NW];
#pragma unroll
  for (int w = 0; w < NW; ++w) {
    // (24-bit multiplies run at full rate: every operand here stays below 2^24)
    const uint32_t bits = __umul24((valid >> (4 * w)) & 0xfu, 0x00204081u);
    keep_even[w] = __umul24(bits & 0x00010001u, 0xffu);
    keep_odd[w] = __umul24((bits >> 8) & 0x00010001u, 0xff00u);
  }
  uint32_t even[NW], odd[NW];  // bytes 0,2 in the low byte / bytes 1,3 in the high byte of a lane
#pragma unroll
  for (int w = 0; w < NW; ++w) even[w] = odd[w] = 0u;
  // Rows outside the image are replaced by the nearest staged row: that row belongs to the
  // same window whenever the window meets the image at all, and a repeated row leaves a
  // maximum unchanged.  A window that lies outside altogether is dealt with at the end.
#pragma unroll
  for (int r = 0; r < K; ++r) {
    const int hh = min(max(h0 + r, row0), row1 - 1);
    const int off = base + __mul24(hh - row0, a.W) + w0;  // staged: < 2^24
    const int wi = off >> 2;
    const uint32_t sft = static_cast<uint32_t>(off & 3);
    uint32_t d[NW + 1];
#pragma unroll
    for (int w = 0; w < NW; ++w) d[w] = words[wi + w];
    d[NW] = 0u;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      const uint32_t x = __builtin_amdgcn_alignbyte(d[w + 1], d[w], sft) ^ bias;
      even[w] = pk_max_u16(even[w], x & keep_even[w]);
      odd[w] = pk_max_u16(odd[w], x & keep_odd[w]);
    }
  }
  // lanes of `even`: bytes 4w, 4w+2; of `odd` (after the shift): bytes 4w+1, 4w+3.
  // outputs 2w, 2w+1 = max(b[4w], b[4w+1], b[4w+2]), max(b[4w+2], b[4w+3], b[4w+4])
  uint32_t res[kPoolItem / 2];
#pragma unroll
  for (int w = 0; w < kPoolItem / 2; ++w) {
    res[w] = pk_max_u16(even[w], odd[w] >> 8);
    if (K == 3)
      res[w] = pk_max_u16(res[w], __builtin_amdgcn_alignbit(even[w + 1], even[w], 16));
  }
  const bool meets_image = h0 < a.H && h0 + K > 0;
#pragma unroll
  for (int w = 0; w < kPoolItem / 4; ++w)
    packed[w] = meets_image ? (__builtin_amdgcn_perm(res[2 * w + 1], res[2 * w], 0x06040200u) ^ bias)
                            : bias;
}

// Sum of the n bytes at LDS byte address `addr`: aligned dwords through the 4-way
// byte dot product against 0x01010101, the partial first and last dwords masked.
template <bool UNSIGNED>
__device__ __forceinline__ int sum_bytes(const uint8_t* lds, int addr, int n) {
  const uint32_t* words = reinterpret_cast<const uint32_t*>(lds);
  const int lo = addr, hi = addr + n;
  const int w0 = lo >> 2, w1 = (hi + 3) >> 2;  // the words [w0, w1) hold the bytes
  if (w0 >= w1) return 0;
  auto dot = [](uint32_t x, int sum) {
    if (UNSIGNED)
      return static_cast<int>(
          __builtin_amdgcn_udot4(x, 0x01010101u, static_cast<uint32_t>(sum), false));
    return __builtin_amdgcn_sdot4(static_cast<int>(x), 0x01010101, sum, false);
  };
  // only the first and the last word are partial: masks there, bare dot products between
  const int tail = hi - 4 * (w1 - 1);  // 1..4 bytes of the last word
  const uint32_t tail_mask = tail >= 4 ? 0xffffffffu : ((1u << (8 * tail)) - 1u);
  uint32_t first = words[w0] & ~((1u << (8 * (lo & 3))) - 1u);
  if (w1 - w0 == 1) first &= tail_mask;
  int sum = dot(first, 0);
  for (int w = w0 + 1; w < w1 - 1; ++w) sum = dot(words[w], sum);
  if (w1 - w0 > 1) sum = dot(words[w1 - 1] & tail_mask, sum);
  return sum;
}

// FAST: 0 generic windows; 1 quads with a 3x3 window, horizontal stride 2; 2 quads 2x2 /
// 2; 3 quads 3x3 / 1; 4 average over full-width windows (global pooling): contiguous sums.
template <bool UNSIGNED, bool AVG, int FAST>
__global__ __launch_bounds__(kPoolThreads) void pool_lds_kernel(PoolArgs a) {
  // the staged bytes start 16 bytes into the array: strips that begin left of column 0
  // read (and discard) what lies in front
  __shared__ __attribute__((aligned(16))) uint8_t lds_raw[kPoolLdsBytes + 96];
  uint8_t* lds = lds_raw + 16;
  const int tid = threadIdx.x;
  if (blockIdx.x == 0 && tid == 0) {
    *a.omin = *a.imin;
    *a.omax = *a.imax;
  }
  int p0, np, oh0, oh1;
  if (a.ppb > 1) {
    p0 = blockIdx.x * a.ppb;
    np = min(a.ppb, a.planes - p0);
    oh0 = 0;
    oh1 = a.OH;
  } else {
    p0 = blockIdx.x / a.bands;
    np = 1;
    oh0 = (blockIdx.x % a.bands) * a.band;
    oh1 = min(oh0 + a.band, a.OH);
  }
  const size_t plane_bytes = static_cast<size_t>(a.H) * a.W;
  int hs = 0, he = a.H;
  if (a.ppb <= 1) {
    hs = min(max(oh0 * a.sh - a.ph, 0), a.H);
    he = max(min((oh1 - 1) * a.sh - a.ph + a.KH, a.H), hs);
  }
  const size_t g0 = static_cast<size_t>(p0) * plane_bytes + static_cast<size_t>(hs) * a.W;
  const size_t len = static_cast<size_t>(np - 1) * plane_bytes + static_cast<size_t>(he - hs) * a.W;
  int shift = 0;
  if (a.vec_ok) {
    // 16-byte chunks from the aligned address below g0 straight into LDS (chunk c lands
    // at byte 16*c), every chunk of the work-group in flight at once.  The descriptor ends
    // at the last whole dword of the tensor: what lies past it arrives as zeros and the
    // tensor's last 1..3 bytes are patched in below.
    const size_t a0 = g0 & ~static_cast<size_t>(15);
    shift = static_cast<int>(g0 - a0);
    const int chunks = static_cast<int>((shift + len + 15) / 16);
    const size_t whole = a.total_in & ~static_cast<size_t>(3);
    const size_t avail = whole > a0 ? whole - a0 : 0;
    const v4i rsrc = make_rsrc(a.in + a0, static_cast<uint32_t>(avail < 0xffffffffu ? avail
                                                                                      : 0xffffffffu));
    const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds));
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    for (int c0 = wave * 64; c0 < chunks; c0 += (kPoolThreads / 64) * 64) {
      if (c0 + lane < chunks)
        dma_buffer(lds0 + static_cast<uint32_t>(c0) * 16, static_cast<uint32_t>(c0 + lane) * 16,
                   rsrc);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    const size_t end = g0 + len;
    if (tid < 3 && whole + tid < a.total_in && whole + tid >= g0 && whole + tid < end)
      lds[whole + tid - a0] = a.in[whole + tid];
  } else {
    for (size_t i = tid; i < len; i += kPoolThreads) lds[i] = a.in[g0 + i];
  }
  __syncthreads();
  const int rows = oh1 - oh0;
  if (FAST == 4) {
    // OW == 1 and every window spans the full width: rows [hstart, hend) of a plane are
    // one contiguous run of bytes
    constexpr int lo = UNSIGNED ? 0 : -128, hi = UNSIGNED ? 255 : 127;
    const int outputs = np * rows;
    for (int o = tid; o < outputs; o += kPoolThreads) {
      const int p = o / rows, oh = oh0 + (o - p * rows);
      int hstart = oh * a.sh - a.ph;
      int hend = min(hstart + a.KH, a.H + a.ph);
      const int padded = (hend - hstart) * a.W;  // pad_w == 0 and kernel_w == W here
      hstart = max(hstart, 0);
      hend = min(hend, a.H);
      const int addr = shift + p * static_cast<int>(plane_bytes) + (hstart - hs) * a.W;
      const int n = max(hend - hstart, 0) * a.W;
      const int sum = sum_bytes<UNSIGNED>(lds, addr, n);
      const int pool_size = a.count_pad ? padded : n;
      const float avg =
          pool_size > 0 ? static_cast<float>(sum) / static_cast<float>(pool_size) : 0.f;
      const int q = min(max(static_cast<int>(rintf(avg)), lo), hi);
      a.out[static_cast<size_t>(p0 + p) * a.OH + oh] = static_cast<uint8_t>(q);
    }
    return;
  }
  // items of kPoolItem adjacent outputs of one row
  const int per_row = (a.OW + kPoolItem - 1) / kPoolItem;
  const int per_plane = rows * per_row;
  const int items = np * per_plane;
  constexpr int K = FAST == 2 ? 2 : 3;
  constexpr int SW = FAST == 3 ? 1 : 2;
  for (int it = tid; it < items; it += kPoolThreads) {
    const int p = a.ppb > 1 ? fast_div(it, a.magic_per_plane) : 0, r = it - p * per_plane;
    const int orow = fast_div(r, a.magic_per_row), ow0 = (r - orow * per_row) * kPoolItem;
    const int oh = oh0 + orow;
    const int nout = min(kPoolItem, a.OW - ow0);
    uint32_t packed[kPoolItem / 4];
    if (!AVG && (FAST == 1 || FAST == 2)) {
      const int base = 16 + shift + p * static_cast<int>(plane_bytes);
      pool_strip_max2<UNSIGNED, K>(lds_raw, base, hs, he, a, oh, ow0, packed);
    } else {
      int q[kPoolItem];
#pragma unroll
      for (int i = 0; i < kPoolItem; ++i) q[i] = 0;
      if (FAST != 0) {
        const int base = 16 + shift + p * static_cast<int>(plane_bytes);
        pool_strip<UNSIGNED, AVG, K, SW>(lds_raw, base, hs, he, a, oh, ow0, q);
      } else {
        const uint8_t* img = lds + shift + static_cast<size_t>(p) * plane_bytes;
        // (fixed trip count: a runtime-indexed q[] would live in scratch memory)
#pragma unroll
        for (int i = 0; i < kPoolItem; ++i)
          if (i < nout) q[i] = pool_window<UNSIGNED>(img, hs, a, oh, ow0 + i);
      }
#pragma unroll
      for (int w = 0; w < kPoolItem / 4; ++w)
        packed[w] = (static_cast<uint32_t>(q[4 * w]) & 0xffu) |
                    ((static_cast<uint32_t>(q[4 * w + 1]) & 0xffu) << 8) |
                    ((static_cast<uint32_t>(q[4 * w + 2]) & 0xffu) << 16) |
                    (static_cast<uint32_t>(q[4 * w + 3]) << 24);
    }
    const size_t off = (static_cast<size_t>(p0 + p) * a.OH + oh) * a.OW + ow0;
    if (nout == kPoolItem && ((reinterpret_cast<uintptr_t>(a.out) + off) & 3u) == 0) {
#pragma unroll
      for (int w = 0; w < kPoolItem / 4; ++w)
        reinterpret_cast<uint32_t*>(a.out + off)[w] = packed[w];
    } else {
#pragma unroll
      for (int i = 0; i < kPoolItem; ++i)
        if (i < nout) a.out[off + i] = static_cast<uint8_t>(packed[i / 4] >> (8 * (i % 4)));
    }
  }
}

// Fallback for images whose single window band does not fit the LDS budget.
template <bool UNSIGNED>
__global__ __launch_bounds__(kPoolThreads) void pool_direct_kernel(PoolArgs a) {
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    *a.omin = *a.imin;
    *a.omax = *a.imax;
  }
  const size_t total = static_cast<size_t>(a.planes) * a.OH * a.OW;
  for (size_t o = static_cast<size_t>(blockIdx.x) * kPoolThreads + threadIdx.x; o < total;
       o += static_cast<size_t>(gridDim.x) * kPoolThreads) {
    const size_t p = o / (static_cast<size_t>(a.OH) * a.OW);
    const int r = static_cast<int>(o - p * a.OH * a.OW);
    const int oh = r / a.OW, ow = r - oh * a.OW;
    const uint8_t* img = a.in + p * static_cast<size_t>(a.H) * a.W;
    a.out[o] = static_cast<uint8_t>(pool_window<UNSIGNED>(img, 0, a, oh, ow));
  }
}

__global__ void copy_range_kernel(const float* imin, const float* imax, float* omin,
                                  float* omax) {
  *omin = *imin;
  *omax = *imax;
}

// Flat byte copy, 16 bytes per lane where both pointers allow it.
__global__ __launch_bounds__(256) void copy_bytes_kernel(const uint8_t* __restrict__ in,
                                                         uint8_t* __restrict__ out, size_t n,
                                                         int vec_ok, const float* imin,
                                                         const float* imax, float* omin,
                                                         float* omax) {
  const size_t stride = static_cast<size_t>(gridDim.x) * 256;
  const size_t t = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
  if (t == 0 && omin != nullptr) {  // the range goes with the data (null: it is in place)
    *omin = *imin;
    *omax = *imax;
  }
  if (vec_ok) {
    const size_t nv = n / 16;
    for (size_t i = t; i < nv; i += stride)
      reinterpret_cast<uint4*>(out)[i] = reinterpret_cast<const uint4*>(in)[i];
    for (size_t i = nv * 16 + t; i < n; i += stride) out[i] = in[i];
  } else {
    for (size_t i = t; i < n; i += stride) out[i] = in[i];
  }
}

}  // namespace
}  // namespace mxq

using namespace mxq;

extern "C" {

int mxq_quantized_pooling_nchw(void* stream, const void* in, int in_type, int N, int C, int H,
                               int W, int kernel_h, int kernel_w, int stride_h, int stride_w,
                               int pad_h, int pad_w, int OH, int OW, int pool_type,
                               int count_include_pad, const float* imin, const float* imax,
                               void* out, float* omin, float* omax) {
  MXQ_API_BEGIN();
  MXQ_CHECK(in_type == MXQ_INT8 || in_type == MXQ_UINT8, "pooling takes int8 or uint8 data");
  MXQ_CHECK(pool_type == MXQ_POOL_MAX || pool_type == MXQ_POOL_AVG,
            "QuantizedPoolingOp only supports pool_type=max/avg for now");
  MXQ_CHECK(N >= 0 && C >= 0 && H > 0 && W > 0 && OH > 0 && OW > 0, "bad shape");
  MXQ_CHECK(kernel_h > 0 && kernel_w > 0 && stride_h > 0 && stride_w > 0 && pad_h >= 0 &&
                pad_w >= 0,
            "bad kernel/stride/pad");
  MXQ_CHECK(kernel_h <= H + 2 * pad_h && kernel_w <= W + 2 * pad_w,
            "kernel size exceeds the padded input");
  MXQ_CHECK(imin && imax && omin && omax, "null range pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const long long planes = static_cast<long long>(N) * C;
  if (planes == 0 || static_cast<long long>(OH) * OW == 0) {
    hipLaunchKernelGGL(copy_range_kernel, dim3(1), dim3(1), 0, s, imin, imax, omin, omax);
    MXQ_LAUNCH_CHECK();
    return 0;
  }
  MXQ_CHECK(in != nullptr && out != nullptr, "null data pointer");
  MXQ_CHECK(planes < (1LL << 31) && static_cast<long long>(OH) * OW < (1LL << 31) &&
                static_cast<long long>(H) * W < (1LL << 31),
            "problem too large for 32-bit plane indices");
  PoolArgs a;
  a.in = static_cast<const uint8_t*>(in);
  a.out = static_cast<uint8_t*>(out);
  a.imin = imin; a.imax = imax; a.omin = omin; a.omax = omax;
  a.total_in = static_cast<size_t>(planes) * H * W;
  a.planes = static_cast<int>(planes);
  a.H = H; a.W = W; a.OH = OH; a.OW = OW; a.KH = kernel_h; a.KW = kernel_w;
  a.sh = stride_h; a.sw = stride_w; a.ph = pad_h; a.pw = pad_w;
  a.is_avg = pool_type == MXQ_POOL_AVG;
  a.count_pad = count_include_pad != 0;
  a.is_unsigned = in_type == MXQ_UINT8;
  a.vec_ok = aligned16(in) ? 1 : 0;
  const long long plane_bytes = static_cast<long long>(H) * W;
  const int cus = num_cus();
  long long blocks = 0;
  bool direct = false;
  if (2 * plane_bytes <= kPoolLdsBytes) {
    // small planes: several per work-group, but keep at least ~4 groups per CU
    long long ppb = kPoolLdsBytes / plane_bytes;
    const long long spread = (planes + 4LL * cus - 1) / (4LL * cus);
    if (ppb > spread) ppb = spread;
    if (ppb < 1) ppb = 1;
    // a group's work items (one per output row for full-width average windows, else one
    // per kPoolItem outputs) should fill whole passes of its threads: 668 planes of one
    // item each would leave the third pass of 256 threads 39 % full
    const bool full_width = a.is_avg && OW == 1 && pad_w == 0 && kernel_w == W;
    const long long units =
        full_width ? OH : static_cast<long long>((OW + kPoolItem - 1) / kPoolItem) * OH;
    auto fill = [&](long long planes_per_group) {
      const long long items = planes_per_group * units;
      return static_cast<double>(items) /
             static_cast<double>((items + kPoolThreads - 1) / kPoolThreads * kPoolThreads);
    };
    long long best = ppb;
    for (long long c = ppb - 1; c >= 1 && 2 * c >= ppb; --c)
      if (fill(c) > fill(best) + 0.03) best = c;
    ppb = best;
    a.ppb = static_cast<int>(ppb);
    a.band = OH;
    a.bands = 1;
    blocks = (planes + ppb - 1) / ppb;
  } else {
    a.ppb = 1;
    // rows_in(band) = (band - 1) * stride + kernel  <=  budget / W
    const long long rows_fit = kPoolLdsBytes / W;
    long long band = rows_fit >= kernel_h ? (rows_fit - kernel_h) / stride_h + 1 : 0;
    if (band > OH) band = OH;
    if (band < 1) {
      direct = true;
    } else {
      a.band = static_cast<int>(band);
      a.bands = static_cast<int>((OH + band - 1) / band);
      blocks = planes * a.bands;
    }
  }
  if (direct) {
    a.band = OH;
    a.bands = 1;
    const long long total = planes * OH * OW;
    long long g = (total + kPoolThreads - 1) / kPoolThreads;
    if (g > 8LL * cus) g = 8LL * cus;
    if (a.is_unsigned)
      hipLaunchKernelGGL((pool_direct_kernel<true>), dim3(g), dim3(kPoolThreads), 0, s, a);
    else
      hipLaunchKernelGGL((pool_direct_kernel<false>), dim3(g), dim3(kPoolThreads), 0, s, a);
  } else {
    MXQ_CHECK(blocks < (1LL << 31), "pooling grid too large");
    auto magic = [](long long d) {
      return d <= 1 ? 0u : static_cast<uint32_t>((1ULL << 32) / static_cast<unsigned long long>(d) + 1ULL);
    };
    const long long ow4 = (OW + kPoolItem - 1) / kPoolItem;  // items per output row
    // items per work-group stay below 2^17 and the divisors below 2^15 (both bounded by
    // the bytes staged in LDS), so n * d < 2^32 holds
    MXQ_CHECK(ow4 * OH < (1LL << 15) || a.ppb <= 1, "pooling plane too large for the item index");
    MXQ_CHECK(ow4 < (1LL << 15), "pooling row too long for the item index");
    a.magic_per_row = magic(ow4);
    a.magic_per_plane = magic(ow4 * OH);
    int fast = 0;
    if (a.is_avg && OW == 1 && pad_w == 0 && kernel_w == W)
      fast = 4;
    else if (pad_w > 8)
      fast = 0;  // the quad path reads at most 16 bytes in front of a row
    else if (kernel_h == 3 && kernel_w == 3 && stride_w == 2)
      fast = 1;
    else if (kernel_h == 2 && kernel_w == 2 && stride_w == 2)
      fast = 2;
    else if (kernel_h == 3 && kernel_w == 3 && stride_w == 1)
      fast = 3;
#define MXQ_POOL(U, A, F) \
  hipLaunchKernelGGL((pool_lds_kernel<U, A, F>), dim3(blocks), dim3(kPoolThreads), 0, s, a)
#define MXQ_POOL_F(U, A)               \
  switch (fast) {                      \
    case 1: MXQ_POOL(U, A, 1); break;  \
    case 2: MXQ_POOL(U, A, 2); break;  \
    case 3: MXQ_POOL(U, A, 3); break;  \
    default: MXQ_POOL(U, A, 0); break; \
  }
    if (fast == 4) {
      if (a.is_unsigned) {
        MXQ_POOL(true, true, 4);
      } else {
        MXQ_POOL(false, true, 4);
      }
    } else if (a.is_unsigned) {
      if (a.is_avg) {
        MXQ_POOL_F(true, true)
      } else {
        MXQ_POOL_F(true, false)
      }
    } else {
      if (a.is_avg) {
        MXQ_POOL_F(false, true)
      } else {
        MXQ_POOL_F(false, false)
      }
    }
#undef MXQ_POOL_F
#undef MXQ_POOL
  }
  MXQ_LAUNCH_CHECK();
  MXQ_API_END();
}

int mxq_quantized_flatten(void* stream, const void* in, const float* imin, const float* imax,
                          void* out, float* omin, float* omax, size_t n_bytes) {
  MXQ_API_BEGIN();
  MXQ_CHECK(imin && imax && omin && omax, "null range pointer");
  MXQ_CHECK(n_bytes == 0 || (in != nullptr && out != nullptr), "null data pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool range_moves = omin != imin || omax != imax;
  if (n_bytes != 0 && in != out) {
    const int vec_ok = aligned16(in) && aligned16(out);
    size_t g = (n_bytes / (vec_ok ? 16 : 1) + 255) / 256;
    const size_t cap = static_cast<size_t>(num_cus()) * 8;
    if (g > cap) g = cap;
    if (g < 1) g = 1;
    hipLaunchKernelGGL(copy_bytes_kernel, dim3(static_cast<unsigned>(g)), dim3(256), 0, s,
                       static_cast<const uint8_t*>(in), static_cast<uint8_t*>(out), n_bytes,
                       vec_ok, imin, imax, range_moves ? omin : nullptr, omax);
    MXQ_LAUNCH_CHECK();
  } else if (range_moves) {
    hipLaunchKernelGGL(copy_range_kernel, dim3(1), dim3(1), 0, s, imin, imax, omin, omax);
    MXQ_LAUNCH_CHECK();
  }
  MXQ_API_END();
}

}  // extern "C"
