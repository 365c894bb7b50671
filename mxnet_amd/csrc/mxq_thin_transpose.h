// Byte transpose of a tile with one thin extent, shared by the convolution's layout adapters
// and _contrib_quantized_transpose.
#ifndef MXQ_THIN_TRANSPOSE_H_
#define MXQ_THIN_TRANSPOSE_H_
#include <hip/hip_runtime.h>

#include <cstdint>

namespace mxq {

// One extent of at most 64 bytes that the tiled byte transposes cannot take (7 x 7 planes: 49
// bytes, no multiple of 4) against a long one that is a multiple of 128: a work-group of 256
// threads moves 128 long positions x T thin ones.  On the side where the thin extent is
// innermost that tile is one contiguous run of 128 * T bytes, kept in LDS (`flat`, 128 * 64
// bytes) as it lies in memory; the other side's 16-byte pieces (16 long positions of one thin
// position) are gathered from it, or scattered into it, byte by byte.  THIN_IN: the input is
// [L][T] and the output [T][L]; else the reverse.  src / dst point at the [.][.] matrix, both
// 16-byte aligned; l0 is the tile's first long position.
template <bool THIN_IN>
__device__ __forceinline__ void thin_transpose_tile(const uint8_t* __restrict__ src,
                                                    uint8_t* __restrict__ dst, int L, int T,
                                                    int l0, uint8_t* flat) {
  typedef uint32_t u4 __attribute__((ext_vector_type(4)));
  const int pieces = 8 * T;  // 16-byte pieces of the tile, on either side
  const int t0 = threadIdx.x;
  if (THIN_IN) {
    const u4* run = reinterpret_cast<const u4*>(src + static_cast<size_t>(l0) * T);
    for (int c = t0; c < pieces; c += 256)
      *reinterpret_cast<u4*>(flat + 16 * c) = __builtin_nontemporal_load(run + c);
    __syncthreads();
    for (int c = t0; c < pieces; c += 256) {
      const int t = c >> 3, g = c & 7;
      u4 v;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        uint32_t x = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i)
          x |= static_cast<uint32_t>(flat[(16 * g + 4 * w + i) * T + t]) << (8 * i);
        v[w] = x;
      }
      __builtin_nontemporal_store(
          v, reinterpret_cast<u4*>(dst + static_cast<size_t>(t) * L + l0 + 16 * g));
    }
  } else {
    for (int c = t0; c < pieces; c += 256) {
      const int t = c >> 3, g = c & 7;
      const u4 v = __builtin_nontemporal_load(
          reinterpret_cast<const u4*>(src + static_cast<size_t>(t) * L + l0 + 16 * g));
#pragma unroll
      for (int w = 0; w < 4; ++w)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          flat[(16 * g + 4 * w + i) * T + t] = static_cast<uint8_t>(v[w] >> (8 * i));
    }
    __syncthreads();
    u4* run = reinterpret_cast<u4*>(dst + static_cast<size_t>(l0) * T);
    for (int c = t0; c < pieces; c += 256)
      __builtin_nontemporal_store(*reinterpret_cast<const u4*>(flat + 16 * c), run + c);
  }
}

}  // namespace mxq
#endif  // MXQ_THIN_TRANSPOSE_H_
