// bench_probe.so - measurement aid for the benchmark, not part of the operator ABI.
//
// mxq_probe_mfma_i8 runs v_mfma_i32_32x32x32_i8 back to back out of registers: no
// LDS, no global memory in the loop, the register shape of the FC kernel's wave
// tile (4 activation and 2 weight fragments, 8 accumulators).  Timed with zero and
// with random operand bytes it shows how much of the nominal int8 rate the matrix
// pipes sustain on the machine at hand before any data movement is paid for: the
// shader clock follows the power the operands make the multipliers draw.
#include <hip/hip_runtime.h>

#include <cstdint>

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

namespace {

__device__ __forceinline__ uint32_t mix(uint32_t x) {
  x ^= x >> 16;
  x *= 0x7feb352du;
  x ^= x >> 15;
  x *= 0x846ca68bu;
  x ^= x >> 16;
  return x;
}

__global__ __launch_bounds__(256) void mfma_probe_kernel(int iters, int zero, int* sink) {
  const uint32_t t = blockIdx.x * 256 + threadIdx.x;
  v4i a[4], b[2];
  for (int i = 0; i < 4; ++i)
    for (int j = 0; j < 4; ++j) a[i][j] = zero ? 0 : static_cast<int>(mix(t * 64 + i * 4 + j));
  for (int i = 0; i < 2; ++i)
    for (int j = 0; j < 4; ++j)
      b[i][j] = zero ? 0 : static_cast<int>(mix(t * 64 + 32 + i * 4 + j));
  v16i acc[4][2];
  for (int i = 0; i < 4; ++i)
    for (int j = 0; j < 2; ++j)
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(b[j], a[i], acc[i][j], 0, 0, 0);
  }
  int s = 0;
  for (int i = 0; i < 4; ++i)
    for (int j = 0; j < 2; ++j)
      for (int v = 0; v < 16; ++v) s += acc[i][j][v];
  if (s == 0x12345678) sink[t] = s;  // keeps the loop alive; practically never taken
}

}  // namespace

extern "C" {

// Launches `blocks` work-groups of 4 waves, each wave issuing 8 * iters MFMAs
// (65536 integer operations each).  `sink` must hold blocks * 256 ints.  Returns the
// operation count of the launch, or -1.0 if the launch failed.
double mxq_probe_mfma_i8(void* stream, int blocks, int iters, int zero_operands, int* sink) {
  if (blocks <= 0 || iters <= 0 || sink == nullptr) return -1.0;
  hipLaunchKernelGGL(mfma_probe_kernel, dim3(blocks), dim3(256), 0,
                     static_cast<hipStream_t>(stream), iters, zero_operands, sink);
  if (hipGetLastError() != hipSuccess) return -1.0;
  return 8.0 * 65536.0 * iters * 4.0 * blocks;
}

}  // extern "C"
