// _contrib_quantized_fully_connected on gfx950: int8 data [M,K] x int8 weight
// [N,K]^T -> int32, with the int8 bias rescaled to int32 and (optionally) the
// calibrated requantize fused into the epilogue.  Replaces cublasGemmEx +
// QuantizedBiasAddKernel of the reference's GPU operator
// (src/operator/quantization/quantized_fully_connected.cu:58-138) with the exact
// integer semantics of its CPU operator (quantized_fully_connected.cc:149-297).
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>

#include "../../include/mxq.h"
#include "mxq_common.h"
#include "mxq_gemm.cuh"
#include "mxq_tiles.h"

namespace mxq {

int g_fc_config = 0;  // 0 = choose by shape; 1.. force a tile configuration (tuning/tests)

namespace {

struct FcArgs {
  const int8_t* data;    // [M][K]
  const int8_t* weight;  // [N][K]
  int M, N, K;
  int ldo;               // output row pitch in elements (N for the FC)
  Epilogue epi;
};

template <class Cfg, bool ALIGNED>
__global__ __launch_bounds__(Cfg::kThreads) void fc_kernel(FcArgs p) {
  __shared__ __attribute__((aligned(16))) v4i lds[2][Cfg::STAGE_SLOTS];
  const int wave = threadIdx.x >> 6;
  const int wm = wave / Cfg::WN, wn = wave % Cfg::WN;
  const int tiles_m = (p.M + Cfg::BM - 1) / Cfg::BM, tiles_n = (p.N + Cfg::BN - 1) / Cfg::BN;
  int tm, tn;
  tile_coords(blockIdx.x, tiles_m, tiles_n, tm, tn);
  const int m0 = tm * Cfg::BM, n0 = tn * Cfg::BN;

  RowFetch<Cfg, Cfg::A_CHUNKS, ALIGNED> af;
  RowFetch<Cfg, Cfg::B_CHUNKS, ALIGNED> bf;
  af.init(p.data, m0, p.M, p.K);
  bf.init(p.weight, n0, p.N, p.K);

  v16i acc[Cfg::MI][Cfg::NI];
  gemm_mainloop<Cfg>(acc, af, bf, (p.K + Cfg::BK - 1) / Cfg::BK, lds);

  gemm_epilogue<Cfg>(acc, p.epi, m0 + wm * Cfg::TM, n0 + wn * Cfg::TN, p.M, p.N,
                     static_cast<size_t>(p.ldo));
  if (blockIdx.x == 0 && threadIdx.x == 0) epilogue_ranges(p.epi);
}

// Direct-to-LDS variant (see gemm_mainloop_dma); launch_fc() picks it when the
// operands qualify.  BUF selects buffer loads (any K % 16 == 0, zero-filled tails)
// over global loads (K % 64 == 0, clamped rows).
template <class Cfg, int NS, int PIPE, bool BUF>
__global__ __launch_bounds__(Cfg::kThreads) void fc_dma_kernel(FcArgs p) {
  __shared__ __attribute__((aligned(16))) v4i lds[NS * Cfg::STAGE_SLOTS];
  const int tiles_m = (p.M + Cfg::BM - 1) / Cfg::BM, tiles_n = (p.N + Cfg::BN - 1) / Cfg::BN;
  int tm, tn;
  tile_coords(blockIdx.x, tiles_m, tiles_n, tm, tn);
  const int m0 = tm * Cfg::BM, n0 = tn * Cfg::BN;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);

  // what the epilogue needs is fetched while the first operand stages are in flight
  EpiPre pre;
  auto prefetch = [&]() { pre = epi_prefetch<Cfg>(p.epi, n0, p.N); };
  v16i acc[Cfg::MI][Cfg::NI];
  const int KT = (p.K + Cfg::BK - 1) / Cfg::BK;
  if (BUF) {
    RowIssuerBuffer<Cfg, Cfg::A_CHUNKS> ai;
    RowIssuerBuffer<Cfg, Cfg::B_CHUNKS> bi;
    ai.init(p.data, m0, p.M, p.K, wave, lane);
    bi.init(p.weight, n0, p.N, p.K, wave, lane);
    gemm_mainloop_dma<Cfg, NS, PIPE>(acc, ai, bi, KT, lds, prefetch);
  } else {
    RowIssuerGlobal<Cfg, Cfg::A_CHUNKS> ai;
    RowIssuerGlobal<Cfg, Cfg::B_CHUNKS> bi;
    ai.init(p.data, m0, p.M, p.K, wave, lane);
    bi.init(p.weight, n0, p.N, p.K, wave, lane);
    gemm_mainloop_dma<Cfg, NS, PIPE>(acc, ai, bi, KT, lds, prefetch);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

  gemm_epilogue_lds<Cfg, NS * Cfg::STAGE_SLOTS * 16>(acc, p.epi, pre, m0, n0, p.M, p.N,
                                                     static_cast<size_t>(p.ldo), lds);
  if (blockIdx.x == 0 && threadIdx.x == 0) epilogue_ranges(p.epi);
}

typedef GemmCfg<256, 256, 64, 2, 4> CfgL8;    // 8 waves, wave tile 128 x 64
typedef GemmCfg<256, 256, 64, 2, 2> CfgL4;    // 4 waves, wave tile 128 x 128
typedef GemmCfg<256, 128, 64, 4, 2> CfgW128;  // 8 waves, wave tile 64 x 64
typedef GemmCfg<256, 64, 64, 4, 1> CfgW64;    // 4 waves, wave tile 64 x 64
typedef GemmCfg<128, 128, 64, 2, 2> CfgM;     // 4 waves, wave tile 64 x 64
typedef GemmCfg<64, 64, 64, 2, 2> CfgS;       // 4 waves, wave tile 32 x 32
// 128-byte stages: half as many K steps (each costs a barrier and a round of DMA latency)
typedef GemmCfg<256, 256, 128, 2, 4> CfgL8K;   // 8 waves, wave tile 128 x 64
typedef GemmCfg<256, 128, 128, 4, 2> CfgW128K; // 8 waves, wave tile 64 x 64
typedef GemmCfg<128, 128, 128, 2, 2> CfgMK;    // 4 waves, wave tile 64 x 64
typedef GemmCfg<64, 64, 128, 2, 2> CfgSK;      // 4 waves, wave tile 32 x 32
typedef GemmCfg<128, 64, 128, 2, 2> CfgRK;     // 4 waves, wave tile 64 x 32
typedef GemmCfg<64, 128, 128, 2, 2> CfgQK;     // 4 waves, wave tile 32 x 64
typedef GemmCfg<64, 64, 256, 2, 2> CfgSK2;     // 256-byte stages for very long K

template <class Cfg, int NS, int PIPE, bool BUF>
void launch_dma(hipStream_t s, const FcArgs& a) {
  const int tiles = ((a.M + Cfg::BM - 1) / Cfg::BM) * ((a.N + Cfg::BN - 1) / Cfg::BN);
  hipLaunchKernelGGL((fc_dma_kernel<Cfg, NS, PIPE, BUF>), dim3(tiles), dim3(Cfg::kThreads), 0,
                     s, a);
  MXQ_LAUNCH_CHECK();
}

template <class Cfg>
void launch_cfg(hipStream_t s, const FcArgs& a, bool aligned) {
  const int tiles = ((a.M + Cfg::BM - 1) / Cfg::BM) * ((a.N + Cfg::BN - 1) / Cfg::BN);
  if (aligned)
    hipLaunchKernelGGL((fc_kernel<Cfg, true>), dim3(tiles), dim3(Cfg::kThreads), 0, s, a);
  else
    hipLaunchKernelGGL((fc_kernel<Cfg, false>), dim3(tiles), dim3(Cfg::kThreads), 0, s, a);
  MXQ_LAUNCH_CHECK();
}

int num_cus() {
  int dev = 0;
  MXQ_HIP(hipGetDevice(&dev));
  static thread_local int cached_dev = -1, cached_cus = 0;
  if (cached_dev != dev) {
    MXQ_HIP(hipDeviceGetAttribute(&cached_cus, hipDeviceAttributeMultiprocessorCount, dev));
    cached_dev = dev;
  }
  return cached_cus;
}

}  // namespace

// Tile configurations:
//   1..4    register-staged kernels (any shape): 256x256x8w, 256x256x4w, 128x128, 64x64
//   11, 12  direct-to-LDS 256x256, 8 waves: compiler-scheduled / pinned pipeline
//   14, 16  direct-to-LDS 256x256, 4 waves: compiler-scheduled / pinned pipeline
//   21..24  direct-to-LDS buffer-load kernels 256x128, 256x64, 128x128, 64x64
//   31, 32  as 12 / 16 with buffer loads (K % 16 == 0 instead of K % 64 == 0)
//   41..44  as 21..24 with a 2-stage ring (short K)
//   51..56  128-byte stages: 64x64 (2, 3 stages), 128x128 (2, 3), 256x256 (2), 256x128 (2)
//   57..59  128x64 and 64x128 with 128-byte stages, 64x64 with 256-byte stages
void launch_fc(hipStream_t s, const int8_t* data, const int8_t* weight, int M, int N, int K,
               int ldo, const Epilogue& epi) {
  FcArgs a;
  a.data = data;
  a.weight = weight;
  a.M = M;
  a.N = N;
  a.K = K;
  a.ldo = ldo;
  a.epi = epi;
  const bool aligned = (K % 16 == 0) && aligned16(data) && aligned16(weight);
  // direct-to-LDS kernels: operands below 2 GiB; K a multiple of the 64-byte stage for
  // the global-load form, of 16 for the buffer-load form
  const bool buf_ok = aligned && K >= 16 && static_cast<long long>(M) * K < (1LL << 31) &&
                      static_cast<long long>(N) * K < (1LL << 31);
  const bool glb_ok = buf_ok && (K % 64 == 0);
  int cfg = g_fc_config;
  if (cfg == 0) {
    const long cus = num_cus();
    auto tiles = [&](int bm, int bn) {
      return static_cast<long>((M + bm - 1) / bm) * ((N + bn - 1) / bn);
    };
    if (buf_ok) {
      switch (choose_tile(M, N, K, cus)) {
        case Tile::kL8: cfg = glb_ok ? 12 : 31; break;
        case Tile::kW128x2: cfg = 41; break;
        case Tile::kW128K2: cfg = 56; break;
        case Tile::kM128x2: cfg = 43; break;
        case Tile::kM128K2: cfg = 53; break;
        case Tile::kS64x2: cfg = 44; break;
        case Tile::kS64x4: cfg = 24; break;
        case Tile::kS64K2: cfg = 51; break;
        case Tile::kR128K2: cfg = 57; break;
        case Tile::kQ128K2: cfg = 58; break;
        case Tile::kS64K4: cfg = 59; break;
      }
    } else {
      if (tiles(256, 256) >= cus)
        cfg = 1;
      else if (tiles(128, 128) >= cus)
        cfg = 3;
      else
        cfg = 4;
    }
  }
  if (cfg >= 11 && cfg <= 16) MXQ_CHECK(glb_ok, "shape does not qualify for the DMA kernels");
  if (cfg >= 21) MXQ_CHECK(buf_ok, "shape does not qualify for the buffer-load DMA kernels");
  switch (cfg) {
    case 1: launch_cfg<CfgL8>(s, a, aligned); break;
    case 2: launch_cfg<CfgL4>(s, a, aligned); break;
    case 3: launch_cfg<CfgM>(s, a, aligned); break;
    case 4: launch_cfg<CfgS>(s, a, aligned); break;
    case 11: launch_dma<CfgL8, 4, 0, false>(s, a); break;
    case 12: launch_dma<CfgL8, 4, 2, false>(s, a); break;
    case 14: launch_dma<CfgL4, 4, 0, false>(s, a); break;
    case 16: launch_dma<CfgL4, 4, 2, false>(s, a); break;
    case 21: launch_dma<CfgW128, 4, 2, true>(s, a); break;
    case 22: launch_dma<CfgW64, 4, 2, true>(s, a); break;
    case 23: launch_dma<CfgM, 4, 2, true>(s, a); break;
    case 24: launch_dma<CfgS, 4, 2, true>(s, a); break;
    case 41: launch_dma<CfgW128, 2, 0, true>(s, a); break;
    case 42: launch_dma<CfgW64, 2, 0, true>(s, a); break;
    case 43: launch_dma<CfgM, 2, 0, true>(s, a); break;
    case 44: launch_dma<CfgS, 2, 0, true>(s, a); break;
    case 51: launch_dma<CfgSK, 2, 0, true>(s, a); break;
    case 52: launch_dma<CfgSK, 3, 0, true>(s, a); break;
    case 53: launch_dma<CfgMK, 2, 0, true>(s, a); break;
    case 54: launch_dma<CfgMK, 3, 0, true>(s, a); break;
    case 55: launch_dma<CfgL8K, 2, 0, true>(s, a); break;
    case 56: launch_dma<CfgW128K, 2, 0, true>(s, a); break;
    case 57: launch_dma<CfgRK, 2, 0, true>(s, a); break;
    case 58: launch_dma<CfgQK, 2, 0, true>(s, a); break;
    case 59: launch_dma<CfgSK2, 2, 0, true>(s, a); break;
    case 31: launch_dma<CfgL8, 4, 2, true>(s, a); break;
    case 32: launch_dma<CfgL4, 4, 2, true>(s, a); break;
    default: MXQ_CHECK(false, "unknown fc tile configuration " << cfg);
  }
}

}  // namespace mxq

using namespace mxq;

extern "C" int mxq_quantized_fc(void* stream, const int8_t* data, const int8_t* weight,
                                const int8_t* bias, int M, int N, int K, const float* min_data,
                                const float* max_data, const float* min_weight,
                                const float* max_weight, const float* min_bias,
                                const float* max_bias, int32_t* out32, float* omin, float* omax,
                                int8_t* out8, float* rmin, float* rmax, int relu,
                                float min_calib, float max_calib) {
  MXQ_API_BEGIN();
  MXQ_CHECK(M >= 0 && N >= 0 && K >= 0, "negative dimension");
  MXQ_CHECK(min_data && max_data && min_weight && max_weight, "null input range pointer");
  MXQ_CHECK(omin && omax, "null output range pointer");
  MXQ_CHECK(bias == nullptr || (min_bias && max_bias), "bias given without its range");
  MXQ_CHECK(out32 != nullptr || out8 != nullptr, "no output buffer");
  MXQ_CHECK(out8 == nullptr || (rmin && rmax), "fused requantize needs rmin/rmax");
  if (M == 0 || N == 0) return 0;
  MXQ_CHECK(data != nullptr && weight != nullptr, "null operand pointer");
  Epilogue e;
  e.bias = bias;
  e.min_data = min_data;
  e.max_data = max_data;
  e.min_weight = min_weight;
  e.max_weight = max_weight;
  e.min_bias = min_bias;
  e.max_bias = max_bias;
  e.out32 = out32;
  e.out8 = out8;
  e.omin = omin;
  e.omax = omax;
  e.rmin = rmin;
  e.rmax = rmax;
  e.relu = relu;
  float a = fabsf(min_calib), b = fabsf(max_calib);
  e.real_range = (a < b) ? b : a;
  e.plane = 0;
  launch_fc(static_cast<hipStream_t>(stream), data, weight, M, N, K, N, e);
  MXQ_API_END();
}
