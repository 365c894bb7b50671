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
#include "mxq_gemm.h"
#include "mxq_tiles.h"

namespace mxq {

namespace {

struct FcArgs {
  const int8_t* data;    // [M][K]
  const int8_t* weight;  // [N][K]
  int M, N, K;
  int ldo;               // output row pitch in elements (N for the FC)
  Epilogue epi;
  SplitK sk;
};

template <class Cfg, bool ALIGNED, int MODE>
__global__ __launch_bounds__(Cfg::kThreads, Cfg::kMinWaves) void fc_kernel(FcArgs p) {
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

  gemm_epilogue<Cfg, MODE>(acc, p.epi, m0 + wm * Cfg::TM, n0 + wn * Cfg::TN, p.M, p.N,
                     static_cast<size_t>(p.ldo));
  if (blockIdx.x == 0 && threadIdx.x == 0) epilogue_ranges<MODE>(p.epi);
}

// Direct-to-LDS variant (see gemm_mainloop_dma); launch_fc() picks it when the
// operands qualify.  BUF selects buffer loads (any K % 16 == 0, zero-filled tails)
// over global loads (K % 64 == 0, clamped rows).
// MODE (kEpiPlain / kEpiF32 / kEpiSum) builds the float output or the residual sum in: kernels
// of their own, so that the int8 and int32 forms do not carry their code.
template <class Cfg, int NS, int PIPE, bool BUF, int MODE>
__global__ __launch_bounds__(Cfg::kThreads, NS <= 2 ? Cfg::kMinWaves : 1) void fc_dma_kernel(FcArgs p) {
  __shared__ __attribute__((aligned(16))) v4i lds[NS * Cfg::STAGE_SLOTS];
  const int tiles_m = (p.M + Cfg::BM - 1) / Cfg::BM, tiles_n = (p.N + Cfg::BN - 1) / Cfg::BN;
  int tm, tn, tile = 0, z = 0;
  if (__builtin_expect(p.sk.splits > 1, 0))
    tile_coords_split(blockIdx.x, tiles_m, tiles_n, p.sk.splits, tm, tn, tile, z);
  else
    tile_coords(blockIdx.x, tiles_m, tiles_n, tm, tn);
  const int m0 = tm * Cfg::BM, n0 = tn * Cfg::BN;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);

  // what the epilogue needs is fetched while the first operand stages are in flight
  EpiPre pre;
  auto prefetch = [&]() { pre = epi_prefetch<Cfg, MODE>(p.epi, n0, p.N); };
  v16i acc[Cfg::MI][Cfg::NI];
  // this work-group's K slice: stages [kt0, kt0 + KT) (all of them without a split)
  const int kt_all = (p.K + Cfg::BK - 1) / Cfg::BK;
  const int kt0 = z * p.sk.kt_per_split;
  const int KT = (kt_all - kt0) < p.sk.kt_per_split ? (kt_all - kt0) : p.sk.kt_per_split;
  const int kbeg = kt0 * Cfg::BK;
  if (BUF) {
    RowIssuerBuffer<Cfg, Cfg::A_CHUNKS> ai;
    RowIssuerBuffer<Cfg, Cfg::B_CHUNKS> bi;
    ai.init(p.data, m0, p.M, p.K, wave, lane, kbeg);
    bi.init(p.weight, n0, p.N, p.K, wave, lane, kbeg);
    gemm_mainloop_dma<Cfg, NS, PIPE>(acc, ai, bi, KT, lds, prefetch);
  } else {
    RowIssuerGlobal<Cfg, Cfg::A_CHUNKS> ai;
    RowIssuerGlobal<Cfg, Cfg::B_CHUNKS> bi;
    ai.init(p.data, m0, p.M, p.K, wave, lane, kbeg);
    bi.init(p.weight, n0, p.N, p.K, wave, lane, kbeg);
    gemm_mainloop_dma<Cfg, NS, PIPE>(acc, ai, bi, KT, lds, prefetch);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  if (blockIdx.x == 0 && threadIdx.x == 0) epilogue_ranges<MODE>(p.epi);
  if (__builtin_expect(p.sk.splits > 1, 0) && !splitk_gather<Cfg>(acc, p.sk, tile, z)) return;

  gemm_epilogue_lds<Cfg, NS * Cfg::STAGE_SLOTS * 16, MODE>(acc, p.epi, pre, m0, n0, p.M, p.N,
                                                           static_cast<size_t>(p.ldo), lds);
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
typedef GemmCfg<256, 192, 128, 4, 2> CfgW192K; // 8 waves, wave tile 64 x 96

// Short-K form (K = 32, 64, 128 or 256; int8 output only).  With one or two K steps a tile of
// the kernels above is all prologue and epilogue: a round of DMA latency, two barriers, and
// an epilogue that keeps the CU's VALUs busy half the time.  Here the weight strip of a
// work-group (up to 256 rows of K bytes, 128 for K = 256) is parked in LDS once, and every wave on its own
// streams work items "32 data rows x 32*NI columns": the data fragment straight from global
// memory into the MFMA layout (a row of K bytes is consumed whole by the wave's K/16 loads),
// the next item's fragment requested before the current one is multiplied, weights read from
// LDS, then the fused epilogue and a transpose of the int8 tile through the wave's own LDS
// scratch.  No barrier after the weights are staged; waves only meet the memory system.
// SUM: the residual operand FcArgs::epi.res is added to the int8 tile on its way out.
template <int KS, int NI, bool SUM>
__global__ __launch_bounds__(256, 2) void fc_stream_kernel(FcArgs p, int bn, int strips) {
  constexpr int K = 32 * KS, CH = 2 * KS;  // bytes and 16-byte chunks per row
  constexpr int TN = 32 * NI, LD = TN + 16;
  constexpr int LPR = TN / 16, RPI = 64 / LPR;
  constexpr int kMaxRows = KS <= 4 ? 256 : 128;  // weight rows per work-group: at most 32 KB
  __shared__ __attribute__((aligned(16))) v4i ldsB[kMaxRows * CH];
  __shared__ __attribute__((aligned(16))) int sbias[256];
  __shared__ __attribute__((aligned(16))) char stage_all[4 * 32 * LD];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n_begin = blockIdx.y * bn;
  const int cols = (p.N - n_begin) < bn ? (p.N - n_begin) : bn;  // a multiple of TN
  for (int i = tid; i < cols * CH; i += 256) {
    const int r = i / CH, c = i - r * CH;
    ldsB[r * CH + (c ^ swz<CH>(r))] = *reinterpret_cast<const v4i*>(
        p.weight + static_cast<size_t>(n_begin + r) * K + c * 16);
  }
  const EpiScalars s = epi_scalars(p.epi);
  SumRule rule = {0.0f, 0.0f, 1};
  if (SUM)
    rule = sum_rule(dev_maxabs(-p.epi.real_range, p.epi.real_range),
                    dev_maxabs(*p.epi.res_min, *p.epi.res_max), p.epi.sum_min_calib,
                    p.epi.sum_max_calib);
  if (tid < cols) sbias[tid] = epi_bias32(p.epi, s, n_begin + tid);
  __syncthreads();

  const int lrow = lane & 31, lgrp = lane >> 5;
  char* stage = stage_all + wave * 32 * LD;
  const int tiles_m = (p.M + 31) / 32;
  const int items = tiles_m * strips;
  const int step = gridDim.x * 4;
  auto load_a = [&](int item, v4i (&f)[KS]) {
    const int m = (item / strips) * 32 + lrow;
    const bool ok = m < p.M;
    const int8_t* row = p.data + static_cast<size_t>(ok ? m : 0) * K + lgrp * 16;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      f[ks] = *reinterpret_cast<const v4i*>(row + ks * 32);
      if (!ok) f[ks] = v4i{0, 0, 0, 0};
    }
  };
  int item = blockIdx.x * 4 + wave;
  v4i fa[KS];
  if (item < items) load_a(item, fa);
  const bool relu = p.epi.relu != 0, stream8 = p.epi.stream8 != 0;
  for (; item < items; item += step) {
    v4i fa_next[KS];
    const bool more = item + step < items;
    if (more) load_a(item + step, fa_next);
    const int tile = item / strips;
    const int s0 = (item - tile * strips) * TN;  // first column of the strip inside the group's
    const int m_base = tile * 32;
    // the residual operand's pieces of this tile, in the layout the tile leaves in
    v4i resv[32 / RPI];
    if (SUM) {
#pragma unroll
      for (int it = 0; it < 32 / RPI; ++it) {
        const int m = m_base + it * RPI + lane / LPR;
        resv[it] = v4i{0, 0, 0, 0};
        if (m < p.M)
          resv[it] = __builtin_nontemporal_load(reinterpret_cast<const v4i*>(
              p.epi.res + static_cast<size_t>(m) * p.ldo + n_begin + s0 + (lane % LPR) * 16));
      }
    }
    // the accumulators start at the int32 bias of their columns (read from LDS straight
    // into the registers the MFMAs add to): the epilogue has no bias add left
    v16i acc[NI];
#pragma unroll
    for (int ni = 0; ni < NI; ++ni)
#pragma unroll
      for (int vq = 0; vq < 4; ++vq) {
        const v4i b = *reinterpret_cast<const v4i*>(sbias + s0 + ni * 32 + 8 * vq + 4 * lgrp);
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[ni][4 * vq + i] = b[i];
      }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int ni = 0; ni < NI; ++ni) {
        const int r = s0 + ni * 32 + lrow;
        const v4i fb = ldsB[r * CH + ((ks * 2 + lgrp) ^ swz<CH>(r))];
        acc[ni] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb, fa[ks], acc[ni], 0, 0, 0);
      }
    auto requantize_tile = [&](auto with_relu) {
#pragma unroll
      for (int ni = 0; ni < NI; ++ni)
#pragma unroll
        for (int vq = 0; vq < 4; ++vq) {
          const int nl = ni * 32 + 8 * vq + 4 * lgrp;
          *reinterpret_cast<uint32_t*>(stage + lrow * LD + nl) =
              epi_requant_pack<decltype(with_relu)::value>(acc[ni][4 * vq], acc[ni][4 * vq + 1],
                                                           acc[ni][4 * vq + 2],
                                                           acc[ni][4 * vq + 3], s);
        }
    };
    if (relu)
      requantize_tile(std::true_type());
    else
      requantize_tile(std::false_type());
    // the wave reads back what its own lanes wrote: LDS executes a wave's instructions in
    // order, the wait makes the writes complete first
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_wave_barrier();
    auto store_tile = [&](auto stream, auto sum_relu, auto sum_fast) {
#pragma unroll
      for (int it = 0; it < 32 / RPI; ++it) {
        const int rr = it * RPI + lane / LPR, c16 = lane % LPR;
        v4i val = *reinterpret_cast<const v4i*>(stage + rr * LD + c16 * 16);
        if (SUM) {
#pragma unroll
          for (int w = 0; w < 4; ++w)
            val[w] = static_cast<int>(
                sum4<decltype(sum_relu)::value, decltype(sum_fast)::value>(
                    static_cast<uint32_t>(val[w]), static_cast<uint32_t>(resv[it][w]), rule));
        }
        const int m = m_base + rr;
        if (m < p.M)
          epi_store16<decltype(stream)::value>(
              val, p.epi.out8 + static_cast<size_t>(m) * p.ldo + n_begin + s0 + c16 * 16);
      }
    };
    auto store_flavour = [&](auto sum_relu, auto sum_fast) {
      if (stream8)
        store_tile(std::true_type(), sum_relu, sum_fast);
      else
        store_tile(std::false_type(), sum_relu, sum_fast);
    };
    if (SUM && !rule.fast) {
      if (p.epi.sum_relu)
        store_flavour(std::true_type(), std::integral_constant<bool, !SUM>());
      else
        store_flavour(std::false_type(), std::integral_constant<bool, !SUM>());
    } else if (SUM && p.epi.sum_relu) {
      store_flavour(std::true_type(), std::true_type());
    } else {
      store_flavour(std::false_type(), std::true_type());
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_wave_barrier();
    if (more) {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) fa[ks] = fa_next[ks];
    }
  }
  if (blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) epilogue_ranges<SUM ? kEpiSum : kEpiPlain>(p.epi);
}

template <int KS, int NI>
void launch_stream(hipStream_t s, const FcArgs& a, long cus, int groups_per_cu) {
  // the residual operand is read in 16-byte pieces, like the output is written
  MXQ_CHECK(a.epi.res == nullptr || aligned16(a.epi.res), "unaligned residual operand");
  constexpr int TN = 32 * NI;
  const int max_rows = KS <= 4 ? 256 : 128;
  const int bn = a.N < max_rows ? a.N : max_rows;
  const int ny = (a.N + bn - 1) / bn;
  const int strips = bn / TN;
  const long items = static_cast<long>((a.M + 31) / 32) * strips;
  long gx = cus * groups_per_cu / ny;
  if (gx < 1) gx = 1;
  if (gx * 4 > items) gx = (items + 3) / 4;
  if (a.epi.res != nullptr)
    hipLaunchKernelGGL((fc_stream_kernel<KS, NI, true>), dim3(static_cast<unsigned>(gx), ny),
                       dim3(256), 0, s, a, bn, strips);
  else
    hipLaunchKernelGGL((fc_stream_kernel<KS, NI, false>), dim3(static_cast<unsigned>(gx), ny),
                       dim3(256), 0, s, a, bn, strips);
  MXQ_LAUNCH_CHECK();
}

template <class Cfg, int NS, int PIPE, bool BUF>
void launch_dma(hipStream_t s, FcArgs a, int splits, const Workspace& ws) {
  const long tiles = static_cast<long>((a.M + Cfg::BM - 1) / Cfg::BM) * ((a.N + Cfg::BN - 1) / Cfg::BN);
  splitk_setup<Cfg>(s, a.sk, tiles, a.K, splits, ws.ptr, ws.bytes);
  const dim3 grid(static_cast<unsigned>(tiles * a.sk.splits));
  switch (epi_mode(a.epi)) {
    case kEpiF32:
      hipLaunchKernelGGL((fc_dma_kernel<Cfg, NS, PIPE, BUF, kEpiF32>), grid, dim3(Cfg::kThreads),
                         0, s, a);
      break;
    case kEpiSum:
      hipLaunchKernelGGL((fc_dma_kernel<Cfg, NS, PIPE, BUF, kEpiSum>), grid, dim3(Cfg::kThreads),
                         0, s, a);
      break;
    default:
      hipLaunchKernelGGL((fc_dma_kernel<Cfg, NS, PIPE, BUF, kEpiPlain>), grid,
                         dim3(Cfg::kThreads), 0, s, a);
  }
  MXQ_LAUNCH_CHECK();
}

template <class Cfg>
void launch_cfg(hipStream_t s, const FcArgs& a, bool aligned) {
  const int tiles = ((a.M + Cfg::BM - 1) / Cfg::BM) * ((a.N + Cfg::BN - 1) / Cfg::BN);
  const int mode = epi_mode(a.epi);
#define MXQ_FC_KERNEL(ALIGNED, MODE) \
  hipLaunchKernelGGL((fc_kernel<Cfg, ALIGNED, MODE>), dim3(tiles), dim3(Cfg::kThreads), 0, s, a)
  if (aligned) {
    if (mode == kEpiF32) MXQ_FC_KERNEL(true, kEpiF32);
    else if (mode == kEpiSum) MXQ_FC_KERNEL(true, kEpiSum);
    else MXQ_FC_KERNEL(true, kEpiPlain);
  } else {
    if (mode == kEpiF32) MXQ_FC_KERNEL(false, kEpiF32);
    else if (mode == kEpiSum) MXQ_FC_KERNEL(false, kEpiSum);
    else MXQ_FC_KERNEL(false, kEpiPlain);
  }
#undef MXQ_FC_KERNEL
  MXQ_LAUNCH_CHECK();
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
//   60      256x192 with 128-byte stages (outputs whose width is a multiple of 192)
//   61, 62  the short-K streaming kernel with 64- / 128-column strips
// Output tile of a direct-to-LDS configuration (what a split-K work-group leaves in the
// workspace); false for every other configuration.
bool fc_cfg_tile(int cfg, int& bm, int& bn) {
  switch (cfg) {
    case 11: case 12: case 14: case 16: case 31: case 32: case 55: bm = 256; bn = 256; return true;
    case 21: case 41: case 56: bm = 256; bn = 128; return true;
    case 22: case 42: bm = 256; bn = 64; return true;
    case 23: case 43: case 53: case 54: bm = 128; bn = 128; return true;
    case 24: case 44: case 51: case 52: case 59: bm = 64; bn = 64; return true;
    case 57: bm = 128; bn = 64; return true;
    case 58: bm = 64; bn = 128; return true;
    case 60: bm = 256; bn = 192; return true;
    default: return false;
  }
}

struct FcPlan {
  int cfg;
  int splits;
  int stream_groups;
};

// What launch_fc would run for this shape.  `aligned`: K % 16 == 0 and 16-byte aligned
// operands; `fused8`: int8 output only, 16-byte aligned with a row pitch that is a
// multiple of 16 (what the streaming kernel stores).
// `sum`: the residual-sum form, whose epilogue does twice the arithmetic per output.
FcPlan plan_fc(int M, int N, int K, bool aligned, bool fused8, const GemmForce& force,
               bool sum = false) {
  FcPlan plan = {force.cfg, force.splits, force.stream_groups > 0 ? force.stream_groups : 2};
  const bool buf_ok = aligned && K >= 16 && static_cast<long long>(M) * K < (1LL << 31) &&
                      static_cast<long long>(N) * K < (1LL << 31);
  const bool glb_ok = buf_ok && (K % 64 == 0);
  const long cus = num_cus();
  if (plan.cfg == 0) {
    auto tiles = [&](int bm, int bn) {
      return static_cast<long>((M + bm - 1) / bm) * ((N + bn - 1) / bn);
    };
    int auto_splits = 1;
    if (buf_ok) {
      switch (choose_tile(M, N, K, cus, false, &auto_splits)) {
        case Tile::kL8: plan.cfg = glb_ok ? 12 : 31; break;
        case Tile::kW128x2: plan.cfg = 41; break;
        case Tile::kW128K2: plan.cfg = 56; break;
        case Tile::kM128x2: plan.cfg = 43; break;
        case Tile::kM128K2: plan.cfg = 53; break;
        case Tile::kS64x2: plan.cfg = 44; break;
        case Tile::kS64x4: plan.cfg = 24; break;
        case Tile::kS64K2: plan.cfg = 51; break;
        case Tile::kR128K2: plan.cfg = 57; break;
        case Tile::kQ128K2: plan.cfg = 58; break;
        case Tile::kS64K4: plan.cfg = 59; break;
        case Tile::kW192K2: plan.cfg = 60; break;
      }
    } else {
      if (tiles(256, 256) >= cus)
        plan.cfg = 1;
      else if (tiles(128, 128) >= cus)
        plan.cfg = 3;
      else
        plan.cfg = 4;
    }
    if (plan.splits == 0) plan.splits = auto_splits;
    // With the residual sum in the epilogue the balance moves (sweeps of every configuration
    // per layer inside the chained ResNet-50 body at batch 64): where the plain form takes
    // 256 x 128 tiles on 64-byte stages, 256 x 256 tiles on 128-byte stages are ahead once
    // they cover 0.56 of the CUs (12544 x 256 -> 1024: -1.9 us per layer) and 128 x 128
    // tiles otherwise (50176 x 128 -> 512: -1.2 us per layer).
    if (sum && plan.cfg == 41) {
      if (K >= 256 && N > 128 && 16 * tiles(256, 256) >= 9 * cus)
        plan.cfg = 55;
      else
        plan.cfg = 43;
    }
    // the short-K streaming kernel: chosen for tall outputs of at most 256 columns
    // (200704 x 64 -> 64: 8.5 us against 10.2; -> 256: 18.5 against 21.9; 200704 x 128 ->
    // 128: 15.3 against 17.1); from 512 columns on the tiled kernels are level or ahead
    const int stream_rows = K == 256 ? 128 : 256;
    const bool stream_ok = aligned && fused8 && (K == 32 || K == 64 || K == 128 || K == 256) &&
                           N % 64 == 0 && (N <= stream_rows || N % stream_rows == 0);
    if (stream_ok && N <= 256 && K <= 128 && M >= 32768) {
      plan.cfg = (N % 128 == 0) ? 62 : 61;
      plan.splits = 1;
      if (force.stream_groups <= 0) plan.stream_groups = K <= 64 ? 4 : 3;
      // the sum's extra registers and arithmetic favour the 64-column strips with more
      // groups in flight (200704 x 64 -> 256 inside the chain: -7 us per layer)
      if (sum && K <= 64) {
        plan.cfg = 61;
        if (force.stream_groups <= 0) plan.stream_groups = 5;
      }
    }
  }
  if (plan.splits <= 0) plan.splits = 1;
  return plan;
}

size_t fc_plan_workspace(const FcPlan& plan, int M, int N) {
  int bm, bn;
  if (plan.splits <= 1 || !fc_cfg_tile(plan.cfg, bm, bn)) return 0;
  const long tiles = static_cast<long>((M + bm - 1) / bm) * ((N + bn - 1) / bn);
  return splitk_workspace_bytes(tiles, plan.splits, bm, bn);
}

// an output without elements still owes its range scalars
__global__ void gemm_ranges_kernel(Epilogue e) { epilogue_ranges<kEpiSum>(e); }

void launch_fc(hipStream_t s, const int8_t* data, const int8_t* weight, int M, int N, int K,
               int ldo, const Epilogue& epi, const GemmForce& force, const Workspace& ws) {
  if (M == 0 || N == 0) {
    hipLaunchKernelGGL(gemm_ranges_kernel, dim3(1), dim3(1), 0, s, epi);
    MXQ_LAUNCH_CHECK();
    return;
  }
  FcArgs a;
  a.data = data;
  a.weight = weight;
  a.M = M;
  a.N = N;
  a.K = K;
  a.ldo = ldo;
  a.epi = epi;
  a.epi.stream8 = epi_stream_rows(M);
  a.sk.splits = 1;
  a.sk.kt_per_split = 1 << 30;
  a.sk.counters = nullptr;
  a.sk.partials = nullptr;
  const bool aligned = (K % 16 == 0) && aligned16(data) && aligned16(weight);
  // direct-to-LDS kernels: operands below 2 GiB; K a multiple of the 64-byte stage for
  // the global-load form, of 16 for the buffer-load form
  const bool buf_ok = aligned && K >= 16 && static_cast<long long>(M) * K < (1LL << 31) &&
                      static_cast<long long>(N) * K < (1LL << 31);
  const bool glb_ok = buf_ok && (K % 64 == 0);
  const bool fused8 = epi.out32 == nullptr && epi.outf == nullptr && epi.out8 != nullptr &&
                      ldo % 16 == 0 && aligned16(epi.out8) &&
                      (epi.res == nullptr || aligned16(epi.res));
  const bool sum = epi.res != nullptr;
  FcPlan plan = plan_fc(M, N, K, aligned, fused8, force, sum);
  // a split the chooser proposed is dropped when the caller brought no room for it
  if (force.splits == 0 && plan.splits > 1 &&
      (ws.ptr == nullptr || !aligned16(ws.ptr) || ws.bytes < fc_plan_workspace(plan, M, N))) {
    GemmForce unsplit = force;
    unsplit.splits = 1;
    plan = plan_fc(M, N, K, aligned, fused8, unsplit, sum);
  }
  const int cfg = plan.cfg;
  if (cfg >= 11 && cfg <= 16) MXQ_CHECK(glb_ok, "shape does not qualify for the DMA kernels");
  if (cfg == 61 || cfg == 62) {
    const int stream_rows = K == 256 ? 128 : 256;  // weight rows one work-group parks in LDS
    const bool stream_ok = aligned && fused8 && (K == 32 || K == 64 || K == 128 || K == 256) &&
                           N % 64 == 0 && (N <= stream_rows || N % stream_rows == 0);
    MXQ_CHECK(stream_ok && (cfg == 61 || N % 128 == 0),
              "shape does not qualify for the short-K streaming kernel");
    MXQ_CHECK(plan.stream_groups >= 1 && plan.stream_groups <= 16, "stream_groups out of range");
    const long cus = num_cus();
#define MXQ_STREAM(NI)                                                          \
  do {                                                                          \
    if (K == 32) launch_stream<1, NI>(s, a, cus, plan.stream_groups);           \
    else if (K == 64) launch_stream<2, NI>(s, a, cus, plan.stream_groups);      \
    else if (K == 128) launch_stream<4, NI>(s, a, cus, plan.stream_groups);     \
    else launch_stream<8, NI>(s, a, cus, plan.stream_groups);                   \
  } while (0)
    if (cfg == 61) MXQ_STREAM(2); else MXQ_STREAM(4);
#undef MXQ_STREAM
    return;
  }
  if (cfg >= 21) MXQ_CHECK(buf_ok, "shape does not qualify for the buffer-load DMA kernels");
  if (cfg < 11) MXQ_CHECK(plan.splits <= 1, "the register-staged kernels have no split-K form");
  const int sp = plan.splits;
  switch (cfg) {
    case 1: launch_cfg<CfgL8>(s, a, aligned); break;
    case 2: launch_cfg<CfgL4>(s, a, aligned); break;
    case 3: launch_cfg<CfgM>(s, a, aligned); break;
    case 4: launch_cfg<CfgS>(s, a, aligned); break;
    case 11: launch_dma<CfgL8, 4, 0, false>(s, a, sp, ws); break;
    case 12: launch_dma<CfgL8, 4, 2, false>(s, a, sp, ws); break;
    case 14: launch_dma<CfgL4, 4, 0, false>(s, a, sp, ws); break;
    case 16: launch_dma<CfgL4, 4, 2, false>(s, a, sp, ws); break;
    case 21: launch_dma<CfgW128, 4, 2, true>(s, a, sp, ws); break;
    case 22: launch_dma<CfgW64, 4, 2, true>(s, a, sp, ws); break;
    case 23: launch_dma<CfgM, 4, 2, true>(s, a, sp, ws); break;
    case 24: launch_dma<CfgS, 4, 2, true>(s, a, sp, ws); break;
    case 41: launch_dma<CfgW128, 2, 0, true>(s, a, sp, ws); break;
    case 42: launch_dma<CfgW64, 2, 0, true>(s, a, sp, ws); break;
    case 43: launch_dma<CfgM, 2, 0, true>(s, a, sp, ws); break;
    case 44: launch_dma<CfgS, 2, 0, true>(s, a, sp, ws); break;
    case 51: launch_dma<CfgSK, 2, 0, true>(s, a, sp, ws); break;
    case 52: launch_dma<CfgSK, 3, 0, true>(s, a, sp, ws); break;
    case 53: launch_dma<CfgMK, 2, 0, true>(s, a, sp, ws); break;
    case 54: launch_dma<CfgMK, 3, 0, true>(s, a, sp, ws); break;
    case 55: launch_dma<CfgL8K, 2, 0, true>(s, a, sp, ws); break;
    case 56: launch_dma<CfgW128K, 2, 0, true>(s, a, sp, ws); break;
    case 57: launch_dma<CfgRK, 2, 0, true>(s, a, sp, ws); break;
    case 58: launch_dma<CfgQK, 2, 0, true>(s, a, sp, ws); break;
    case 59: launch_dma<CfgSK2, 2, 0, true>(s, a, sp, ws); break;
    case 60: launch_dma<CfgW192K, 2, 0, true>(s, a, sp, ws); break;
    case 31: launch_dma<CfgL8, 4, 2, true>(s, a, sp, ws); break;
    case 32: launch_dma<CfgL4, 4, 2, true>(s, a, sp, ws); break;
    default: MXQ_CHECK(false, "unknown fc tile configuration " << cfg);
  }
}

// Scratch bytes with which launch_fc takes its fastest route for this shape (0 when it
// would not split).  Assumes 16-byte aligned operands.
size_t fc_workspace_bytes(int M, int N, int K, bool fused8) {
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  const FcPlan plan = plan_fc(M, N, K, K % 16 == 0, fused8, GemmForce());
  return fc_plan_workspace(plan, M, N);
}

}  // namespace mxq

using namespace mxq;

namespace {

// The residual sum fused behind the requantization (mxq_quantized_fc_sum).
struct SumArgs {
  const int8_t* res;
  const float* res_min;
  const float* res_max;
  float min_calib, max_calib;
  int relu;
};

void fc_entry(void* stream, const int8_t* data, const int8_t* weight, const int8_t* bias, int M,
              int N, int K, const float* min_data, const float* max_data,
              const float* min_weight, const float* max_weight, const float* min_bias,
              const float* max_bias, int32_t* out32, float* omin, float* omax, int8_t* out8,
              float* out_f32, float* rmin, float* rmax, int relu, float min_calib,
              float max_calib, void* workspace, size_t workspace_bytes, const GemmForce& force,
              const SumArgs* sum = nullptr) {
  MXQ_CHECK(M >= 0 && N >= 0 && K >= 0, "negative dimension");
  MXQ_CHECK(min_data && max_data && min_weight && max_weight, "null input range pointer");
  MXQ_CHECK(omin && omax, "null output range pointer");
  MXQ_CHECK(bias == nullptr || (min_bias && max_bias), "bias given without its range");
  MXQ_CHECK(M == 0 || N == 0 || out32 != nullptr || out8 != nullptr || out_f32 != nullptr,
            "no output buffer");
  MXQ_CHECK((out8 == nullptr && out_f32 == nullptr) || (rmin && rmax),
            "fused requantize needs rmin/rmax");
  MXQ_CHECK(M == 0 || N == 0 || K == 0 || (data != nullptr && weight != nullptr),
            "null operand pointer");
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
  e.outf = out_f32;
  e.res = nullptr;
  e.res_min = e.res_max = nullptr;
  e.sum_min_calib = e.sum_max_calib = 0.f;
  e.sum_relu = 0;
  e.with_sum = 0;
  if (sum != nullptr) {
    MXQ_CHECK((M == 0 || N == 0 || out8 != nullptr) && out32 == nullptr && out_f32 == nullptr,
              "the fused sum writes the int8 output only");
    MXQ_CHECK(sum->res_min && sum->res_max, "null residual range pointer");
    MXQ_CHECK(M == 0 || N == 0 || sum->res != nullptr, "null residual operand");
    if (M != 0 && N != 0) {  // without elements only the ranges are written
      e.res = sum->res;
      e.res_min = sum->res_min;
      e.res_max = sum->res_max;
    }
    e.sum_min_calib = sum->min_calib;
    e.sum_max_calib = sum->max_calib;
    e.sum_relu = sum->relu;
    e.with_sum = 1;
  }
  e.omin = omin;
  e.omax = omax;
  e.rmin = rmin;
  e.rmax = rmax;
  e.relu = relu;
  float a = fabsf(min_calib), b = fabsf(max_calib);
  e.real_range = (a < b) ? b : a;
  e.plane = 0;
  Workspace ws;
  ws.ptr = workspace;
  ws.bytes = workspace_bytes;
  launch_fc(static_cast<hipStream_t>(stream), data, weight, M, N, K, N, e, force, ws);
}

}  // namespace

extern "C" {

size_t mxq_quantized_fc_workspace(int M, int N, int K, int fused_int8_only) {
  try {
    return fc_workspace_bytes(M, N, K, fused_int8_only != 0 && N % 16 == 0);
  } catch (...) {
    return 0;
  }
}

int mxq_quantized_fc(void* stream, const int8_t* data, const int8_t* weight, const int8_t* bias,
                     int M, int N, int K, const float* min_data, const float* max_data,
                     const float* min_weight, const float* max_weight, const float* min_bias,
                     const float* max_bias, int32_t* out32, float* omin, float* omax,
                     int8_t* out8, float* rmin, float* rmax, int relu, float min_calib,
                     float max_calib, void* workspace, size_t workspace_bytes) {
  MXQ_API_BEGIN();
  fc_entry(stream, data, weight, bias, M, N, K, min_data, max_data, min_weight, max_weight,
           min_bias, max_bias, out32, omin, omax, out8, nullptr, rmin, rmax, relu, min_calib,
           max_calib, workspace, workspace_bytes, GemmForce());
  MXQ_API_END();
}

// Test-only twin of mxq_quantized_fc (declared in tests/mxq_test_hooks.h, not in the
// operator header): the tile configuration, the split-K factor and the streaming kernel's
// work-groups per CU come as arguments (0 = let the launcher choose), so tests can drive
// every kernel variant on any shape without process-wide state.
int mxq_test_quantized_fc(void* stream, const int8_t* data, const int8_t* weight,
                          const int8_t* bias, int M, int N, int K, const float* min_data,
                          const float* max_data, const float* min_weight,
                          const float* max_weight, const float* min_bias, const float* max_bias,
                          int32_t* out32, float* omin, float* omax, int8_t* out8, float* rmin,
                          float* rmax, int relu, float min_calib, float max_calib,
                          void* workspace, size_t workspace_bytes, int cfg, int splits,
                          int stream_groups) {
  MXQ_API_BEGIN();
  GemmForce force;
  force.cfg = cfg;
  force.splits = splits;
  force.stream_groups = stream_groups;
  fc_entry(stream, data, weight, bias, M, N, K, min_data, max_data, min_weight, max_weight,
           min_bias, max_bias, out32, omin, omax, out8, nullptr, rmin, rmax, relu, min_calib,
           max_calib, workspace, workspace_bytes, force);
  MXQ_API_END();
}

int mxq_quantized_fc_f32(void* stream, const int8_t* data, const int8_t* weight,
                         const int8_t* bias, int M, int N, int K, const float* min_data,
                         const float* max_data, const float* min_weight, const float* max_weight,
                         const float* min_bias, const float* max_bias, float* out_f32,
                         float* omin, float* omax, float* rmin, float* rmax, int relu,
                         float min_calib, float max_calib, void* workspace,
                         size_t workspace_bytes) {
  MXQ_API_BEGIN();
  MXQ_CHECK(M == 0 || N == 0 || out_f32 != nullptr, "no output buffer");
  fc_entry(stream, data, weight, bias, M, N, K, min_data, max_data, min_weight, max_weight,
           min_bias, max_bias, nullptr, omin, omax, nullptr, out_f32, rmin, rmax, relu,
           min_calib, max_calib, workspace, workspace_bytes, GemmForce());
  MXQ_API_END();
}

int mxq_quantized_fc_sum(void* stream, const int8_t* data, const int8_t* weight,
                         const int8_t* bias, int M, int N, int K, const float* min_data,
                         const float* max_data, const float* min_weight, const float* max_weight,
                         const float* min_bias, const float* max_bias, const int8_t* residual,
                         const float* min_residual, const float* max_residual, int8_t* out8,
                         float* omin, float* omax, float* rmin, float* rmax, float min_calib,
                         float max_calib, float sum_min_calib, float sum_max_calib, int sum_relu,
                         void* workspace, size_t workspace_bytes) {
  MXQ_API_BEGIN();
  const SumArgs sum = {residual, min_residual, max_residual, sum_min_calib, sum_max_calib,
                       sum_relu};
  fc_entry(stream, data, weight, bias, M, N, K, min_data, max_data, min_weight, max_weight,
           min_bias, max_bias, nullptr, omin, omax, out8, nullptr, rmin, rmax, 0, min_calib,
           max_calib, workspace, workspace_bytes, GemmForce(), &sum);
  MXQ_API_END();
}

// Test-only twin of mxq_quantized_fc_sum with the kernel variant pinned
// (tests/mxq_test_hooks.h).
int mxq_test_quantized_fc_sum(void* stream, const int8_t* data, const int8_t* weight,
                              const int8_t* bias, int M, int N, int K, const float* min_data,
                              const float* max_data, const float* min_weight,
                              const float* max_weight, const float* min_bias,
                              const float* max_bias, const int8_t* residual,
                              const float* min_residual, const float* max_residual,
                              int8_t* out8, float* omin, float* omax, float* rmin, float* rmax,
                              float min_calib, float max_calib, float sum_min_calib,
                              float sum_max_calib, int sum_relu, void* workspace,
                              size_t workspace_bytes, int cfg, int splits, int stream_groups) {
  MXQ_API_BEGIN();
  const SumArgs sum = {residual, min_residual, max_residual, sum_min_calib, sum_max_calib,
                       sum_relu};
  GemmForce force;
  force.cfg = cfg;
  force.splits = splits;
  force.stream_groups = stream_groups;
  fc_entry(stream, data, weight, bias, M, N, K, min_data, max_data, min_weight, max_weight,
           min_bias, max_bias, nullptr, omin, omax, out8, nullptr, rmin, rmax, 0, min_calib,
           max_calib, workspace, workspace_bytes, force, &sum);
  MXQ_API_END();
}

// Test-only twin of mxq_quantized_fc_f32 with the tile configuration and the split-K factor
// pinned (tests/mxq_test_hooks.h).
int mxq_test_quantized_fc_f32(void* stream, const int8_t* data, const int8_t* weight,
                              const int8_t* bias, int M, int N, int K, const float* min_data,
                              const float* max_data, const float* min_weight,
                              const float* max_weight, const float* min_bias,
                              const float* max_bias, float* out_f32, float* omin, float* omax,
                              float* rmin, float* rmax, int relu, float min_calib,
                              float max_calib, void* workspace, size_t workspace_bytes, int cfg,
                              int splits) {
  MXQ_API_BEGIN();
  MXQ_CHECK(M == 0 || N == 0 || out_f32 != nullptr, "no output buffer");
  GemmForce force;
  force.cfg = cfg;
  force.splits = splits;
  force.stream_groups = 0;
  fc_entry(stream, data, weight, bias, M, N, K, min_data, max_data, min_weight, max_weight,
           min_bias, max_bias, nullptr, omin, omax, nullptr, out_f32, rmin, rmax, relu,
           min_calib, max_calib, workspace, workspace_bytes, force);
  MXQ_API_END();
}

}  // extern "C"
