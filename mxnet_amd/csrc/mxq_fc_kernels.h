// The fully-connected kernels and their launch templates (see mxq_fc.hip for the operator
// they serve and the list of tile configurations).  Included by one translation unit per
// epilogue mode, which instantiates every configuration for that mode through
// fc_launch_mode<MODE>.
#ifndef MXQ_FC_KERNELS_H_
#define MXQ_FC_KERNELS_H_

#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <type_traits>

#include "../../include/mxq.h"
#include "mxq_common.h"
#include "mxq_fc_args.h"
#include "mxq_gemm.h"
#include "mxq_tiles.h"

namespace mxq {

namespace {


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

template <int KS, int NI, bool SUM>
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
  hipLaunchKernelGGL((fc_stream_kernel<KS, NI, SUM>), dim3(static_cast<unsigned>(gx), ny),
                     dim3(256), 0, s, a, bn, strips);
  MXQ_LAUNCH_CHECK();
}

template <class Cfg, int NS, int PIPE, bool BUF, int MODE>
void launch_dma(hipStream_t s, FcArgs a, int splits, const Workspace& ws) {
  const long tiles = static_cast<long>((a.M + Cfg::BM - 1) / Cfg::BM) * ((a.N + Cfg::BN - 1) / Cfg::BN);
  splitk_setup<Cfg>(s, a.sk, tiles, a.K, splits, ws.ptr, ws.bytes);
  hipLaunchKernelGGL((fc_dma_kernel<Cfg, NS, PIPE, BUF, MODE>),
                     dim3(static_cast<unsigned>(tiles * a.sk.splits)), dim3(Cfg::kThreads), 0, s,
                     a);
  MXQ_LAUNCH_CHECK();
}

template <class Cfg, int MODE>
void launch_cfg(hipStream_t s, const FcArgs& a, bool aligned) {
  const int tiles = ((a.M + Cfg::BM - 1) / Cfg::BM) * ((a.N + Cfg::BN - 1) / Cfg::BN);
  if (aligned)
    hipLaunchKernelGGL((fc_kernel<Cfg, true, MODE>), dim3(tiles), dim3(Cfg::kThreads), 0, s, a);
  else
    hipLaunchKernelGGL((fc_kernel<Cfg, false, MODE>), dim3(tiles), dim3(Cfg::kThreads), 0, s, a);
  MXQ_LAUNCH_CHECK();
}

// Every configuration for one epilogue mode.
template <int MODE>
void fc_launch_mode(hipStream_t s, const FcArgs& a, const FcLaunch& how, const Workspace& ws) {
  const int cfg = how.cfg, sp = how.splits;
  if (cfg == 61 || cfg == 62) {
    // the streaming kernel writes the int8 output (with or without the residual sum)
    if constexpr (MODE == kEpiF32) {
      MXQ_CHECK(false, "the short-K streaming kernel has no float-output form");
    } else {
      constexpr bool SUM = MODE == kEpiSum;
      const long cus = num_cus();
#define MXQ_STREAM(NI)                                                             \
  do {                                                                             \
    if (a.K == 32) launch_stream<1, NI, SUM>(s, a, cus, how.stream_groups);        \
    else if (a.K == 64) launch_stream<2, NI, SUM>(s, a, cus, how.stream_groups);   \
    else if (a.K == 128) launch_stream<4, NI, SUM>(s, a, cus, how.stream_groups);  \
    else launch_stream<8, NI, SUM>(s, a, cus, how.stream_groups);                  \
  } while (0)
      if (cfg == 61) MXQ_STREAM(2); else MXQ_STREAM(4);
#undef MXQ_STREAM
    }
    return;
  }
  switch (cfg) {
    case 1: launch_cfg<CfgL8, MODE>(s, a, how.aligned); break;
    case 2: launch_cfg<CfgL4, MODE>(s, a, how.aligned); break;
    case 3: launch_cfg<CfgM, MODE>(s, a, how.aligned); break;
    case 4: launch_cfg<CfgS, MODE>(s, a, how.aligned); break;
    case 11: launch_dma<CfgL8, 4, 0, false, MODE>(s, a, sp, ws); break;
    case 12: launch_dma<CfgL8, 4, 2, false, MODE>(s, a, sp, ws); break;
    case 14: launch_dma<CfgL4, 4, 0, false, MODE>(s, a, sp, ws); break;
    case 16: launch_dma<CfgL4, 4, 2, false, MODE>(s, a, sp, ws); break;
    case 21: launch_dma<CfgW128, 4, 2, true, MODE>(s, a, sp, ws); break;
    case 22: launch_dma<CfgW64, 4, 2, true, MODE>(s, a, sp, ws); break;
    case 23: launch_dma<CfgM, 4, 2, true, MODE>(s, a, sp, ws); break;
    case 24: launch_dma<CfgS, 4, 2, true, MODE>(s, a, sp, ws); break;
    case 41: launch_dma<CfgW128, 2, 0, true, MODE>(s, a, sp, ws); break;
    case 42: launch_dma<CfgW64, 2, 0, true, MODE>(s, a, sp, ws); break;
    case 43: launch_dma<CfgM, 2, 0, true, MODE>(s, a, sp, ws); break;
    case 44: launch_dma<CfgS, 2, 0, true, MODE>(s, a, sp, ws); break;
    case 51: launch_dma<CfgSK, 2, 0, true, MODE>(s, a, sp, ws); break;
    case 52: launch_dma<CfgSK, 3, 0, true, MODE>(s, a, sp, ws); break;
    case 53: launch_dma<CfgMK, 2, 0, true, MODE>(s, a, sp, ws); break;
    case 54: launch_dma<CfgMK, 3, 0, true, MODE>(s, a, sp, ws); break;
    case 55: launch_dma<CfgL8K, 2, 0, true, MODE>(s, a, sp, ws); break;
    case 56: launch_dma<CfgW128K, 2, 0, true, MODE>(s, a, sp, ws); break;
    case 57: launch_dma<CfgRK, 2, 0, true, MODE>(s, a, sp, ws); break;
    case 58: launch_dma<CfgQK, 2, 0, true, MODE>(s, a, sp, ws); break;
    case 59: launch_dma<CfgSK2, 2, 0, true, MODE>(s, a, sp, ws); break;
    case 60: launch_dma<CfgW192K, 2, 0, true, MODE>(s, a, sp, ws); break;
    case 31: launch_dma<CfgL8, 4, 2, true, MODE>(s, a, sp, ws); break;
    case 32: launch_dma<CfgL4, 4, 2, true, MODE>(s, a, sp, ws); break;
    default: MXQ_CHECK(false, "unknown fc tile configuration " << cfg);
  }
}

}  // namespace

}  // namespace mxq
#endif  // MXQ_FC_KERNELS_H_
