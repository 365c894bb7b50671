// _contrib_quantized_conv on gfx950: implicit-GEMM int8 convolution on NHWC
// operands with the same MFMA core and epilogue as the fully-connected kernel.
// Replaces cudnnConvolutionForward (NHWC int8, IMPLICIT_PRECOMP_GEMM), the
// float->int32 cast and QuantizedBiasAddKernel of the reference's GPU operator
// (src/operator/quantization/quantized_conv.cu:101-219); the accumulator stays an
// exact int32 and the bias is added in integers.
//
// GEMM view: rows m = (n, oh, ow), columns = output channel o, reduction
// k = (kh, kw, c) with c fastest, which is the memory order of both the NHWC
// activation pixel and the OHWI weight row.  Out-of-image taps and the K tail are
// zero-filled by the loader, so no padded copy of the input is ever made.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>

#include "../../include/mxq.h"
#include "mxq_common.h"
#include "mxq_thin_transpose.h"
#include "mxq_gemm.h"
#include "mxq_tiles.h"

namespace mxq {

void launch_fc(hipStream_t s, const int8_t* data, const int8_t* weight, int M, int N, int K,
               int ldo, const Epilogue& epi, const GemmForce& force, const Workspace& ws);
size_t fc_workspace_bytes(int M, int N, int K, bool fused8);

namespace {

struct ConvArgs {
  const int8_t* data;    // [N][H][W][C]
  const int8_t* weight;  // [O][KH][KW][C]
  int N, H, W, C, O, KH, KW;
  int sh, sw, ph, pw, dh, dw, OH, OW;
  int M, K;  // N*OH*OW, KH*KW*C
  Epilogue epi;
  SplitK sk;
};

// Activation loader: row = output pixel, chunk = 16 channels of one filter tap.
template <class Cfg, int CHUNKS, bool ALIGNED>
struct ConvFetch {
  const int8_t* img[CHUNKS];  // start of image n
  int ih0[CHUNKS], iw0[CHUNKS];
  bool ok[CHUNKS];
  int lc;
  int C, KW, H, W, K, dh, dw;

  __device__ __forceinline__ void init(const ConvArgs& args, int row0) {
    C = args.C; KW = args.KW; H = args.H; W = args.W; K = args.K;
    dh = args.dh; dw = args.dw;
    lc = threadIdx.x % Cfg::CH;
    const int lr = threadIdx.x / Cfg::CH;
    const int ohow = args.OH * args.OW;
#pragma unroll
    for (int j = 0; j < CHUNKS; ++j) {
      const int m = row0 + lr + j * Cfg::ROWS_PER_PASS;
      ok[j] = m < args.M;
      const int mm = ok[j] ? m : 0;
      const int n = mm / ohow;
      const int rem = mm - n * ohow;
      const int oh = rem / args.OW;
      const int ow = rem - oh * args.OW;
      img[j] = args.data + static_cast<size_t>(n) * args.H * args.W * args.C;
      ih0[j] = oh * args.sh - args.ph;
      iw0[j] = ow * args.sw - args.pw;
    }
  }

  __device__ __forceinline__ void fetch(int kt, v4i (&reg)[CHUNKS]) {
    const int k0 = kt * Cfg::BK + lc * 16;
    if (ALIGNED) {
      // C % 16 == 0: the 16 bytes lie inside one tap
      const bool k_ok = k0 < K;
      const int tap = k0 / C;
      const int c = k0 - tap * C;
      const int kh = tap / KW;
      const int kw = tap - kh * KW;
      const int dih = kh * dh, diw = kw * dw;
#pragma unroll
      for (int j = 0; j < CHUNKS; ++j) {
        const int ih = ih0[j] + dih, iw = iw0[j] + diw;
        const bool v = ok[j] && k_ok && ih >= 0 && ih < H && iw >= 0 && iw < W;
        v4i r = {0, 0, 0, 0};
        if (v)
          r = *reinterpret_cast<const v4i*>(img[j] +
                                            (static_cast<size_t>(ih) * W + iw) * C + c);
        reg[j] = r;
      }
    } else {
#pragma unroll
      for (int j = 0; j < CHUNKS; ++j) {
        v4i r = {0, 0, 0, 0};
        if (ok[j]) {
          for (int i = 0; i < 16; ++i) {
            const int k = k0 + i;
            if (k >= K) break;
            const int tap = k / C;
            const int c = k - tap * C;
            const int kh = tap / KW;
            const int kw = tap - kh * KW;
            const int ih = ih0[j] + kh * dh, iw = iw0[j] + kw * dw;
            if (ih >= 0 && ih < H && iw >= 0 && iw < W) {
              uint32_t b =
                  static_cast<uint8_t>(img[j][(static_cast<size_t>(ih) * W + iw) * C + c]);
              r[i >> 2] |= static_cast<int>(b << (8 * (i & 3)));
            }
          }
        }
        reg[j] = r;
      }
    }
  }
};

template <class Cfg, bool ALIGNED>
__global__ __launch_bounds__(Cfg::kThreads, Cfg::kMinWaves) void conv_kernel(ConvArgs p) {
  __shared__ __attribute__((aligned(16))) v4i lds[2][Cfg::STAGE_SLOTS];
  const int wave = threadIdx.x >> 6;
  const int wm = wave / Cfg::WN, wn = wave % Cfg::WN;
  const int tiles_m = (p.M + Cfg::BM - 1) / Cfg::BM, tiles_n = (p.O + Cfg::BN - 1) / Cfg::BN;
  int tm, tn;
  tile_coords(blockIdx.x, tiles_m, tiles_n, tm, tn);
  const int m0 = tm * Cfg::BM, n0 = tn * Cfg::BN;

  ConvFetch<Cfg, Cfg::A_CHUNKS, ALIGNED> af;
  RowFetch<Cfg, Cfg::B_CHUNKS, ALIGNED> bf;
  af.init(p, m0);
  bf.init(p.weight, n0, p.O, p.K);

  v16i acc[Cfg::MI][Cfg::NI];
  gemm_mainloop<Cfg>(acc, af, bf, (p.K + Cfg::BK - 1) / Cfg::BK, lds);

  gemm_epilogue<Cfg>(acc, p.epi, m0 + wm * Cfg::TM, n0 + wn * Cfg::TN, p.M, p.O,
                     static_cast<size_t>(p.O));
  if (blockIdx.x == 0 && threadIdx.x == 0) epilogue_ranges(p.epi);
}

// Activation operand of the direct-to-LDS main loop: lane state for "16 channels of
// one filter tap of one output pixel", advanced stage by stage without divisions.
// Halo taps, rows past the last pixel and the K tail are sent to an out-of-range
// buffer offset and arrive in LDS as zeros.  Needs C % 16 == 0.
template <class Cfg, int INSTR>
struct ConvIssuer {
  int pix[INSTR];           // byte offset of pixel (n, ih0, iw0), may be negative
  int ih0[INSTR], iw0[INSTR];
  bool ok[INSTR];
  int cc, kh, kw;           // position of this lane's chunk in the stage issued next
  int dih, diw, tapoff;     // kh*dilate_h, kw*dilate_w, ((kh*dh)*W + kw*dw)*C
  int C, H, W, KH, KW, dh, dw;
  v4i rsrc;

  // kbeg: reduction index (a multiple of the stage depth) at which stage 0 starts
  __device__ __forceinline__ void init(const ConvArgs& a, int row_begin, int wave, int lane,
                                       int kbeg = 0) {
    C = a.C; H = a.H; W = a.W; KH = a.KH; KW = a.KW; dh = a.dh; dw = a.dw;
    rsrc = make_rsrc(a.data, static_cast<uint32_t>(a.N) * a.H * a.W * a.C);
    DmaLane<Cfg> g;
    g.init(wave, lane);
    const int k = kbeg + g.c16;
    const int tap = k / C;
    cc = k - tap * C;
    kh = tap / KW;
    kw = tap - kh * KW;
    retap();
    const int ohow = a.OH * a.OW;
#pragma unroll
    for (int i = 0; i < INSTR; ++i) {
      const int m = row_begin + g.row0 + i * DmaLane<Cfg>::kRowStep;
      ok[i] = m < a.M;
      const int mm = ok[i] ? m : 0;
      const int n = mm / ohow;
      const int rem = mm - n * ohow;
      const int oh = rem / a.OW;
      const int ow = rem - oh * a.OW;
      ih0[i] = oh * a.sh - a.ph;
      iw0[i] = ow * a.sw - a.pw;
      pix[i] = ((n * H + ih0[i]) * W + iw0[i]) * C;
    }
  }
  __device__ __forceinline__ void retap() {
    dih = kh * dh;
    diw = kw * dw;
    tapoff = (dih * W + diw) * C;
  }
  __device__ __forceinline__ void issue(int i, int, uint32_t lds_addr) {
    const int ih = ih0[i] + dih, iw = iw0[i] + diw;
    const bool v = ok[i] && kh < KH && static_cast<unsigned>(ih) < static_cast<unsigned>(H) &&
                   static_cast<unsigned>(iw) < static_cast<unsigned>(W);
    const uint32_t off = v ? static_cast<uint32_t>(pix[i] + tapoff + cc) : kOutOfRange;
    dma_buffer(lds_addr, off, rsrc);
  }
  __device__ __forceinline__ void stage_done() {
    cc += Cfg::BK;
    while (cc >= C) {
      cc -= C;
      if (++kw == KW) {
        kw = 0;
        ++kh;
      }
    }
    retap();
  }
};

template <class Cfg, int NS, int PIPE>
__global__ __launch_bounds__(Cfg::kThreads, NS <= 2 ? Cfg::kMinWaves : 1) void conv_dma_kernel(ConvArgs p) {
  __shared__ __attribute__((aligned(16))) v4i lds[NS * Cfg::STAGE_SLOTS];
  const int tiles_m = (p.M + Cfg::BM - 1) / Cfg::BM, tiles_n = (p.O + Cfg::BN - 1) / Cfg::BN;
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
  auto prefetch = [&]() { pre = epi_prefetch<Cfg>(p.epi, n0, p.O); };
  // this work-group's K slice: stages [kt0, kt0 + KT) (all of them without a split)
  const int kt_all = (p.K + Cfg::BK - 1) / Cfg::BK;
  const int kt0 = z * p.sk.kt_per_split;
  const int KT = (kt_all - kt0) < p.sk.kt_per_split ? (kt_all - kt0) : p.sk.kt_per_split;
  const int kbeg = kt0 * Cfg::BK;
  ConvIssuer<Cfg, Cfg::A_CHUNKS> ai;
  RowIssuerBuffer<Cfg, Cfg::B_CHUNKS> bi;
  ai.init(p, m0, wave, lane, kbeg);
  bi.init(p.weight, n0, p.O, p.K, wave, lane, kbeg);

  v16i acc[Cfg::MI][Cfg::NI];
  gemm_mainloop_dma<Cfg, NS, PIPE>(acc, ai, bi, KT, lds, prefetch);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  if (blockIdx.x == 0 && threadIdx.x == 0) epilogue_ranges(p.epi);
  if (__builtin_expect(p.sk.splits > 1, 0) && !splitk_gather<Cfg>(acc, p.sk, tile, z)) return;

  gemm_epilogue_lds<Cfg, NS * Cfg::STAGE_SLOTS * 16>(acc, p.epi, pre, m0, n0, p.M, p.O,
                                                     static_cast<size_t>(p.O), lds);
}

// ---- 3 x 3 convolution over 64 channels with the weights parked in LDS --------------
// A layer like ResNet's 56 x 56, 64 -> 64 has a short reduction (K = 576) and a weight
// tensor of 36 KB: as an implicit GEMM every tile is prologue and epilogue, and the nine
// taps re-fetch every input pixel nine times.  Here a work-group of 8 waves parks the whole
// weight tensor in LDS once; after that one barrier every wave works on its own.  An item
// is R consecutive output rows of one image: the wave brings their R + 2 input rows (with
// the zero halo left and right, zero rows above and below the image) into its private LDS
// patch with buffer loads ... lds, then for each output row runs the 9 taps x 2 k-steps x
// (2 x 2) MFMAs out of LDS, adds the bias, requantizes and stores the row; the int8 tile is
// transposed through the patch row that has just become dead.  No barrier per K step,
// every input row is fetched (R + 2) / R times instead of nine, and with two waves per SIMD
// one wave's fetch and epilogue overlap the other's MFMAs.  int8 output with the fused
// requantize only (the form the quantized graph runs with a calibrated convolution);
// everything else takes the tiled kernels.
constexpr int kRowsC = 64;        // input channels = bytes per pixel
constexpr int kRowsO = 64;        // output channels
constexpr int kRowsPitch = 60;    // patch pixels per row
constexpr int kRowsMaxW = kRowsPitch - 2;
constexpr int kRowsWaves = 8;

// (row & 3) ^ (row >> 2 & 3): spreads the 16-byte pieces of the transposed int8 tile (row
// pitch 64 bytes) over the banks for the column-wise writes and the row-wise reads alike
__device__ __forceinline__ int tile_swz(int row) { return (row ^ (row >> 2)) & 3; }

template <int R>
__global__ __launch_bounds__(64 * kRowsWaves, 1) void conv3x3_rows_kernel(ConvArgs p) {
  constexpr int CH = kRowsC / 16;                       // 16-byte chunks per pixel
  constexpr int kPatchPixels = (R + 2) * kRowsPitch;
  constexpr int kFetches = (kPatchPixels + 15) / 16;    // buffer loads of 16 pixels each
  __shared__ __attribute__((aligned(16))) v4i wl[9 * kRowsO * CH];               // 36 KB
  __shared__ __attribute__((aligned(16))) v4i patch_all[kRowsWaves * kPatchPixels * CH];
  __shared__ __attribute__((aligned(16))) int sbias[kRowsO];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  v4i* patch = patch_all + wave * kPatchPixels * CH;
  const uint32_t patch_addr = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(patch));
  const v4i rsrc = make_rsrc(p.data, static_cast<uint32_t>(p.N) * p.H * p.W * kRowsC);
  const int chunks_per_image = (p.OH + R - 1) / R;
  const int items = p.N * chunks_per_image;
  // lane geometry of the fetches: flat patch pixel 16 * j + lane / 4, chunk slot lane % 4
  auto fetch = [&](int item) {
    const int n = item / chunks_per_image, oh0 = (item - n * chunks_per_image) * R;
#pragma unroll
    for (int j = 0; j < kFetches; ++j) {
      const int flat = 16 * j + (lane >> 2);
      const int row = flat / kRowsPitch, px = flat - row * kRowsPitch;
      const int ih = oh0 + row - 1, iw = px - 1;
      const int chunk = (lane & 3) ^ swz<CH>(px);
      const bool ok = static_cast<unsigned>(ih) < static_cast<unsigned>(p.H) &&
                      static_cast<unsigned>(iw) < static_cast<unsigned>(p.W);
      const uint32_t off =
          ok ? static_cast<uint32_t>(((n * p.H + ih) * p.W + iw) * kRowsC + chunk * 16)
             : kOutOfRange;
      if (flat < kPatchPixels) dma_buffer(patch_addr + j * 1024, off, rsrc);
    }
  };
  int item = blockIdx.x * kRowsWaves + wave;
  if (item < items) fetch(item);  // on its way while the weights are staged

  // weights [o][tap][c] -> LDS [tap][o][chunk ^ swz(o)], straight into LDS as well: fetch
  // j fills the 16 rows (tap, o) = 16 * j ... + 15, lane / 4 the row, lane % 4 the slot
  {
    const v4i wrsrc = make_rsrc(p.weight, 9 * kRowsO * kRowsC);
    const uint32_t wl_addr = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(wl));
    constexpr int kWeightFetches = 9 * kRowsO / 16;  // 36
    for (int j = wave; j < kWeightFetches; j += kRowsWaves) {
      const int row = 16 * j + (lane >> 2);
      const int t = row / kRowsO, o = row - t * kRowsO;
      const int chunk = (lane & 3) ^ swz<CH>(o);
      dma_buffer(wl_addr + j * 1024, static_cast<uint32_t>((o * 9 + t) * kRowsC + chunk * 16),
                 wrsrc);
    }
  }
  const EpiScalars s = epi_scalars(p.epi);
  if (tid < kRowsO) sbias[tid] = epi_bias32(p.epi, s, tid);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();

  const int lrow = lane & 31, lgrp = lane >> 5;
  const bool relu = p.epi.relu != 0, stream8 = p.epi.stream8 != 0;
  // patch pixel of output column mi * 32 + lrow under tap column kw; columns past the row
  // (their results are never stored) are kept inside it
  int apx[2][3];
#pragma unroll
  for (int mi = 0; mi < 2; ++mi)
#pragma unroll
    for (int kw = 0; kw < 3; ++kw) {
      const int px = mi * 32 + lrow + kw;
      apx[mi][kw] = px < kRowsPitch ? px : kRowsPitch - 1;
    }
  for (; item < items; item += gridDim.x * kRowsWaves) {
    const int n = item / chunks_per_image, oh0 = (item - n * chunks_per_image) * R;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __builtin_amdgcn_wave_barrier();
    // a real loop: the second row re-runs the first row's instructions out of the
    // instruction cache instead of fetching a second copy of them
#pragma unroll 1
    for (int r = 0; r < R; ++r) {
      if (oh0 + r >= p.OH) break;
      // accumulators start at the int32 bias of their columns, read from LDS straight into
      // the registers the MFMAs add to: no bias add in the epilogue
      v16i acc[2][2];
#pragma unroll
      for (int ni = 0; ni < 2; ++ni)
#pragma unroll
        for (int vq = 0; vq < 4; ++vq) {
          const v4i b = *reinterpret_cast<const v4i*>(sbias + ni * 32 + 8 * vq + 4 * lgrp);
#pragma unroll
          for (int mi = 0; mi < 2; ++mi)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[mi][ni][4 * vq + i] = b[i];
        }
#pragma unroll
      for (int kh = 0; kh < 3; ++kh)
#pragma unroll
        for (int kw = 0; kw < 3; ++kw)
#pragma unroll
          for (int ks = 0; ks < 2; ++ks) {
            v4i fa[2], fb[2];
#pragma unroll
            for (int mi = 0; mi < 2; ++mi) {
              const int px = apx[mi][kw];
              fa[mi] = patch[((r + kh) * kRowsPitch + px) * CH + ((ks * 2 + lgrp) ^ swz<CH>(px))];
            }
#pragma unroll
            for (int ni = 0; ni < 2; ++ni)
              fb[ni] = wl[((kh * 3 + kw) * kRowsO + ni * 32 + lrow) * CH +
                          ((ks * 2 + lgrp) ^ swz<CH>(lrow))];
#pragma unroll
            for (int mi = 0; mi < 2; ++mi)
#pragma unroll
              for (int ni = 0; ni < 2; ++ni)
                acc[mi][ni] =
                    __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[ni], fa[mi], acc[mi][ni], 0, 0, 0);
          }
      // patch row r is dead now (output row r + 1 starts at patch row r + 1): the int8 tile
      // of up to 58 pixels x 64 channels is transposed through it, 64 bytes per pixel
      char* stage = reinterpret_cast<char*>(patch + r * kRowsPitch * CH);
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      __builtin_amdgcn_wave_barrier();
      auto requantize_tile = [&](auto with_relu) {
#pragma unroll
        for (int mi = 0; mi < 2; ++mi) {
          const int px = mi * 32 + lrow;
#pragma unroll
          for (int ni = 0; ni < 2; ++ni)
#pragma unroll
            for (int vq = 0; vq < 4; ++vq) {
              const int nl = ni * 32 + 8 * vq + 4 * lgrp;
              const uint32_t w = epi_requant_pack<decltype(with_relu)::value>(
                  acc[mi][ni][4 * vq], acc[mi][ni][4 * vq + 1], acc[mi][ni][4 * vq + 2],
                  acc[mi][ni][4 * vq + 3], s);
              if (px < p.OW)
                *reinterpret_cast<uint32_t*>(stage + px * kRowsO +
                                             (((nl >> 4) ^ tile_swz(px)) << 4) + (nl & 15)) = w;
            }
        }
      };
      if (relu)
        requantize_tile(std::true_type());
      else
        requantize_tile(std::false_type());
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      __builtin_amdgcn_wave_barrier();
      int8_t* orow = p.epi.out8 +
                     (static_cast<size_t>(n) * p.OH + oh0 + r) * p.OW * kRowsO;
      auto store_row = [&](auto stream) {
#pragma unroll
        for (int it = 0; it < 4; ++it) {
          const int px = it * 16 + (lane >> 2), c16 = lane & 3;
          if (px < p.OW) {
            const v4i val =
                *reinterpret_cast<const v4i*>(stage + px * kRowsO + ((c16 ^ tile_swz(px)) << 4));
            epi_store16<decltype(stream)::value>(val, orow + px * kRowsO + c16 * 16);
          }
        }
      };
      if (stream8)
        store_row(std::true_type());
      else
        store_row(std::false_type());
    }
    // the next item's fetches overwrite the patch: every LDS read above must have returned
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_wave_barrier();
    const int next = item + gridDim.x * kRowsWaves;
    if (next < items) fetch(next);
  }
  if (blockIdx.x == 0 && threadIdx.x == 0) epilogue_ranges(p.epi);
}

bool conv3x3_rows_ok(const ConvArgs& a) {
  const long long data_bytes = static_cast<long long>(a.N) * a.H * a.W * a.C;
  return a.KH == 3 && a.KW == 3 && a.sh == 1 && a.sw == 1 && a.ph == 1 && a.pw == 1 &&
         a.dh == 1 && a.dw == 1 && a.C == kRowsC && a.O == kRowsO && a.W <= kRowsMaxW &&
         a.epi.out32 == nullptr && a.epi.out8 != nullptr && aligned16(a.data) &&
         aligned16(a.weight) && aligned16(a.epi.out8) && data_bytes < (1LL << 31);
}

void launch_conv3x3_rows(hipStream_t s, const ConvArgs& a) {
  const long cus = num_cus();
  // two output rows per item once that still gives most waves of the chip an item: a third
  // fewer input rows to fetch per output row
  const long items2 = static_cast<long>(a.N) * ((a.OH + 1) / 2);
  const bool two = 5 * items2 >= 3 * kRowsWaves * cus;
  const long items = two ? items2 : static_cast<long>(a.N) * a.OH;
  long grid = (items + kRowsWaves - 1) / kRowsWaves;
  if (grid > cus) grid = cus;
  if (two)
    hipLaunchKernelGGL(conv3x3_rows_kernel<2>, dim3(static_cast<unsigned>(grid)),
                       dim3(64 * kRowsWaves), 0, s, a);
  else
    hipLaunchKernelGGL(conv3x3_rows_kernel<1>, dim3(static_cast<unsigned>(grid)),
                       dim3(64 * kRowsWaves), 0, s, a);
  MXQ_LAUNCH_CHECK();
}

// ---- 3 x 3 convolution with the input patch resident in LDS -------------------------
// The implicit GEMM above stages every input pixel nine times, once per tap, through the
// CU's 64 bytes per clock from L1 into LDS, which is what bounds every tile below 256 x 256.
// Here a work-group takes 128 consecutive output pixels (in (n, oh, ow) order, regardless
// of where a row or an image ends) and 128 output channels, brings the input rows those
// pixels touch into LDS ONCE -- "virtual rows" n * (H + 2) + ih + 1, so that the zero rows
// above and below an image are rows like any other and a tile that passes from one image
// to the next still reads a contiguous range -- and forms the nine taps' activation
// fragments by address arithmetic: the patch pixel of output pixel (n, oh, ow) under tap
// (kh, kw) is pp0 + kh * (W + 2) + kw.  Only the weights go through the stage ring (128
// rows x 128 bytes per stage: one tap's 128 channels), so a K step moves half the bytes of
// the implicit GEMM's and the ring is half as large: two work-groups of 8 waves share a CU
// and one's loads and epilogue overlap the other's MFMAs.  Stride 1, pad 1, no dilation,
// C a multiple of 128; int8 fused or int32 output through the common epilogue.
constexpr int kPatchBytes = 40 * 1024;   // room for the patch of one tile
#ifdef MXQ_STAMPS
__device__ long long mxq_dbg_stamps[8 * 4096];
#define MXQ_STAMP(k)                                                                  \
  do {                                                                                \
    if (lane == 0 && wave == 0 && blockIdx.x < 4096)                                  \
      mxq_dbg_stamps[blockIdx.x * 8 + (k)] = __builtin_readcyclecounter();            \
  } while (0)
#else
#define MXQ_STAMP(k)
#endif
typedef GemmCfg<128, 128, 128, 4, 2> CfgPatch;  // 8 waves, wave tile 32 pixels x 64 channels

template <int NS>
__global__ __launch_bounds__(512, 2) void conv3x3_patch_kernel(ConvArgs p) {
  typedef CfgPatch Cfg;
  constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK, CHW = Cfg::CH;   // CHW: chunks per weight row of a stage
  constexpr int NW = 8, BI = Cfg::B_CHUNKS, KS = Cfg::KS, NI = Cfg::NI;
  constexpr int STAGE_BYTES = BN * BK, RING_BYTES = NS * STAGE_BYTES;
  static_assert(Cfg::MI == 1 && NI == 2 && BI == 2, "wave tile 32 x 64");
  __shared__ __attribute__((aligned(16))) v4i lds[(kPatchBytes + RING_BYTES) / 16];
  char* patch = reinterpret_cast<char*>(lds);
  char* ring = patch + kPatchBytes;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / Cfg::WN, wn = wave % Cfg::WN;
  MXQ_STAMP(4);
  const int tiles_m = (p.M + BM - 1) / BM, tiles_n = (p.O + BN - 1) / BN;
  // channel tiles of one pixel tile are neighbours (they share the patch's cache lines)
  const int lid = xcd_remap(blockIdx.x, tiles_m * tiles_n);
  const int tn = lid % tiles_n, tm = lid / tiles_n;
  const int m0 = tm * BM, n0 = tn * BN;
  const int PW = p.W + 2, CH = p.C >> 4;   // patch pixels per row, 16-byte chunks per pixel
  const int ohow = p.OH * p.OW;

  // the range of virtual rows this tile touches
  const int ma = m0, mb = (m0 + BM - 1 < p.M) ? m0 + BM - 1 : p.M - 1;
  const int na = ma / ohow, oha = (ma - na * ohow) / p.OW;
  const int nb = mb / ohow, ohb = (mb - nb * ohow) / p.OW;
  const int vr0 = na * (p.H + 2) + oha;
  const int rows = nb * (p.H + 2) + ohb + 2 - vr0 + 1;

  // The patch: a row of it is RP pixels (the W + 2 real ones padded so that a row is whole
  // load instructions of 64 slots: the row of an instruction is then wave-uniform and no lane
  // divides anything), chunk j of patch pixel pp at slot pp * CH + (j ^ patch_swz(pp)).  A
  // fragment read is 16 consecutive pixels per LDS pass; with 128-byte pixels two of them
  // fill the banks once, so the XOR advances every second pixel, with wider pixels every one.
  const int ch_shift = __builtin_ctz(CH);
  const int per_row = (PW * CH + 63) >> 6;        // load instructions per patch row
  const int RP = (per_row << 6) >> ch_shift;      // pixels per patch row
  const int swz_shift = CH == 8 ? 1 : 0;
  auto patch_swz = [&](int pixel) { return (pixel >> swz_shift) & (CH - 1); };
  {
    const v4i rsrc = make_rsrc(p.data, static_cast<uint32_t>(p.N) * p.H * p.W * p.C);
    const uint32_t patch_addr = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(patch));
    const int instrs = rows * per_row;
    for (int it = wave; it < instrs; it += NW) {
      const int r = it / per_row, part = it - r * per_row;    // wave-uniform
      const int vabs = vr0 + r;
      const int n = vabs / (p.H + 2), ih = vabs - n * (p.H + 2) - 1;
      const bool row_ok = n < p.N && static_cast<unsigned>(ih) < static_cast<unsigned>(p.H);
      const int q = part * 64 + lane;                          // slot inside the row
      const int px = q >> ch_shift, pp = r * RP + px;
      const int j = (q & (CH - 1)) ^ patch_swz(pp);
      const int iw = px - 1;
      const bool ok = row_ok && static_cast<unsigned>(iw) < static_cast<unsigned>(p.W);
      const uint32_t off =
          ok ? static_cast<uint32_t>(((n * p.H + ih) * p.W + iw) * p.C + 16 * j) : kOutOfRange;
      dma_buffer(patch_addr + it * 1024, off, rsrc);
    }
  }
  // the weights: stage s = tap s / (C / BK), channel block s % (C / BK); OHWI rows are K-contiguous
  RowIssuerBuffer<Cfg, BI> bi;
  bi.init(p.weight, n0, p.O, p.K, wave, lane, 0);
  const uint32_t ring_addr = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(ring));
  const int KT = p.K / BK;
  auto issue = [&](int stage) {
    if (stage >= KT) return;
    const uint32_t sb = ring_addr + static_cast<uint32_t>(stage % NS) * STAGE_BYTES;
#pragma unroll
    for (int j = 0; j < BI; ++j) bi.issue(j, stage, sb + (j * NW + wave) * 1024);
  };
#pragma unroll
  for (int st = 0; st < NS - 1; ++st) issue(st);
  MXQ_STAMP(5);
  EpiPre pre = epi_prefetch<Cfg>(p.epi, n0, p.O);
  MXQ_STAMP(6);

  // this lane's output pixel and its patch pixel under tap (0, 0)
  const int frow = lane & 31, fgrp = lane >> 5;
  int m = m0 + wm * Cfg::TM + frow;
  m = m < p.M ? m : p.M - 1;   // rows past the end repeat the last pixel; never stored
  const int n = m / ohow, rem = m - n * ohow;
  const int oh = rem / p.OW, ow = rem - oh * p.OW;
  const int pp0 = (n * (p.H + 2) + oh - vr0) * RP + ow;
  const int rb = wn * Cfg::TN + frow;
  int fb0[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) fb0[ks] = rb * CHW + ((ks * 2 + fgrp) ^ swz<CHW>(rb));

  v16i acc[1][NI];
#pragma unroll
  for (int ni = 0; ni < NI; ++ni)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[0][ni][v] = 0;

  const int blocks = p.C / BK;   // stages per tap
  int tap = 0, cblk = 0, pp = pp0;   // of the stage computed next
  MXQ_STAMP(0);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the patch and the first stages
  MXQ_STAMP(1);
  for (int kt = 0; kt < KT; ++kt) {
    if (kt > 0) {
      const int newest = (kt + NS - 2) < (KT - 1) ? (kt + NS - 2) : (KT - 1);
      wait_ahead<BI, NS - 2>(newest - kt);
    }
    __builtin_amdgcn_s_barrier();
    issue(kt + NS - 1);
    const v4i* sbw = reinterpret_cast<const v4i*>(ring + (kt % NS) * STAGE_BYTES);
    const v4i* pix = reinterpret_cast<const v4i*>(patch) + pp * CH;
    const int sw_ = patch_swz(pp);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const v4i fa = pix[(cblk * (BK / 16) + ks * 2 + fgrp) ^ sw_];
      v4i fb[NI];
#pragma unroll
      for (int ni = 0; ni < NI; ++ni) fb[ni] = sbw[fb0[ks] + ni * 32 * CHW];
#pragma unroll
      for (int ni = 0; ni < NI; ++ni)
        acc[0][ni] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[ni], fa, acc[0][ni], 0, 0, 0);
    }
    if (++cblk == blocks) {
      cblk = 0;
      ++tap;
      const int kh = tap / 3, kw = tap - 3 * kh;
      pp = pp0 + kh * RP + kw;
    }
  }
  MXQ_STAMP(2);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  if (blockIdx.x == 0 && tid == 0) epilogue_ranges(p.epi);
  gemm_epilogue_lds<Cfg, kPatchBytes + RING_BYTES>(acc, p.epi, pre, m0, n0, p.M, p.O,
                                                   static_cast<size_t>(p.O), lds);
  MXQ_STAMP(3);
}

#ifdef MXQ_STAMPS
extern "C" int mxq_dbg_read_stamps(long long* host, int count) {
  return hipMemcpyFromSymbol(host, HIP_SYMBOL(mxq_dbg_stamps), sizeof(long long) * count) ==
                 hipSuccess
             ? 0
             : -1;
}
#endif

// Virtual rows the patch of a 128-pixel tile can span: the rows its pixels lie in, one
// above, one below, and two halo rows for every image boundary inside the tile.
inline int conv3x3_patch_rows(int OH, int OW) {
  const int out_rows = (128 + OW - 2) / OW + 1;
  const int crossings = (128 + OH * OW - 2) / (OH * OW);
  return out_rows + 2 + 2 * crossings;
}

bool conv3x3_patch_ok(const ConvArgs& a) {
  const long long data_bytes = static_cast<long long>(a.N) * a.H * a.W * a.C;
  const int ch = a.C / 16;
  return a.KH == 3 && a.KW == 3 && a.sh == 1 && a.sw == 1 && a.ph == 1 && a.pw == 1 &&
         a.dh == 1 && a.dw == 1 && a.C % 128 == 0 && (ch & (ch - 1)) == 0 && a.O % 16 == 0 &&
         aligned16(a.data) && aligned16(a.weight) && data_bytes < (1LL << 31) &&
         static_cast<long long>(a.O) * a.K < (1LL << 31) &&
         // (a patch row is whole load instructions of 1 KiB)
         static_cast<long long>(conv3x3_patch_rows(a.OH, a.OW)) *
                 (((a.W + 2) * ch + 63) / 64 * 1024) <=
             kPatchBytes;
}

void launch_conv3x3_patch(hipStream_t s, const ConvArgs& a) {
  const long tiles = static_cast<long>((a.M + 127) / 128) * ((a.O + 127) / 128);
  hipLaunchKernelGGL(conv3x3_patch_kernel<2>, dim3(static_cast<unsigned>(tiles)), dim3(512), 0, s,
                     a);
  MXQ_LAUNCH_CHECK();
}

typedef GemmCfg<256, 256, 64, 2, 4> CfgL8;   // 8 waves, wave tile 128 x 64
typedef GemmCfg<256, 128, 64, 4, 2> CfgW128; // 8 waves, wave tile 64 x 64
typedef GemmCfg<256, 64, 64, 4, 1> CfgW64;   // 4 waves, wave tile 64 x 64
typedef GemmCfg<128, 128, 64, 2, 2> CfgM;    // 4 waves, wave tile 64 x 64
typedef GemmCfg<64, 64, 64, 2, 2> CfgS;      // 4 waves, wave tile 32 x 32
typedef GemmCfg<256, 256, 64, 2, 2> CfgL4;   // 4 waves, wave tile 128 x 128
// 128-byte stages: half as many K steps
typedef GemmCfg<256, 256, 128, 2, 4> CfgL8K;
typedef GemmCfg<256, 128, 128, 4, 2> CfgW128K;
typedef GemmCfg<128, 128, 128, 2, 2> CfgMK;
typedef GemmCfg<64, 64, 128, 2, 2> CfgSK;
typedef GemmCfg<128, 64, 128, 2, 2> CfgRK;
typedef GemmCfg<64, 128, 128, 2, 2> CfgQK;
typedef GemmCfg<64, 64, 256, 2, 2> CfgSK2;

template <class Cfg, int NS, int PIPE>
void launch_dma(hipStream_t s, ConvArgs a, int splits, const Workspace& ws) {
  const long tiles =
      static_cast<long>((a.M + Cfg::BM - 1) / Cfg::BM) * ((a.O + Cfg::BN - 1) / Cfg::BN);
  splitk_setup<Cfg>(s, a.sk, tiles, a.K, splits, ws.ptr, ws.bytes);
  hipLaunchKernelGGL((conv_dma_kernel<Cfg, NS, PIPE>),
                     dim3(static_cast<unsigned>(tiles * a.sk.splits)), dim3(Cfg::kThreads), 0, s,
                     a);
  MXQ_LAUNCH_CHECK();
}

template <class Cfg>
void launch_cfg(hipStream_t s, const ConvArgs& a, bool aligned) {
  const int tiles = ((a.M + Cfg::BM - 1) / Cfg::BM) * ((a.O + Cfg::BN - 1) / Cfg::BN);
  if (aligned)
    hipLaunchKernelGGL((conv_kernel<Cfg, true>), dim3(tiles), dim3(Cfg::kThreads), 0, s, a);
  else
    hipLaunchKernelGGL((conv_kernel<Cfg, false>), dim3(tiles), dim3(Cfg::kThreads), 0, s, a);
  MXQ_LAUNCH_CHECK();
}

// ---- layout adapters ------------------------------------------------------------
// A second, small transpose that rides along in the launch of a large one: the weights of
// a convolution ([O][C][taps] -> [O][taps][C]) next to its data.  A launch of its own costs
// 4.6-5.9 us inside a network however little it moves (launch, then a cold round trip to
// memory), which for four 3 x 3 layers was 20 us of a 520 us pass.  [B][R][S] -> [B][S][R]
// with 16 | R and S small: a thread gathers 16 bytes S apart and stores them as one piece.
struct SmallJob {
  const uint8_t* in;
  uint8_t* out;
  int R, S;
  unsigned pieces;   // B * S * R / 16; 0 = no job
};

__device__ __forceinline__ void small_transpose_job(const SmallJob& j, unsigned block,
                                                    unsigned nblocks) {
  typedef uint32_t u4 __attribute__((ext_vector_type(4)));
  const unsigned per_row = static_cast<unsigned>(j.R) >> 4;     // pieces per output row [b][s]
  for (unsigned t = block * 256u + threadIdx.x; t < j.pieces; t += nblocks * 256u) {
    const unsigned row = t / per_row, k = t - row * per_row;    // row = b * S + s
    const unsigned b = row / static_cast<unsigned>(j.S), s = row - b * j.S;
    const uint8_t* src = j.in + (static_cast<size_t>(b) * j.R + 16 * k) * j.S + s;
    uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < 16; ++i)
      w[i >> 2] |= static_cast<uint32_t>(src[static_cast<size_t>(i) * j.S]) << (8 * (i & 3));
    *reinterpret_cast<u4*>(j.out + static_cast<size_t>(row) * j.R + 16 * k) =
        u4{w[0], w[1], w[2], w[3]};
  }
}

// Batched transpose [B][R][S] -> [B][S][RP] through a padded LDS tile; reads are
// contiguous along S, writes contiguous along R.  RP >= R: positions R..RP-1 of every
// output row are written as zeros (channel padding).
template <typename T>
__global__ __launch_bounds__(256) void transpose_kernel(const T* __restrict__ in,
                                                        T* __restrict__ out, int R, int S,
                                                        int RP) {
  __shared__ T tile[64][65];
  const size_t b = blockIdx.z;
  const int r0 = blockIdx.y * 64, s0 = blockIdx.x * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  const T* src = in + b * static_cast<size_t>(R) * S;
  T* dst = out + b * static_cast<size_t>(RP) * S;
  for (int i = ty; i < 64; i += 4) {
    const int r = r0 + i, s = s0 + tx;
    tile[i][tx] = (r < R && s < S) ? src[static_cast<size_t>(r) * S + s] : T(0);
  }
  __syncthreads();
  for (int i = ty; i < 64; i += 4) {
    const int s = s0 + i, r = r0 + tx;
    if (r < RP && s < S) dst[static_cast<size_t>(s) * RP + r] = tile[tx][i];
  }
}

// The byte form of the same transpose for friendly shapes (S % 4 == 0, RP % 16 == 0,
// aligned pointers): a work-group takes 64 rows x 128 columns, every thread loads dwords
// along S (a wave reads whole 128-byte runs), transposes 4 x 4 bytes in registers with
// v_perm and parks the result in LDS, from where 16-byte pieces of the output rows leave
// (a wave writes 1 KiB contiguous when the group covers all RP positions of its rows).
__global__ __launch_bounds__(256) void transpose_i8_kernel(const uint8_t* __restrict__ in,
                                                           uint8_t* __restrict__ out, int R,
                                                           int S, int RP, int B, SmallJob job) {
  constexpr int kPitch = 17;  // dwords per transposed row: 64 bytes + 4 of padding
  __shared__ uint32_t tile[128 * kPitch];
  if (static_cast<int>(blockIdx.z) >= B) {   // the extra z slices carry the riding job
    const unsigned per_z = gridDim.x * gridDim.y;
    small_transpose_job(job, (blockIdx.z - B) * per_z + blockIdx.y * gridDim.x + blockIdx.x,
                        (gridDim.z - B) * per_z);
    return;
  }
  const size_t b = blockIdx.z;
  const int r0 = blockIdx.y * 64, s0 = blockIdx.x * 128;
  const int t = threadIdx.x;
  const uint8_t* src = in + b * static_cast<size_t>(R) * S;
  uint8_t* dst = out + b * static_cast<size_t>(RP) * S;
  const int sq = t & 31;
#pragma unroll
  for (int pass = 0; pass < 2; ++pass) {
    const int rq = (t >> 5) + 8 * pass;
    const int s = s0 + 4 * sq;
    uint32_t w[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int r = r0 + 4 * rq + j;
      w[j] = (r < R && s < S)
                 ? *reinterpret_cast<const uint32_t*>(src + static_cast<size_t>(r) * S + s)
                 : 0u;
    }
    // x[i] = byte i of w[0..3]
    const uint32_t t0 = __builtin_amdgcn_perm(w[1], w[0], 0x05010400u);
    const uint32_t t1 = __builtin_amdgcn_perm(w[1], w[0], 0x07030602u);
    const uint32_t t2 = __builtin_amdgcn_perm(w[3], w[2], 0x05010400u);
    const uint32_t t3 = __builtin_amdgcn_perm(w[3], w[2], 0x07030602u);
    tile[(4 * sq + 0) * kPitch + rq] = __builtin_amdgcn_perm(t2, t0, 0x05040100u);
    tile[(4 * sq + 1) * kPitch + rq] = __builtin_amdgcn_perm(t2, t0, 0x07060302u);
    tile[(4 * sq + 2) * kPitch + rq] = __builtin_amdgcn_perm(t3, t1, 0x05040100u);
    tile[(4 * sq + 3) * kPitch + rq] = __builtin_amdgcn_perm(t3, t1, 0x07060302u);
  }
  __syncthreads();
  const int nb = min(64, RP - r0);  // bytes of every output row this group owns (16 | nb)
  const int per_row = nb >> 4;      // 16-byte pieces per row: 1..4
  const int pieces = 128 * per_row;
  for (int c = t; c < pieces; c += 256) {
    const int sl = per_row == 4 ? (c >> 2) : (per_row == 2 ? (c >> 1) : (per_row == 1 ? c : c / 3));
    const int k = c - sl * per_row;
    if (s0 + sl >= S) continue;
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    u4 v;
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = tile[sl * kPitch + 4 * k + i];
    *reinterpret_cast<u4*>(dst + static_cast<size_t>(s0 + sl) * RP + r0 + 16 * k) = v;
  }
}

// The same on 128 rows x 128 columns with 16-byte loads (S % 16 == 0, S and RP >= 128,
// 16-byte aligned input as well): a thread takes 16 bytes along S of four consecutive rows, four load
// instructions instead of sixteen, and the output runs are whole 128-byte lines.
struct WideOrder {
  unsigned tiles_s, tiles_r, total, per_xcd;
  unsigned grid;   // work-groups of the tile grid
};

template <int PIECE>
__global__ __launch_bounds__(256) void transpose_i8_wide_kernel(const uint8_t* __restrict__ in,
                                                                uint8_t* __restrict__ out,
                                                                int R, int S, int RP,
                                                                WideOrder o, SmallJob job) {
  typedef uint32_t u4 __attribute__((ext_vector_type(4)));
  constexpr int kPitch = 33;  // dwords per transposed row: 128 bytes + 4 of padding
  __shared__ uint32_t tile[128 * kPitch];
  if (blockIdx.x >= o.grid) {   // blocks past the tile grid carry the riding job
    small_transpose_job(job, blockIdx.x - o.grid, gridDim.x - o.grid);
    return;
  }
  // the tile sequence runs along S first, then R, then the batch; with o.per_xcd != 0 the
  // round-robin of work-group ids over the 8 XCDs is undone, so that every XCD owns a
  // contiguous range of it and tiles that share input cache lines meet in one L2
  unsigned item = blockIdx.x;
  if (o.per_xcd != 0) {
    item = (blockIdx.x & 7u) * o.per_xcd + (blockIdx.x >> 3);
    if (item >= o.total) return;
  }
  const unsigned rest = item / o.tiles_s, ts = item - rest * o.tiles_s;
  const unsigned bq = rest / o.tiles_r, tr = rest - bq * o.tiles_r;
  const size_t b = bq;
  const int r0 = tr * 128, s0 = ts * 128;
  const int t = threadIdx.x;
  const uint8_t* src = in + b * static_cast<size_t>(R) * S;
  uint8_t* dst = out + b * static_cast<size_t>(RP) * S;
  const int sq = t & 7, rq = t >> 3;
  const int s = s0 + 16 * sq;
  u4 w[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int r = r0 + 4 * rq + j;
    w[j] = (r < R && s < S) ? __builtin_nontemporal_load(reinterpret_cast<const u4*>(
                                  src + static_cast<size_t>(r) * S + s))
                            : u4{0, 0, 0, 0};
  }
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    // x[i] = byte i of w[0..3][d]
    const uint32_t t0 = __builtin_amdgcn_perm(w[1][d], w[0][d], 0x05010400u);
    const uint32_t t1 = __builtin_amdgcn_perm(w[1][d], w[0][d], 0x07030602u);
    const uint32_t t2 = __builtin_amdgcn_perm(w[3][d], w[2][d], 0x05010400u);
    const uint32_t t3 = __builtin_amdgcn_perm(w[3][d], w[2][d], 0x07030602u);
    const int row = 16 * sq + 4 * d;
    tile[(row + 0) * kPitch + rq] = __builtin_amdgcn_perm(t2, t0, 0x05040100u);
    tile[(row + 1) * kPitch + rq] = __builtin_amdgcn_perm(t2, t0, 0x07060302u);
    tile[(row + 2) * kPitch + rq] = __builtin_amdgcn_perm(t3, t1, 0x05040100u);
    tile[(row + 3) * kPitch + rq] = __builtin_amdgcn_perm(t3, t1, 0x07060302u);
  }
  __syncthreads();
  const int nb = min(128, RP - r0);  // bytes of every output row this group owns (PIECE | nb)
  const int per_row = nb / PIECE;
  const int pieces = 128 * per_row;
  for (int c = t; c < pieces; c += 256) {
    const int sl = per_row == 128 / PIECE ? c / (128 / PIECE) : c / per_row;
    const int k = c - sl * per_row;
    if (s0 + sl < S) {
      uint8_t* to = dst + static_cast<size_t>(s0 + sl) * RP + r0 + PIECE * k;
      if (PIECE == 16) {
        u4 v;
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = tile[sl * kPitch + 4 * k + i];
        __builtin_nontemporal_store(v, reinterpret_cast<u4*>(to));
      } else {
        // rows of 4 | RP bytes (14 x 14 planes): dword pieces, a wave still writes whole runs
        __builtin_nontemporal_store(tile[sl * kPitch + k], reinterpret_cast<uint32_t*>(to));
      }
    }
  }
}

__global__ __launch_bounds__(256) void copy16_kernel(const uint8_t* __restrict__ in,
                                                     uint8_t* __restrict__ out, size_t pieces) {
  typedef uint32_t u4 __attribute__((ext_vector_type(4)));
  const size_t stride = static_cast<size_t>(gridDim.x) * 256;
  for (size_t q = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x; q < pieces; q += stride)
    reinterpret_cast<u4*>(out)[q] = reinterpret_cast<const u4*>(in)[q];
}

// Small tensors with a thin inner extent on their own (7 x 7 planes of up to 4 MiB, or a
// weight tensor whose data took a kernel that carries no rider): the job body as a kernel,
// up to two jobs per launch.
__global__ __launch_bounds__(256) void small_transpose_kernel(SmallJob first, SmallJob second,
                                                              unsigned first_blocks) {
  if (blockIdx.x < first_blocks)
    small_transpose_job(first, blockIdx.x, first_blocks);
  else
    small_transpose_job(second, blockIdx.x - first_blocks, gridDim.x - first_blocks);
}

// A thin extent (at most 64 bytes, e.g. 7 x 7 planes) beside a long one that is a multiple of
// 128: see thin_transpose_tile.  One matrix per blockIdx.y.
template <bool THIN_IN>
__global__ __launch_bounds__(256) void transpose_i8_thin_kernel(const uint8_t* __restrict__ in,
                                                                uint8_t* __restrict__ out,
                                                                int L, int T) {
  __shared__ __attribute__((aligned(16))) uint8_t flat[128 * 64];
  const size_t plane = static_cast<size_t>(L) * T;
  thin_transpose_tile<THIN_IN>(in + blockIdx.y * plane, out + blockIdx.y * plane, L, T,
                               blockIdx.x * 128, flat);
}

// Space-to-depth by 2 while going from planes to pixels: out[b][h2][w2][(dh*2+dw)*C + c] =
// in[b][c][2*h2 - off_h + dh][2*w2 - off_w + dw] (zero outside the plane), the channel run
// of every output pixel zero-padded to CP bytes.  A stride-2 convolution over few channels
// becomes a unit-stride one over 4*C channels and half the window, which suits the
// direct-to-LDS kernels (16-byte channel runs) far better than 3 or 4 channels do.
__global__ __launch_bounds__(256) void s2d_nhwc_kernel(const int8_t* __restrict__ in,
                                                       int8_t* __restrict__ out, int C, int H,
                                                       int W, int H2, int W2, int off_h,
                                                       int off_w, int CP, size_t pixels) {
  for (size_t p = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x; p < pixels;
       p += static_cast<size_t>(gridDim.x) * 256) {
    const int w2 = static_cast<int>(p % W2);
    const size_t t = p / W2;
    const int h2 = static_cast<int>(t % H2);
    const size_t b = t / H2;
    const int8_t* img = in + b * static_cast<size_t>(C) * H * W;
    int8_t* dst = out + p * CP;
    for (int d = 0; d < 4; ++d) {
      const int h = 2 * h2 - off_h + (d >> 1), w = 2 * w2 - off_w + (d & 1);
      const bool inside = static_cast<unsigned>(h) < static_cast<unsigned>(H) &&
                          static_cast<unsigned>(w) < static_cast<unsigned>(W);
      for (int c = 0; c < C; ++c)
        dst[d * C + c] = inside ? img[(static_cast<size_t>(c) * H + h) * W + w] : int8_t(0);
    }
    for (int c = 4 * C; c < CP; ++c) dst[c] = 0;
  }
}

// Input rows that do not start on 128-byte marks (56 x 56 and 28 x 28 planes on the way to
// pixels) share cache lines between neighbouring tiles along S: there the round-robin of
// work-group ids over the XCDs is undone (64 x 256 x 56 x 56: 22.6 -> 21.1 us, 64 x 512 x 28 x 28:
// 14.3 -> 12.1 us).  Rows on the marks lose 10 % that way (64 x 64 planes: 25.6 -> 28.9 us) and
// the way back to planes gains nothing reliably, so those keep the plain order.
// work-groups a riding job gets: enough to be done when the carrier is
inline unsigned job_blocks(const SmallJob& job) {
  if (job.pieces == 0) return 0;
  const unsigned want = (job.pieces + 255u) / 256u;
  return want < 1024u ? want : 1024u;
}

template <int PIECE>
void launch_wide(hipStream_t s, const void* in, void* out, int B, int R, int S, int RP,
                 const SmallJob& job) {
  WideOrder o;
  o.tiles_s = static_cast<unsigned>((S + 127) / 128);
  o.tiles_r = static_cast<unsigned>((RP + 127) / 128);
  const unsigned long long total = 1ull * o.tiles_s * o.tiles_r * static_cast<unsigned>(B);
  MXQ_CHECK(total < (1ull << 31) - 256, "transpose grid too large");
  o.total = static_cast<unsigned>(total);
  o.per_xcd = (S % 128 != 0) ? (o.total + 7u) / 8u : 0u;
  o.grid = o.per_xcd != 0 ? o.per_xcd * 8u : o.total;
  hipLaunchKernelGGL(transpose_i8_wide_kernel<PIECE>, dim3(o.grid + job_blocks(job)), dim3(256), 0,
                     s, static_cast<const uint8_t*>(in), static_cast<uint8_t*>(out), R, S, RP, o,
                     job);
  MXQ_LAUNCH_CHECK();
}

// [B][R][S] -> [B][S][RP].  `rider`, when given, is a small job the launch carries along if
// its kernel can (then rider->pieces is cleared); the caller launches what is left.
template <typename T>
void launch_transpose(hipStream_t s, const void* in, void* out, int B, int R, int S, int RP,
                      SmallJob* rider = nullptr) {
  if (B == 0 || RP == 0 || S == 0) return;
  MXQ_CHECK(RP >= R, "padded extent below the extent");
  SmallJob none = {nullptr, nullptr, 16, 1, 0};
  SmallJob job = rider != nullptr ? *rider : none;
  auto carried = [&]() {
    if (rider != nullptr) rider->pieces = 0;
  };
  // only the kernels that put batches and row tiles on grid.y / grid.z have their limit
  auto check_yz = [&]() {
    MXQ_CHECK(B < 65535 && (RP + 63) / 64 <= 65535, "transpose grid too large");
  };
  if (sizeof(T) == 1 && S % 16 == 0 && S >= 128 && RP >= 128 && RP % 4 == 0 && RP % 16 != 0 &&
      aligned16(in) && (reinterpret_cast<uintptr_t>(out) & 3u) == 0) {
    launch_wide<4>(s, in, out, B, R, S, RP, job);
    carried();
    return;
  }
  if (sizeof(T) == 1 && S % 4 == 0 && RP % 16 == 0 &&
      (reinterpret_cast<uintptr_t>(in) & 3u) == 0 && aligned16(out)) {
    // (with fewer than 128 columns half of the wide tile's lanes would idle: 64 x 56 x 56 x 64
    // back to planes takes 7.8 us that way against 6.0 us)
    if (S % 16 == 0 && S >= 128 && RP >= 128 && aligned16(in)) {
      launch_wide<16>(s, in, out, B, R, S, RP, job);
      carried();
      return;
    }
    check_yz();
    const unsigned per_z = static_cast<unsigned>((S + 127) / 128) * ((RP + 63) / 64);
    const unsigned extra_z = (job_blocks(job) + per_z - 1) / per_z;
    MXQ_CHECK(B + extra_z <= 65535u, "transpose grid too large");
    dim3 grid128((S + 127) / 128, (RP + 63) / 64, B + extra_z);
    hipLaunchKernelGGL(transpose_i8_kernel, grid128, dim3(256), 0, s,
                       static_cast<const uint8_t*>(in), static_cast<uint8_t*>(out), R, S, RP, B,
                       job);
    MXQ_LAUNCH_CHECK();
    carried();
    return;
  }
  if (sizeof(T) == 1 && RP == R && R % 16 == 0 && S > 1 && S <= 64 && aligned16(out) &&
      static_cast<long long>(B) * R * S <= (4LL << 20)) {
    // a small tensor with a thin inner extent (3 x 3 weights, 7 x 7 planes)
    SmallJob me = {static_cast<const uint8_t*>(in), static_cast<uint8_t*>(out), R, S,
                   static_cast<unsigned>(static_cast<long long>(B) * S * (R / 16))};
    const unsigned mine = (me.pieces + 255u) / 256u;
    hipLaunchKernelGGL(small_transpose_kernel, dim3(mine + job_blocks(job)), dim3(256), 0, s, me,
                       job, mine);
    MXQ_LAUNCH_CHECK();
    carried();
    return;
  }
  if (sizeof(T) == 1 && RP == R && aligned16(in) && aligned16(out)) {
    // a thin extent (<= 64) beside a long one that is a multiple of 128
    const bool thin_in = S <= 64 && R % 128 == 0;
    const bool thin_out = R <= 64 && S % 128 == 0;
    if ((thin_in && S == 1) || (thin_out && R == 1)) {
      // a thin extent of 1 (the weights of a 1 x 1 convolution): the transpose is a copy
      const size_t pieces = static_cast<size_t>(B) * R * S / 16;  // 128 | R * S
      const size_t want = (pieces + 255) / 256;
      const size_t cap = static_cast<size_t>(num_cus()) * 8;
      hipLaunchKernelGGL(copy16_kernel, dim3(static_cast<unsigned>(want < cap ? want : cap)),
                         dim3(256), 0, s, static_cast<const uint8_t*>(in),
                         static_cast<uint8_t*>(out), pieces);
      MXQ_LAUNCH_CHECK();
      return;
    }
    if (thin_in || thin_out) {
      const int L = thin_in ? R : S, thin = thin_in ? S : R;
      MXQ_CHECK(B <= 65535, "transpose grid too large");
      dim3 grid(L / 128, B);
      if (thin_in)
        hipLaunchKernelGGL(transpose_i8_thin_kernel<true>, grid, dim3(256), 0, s,
                           static_cast<const uint8_t*>(in), static_cast<uint8_t*>(out), L, thin);
      else
        hipLaunchKernelGGL(transpose_i8_thin_kernel<false>, grid, dim3(256), 0, s,
                           static_cast<const uint8_t*>(in), static_cast<uint8_t*>(out), L, thin);
      MXQ_LAUNCH_CHECK();
      return;
    }
  }
  check_yz();
  dim3 grid((S + 63) / 64, (RP + 63) / 64, B);
  hipLaunchKernelGGL((transpose_kernel<T>), grid, dim3(256), 0, s, static_cast<const T*>(in),
                     static_cast<T*>(out), R, S, RP);
  MXQ_LAUNCH_CHECK();
}

// Output tile of a direct-to-LDS configuration of this file (what a split-K work-group
// leaves in the workspace); false for the register-staged ones.
bool conv_cfg_tile(int cfg, int& bm, int& bn) {
  switch (cfg) {
    case 11: case 16: case 35: bm = 256; bn = 256; return true;
    case 12: case 22: case 36: bm = 256; bn = 128; return true;
    case 13: case 23: bm = 256; bn = 64; return true;
    case 14: case 24: case 33: case 34: bm = 128; bn = 128; return true;
    case 15: case 25: case 31: case 32: case 39: bm = 64; bn = 64; return true;
    case 37: bm = 128; bn = 64; return true;
    case 38: bm = 64; bn = 128; return true;
    default: return false;
  }
}

struct ConvGeometry {
  int N, H, W, C, O, KH, KW, sh, sw, ph, pw, dh, dw;
  int OH, OW;
  long long M, K;
  bool is_fc;  // 1x1, unit stride, no padding: the FC of the flattened pixels
};

ConvGeometry conv_geometry(int N, int H, int W, int C, int O, int KH, int KW, int stride_h,
                           int stride_w, int pad_h, int pad_w, int dilate_h, int dilate_w) {
  MXQ_CHECK(N >= 0 && H > 0 && W > 0 && C > 0 && O > 0 && KH > 0 && KW > 0, "bad shape");
  MXQ_CHECK(stride_h > 0 && stride_w > 0 && dilate_h > 0 && dilate_w > 0 && pad_h >= 0 &&
                pad_w >= 0,
            "bad stride/dilate/pad");
  const int eh = dilate_h * (KH - 1) + 1, ew = dilate_w * (KW - 1) + 1;
  MXQ_CHECK(H + 2 * pad_h >= eh && W + 2 * pad_w >= ew, "kernel larger than padded input");
  ConvGeometry g = {N, H, W, C, O, KH, KW, stride_h, stride_w, pad_h, pad_w, dilate_h, dilate_w,
                    0, 0, 0, 0, false};
  g.OH = (H + 2 * pad_h - eh) / stride_h + 1;
  g.OW = (W + 2 * pad_w - ew) / stride_w + 1;
  g.M = static_cast<long long>(N) * g.OH * g.OW;
  g.K = static_cast<long long>(KH) * KW * C;
  MXQ_CHECK(g.M < (1LL << 31) && g.K < (1LL << 31), "problem too large for 32-bit tile indices");
  g.is_fc = KH == 1 && KW == 1 && stride_h == 1 && stride_w == 1 && pad_h == 0 && pad_w == 0;
  return g;
}

struct ConvPlan {
  int cfg;
  int splits;
};

// What conv_nhwc would launch for a convolution that does not reduce to the FC.  `aligned`:
// C % 16 == 0 and 16-byte aligned operands.
ConvPlan plan_conv(const ConvGeometry& g, bool aligned, const GemmForce& force) {
  ConvPlan plan = {force.cfg, force.splits};
  const int M = static_cast<int>(g.M), K = static_cast<int>(g.K), O = g.O;
  const long long data_bytes = static_cast<long long>(g.N) * g.H * g.W * g.C;
  const bool dma_ok = aligned && data_bytes < (1LL << 31) &&
                      static_cast<long long>(O) * K < (1LL << 31);
  if (plan.cfg == 0) {
    const long cus = num_cus();
    auto tiles = [&](int bm, int bn) {
      return static_cast<long>((M + bm - 1) / bm) * ((O + bn - 1) / bn);
    };
    int auto_splits = 1;
    if (dma_ok) {
      switch (choose_tile(M, O, K, cus, true, &auto_splits)) {
        case Tile::kL8: plan.cfg = 11; break;
        case Tile::kW128x2: plan.cfg = 22; break;
        case Tile::kW128K2: plan.cfg = 36; break;
        case Tile::kM128x2: plan.cfg = 24; break;
        case Tile::kM128K2: plan.cfg = 33; break;
        case Tile::kS64x2: plan.cfg = 25; break;
        case Tile::kS64x4: plan.cfg = 15; break;
        case Tile::kS64K2: plan.cfg = 31; break;
        case Tile::kR128K2: plan.cfg = 37; break;
        case Tile::kQ128K2: plan.cfg = 38; break;
        case Tile::kS64K4: plan.cfg = 39; break;
        case Tile::kW192K2: plan.cfg = 11; break;  // not proposed for gathered operands
      }
    } else if (O > 128 && tiles(256, 256) >= cus) {
      plan.cfg = 1;
    } else if (O > 64 && tiles(256, 128) >= cus) {
      plan.cfg = 2;
    } else if (O <= 64 && tiles(256, 64) >= cus) {
      plan.cfg = 3;
    } else if (tiles(128, 128) >= cus) {
      plan.cfg = 4;
    } else {
      plan.cfg = 5;
    }
    if (plan.splits == 0) plan.splits = auto_splits;
  }
  if (plan.splits <= 0) plan.splits = 1;
  return plan;
}

size_t conv_plan_workspace(const ConvPlan& plan, const ConvGeometry& g) {
  int bm, bn;
  if (plan.splits <= 1 || !conv_cfg_tile(plan.cfg, bm, bn)) return 0;
  const long tiles = static_cast<long>((g.M + bm - 1) / bm) * ((g.O + bn - 1) / bn);
  return splitk_workspace_bytes(tiles, plan.splits, bm, bn);
}

// Both C entry points: `planar` writes out32 as [N][O][OH][OW] instead of [N][OH][OW][O].
void conv_nhwc(void* stream, const int8_t* data, const int8_t* weight, const int8_t* bias, int N,
               int H, int W, int C, int O, int KH, int KW, int stride_h, int stride_w, int pad_h,
               int pad_w, int dilate_h, int dilate_w, const float* min_data,
               const float* max_data, const float* min_weight, const float* max_weight,
               const float* min_bias, const float* max_bias, int32_t* out32, float* omin,
               float* omax, int8_t* out8, float* rmin, float* rmax, int relu, float min_calib,
               float max_calib, bool planar, const GemmForce& force, const Workspace& ws) {
  const ConvGeometry g = conv_geometry(N, H, W, C, O, KH, KW, stride_h, stride_w, pad_h, pad_w,
                                       dilate_h, dilate_w);
  MXQ_CHECK(min_data && max_data && min_weight && max_weight, "null input range pointer");
  MXQ_CHECK(omin && omax, "null output range pointer");
  MXQ_CHECK(bias == nullptr || (min_bias && max_bias), "bias given without its range");
  MXQ_CHECK(N == 0 || out32 != nullptr || out8 != nullptr, "no output buffer");
  MXQ_CHECK(out8 == nullptr || (rmin && rmax), "fused requantize needs rmin/rmax");
  ConvArgs a;
  a.data = data;
  a.weight = weight;
  a.N = N; a.H = H; a.W = W; a.C = C; a.O = O; a.KH = KH; a.KW = KW;
  a.sh = stride_h; a.sw = stride_w; a.ph = pad_h; a.pw = pad_w; a.dh = dilate_h; a.dw = dilate_w;
  a.OH = g.OH;
  a.OW = g.OW;
  a.M = static_cast<int>(g.M);
  a.K = static_cast<int>(g.K);
  a.sk.splits = 1;
  a.sk.kt_per_split = 1 << 30;
  a.sk.counters = nullptr;
  a.sk.partials = nullptr;
  MXQ_CHECK(a.M == 0 || O == 0 || (data != nullptr && weight != nullptr),
            "null operand pointer");
  Epilogue& e = a.epi;
  e.bias = bias;
  e.min_data = min_data; e.max_data = max_data;
  e.min_weight = min_weight; e.max_weight = max_weight;
  e.min_bias = min_bias; e.max_bias = max_bias;
  e.out32 = out32; e.out8 = out8; e.outf = nullptr;
  e.res = nullptr; e.res_min = nullptr; e.res_max = nullptr;
  e.sum_min_calib = 0.f; e.sum_max_calib = 0.f; e.sum_relu = 0; e.with_sum = 0;
  e.omin = omin; e.omax = omax; e.rmin = rmin; e.rmax = rmax;
  e.relu = relu;
  float x = fabsf(min_calib), y = fabsf(max_calib);
  e.real_range = (x < y) ? y : x;
  e.plane = planar ? a.OH * a.OW : 0;
  e.stream8 = epi_stream_rows(a.M);

  hipStream_t s = static_cast<hipStream_t>(stream);
  if (a.M == 0 || O == 0) {
    // no output elements: launch_fc writes the range scalars alone
    launch_fc(s, data, weight, a.M, O, C, O, e, GemmForce(), Workspace());
    return;
  }
  // a 1x1, unit-stride, unpadded convolution is the FC of the flattened pixels
  if (force.cfg == 0 && g.is_fc) {
    launch_fc(s, data, weight, a.M, O, C, O, e, force, ws);
    return;
  }
  const bool aligned = (C % 16 == 0) && aligned16(data) && aligned16(weight);
  const long long data_bytes = static_cast<long long>(N) * H * W * C;
  const bool dma_ok = aligned && data_bytes < (1LL << 31) &&
                      static_cast<long long>(O) * a.K < (1LL << 31);
  ConvPlan plan = plan_conv(g, aligned, force);
  // a split the chooser proposed is dropped when the caller brought no room for it
  if (force.splits == 0 && plan.splits > 1 &&
      (ws.ptr == nullptr || !aligned16(ws.ptr) || ws.bytes < conv_plan_workspace(plan, g))) {
    GemmForce unsplit = force;
    unsplit.splits = 1;
    plan = plan_conv(g, aligned, unsplit);
  }
  // 61: the parked-weights row kernel (3 x 3 over 64 -> 64 channels, fused int8 output);
  // chosen for it whenever the launch has rows for every wave of the chip
  if (plan.cfg == 61 || (force.cfg == 0 && conv3x3_rows_ok(a) &&
                         static_cast<long>(a.N) * a.OH >= 1L * kRowsWaves * num_cus())) {
    MXQ_CHECK(conv3x3_rows_ok(a), "shape does not qualify for the parked-weights 3x3 kernel");
    MXQ_CHECK(plan.splits <= 1 || force.splits == 0, "the 3x3 row kernel has no split-K form");
    launch_conv3x3_rows(s, a);
    return;
  }
  // 62: the resident-patch 3 x 3 kernel; chosen where it was measured ahead of the tiled
  // kernels (28 x 28 planes over 128 channels at batch 64: 15.4 against 16.6 us of kernel time)
  const long patch_tiles = static_cast<long>((a.M + 127) / 128) * ((a.O + 127) / 128);
  if (plan.cfg == 62 || (force.cfg == 0 && plan.splits <= 1 && conv3x3_patch_ok(a) &&
                         patch_tiles >= num_cus())) {
    MXQ_CHECK(conv3x3_patch_ok(a), "shape does not qualify for the resident-patch 3x3 kernel");
    MXQ_CHECK(plan.splits <= 1 || force.splits == 0, "the patch kernel has no split-K form");
    launch_conv3x3_patch(s, a);
    return;
  }
  const int cfg = plan.cfg, sp = plan.splits;
  if (cfg > 10) MXQ_CHECK(dma_ok, "shape does not qualify for the direct-to-LDS conv kernels");
  if (cfg <= 10) MXQ_CHECK(sp <= 1, "the register-staged kernels have no split-K form");
  switch (cfg) {
    case 1: launch_cfg<CfgL8>(s, a, aligned); break;
    case 2: launch_cfg<CfgW128>(s, a, aligned); break;
    case 3: launch_cfg<CfgW64>(s, a, aligned); break;
    case 4: launch_cfg<CfgM>(s, a, aligned); break;
    case 5: launch_cfg<CfgS>(s, a, aligned); break;
    case 11: launch_dma<CfgL8, 4, 2>(s, a, sp, ws); break;
    case 12: launch_dma<CfgW128, 4, 2>(s, a, sp, ws); break;
    case 13: launch_dma<CfgW64, 4, 2>(s, a, sp, ws); break;
    case 14: launch_dma<CfgM, 4, 2>(s, a, sp, ws); break;
    case 15: launch_dma<CfgS, 4, 2>(s, a, sp, ws); break;
    case 16: launch_dma<CfgL4, 4, 2>(s, a, sp, ws); break;
    case 31: launch_dma<CfgSK, 2, 0>(s, a, sp, ws); break;
    case 32: launch_dma<CfgSK, 3, 0>(s, a, sp, ws); break;
    case 33: launch_dma<CfgMK, 2, 0>(s, a, sp, ws); break;
    case 34: launch_dma<CfgMK, 3, 0>(s, a, sp, ws); break;
    case 35: launch_dma<CfgL8K, 2, 0>(s, a, sp, ws); break;
    case 36: launch_dma<CfgW128K, 2, 0>(s, a, sp, ws); break;
    case 37: launch_dma<CfgRK, 2, 0>(s, a, sp, ws); break;
    case 38: launch_dma<CfgQK, 2, 0>(s, a, sp, ws); break;
    case 39: launch_dma<CfgSK2, 2, 0>(s, a, sp, ws); break;
    case 22: launch_dma<CfgW128, 2, 0>(s, a, sp, ws); break;
    case 23: launch_dma<CfgW64, 2, 0>(s, a, sp, ws); break;
    case 24: launch_dma<CfgM, 2, 0>(s, a, sp, ws); break;
    case 25: launch_dma<CfgS, 2, 0>(s, a, sp, ws); break;
    default: MXQ_CHECK(false, "unknown conv tile configuration " << cfg);
  }
}

}  // namespace

// Data [N][C][H][W] -> [N][H][W][Cp] and weights [O][C][KH][KW] -> [O][KH][KW][Cp] for the
// NCHW operator's adapter route, in one launch where the data's kernel can carry the weights.
void nchw_to_nhwc_pair(hipStream_t s, const int8_t* data, int8_t* d_out, int N, int C, int H,
                       int W, int Cp, const int8_t* weight, int8_t* w_out, int O, int KH, int KW) {
  MXQ_CHECK(static_cast<long long>(H) * W < (1LL << 31), "image too large");
  const int taps = KH * KW;
  const long long wpieces = static_cast<long long>(O) * taps * (C / 16);
  SmallJob job = {reinterpret_cast<const uint8_t*>(weight), reinterpret_cast<uint8_t*>(w_out), C,
                  taps, 0};
  const bool rides = w_out != nullptr && Cp == C && C % 16 == 0 && taps > 1 && taps <= 64 &&
                     aligned16(w_out) && wpieces < (1LL << 31);
  if (rides) job.pieces = static_cast<unsigned>(wpieces);
  if (static_cast<long long>(N) * Cp * H * W != 0)
    launch_transpose<int8_t>(s, data, d_out, N, C, H * W, Cp, &job);
  if (w_out == nullptr) return;
  if (rides && job.pieces == 0) return;   // carried
  launch_transpose<int8_t>(s, weight, w_out, O, C, taps, Cp);
}

}  // namespace mxq

using namespace mxq;

extern "C" {

size_t mxq_quantized_conv_workspace(int N, int H, int W, int C, int O, int KH, int KW,
                                    int stride_h, int stride_w, int pad_h, int pad_w,
                                    int dilate_h, int dilate_w, int fused_int8_only) {
  try {
    const ConvGeometry g = conv_geometry(N, H, W, C, O, KH, KW, stride_h, stride_w, pad_h, pad_w,
                                         dilate_h, dilate_w);
    if (g.M == 0) return 0;
    if (g.is_fc)
      return fc_workspace_bytes(static_cast<int>(g.M), O, C, fused_int8_only != 0 && O % 16 == 0);
    return conv_plan_workspace(plan_conv(g, C % 16 == 0, GemmForce()), g);
  } catch (...) {
    return 0;
  }
}

int mxq_quantized_conv_nhwc(void* stream, const int8_t* data, const int8_t* weight,
                            const int8_t* bias, int N, int H, int W, int C, int O, int KH,
                            int KW, int stride_h, int stride_w, int pad_h, int pad_w,
                            int dilate_h, int dilate_w, const float* min_data,
                            const float* max_data, const float* min_weight,
                            const float* max_weight, const float* min_bias,
                            const float* max_bias, int32_t* out32, float* omin, float* omax,
                            int8_t* out8, float* rmin, float* rmax, int relu, float min_calib,
                            float max_calib, void* workspace, size_t workspace_bytes) {
  MXQ_API_BEGIN();
  Workspace ws;
  ws.ptr = workspace;
  ws.bytes = workspace_bytes;
  conv_nhwc(stream, data, weight, bias, N, H, W, C, O, KH, KW, stride_h, stride_w, pad_h, pad_w,
            dilate_h, dilate_w, min_data, max_data, min_weight, max_weight, min_bias, max_bias,
            out32, omin, omax, out8, rmin, rmax, relu, min_calib, max_calib, false, GemmForce(),
            ws);
  MXQ_API_END();
}

#ifdef MXQ_TEST_HOOKS
// Test-only twin of mxq_quantized_conv_nhwc (declared in tests/mxq_test_hooks.h): the tile
// configuration and the split-K factor come as arguments (0 = let the launcher choose).
int mxq_test_quantized_conv_nhwc(void* stream, const int8_t* data, const int8_t* weight,
                                 const int8_t* bias, int N, int H, int W, int C, int O, int KH,
                                 int KW, int stride_h, int stride_w, int pad_h, int pad_w,
                                 int dilate_h, int dilate_w, const float* min_data,
                                 const float* max_data, const float* min_weight,
                                 const float* max_weight, const float* min_bias,
                                 const float* max_bias, int32_t* out32, float* omin,
                                 float* omax, int8_t* out8, float* rmin, float* rmax, int relu,
                                 float min_calib, float max_calib, void* workspace,
                                 size_t workspace_bytes, int cfg, int splits) {
  MXQ_API_BEGIN();
  Workspace ws;
  ws.ptr = workspace;
  ws.bytes = workspace_bytes;
  GemmForce force;
  force.cfg = cfg;
  force.splits = splits;
  conv_nhwc(stream, data, weight, bias, N, H, W, C, O, KH, KW, stride_h, stride_w, pad_h, pad_w,
            dilate_h, dilate_w, min_data, max_data, min_weight, max_weight, min_bias, max_bias,
            out32, omin, omax, out8, rmin, rmax, relu, min_calib, max_calib, false, force, ws);
  MXQ_API_END();
}
#endif  // MXQ_TEST_HOOKS

int mxq_quantized_conv_nhwc_out_nchw(void* stream, const int8_t* data, const int8_t* weight,
                                     const int8_t* bias, int N, int H, int W, int C, int O,
                                     int KH, int KW, int stride_h, int stride_w, int pad_h,
                                     int pad_w, int dilate_h, int dilate_w,
                                     const float* min_data, const float* max_data,
                                     const float* min_weight, const float* max_weight,
                                     const float* min_bias, const float* max_bias,
                                     int32_t* out32_nchw, float* omin, float* omax,
                                     void* workspace, size_t workspace_bytes) {
  MXQ_API_BEGIN();
  MXQ_CHECK(out32_nchw != nullptr, "no output buffer");
  Workspace ws;
  ws.ptr = workspace;
  ws.bytes = workspace_bytes;
  conv_nhwc(stream, data, weight, bias, N, H, W, C, O, KH, KW, stride_h, stride_w, pad_h, pad_w,
            dilate_h, dilate_w, min_data, max_data, min_weight, max_weight, min_bias, max_bias,
            out32_nchw, omin, omax, nullptr, nullptr, nullptr, 0, 0.f, 0.f, true, GemmForce(), ws);
  MXQ_API_END();
}


int mxq_nchw_to_nhwc_i8(void* stream, const int8_t* in, int8_t* out, int N, int C, int H,
                        int W) {
  MXQ_API_BEGIN();
  MXQ_CHECK(N >= 0 && C >= 0 && H >= 0 && W >= 0, "negative dimension");
  MXQ_CHECK((static_cast<long long>(H) * W) < (1LL << 31), "image too large");
  if (static_cast<long long>(N) * C * H * W == 0) return 0;
  MXQ_CHECK(in != nullptr && out != nullptr, "null pointer");
  launch_transpose<int8_t>(static_cast<hipStream_t>(stream), in, out, N, C, H * W, C);
  MXQ_API_END();
}

int mxq_nchw_to_nhwc_pad_i8(void* stream, const int8_t* in, int8_t* out, int N, int C, int H,
                            int W, int C_padded) {
  MXQ_API_BEGIN();
  MXQ_CHECK(N >= 0 && C >= 0 && H >= 0 && W >= 0, "negative dimension");
  MXQ_CHECK(C_padded >= C, "C_padded must be at least C");
  MXQ_CHECK((static_cast<long long>(H) * W) < (1LL << 31), "image too large");
  if (static_cast<long long>(N) * C_padded * H * W == 0) return 0;
  MXQ_CHECK(in != nullptr && out != nullptr, "null pointer");
  launch_transpose<int8_t>(static_cast<hipStream_t>(stream), in, out, N, C, H * W, C_padded);
  MXQ_API_END();
}

int mxq_nchw_to_s2d_nhwc_i8(void* stream, const int8_t* in, int8_t* out, int N, int C, int H,
                            int W, int off_h, int off_w, int C_padded) {
  MXQ_API_BEGIN();
  MXQ_CHECK(N >= 0 && C >= 0 && H >= 0 && W >= 0, "negative dimension");
  MXQ_CHECK((off_h == 0 || off_h == 1) && (off_w == 0 || off_w == 1), "offsets are 0 or 1");
  MXQ_CHECK(C_padded >= 4 * C, "C_padded must be at least 4 * C");
  const int H2 = (H + off_h + 1) / 2, W2 = (W + off_w + 1) / 2;
  const size_t pixels = static_cast<size_t>(N) * H2 * W2;
  if (pixels == 0 || C_padded == 0) return 0;
  MXQ_CHECK(in != nullptr && out != nullptr, "null pointer");
  size_t g = (pixels + 255) / 256;
  if (g > 65535u * 16u) g = 65535u * 16u;
  hipLaunchKernelGGL(s2d_nhwc_kernel, dim3(static_cast<unsigned>(g)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), in, out, C, H, W, H2, W2, off_h, off_w,
                     C_padded, pixels);
  MXQ_LAUNCH_CHECK();
  MXQ_API_END();
}

int mxq_nhwc_to_nchw(void* stream, const void* in, void* out, int N, int C, int H, int W,
                     int elem_bytes) {
  MXQ_API_BEGIN();
  MXQ_CHECK(N >= 0 && C >= 0 && H >= 0 && W >= 0, "negative dimension");
  MXQ_CHECK(elem_bytes == 1 || elem_bytes == 4, "elem_bytes must be 1 or 4");
  MXQ_CHECK((static_cast<long long>(H) * W) < (1LL << 31), "image too large");
  if (static_cast<long long>(N) * C * H * W == 0) return 0;
  MXQ_CHECK(in != nullptr && out != nullptr, "null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (elem_bytes == 1)
    launch_transpose<int8_t>(s, in, out, N, H * W, C, H * W);
  else
    launch_transpose<int32_t>(s, in, out, N, H * W, C, H * W);
  MXQ_API_END();
}

}  // extern "C"
