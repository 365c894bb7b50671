// int8 x int8 -> int32 MFMA contraction core for gfx950, shared by the quantized
// fully-connected and convolution kernels.
//
//   out[m][n] = bias32[n] + sum_k A[m][k] * B[n][k]        (both operands K-contiguous)
//
// A is the activation operand (FC data rows, or the implicit im2col rows of an
// NHWC convolution), B the weight [N][K].  The work-group tile is BM x BN, the
// K loop advances BK bytes per step through a double-buffered LDS stage; each
// wave owns a (BM/WM) x (BN/WN) sub-tile built from 32x32x32 i8 MFMAs.
//
// MFMA operand roles: the weight fragment is source A and the activation
// fragment source B of v_mfma_i32_32x32x32_i8, so that in the result lane l
// holds activation row (l % 32) and registers v hold 4 consecutive output
// columns n = 8*(v/4) + 4*(l/32) + (v%4): the epilogue then stores 4 adjacent
// int32 (one 16-byte store) or 4 adjacent int8 (one dword) per lane.
// Both fragments take, for k-group g = l/32, the 16 bytes at k = 32*ks + 16*g of
// their row, so whatever order the hardware assigns to those bytes inside the
// instruction is the same for the two operands and the dot product is exact.
//
// LDS layout: a stage holds rows of BK bytes = CH 16-byte chunks; chunk c of row
// r lives in slot r*CH + (c ^ swz(r)).  swz() spreads the 32 rows a fragment
// read touches over all banks (see swz()).
//
// Epilogue (exact integers, then the native requantize arithmetic):
//   bias32[n] = trunc(float(bias[n]) * fbq / foq)      quantized_fully_connected.cc:149-174
//   acc      += bias32[n]                               (wrap-around int32)
//   out32     = acc                                      optional
//   out8      = FloatToQuantized(float(acc) * (max_out / 2^31), -R, R)   requantize-inl.h:89-105
//               optionally max(out8, 0)
#ifndef MXQ_GEMM_H_
#define MXQ_GEMM_H_

#include <hip/hip_runtime.h>

#include <type_traits>

#include <cstdint>

#include "mxq_common.h"
#include "mxq_sum.h"

namespace mxq {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

struct Epilogue {
  const int8_t* bias;      // int8 [N] or null
  const float* min_data;   // device scalars
  const float* max_data;
  const float* min_weight;
  const float* max_weight;
  const float* min_bias;
  const float* max_bias;
  int32_t* out32;          // [M][ldo] or null
  int8_t* out8;            // [M][ldo] or null
  // [M][ldo] or null: the int8 result above taken back to float, q * (R / 127), i.e.
  // what dequantize makes of the requantized output (dequantize-inl.h:64-75)
  float* outf;
  // int8 [M][ldo] or null: a second operand that is added to the requantized int8 result
  // before it is stored (the residual sum that follows the layer, then optionally the int8
  // relu): out8 = relu?(add(requantize(acc), res)) over the calibrated range
  // (sum_min_calib, sum_max_calib), which rmin / rmax then receive.
  const int8_t* res;
  const float* res_min;    // device scalars: the range of res
  const float* res_max;
  float sum_min_calib, sum_max_calib;
  int sum_relu;
  int with_sum;            // rmin / rmax report the sum's range (also for an empty output)
  float* omin;             // int32 output range
  float* omax;
  float* rmin;             // requantized range (only with out8)
  float* rmax;
  int relu;
  float real_range;        // MaxAbs(min_calib, max_calib), host-computed
  // 0: out32 is row-major [M][ldo].  > 0: the rows are pixels of images of `plane` pixels
  // and out32 is written planar, [M / plane][N][plane] (NCHW for an NHWC convolution);
  // only out32 has this form.
  int plane;
  // out8 is written with non-temporal stores (see epi_stream_rows)
  int stream8;
};

// Outputs of at least this many rows are written with non-temporal stores: plain stores
// leave the int8 tiles as dirty lines in the XCDs' L2s, where they displace the operand
// rows other tiles of the launch still share and have to be written back when the next
// launch needs the space.  The layer that consumes the output then reads it from memory
// instead of the memory-side cache.  Measured at batch 64 (one box each, two rounds):
//   the 19 ResNet-50 layers on operands of their own: plain 304-309 us, streaming from
//     32768 rows 277, from 8192 rows 267, every layer 263;
//   the ResNet-50 bottleneck body as a real chain (52 convolutions, every layer reading
//     what the one before wrote): plain 1095 us, from 32768 rows 1074, from 8192 rows 1065,
//     every layer 1064.5;
//   producer -> consumer pairs (1x1 -> 1x1, 1x1 -> 3x3, 3x3 -> 1x1): -14 ... 0 % for the
//     pair at 200704 and 50176 rows, -3 ... +5 % at 12544 rows, +1 ... +11 % at 3136 and
//     4096 rows; BERT's chain at 4096 rows (a dequantize consumes each output) +2.5 %.
// 8192 keeps everything from 14 x 14 planes at batch 64 up and leaves the 4096-row
// fully-connected layers alone.
constexpr int kEpiStreamRows = 8192;
inline int epi_stream_rows(long long rows) { return rows >= kEpiStreamRows ? 1 : 0; }

// 16 bytes of the int8 output tile.  The flavour is a compile-time parameter and callers
// branch around whole store loops: two stores to one address that differ only in the
// non-temporal hint are merged into a plain one by the compiler.
template <bool STREAM>
__device__ __forceinline__ void epi_store16(v4i val, void* p) {
  if (STREAM)
    __builtin_nontemporal_store(val, reinterpret_cast<v4i*>(p));
  else
    *reinterpret_cast<v4i*>(p) = val;
}

__device__ __forceinline__ float dev_maxabs(float a, float b) {
  float x = fabsf(a), y = fabsf(b);
  return (x < y) ? y : x;
}

// Scalars every thread needs in the epilogue.
struct EpiScalars {
  float max_out;   // QuantizationRangeForMultiplication, quantization_utils.h:141-157
  float foq, fbq;  // float per int32 level / per int8 bias level
  float in_scale;  // max_out / 2^31
  float qscale;    // 127 / R
  float dqscale;   // R / 127: float per int8 level of the requantized output
};

__device__ __forceinline__ EpiScalars epi_scalars(const Epilogue& e) {
  EpiScalars s;
  const float la = dev_maxabs(*e.min_data, *e.max_data) / 127.0f;
  const float lb = dev_maxabs(*e.min_weight, *e.max_weight) / 127.0f;
  const float lc = la * lb;
  s.max_out = lc * 2147483648.0f;
  s.foq = static_cast<float>(static_cast<double>(dev_maxabs(-s.max_out, s.max_out)) /
                             2147483647.0);
  s.fbq = 0.f;
  if (e.bias != nullptr)
    s.fbq = static_cast<float>(static_cast<double>(dev_maxabs(*e.min_bias, *e.max_bias)) / 127.0);
  s.in_scale = dev_maxabs(-s.max_out, s.max_out) / 2147483648.0f;
  s.qscale = 127.0f / dev_maxabs(-e.real_range, e.real_range);
  s.dqscale = dev_maxabs(-e.real_range, e.real_range) / 127.0f;
  return s;
}

__device__ __forceinline__ int epi_bias32(const Epilogue& e, const EpiScalars& s, int n) {
  if (e.bias == nullptr || s.foq == 0.0f) return 0;
  float p = static_cast<float>(static_cast<int>(e.bias[n])) * s.fbq;
  return static_cast<int>(p / s.foq);
}

// FloatToQuantized<int8>(float(acc) * in_scale): trunc(sign(f) * min(|f|*s + 0.5, 127)),
// optionally followed by the int8 relu.  The magnitude |f|*s + 0.5 is >= 0.5, so giving
// it f's sign and clamping the signed value to [lo, 127] (lo = -127, or 0 with relu)
// before the truncating convert yields the same integer: copysign and clamp commute,
// trunc(+-0.5) = 0 covers f = +-0, and a negative value clamped to 0 is what relu makes
// of the negative int8.  One v_med3_f32 replaces the min and the integer max.
__device__ __forceinline__ int epi_requant(int acc, const EpiScalars& s, float lo) {
  float f = static_cast<float>(acc) * s.in_scale;
  float t = fabsf(f) * s.qscale;
  float u = copysignf(t + 0.5f, f);
  return static_cast<int>(__builtin_amdgcn_fmed3f(u, lo, 127.0f));
}
// The same with the relu, without the sign handling: for f > 0 these are the operations
// above (|f| = f); for f <= 0 the product is the exact negative of |f|*s, so the sum is at
// most 0.5 and the clamp to [0, 127] followed by the truncation gives the 0 that relu makes
// of a non-positive int8.
__device__ __forceinline__ int epi_requant_relu(int acc, const EpiScalars& s) {
  float f = static_cast<float>(acc) * s.in_scale;
  float u = f * s.qscale + 0.5f;
  return static_cast<int>(__builtin_amdgcn_fmed3f(u, 0.0f, 127.0f));
}

// The requantized int8 value taken back to float (an int8 dequantize over the calibrated
// range): float(q) * (R / 127), as bits.  The detour through the integer keeps +0 for a
// magnitude that truncates to zero from below.
__device__ __forceinline__ int epi_dequant_bits(int q, const EpiScalars& s) {
  return __builtin_bit_cast(int, static_cast<float>(q) * s.dqscale);
}

// {a,b,c,d} low bytes -> one dword (a in byte 0).
__device__ __forceinline__ uint32_t pack_bytes(int a, int b, int c, int d) {
  const uint32_t lo = __builtin_amdgcn_perm(static_cast<uint32_t>(b), static_cast<uint32_t>(a),
                                            0x0c0c0400u);
  const uint32_t hi = __builtin_amdgcn_perm(static_cast<uint32_t>(d), static_cast<uint32_t>(c),
                                            0x04000c0cu);
  return lo | hi;
}

// Four requantized outputs as one dword (first in byte 0).  (Converting the relu'd values as
// unsigned and or-ing them without byte masks saves a quarter instruction per output and
// measures the same: 19-layer stack 261.7 against 260.3 us.)
// With the relu the four values are in [0, 127] and v_cvt_pk_u8_f32 can take the place of
// the clamp's lower side, the truncating convert and the pack: it saturates at 0, writes
// byte k of its destination, and rounds as the wave's float rounding mode says.  The mode
// is switched to round-toward-zero for exactly the four converts (one asm statement, so
// that no multiply or add of the requantization can be scheduled into the stretch) and
// back: u = f * s + 0.5 itself is computed in round-to-nearest as before, only its
// truncation changes hands.  6.25 VALU instructions per output instead of 7.
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
__device__ __forceinline__ uint32_t epi_requant_relu_pack(int a0, int a1, int a2, int a3,
                                                          const EpiScalars& s) {
  auto level = [&](int a) {
    const float f = static_cast<float>(a) * s.in_scale;
    const float u = f * s.qscale + 0.5f;
    return (u < 127.0f) ? u : 127.0f;   // the reference's min(|f| * s + 0.5, 127)
  };
  const float u0 = level(a0), u1 = level(a1), u2 = level(a2), u3 = level(a3);
  uint32_t w;
  asm volatile(
      "s_setreg_imm32_b32 hwreg(HW_REG_MODE, 0, 2), 3\n\t"
      "v_cvt_pk_u8_f32 %0, %1, 0, 0\n\t"
      "v_cvt_pk_u8_f32 %0, %2, 1, %0\n\t"
      "v_cvt_pk_u8_f32 %0, %3, 2, %0\n\t"
      "v_cvt_pk_u8_f32 %0, %4, 3, %0\n\t"
      "s_setreg_imm32_b32 hwreg(HW_REG_MODE, 0, 2), 0"
      : "=&v"(w)
      : "v"(u0), "v"(u1), "v"(u2), "v"(u3));
  return w;
}
#pragma clang diagnostic pop

template <bool RELU>
__device__ __forceinline__ uint32_t epi_requant_pack(int a0, int a1, int a2, int a3,
                                                     const EpiScalars& s) {
  if (RELU) return epi_requant_relu_pack(a0, a1, a2, a3, s);
  return pack_bytes(epi_requant(a0, s, -127.0f), epi_requant(a1, s, -127.0f),
                    epi_requant(a2, s, -127.0f), epi_requant(a3, s, -127.0f));
}

// Bank-spreading XOR for the chunk index.  A fragment read is 32 consecutive
// rows at one logical chunk, 16 bytes per lane.  For CH = 4 the function is a
// bijection of row bits (1,2) for fixed bits (0,3) and of bits (2,3) for fixed
// bits (0,1), which makes any aligned group of 8 or of 16 consecutive rows hit
// distinct 16-byte bank groups whether the LDS serves 128 or 256 bytes per clock.
// For CH = 8 (r ^ r>>3) & 7 has the same two properties.
template <int CH>
__device__ __forceinline__ int swz(int r) {
  if (CH == 4) return (((r >> 1) ^ (r >> 3)) & 1) | (((r >> 2) & 1) << 1);
  if (CH == 8) return (r ^ (r >> 2)) & 7;
  if (CH == 16) return r & 15;
  return 0;
}

template <int BM_, int BN_, int BK_, int WM_, int WN_>
struct GemmCfg {
  static constexpr int BM = BM_, BN = BN_, BK = BK_, WM = WM_, WN = WN_;
  static constexpr int kThreads = 64 * WM * WN;
  static constexpr int CH = BK / 16;       // 16-byte chunks per tile row
  static constexpr int TM = BM / WM;       // wave tile
  static constexpr int TN = BN / WN;
  static constexpr int MI = TM / 32;       // 32x32 MFMA tiles per wave
  static constexpr int NI = TN / 32;
  static constexpr int KS = BK / 32;       // MFMA k-steps per stage
  static constexpr int A_CHUNKS = BM * CH / kThreads;
  static constexpr int B_CHUNKS = BN * CH / kThreads;
  static constexpr int ROWS_PER_PASS = kThreads / CH;
  static constexpr int STAGE_SLOTS = (BM + BN) * CH;
  // Second __launch_bounds__ argument (minimum waves per SIMD).  A 4-wave work-group alone
  // asks for 1, which lets the compiler budget 512 registers per lane and put the MFMA
  // results in the accumulation half of the file, from where every value costs the epilogue
  // a v_accvgpr_read (and a v_accvgpr_write to zero it).  Asking for 2 caps the budget at
  // 256 architected registers and selects the MFMA form that writes them directly; only
  // done where the accumulators leave room (not for 256 x 256 on 4 waves).
  static constexpr int kMinWaves = (kThreads <= 256 && MI * NI * 16 <= 128) ? 2 : 1;
  static_assert(BM % (32 * WM) == 0 && BN % (32 * WN) == 0, "wave tile");
  static_assert((BM * CH) % kThreads == 0 && (BN * CH) % kThreads == 0, "loader");
  static_assert(kThreads % CH == 0, "loader rows");
};

// Work-group -> tile mapping.  Hardware hands consecutive work-group ids to the
// 8 XCDs round-robin; remap so that each XCD (own L2) owns a contiguous run of
// logical tile ids, and order logical ids in bands of GROUP tile-rows so the run
// is a compact rectangle that shares activation rows and weight rows in L2.
__device__ __forceinline__ int xcd_remap(int bid, int total) {
  return ((total & 7) == 0) ? (bid & 7) * (total >> 3) + (bid >> 3) : bid;
}
__device__ __forceinline__ void band_coords(int lid, int tiles_m, int tiles_n, int& tm, int& tn) {
  constexpr int GROUP = 4;
  const int band = GROUP * tiles_n;
  const int g = lid / band;
  const int first_m = g * GROUP;
  const int rows = (tiles_m - first_m) < GROUP ? (tiles_m - first_m) : GROUP;
  const int in_band = lid - g * band;
  tm = first_m + in_band % rows;
  tn = in_band / rows;
}
__device__ __forceinline__ void tile_coords(int bid, int tiles_m, int tiles_n, int& tm,
                                            int& tn) {
  band_coords(xcd_remap(bid, tiles_m * tiles_n), tiles_m, tiles_n, tm, tn);
}
// The same for a grid of tiles x splits work-groups (split-K): consecutive logical ids walk
// the tiles of one K slice, so the work-groups an XCD owns share operand rows in its L2.
// `tile` is the tile's index in the counter and partial arrays.
__device__ __forceinline__ void tile_coords_split(int bid, int tiles_m, int tiles_n, int splits,
                                                  int& tm, int& tn, int& tile, int& z) {
  const int tiles = tiles_m * tiles_n;
  const int lid = xcd_remap(bid, tiles * splits);
  z = lid / tiles;
  tile = lid - z * tiles;
  band_coords(tile, tiles_m, tiles_n, tm, tn);
}

// 16 bytes of row `row` at byte offset k0; zero outside [0,K).  With ALIGNED the
// row start and K are multiples of 16 so a chunk is entirely in or out.
template <bool ALIGNED>
__device__ __forceinline__ v4i load_chunk(const int8_t* __restrict__ rowptr, bool row_ok, int k0,
                                          int K) {
  v4i r = {0, 0, 0, 0};
  if (!row_ok) return r;
  if (ALIGNED) {
    if (k0 < K) r = *reinterpret_cast<const v4i*>(rowptr + k0);
  } else {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      if (k0 + i < K) {
        uint32_t b = static_cast<uint8_t>(rowptr[k0 + i]);
        r[i >> 2] |= static_cast<int>(b << (8 * (i & 3)));
      }
    }
  }
  return r;
}

// Row-major operand with K contiguous: chunk (row, k0) = 16 bytes at base + row*K + k0.
// Used for the FC activation and for every weight operand.
template <class Cfg, int CHUNKS, bool ALIGNED>
struct RowFetch {
  const int8_t* ptr[CHUNKS];
  bool ok[CHUNKS];
  int K, lc;
  __device__ __forceinline__ void init(const int8_t* base, int row0, int rows, int K_) {
    K = K_;
    lc = threadIdx.x % Cfg::CH;
    const int lr = threadIdx.x / Cfg::CH;
#pragma unroll
    for (int j = 0; j < CHUNKS; ++j) {
      const int r = row0 + lr + j * Cfg::ROWS_PER_PASS;
      ok[j] = r < rows;
      ptr[j] = base + static_cast<size_t>(ok[j] ? r : 0) * K;
    }
  }
  __device__ __forceinline__ void fetch(int kt, v4i (&reg)[CHUNKS]) {
    const int k0 = kt * Cfg::BK + lc * 16;
#pragma unroll
    for (int j = 0; j < CHUNKS; ++j) reg[j] = load_chunk<ALIGNED>(ptr[j], ok[j], k0, K);
  }
};

// The K loop: double-buffered LDS stage, global loads for step kt+1 are issued
// before the MFMAs of step kt and parked in registers until the stage they
// replace has been consumed.  AF / BF provide fetch(kt, regs).
template <class Cfg, class AF, class BF>
__device__ __forceinline__ void gemm_mainloop(v16i (&acc)[Cfg::MI][Cfg::NI], AF& af, BF& bf,
                                              int KT, v4i (*lds)[Cfg::STAGE_SLOTS]) {
  constexpr int CH = Cfg::CH;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / Cfg::WN, wn = wave % Cfg::WN;

  // LDS slots this thread fills (chunk column fixed, rows advance by ROWS_PER_PASS)
  const int lc = tid % CH, lr = tid / CH;
  int a_slot[Cfg::A_CHUNKS], b_slot[Cfg::B_CHUNKS];
#pragma unroll
  for (int j = 0; j < Cfg::A_CHUNKS; ++j) {
    const int r = lr + j * Cfg::ROWS_PER_PASS;
    a_slot[j] = r * CH + (lc ^ swz<CH>(r));
  }
#pragma unroll
  for (int j = 0; j < Cfg::B_CHUNKS; ++j) {
    const int r = lr + j * Cfg::ROWS_PER_PASS;
    b_slot[j] = Cfg::BM * CH + r * CH + (lc ^ swz<CH>(r));
  }

  // fragment read slots (stage-relative) per MFMA k-step
  const int frow = lane & 31, fgrp = lane >> 5;
  int fa_slot[Cfg::KS][Cfg::MI], fb_slot[Cfg::KS][Cfg::NI];
#pragma unroll
  for (int ks = 0; ks < Cfg::KS; ++ks) {
    const int c = ks * 2 + fgrp;
#pragma unroll
    for (int mi = 0; mi < Cfg::MI; ++mi) {
      const int r = wm * Cfg::TM + mi * 32 + frow;
      fa_slot[ks][mi] = r * CH + (c ^ swz<CH>(r));
    }
#pragma unroll
    for (int ni = 0; ni < Cfg::NI; ++ni) {
      const int r = wn * Cfg::TN + ni * 32 + frow;
      fb_slot[ks][ni] = Cfg::BM * CH + r * CH + (c ^ swz<CH>(r));
    }
  }

#pragma unroll
  for (int mi = 0; mi < Cfg::MI; ++mi)
#pragma unroll
    for (int ni = 0; ni < Cfg::NI; ++ni)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[mi][ni][v] = 0;

  v4i ra[Cfg::A_CHUNKS], rb[Cfg::B_CHUNKS];
  auto stash = [&](int buf) {
#pragma unroll
    for (int j = 0; j < Cfg::A_CHUNKS; ++j) lds[buf][a_slot[j]] = ra[j];
#pragma unroll
    for (int j = 0; j < Cfg::B_CHUNKS; ++j) lds[buf][b_slot[j]] = rb[j];
  };

  af.fetch(0, ra);
  bf.fetch(0, rb);
  stash(0);
  __syncthreads();

  for (int kt = 0; kt < KT; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < KT) {
      af.fetch(kt + 1, ra);
      bf.fetch(kt + 1, rb);
    }
#pragma unroll
    for (int ks = 0; ks < Cfg::KS; ++ks) {
      v4i fa[Cfg::MI], fb[Cfg::NI];
#pragma unroll
      for (int mi = 0; mi < Cfg::MI; ++mi) fa[mi] = lds[buf][fa_slot[ks][mi]];
#pragma unroll
      for (int ni = 0; ni < Cfg::NI; ++ni) fb[ni] = lds[buf][fb_slot[ks][ni]];
#pragma unroll
      for (int mi = 0; mi < Cfg::MI; ++mi)
#pragma unroll
        for (int ni = 0; ni < Cfg::NI; ++ni)
          acc[mi][ni] =
              __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[ni], fa[mi], acc[mi][ni], 0, 0, 0);
    }
    if (kt + 1 < KT) stash(buf ^ 1);
    __syncthreads();
  }
}

// ---- direct-to-LDS main loop ------------------------------------------------------
// Fast path for 16-byte aligned operands below 2 GiB: tiles go from global memory
// straight into LDS (global_load_lds_dwordx4 / buffer_load_dwordx4 ... lds: no
// staging registers, no ds_write) through an NS-stage ring.  Each wave instruction
// fills 64 consecutive 16-byte slots; the bank swizzle is applied on the global side
// (lane for slot (r, c') fetches chunk c' ^ swz(r) of row r).
//
// The loads are issued through inline assembly, so the compiler's wait-count
// pass does not see them; completion is enforced here by hand: vmcnt counts
// them in issue order, and a wave waits until at most the newer stages' loads
// are outstanding before it joins the work-group barrier that publishes a stage.
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
__device__ __forceinline__ void dma_global(uint32_t lds_byte_addr, uint32_t voffset,
                                           const int8_t* sbase) {
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(lds_byte_addr), "v"(voffset), "s"(sbase)
               : "memory", "m0");
}
// Buffer form: lanes whose offset is outside [0, num_records) deliver zeros, which
// is how image halos, rows past the end of an operand and the K tail are filled.
__device__ __forceinline__ void dma_buffer(uint32_t lds_byte_addr, uint32_t voffset, v4i rsrc) {
  asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
               :
               : "s"(lds_byte_addr), "v"(voffset), "s"(rsrc)
               : "memory", "m0");
}
#pragma clang diagnostic pop

constexpr uint32_t kOutOfRange = 0x80000000u;  // operands are below 2 GiB

// Raw buffer descriptor over [base, base + bytes): stride 0, 32-bit data format.
__device__ __forceinline__ v4i make_rsrc(const void* base, uint32_t bytes) {
  const uint64_t a = reinterpret_cast<uint64_t>(base);
  v4i r;
  r.x = __builtin_amdgcn_readfirstlane(static_cast<int>(static_cast<uint32_t>(a)));
  r.y = __builtin_amdgcn_readfirstlane(static_cast<int>(static_cast<uint32_t>(a >> 32)));
  r.z = __builtin_amdgcn_readfirstlane(static_cast<int>(bytes));
  r.w = 0x00020000;
  return r;
}

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt range");
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
// Wait until at most `ahead` (clamped to [0, MAXS]) stages of CPT loads are outstanding.
template <int CPT, int MAXS>
__device__ __forceinline__ void wait_ahead(int ahead) {
  if constexpr (MAXS <= 0) {
    wait_vmcnt<0>();
  } else {
    if (ahead >= MAXS)
      wait_vmcnt<MAXS * CPT>();
    else
      wait_ahead<CPT, MAXS - 1>(ahead);
  }
}

// Slot geometry of DMA instruction i of a wave: rows (i*NW + wave)*(64/CH) ..., the
// chunk a lane fetches does not depend on i (swz() only looks at row bits the lane
// index provides).
template <class Cfg>
struct DmaLane {
  int row0;   // tile row of instruction 0 for this lane
  int c16;    // byte offset (within a 64-byte stage row) of the chunk this lane fetches
  static constexpr int kRowStep = (Cfg::kThreads / 64) * (64 / Cfg::CH);  // rows between instrs
  __device__ __forceinline__ void init(int wave, int lane) {
    const int slot = wave * 64 + lane;
    row0 = slot / Cfg::CH;
    c16 = ((slot % Cfg::CH) ^ swz<Cfg::CH>(row0)) * 16;
  }
};

// K-contiguous row-major operand (FC activation, every weight) through
// global_load_lds.  Needs K % BK == 0; rows past the end are clamped to the last
// row (they only feed accumulators that are never stored).  `kbeg` is the byte offset
// inside a row at which stage 0 starts (the K slice of a split-K work-group).
template <class Cfg, int INSTR>
struct RowIssuerGlobal {
  uint32_t voff[INSTR];
  const int8_t* base;
  __device__ __forceinline__ void init(const int8_t* b, int row_begin, int rows, int K, int wave,
                                       int lane, int kbeg = 0) {
    base = b + kbeg;
    DmaLane<Cfg> g;
    g.init(wave, lane);
#pragma unroll
    for (int i = 0; i < INSTR; ++i) {
      int row = row_begin + g.row0 + i * DmaLane<Cfg>::kRowStep;
      row = row < rows ? row : rows - 1;
      voff[i] = static_cast<uint32_t>(row) * static_cast<uint32_t>(K) + g.c16;
    }
  }
  __device__ __forceinline__ void issue(int i, int stage, uint32_t lds_addr) {
    dma_global(lds_addr, voff[i], base + static_cast<size_t>(stage) * Cfg::BK);
  }
  __device__ __forceinline__ void stage_done() {}
};

// The same operand through buffer loads: any K that is a multiple of 16; rows past
// the end and chunks past K arrive as zeros.
template <class Cfg, int INSTR>
struct RowIssuerBuffer {
  uint32_t roff[INSTR];
  int c16, K;
  v4i rsrc;
  __device__ __forceinline__ void init(const int8_t* b, int row_begin, int rows, int K_, int wave,
                                       int lane, int kbeg = 0) {
    K = K_;
    rsrc = make_rsrc(b, static_cast<uint32_t>(rows) * static_cast<uint32_t>(K_));
    DmaLane<Cfg> g;
    g.init(wave, lane);
    c16 = g.c16 + kbeg;
#pragma unroll
    for (int i = 0; i < INSTR; ++i) {
      const int row = row_begin + g.row0 + i * DmaLane<Cfg>::kRowStep;
      roff[i] = row < rows ? static_cast<uint32_t>(row) * static_cast<uint32_t>(K_) : kOutOfRange;
    }
  }
  __device__ __forceinline__ void issue(int i, int stage, uint32_t lds_addr) {
    const int k0 = stage * Cfg::BK + c16;
    const uint32_t v = (k0 < K && roff[i] != kOutOfRange) ? roff[i] + k0 : kOutOfRange;
    dma_buffer(lds_addr, v, rsrc);
  }
  __device__ __forceinline__ void stage_done() {}
};

// PIPE selects the software pipeline of the K loop:
//   0  wait + barrier, issue the next stage, read fragments, MFMA (compiler scheduled)
//   2  fragments double-buffered in registers across the barrier and the instruction
//      order pinned: after every MFMA exactly one fragment read for the next k-step
//      (and, in the first k-step, one DMA issue) is placed, so the matrix pipe is fed
//      back-to-back while LDS and DMA work trickles in between.
// AIssuer / BIssuer provide issue(instr, stage, lds_byte_addr) and stage_done(); stages
// are issued in increasing order, each exactly once, and only stages < KT.
// `after_prologue` runs once the first NS-1 stages are on their way: the place for work
// that only the epilogue needs (range scalars, bias) and whose loads and divisions should
// hide behind the first operand fetch rather than in front of it.
template <class Cfg, int NS, int PIPE, class AIssuer, class BIssuer, class AfterPrologue>
__device__ __forceinline__ void gemm_mainloop_dma(v16i (&acc)[Cfg::MI][Cfg::NI], AIssuer& ai,
                                                  BIssuer& bi, int KT, v4i* lds,
                                                  AfterPrologue&& after_prologue) {
  constexpr int CH = Cfg::CH, NW = Cfg::kThreads / 64;
  constexpr int AI = Cfg::A_CHUNKS, BI = Cfg::B_CHUNKS, CPT = AI + BI;
  constexpr int MI = Cfg::MI, NI = Cfg::NI, KS = Cfg::KS;
  constexpr int STAGE_BYTES = Cfg::STAGE_SLOTS * 16;
  static_assert((Cfg::BM * CH) % (NW * 64) == 0 && (Cfg::BN * CH) % (NW * 64) == 0, "dma tiling");
  static_assert(PIPE == 0 || PIPE == 2, "pipeline variant");
  static_assert(PIPE == 0 || NS >= 4, "cross-barrier fragment prefetch needs 4 stages");
  static_assert(CH == 4 || CH == 8 || CH == 16,
                "fragment addressing below needs swz() to ignore row bit 5");
  static_assert((NS - 2) * CPT < 64, "vmcnt range");
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / Cfg::WN, wn = wave % Cfg::WN;
  const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds));

  // DMA instruction j (0 .. CPT-1) of a stage; nothing is issued past the last stage
  auto issue_one = [&](int stage, int j) {
    if (stage >= KT) return;
    const uint32_t sb = lds0 + static_cast<uint32_t>(stage % NS) * STAGE_BYTES;
    if (j < AI)
      ai.issue(j, stage, sb + (j * NW + wave) * 1024);
    else
      bi.issue(j - AI, stage, sb + Cfg::BM * CH * 16 + ((j - AI) * NW + wave) * 1024);
    if (j == CPT - 1) {
      ai.stage_done();
      bi.stage_done();
    }
  };
  auto issue = [&](int stage) {
#pragma unroll
    for (int j = 0; j < CPT; ++j) issue_one(stage, j);
  };

  // Fragment addressing.  Row r = tile_row + 32*i + (lane & 31): 32*i does not touch
  // the row bits swz() looks at, so fragment i sits 32*CH slots after fragment 0, and
  // k-step ks flips bit 1 of the chunk index (chunk = 2*ks + lane/32).
  const int frow = lane & 31, fgrp = lane >> 5;
  const int ra = wm * Cfg::TM + frow, rb = wn * Cfg::TN + frow;
  int fa0[KS], fb0[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    fa0[ks] = ra * CH + ((ks * 2 + fgrp) ^ swz<CH>(ra));
    fb0[ks] = Cfg::BM * CH + rb * CH + ((ks * 2 + fgrp) ^ swz<CH>(rb));
  }
  // fragment f of a k-step: f < MI -> activation fragment f, else weight fragment f-MI
  auto read_one = [&](int stage, int ks, int f, v4i (&fa)[MI], v4i (&fb)[NI]) {
    const v4i* st = lds + (stage % NS) * Cfg::STAGE_SLOTS;
    if (f < MI)
      fa[f] = st[fa0[ks] + f * 32 * CH];
    else
      fb[f - MI] = st[fb0[ks] + (f - MI) * 32 * CH];
  };
  auto read_frags = [&](int stage, int ks, v4i (&fa)[MI], v4i (&fb)[NI]) {
#pragma unroll
    for (int f = 0; f < MI + NI; ++f) read_one(stage, ks, f, fa, fb);
  };

#pragma unroll
  for (int mi = 0; mi < MI; ++mi)
#pragma unroll
    for (int ni = 0; ni < NI; ++ni)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[mi][ni][v] = 0;

#pragma unroll
  for (int s = 0; s < NS - 1; ++s) issue(s);  // stages 0 .. min(KT, NS-1)-1
  after_prologue();
  auto last_issued = [&](int kt_now) {         // newest stage in flight during step kt_now
    const int l = kt_now + NS - 2;
    return l < KT - 1 ? l : KT - 1;
  };

  if (PIPE == 0) {
    for (int kt = 0; kt < KT; ++kt) {
      wait_ahead<CPT, NS - 2>(last_issued(kt) - kt);  // this wave's part of stage kt landed
      __builtin_amdgcn_s_barrier();                    // ... everybody's; stage kt-1 is free
      issue(kt + NS - 1);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        v4i fa[MI], fb[NI];
        read_frags(kt, ks, fa, fb);
#pragma unroll
        for (int mi = 0; mi < MI; ++mi)
#pragma unroll
          for (int ni = 0; ni < NI; ++ni)
            acc[mi][ni] =
                __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[ni], fa[mi], acc[mi][ni], 0, 0, 0);
      }
    }
  } else {
    static_assert(KS % 2 == 0, "fragment ping-pong assumes an even k-step count");
    constexpr int NF = MI + NI, SLOTS = MI * NI;
    v4i fa[2][MI], fb[2][NI];
    // stages 0 and 1 landed: everything newer than stage 1 may stay in flight
    wait_ahead<CPT, NS - 3>(last_issued(0) - 1);
    __builtin_amdgcn_s_barrier();
    read_frags(0, 0, fa[0], fb[0]);
    for (int kt = 0; kt < KT; ++kt) {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const int cur = ks & 1, nxt = cur ^ 1;
        const int nstage = (ks + 1 < KS) ? kt : kt + 1;  // kt+1 was published one barrier ago
        const int nks = (ks + 1 < KS) ? ks + 1 : 0;
#pragma unroll
        for (int mi = 0; mi < MI; ++mi) {
#pragma unroll
          for (int ni = 0; ni < NI; ++ni) {
            const int step = mi * NI + ni;
            acc[mi][ni] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[cur][ni], fa[cur][mi],
                                                                acc[mi][ni], 0, 0, 0);
            // spread NF fragment reads (and, in k-step 0, the CPT DMA issues of stage
            // kt+NS-1, which overwrites stage kt-1) over the MFMA slots of this k-step
#pragma unroll
            for (int f = 0; f < NF; ++f)
              if (f * SLOTS / NF == step) read_one(nstage, nks, f, fa[nxt], fb[nxt]);
            if (ks == 0) {
#pragma unroll
              for (int j = 0; j < CPT; ++j)
                if (j * SLOTS / CPT == step) issue_one(kt + NS - 1, j);
            }
            __builtin_amdgcn_sched_barrier(0);
          }
        }
      }
      // stage kt+2 landed for this wave; newest in flight is min(KT-1, kt+NS-1)
      wait_ahead<CPT, NS - 3>(last_issued(kt + 1) - (kt + 2));
      __builtin_amdgcn_s_barrier();
    }
  }
}

// Stores one wave's accumulators.  m_base/n_base: origin of the wave tile.
// What a kernel's epilogue is built for besides the int32 and int8 outputs.  Only the
// fully-connected kernels are built with the extras, each as an instantiation of its own:
// elsewhere their code is left out, which keeps cold kernels short.
constexpr int kEpiPlain = 0;  // out32 and / or out8
constexpr int kEpiF32 = 1;    // Epilogue::outf
constexpr int kEpiSum = 2;    // out8 with Epilogue::res added

inline int epi_mode(const Epilogue& e) {
  return e.outf != nullptr ? kEpiF32 : (e.res != nullptr ? kEpiSum : kEpiPlain);
}

template <class Cfg, int MODE = kEpiPlain>
__device__ __forceinline__ void gemm_epilogue(v16i (&acc)[Cfg::MI][Cfg::NI], const Epilogue& e,
                                              int m_base, int n_base, int M, int N,
                                              size_t ldo) {
  const int lane = threadIdx.x & 63;
  const EpiScalars s = epi_scalars(e);
  const int lrow = lane & 31, lgrp = lane >> 5;
  const bool n_vec_ok = (N & 3) == 0 && (ldo & 3) == 0;
#pragma unroll
  for (int ni = 0; ni < Cfg::NI; ++ni) {
#pragma unroll
    for (int vq = 0; vq < 4; ++vq) {
      const int n = n_base + ni * 32 + 8 * vq + 4 * lgrp;
      int b32[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) b32[i] = (n + i < N) ? epi_bias32(e, s, n + i) : 0;
#pragma unroll
      for (int mi = 0; mi < Cfg::MI; ++mi) {
        const int m = m_base + mi * 32 + lrow;
        if (m >= M || n >= N) continue;
        int v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
          v[i] = static_cast<int>(static_cast<uint32_t>(acc[mi][ni][4 * vq + i]) +
                                  static_cast<uint32_t>(b32[i]));
        const size_t off = static_cast<size_t>(m) * ldo + n;
        const bool full = n_vec_ok && (n + 3 < N);
        if (e.out32 != nullptr && e.plane > 0) {
          const int img = m / e.plane, pix = m - img * e.plane;
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (n + i < N)
              e.out32[(static_cast<size_t>(img) * N + (n + i)) * e.plane + pix] = v[i];
        } else if (e.out32 != nullptr) {
          if (full) {
            v4i w = {v[0], v[1], v[2], v[3]};
            *reinterpret_cast<v4i*>(e.out32 + off) = w;
          } else {
#pragma unroll
            for (int i = 0; i < 4; ++i)
              if (n + i < N) e.out32[off + i] = v[i];
          }
        }
        if (e.out8 != nullptr || (MODE == kEpiF32 && e.outf != nullptr)) {
          int q[4];
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            q[i] = epi_requant(v[i], s, e.relu ? 0.0f : -127.0f);
          }
          if (MODE == kEpiSum && e.res != nullptr && e.out8 != nullptr) {
            const SumRule r = sum_rule(dev_maxabs(-e.real_range, e.real_range),
                                       dev_maxabs(*e.res_min, *e.res_max), e.sum_min_calib,
                                       e.sum_max_calib);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              if (n + i < N) {
                // the overflow-safe form serves every rule on this rarely taken path
                const int b = static_cast<int>(e.res[off + i]);
                const uint32_t v8 = e.sum_relu ? sum_one<true, false>(q[i], b, r)
                                               : sum_one<false, false>(q[i], b, r);
                e.out8[off + i] = static_cast<int8_t>(v8 & 0xffu);
              }
            }
          } else if (e.out8 != nullptr) {
            if (full) {
              *reinterpret_cast<uint32_t*>(e.out8 + off) = pack_bytes(q[0], q[1], q[2], q[3]);
            } else {
#pragma unroll
              for (int i = 0; i < 4; ++i)
                if (n + i < N) e.out8[off + i] = static_cast<int8_t>(q[i]);
            }
          }
          if (MODE == kEpiF32 && e.outf != nullptr) {
            int* of = reinterpret_cast<int*>(e.outf);
            if (full && (reinterpret_cast<uintptr_t>(e.outf) & 15u) == 0) {
              v4i w = {epi_dequant_bits(q[0], s), epi_dequant_bits(q[1], s),
                       epi_dequant_bits(q[2], s), epi_dequant_bits(q[3], s)};
              *reinterpret_cast<v4i*>(of + off) = w;
            } else {
#pragma unroll
              for (int i = 0; i < 4; ++i)
                if (n + i < N) of[off + i] = epi_dequant_bits(q[i], s);
            }
          }
        }
      }
    }
  }
}

// Epilogue of the direct-to-LDS kernels.  The stage ring is free once the K loop is
// over, so it is reused to (a) hold the block's int32 bias once and (b) transpose
// each wave's int8 tile: lanes own 4 adjacent columns of 32 different rows after
// the MFMA, which would make every store instruction touch 32 cache lines with 8
// bytes each; staged through LDS a store instruction writes whole 64..128-byte row
// segments.  Falls back to gemm_epilogue when the output is not 16-byte friendly.
// What the epilogue needs from global memory, fetched before the K loop so that the
// scalar loads, the divisions and the bias load are hidden behind it: the range
// scalars and the int32 bias of column n0 + threadIdx.x.
struct EpiPre {
  EpiScalars s;
  int bias32;
  SumRule sum;  // the residual sum's scales (kernels built for it)
};
template <class Cfg, int MODE = kEpiPlain>
__device__ __forceinline__ EpiPre epi_prefetch(const Epilogue& e, int n0, int N) {
  static_assert(Cfg::kThreads >= Cfg::BN, "one thread per tile column");
  EpiPre p;
  p.s = epi_scalars(e);
  p.sum = SumRule{0.0f, 0.0f, 1};
  if (MODE == kEpiSum && e.res != nullptr)
    p.sum = sum_rule(dev_maxabs(-e.real_range, e.real_range),
                     dev_maxabs(*e.res_min, *e.res_max), e.sum_min_calib, e.sum_max_calib);
  const int t = threadIdx.x;
  p.bias32 = (t < Cfg::BN && n0 + t < N) ? epi_bias32(e, p.s, n0 + t) : 0;
  return p;
}

// Bytes of the stage ring one wave uses as scratch in gemm_epilogue_lds: its int8 tile
// (row pitch TN + 16) and, when the ring is large enough, one 32 x 32 int32 MFMA tile
// (row pitch 36 dwords: 16-byte aligned rows whose 16-lane write groups cover all banks).
template <class Cfg>
struct EpiScratch {
  static constexpr int kTile8 = Cfg::TM * (Cfg::TN + 16);
  static constexpr int kPitch32 = 36;
  static constexpr int kTile32 = 32 * kPitch32 * 4;
  static constexpr int kPerWave = kTile8 > kTile32 ? kTile8 : kTile32;
  static constexpr int kWaves = Cfg::kThreads / 64;
  // the int8 tile always has to fit; the int32 tile is optional
  static constexpr int kNeed8 = Cfg::BN * 4 + kWaves * kTile8;
  static constexpr int kNeed32 = Cfg::BN * 4 + kWaves * kPerWave;
};

template <class Cfg, int RING_BYTES, int MODE = kEpiPlain>
__device__ __forceinline__ void gemm_epilogue_lds(v16i (&acc)[Cfg::MI][Cfg::NI],
                                                  const Epilogue& e, const EpiPre& pre, int m0,
                                                  int n0, int M, int N, size_t ldo,
                                                  v4i* lds_v) {
  typedef EpiScratch<Cfg> Scratch;
  static_assert(RING_BYTES >= Scratch::kNeed8, "stage ring too small for the epilogue transpose");
  constexpr bool kStage32 = RING_BYTES >= Scratch::kNeed32;
  constexpr int kPerWave = kStage32 ? Scratch::kPerWave : Scratch::kTile8;
  constexpr int TM = Cfg::TM, TN = Cfg::TN, MI = Cfg::MI, NI = Cfg::NI;
  constexpr int LD = TN + 16;        // staged row pitch in bytes (keeps 16-byte alignment)
  constexpr int LPR = TN / 16;       // lanes per staged row on the way out
  constexpr int RPI = 64 / LPR;      // rows per store instruction
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / Cfg::WN, wn = wave % Cfg::WN;
  const int m_base = m0 + wm * TM, n_base = n0 + wn * TN;
  const bool fast8 = e.out8 == nullptr ||
                     ((N % 16 == 0) && (ldo % 16 == 0) &&
                      ((reinterpret_cast<uintptr_t>(e.out8) & 15u) == 0));
  const bool fast32 = e.out32 == nullptr ||
                      ((N % 4 == 0) && (ldo % 4 == 0) &&
                       ((reinterpret_cast<uintptr_t>(e.out32) & 15u) == 0));
  // the sum's scales; a rule whose products could overflow goes the general way with the
  // unaligned outputs
  const SumRule rule = pre.sum;
  const bool fasts = MODE != kEpiSum || e.res == nullptr ||
                     (((reinterpret_cast<uintptr_t>(e.res) & 15u) == 0) && rule.fast);
  const bool fastf = MODE != kEpiF32 || e.outf == nullptr ||
                     ((N % 4 == 0) && (ldo % 4 == 0) &&
                      ((reinterpret_cast<uintptr_t>(e.outf) & 15u) == 0));
  if (__builtin_expect(!(fast8 && fast32 && fastf && fasts), 0)) {
    gemm_epilogue<Cfg, MODE>(acc, e, m_base, n_base, M, N, ldo);
    return;
  }
  char* lds = reinterpret_cast<char*>(lds_v);
  int* sbias = reinterpret_cast<int*>(lds);
  char* stage = lds + Cfg::BN * 4 + wave * kPerWave;
  const EpiScalars s = pre.s;

  __syncthreads();  // every wave is done reading operand stages
  if (tid < Cfg::BN) sbias[tid] = pre.bias32;
  __syncthreads();

  const int lrow = lane & 31, lgrp = lane >> 5;
  // accumulator + bias in place: both outputs below start from it
#pragma unroll
  for (int ni = 0; ni < NI; ++ni) {
#pragma unroll
    for (int vq = 0; vq < 4; ++vq) {
      const int nl = ni * 32 + 8 * vq + 4 * lgrp;  // column inside the wave tile
      const v4i b = *reinterpret_cast<const v4i*>(sbias + wn * TN + nl);
#pragma unroll
      for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          acc[mi][ni][4 * vq + i] = static_cast<int>(
              static_cast<uint32_t>(acc[mi][ni][4 * vq + i]) + static_cast<uint32_t>(b[i]));
    }
  }

  // A 32-bit output, row-major: `quad(mi, ni, vq)` gives the 4 adjacent columns a lane holds
  // of MFMA tile (mi, ni).  One 32 x 32 tile at a time through the wave's scratch: stored
  // directly a lane's quads touch 32 rows with 32 bytes each; read back, 8 lanes cover one
  // 128-byte row and a store instruction writes 8 whole cache lines.
  auto store_rows32 = [&](int* out, auto quad) {
    if (kStage32) {
      int* t32 = reinterpret_cast<int*>(stage);
#pragma unroll
      for (int mi = 0; mi < MI; ++mi) {
#pragma unroll
        for (int ni = 0; ni < NI; ++ni) {
#pragma unroll
          for (int vq = 0; vq < 4; ++vq)
            *reinterpret_cast<v4i*>(t32 + lrow * Scratch::kPitch32 + 8 * vq + 4 * lgrp) =
                quad(mi, ni, vq);
          asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
          __builtin_amdgcn_wave_barrier();
          v4i back[4];
#pragma unroll
          for (int it = 0; it < 4; ++it)
            back[it] = *reinterpret_cast<const v4i*>(t32 + (it * 8 + (lane >> 3)) *
                                                               Scratch::kPitch32 +
                                                     (lane & 7) * 4);
          asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
          __builtin_amdgcn_wave_barrier();
#pragma unroll
          for (int it = 0; it < 4; ++it) {
            const int m = m_base + mi * 32 + it * 8 + (lane >> 3);
            const int n = n_base + ni * 32 + (lane & 7) * 4;
            if (m < M && n < N)
              *reinterpret_cast<v4i*>(out + static_cast<size_t>(m) * ldo + n) = back[it];
          }
        }
      }
    } else {
#pragma unroll
      for (int ni = 0; ni < NI; ++ni)
#pragma unroll
        for (int vq = 0; vq < 4; ++vq)
#pragma unroll
          for (int mi = 0; mi < MI; ++mi) {
            const int m = m_base + mi * 32 + lrow, n = n_base + ni * 32 + 8 * vq + 4 * lgrp;
            if (m < M && n < N)
              *reinterpret_cast<v4i*>(out + static_cast<size_t>(m) * ldo + n) = quad(mi, ni, vq);
          }
    }
  };
  auto acc_quad = [&](int mi, int ni, int vq) {
    return v4i{acc[mi][ni][4 * vq], acc[mi][ni][4 * vq + 1], acc[mi][ni][4 * vq + 2],
               acc[mi][ni][4 * vq + 3]};
  };

  // Branch weights only place code: the fused int8 path, the one short launches take, stays
  // contiguous, which shortens the instruction fetch of a launch whose code is cold (19-layer
  // ResNet stack 264.8 -> 260.4 us; int32-output launches +0.4 %).
  if (__builtin_expect(e.out32 != nullptr, 0)) {
    if (e.plane == 0) {
      store_rows32(e.out32, acc_quad);
    } else if (kStage32) {
      // planar: the tile goes into the scratch channel-major (a lane's 16 values are
      // one pixel of 16 channels; 32 lanes write 32 adjacent dwords), so that read
      // back a lane holds 4 adjacent pixels of one channel and 8 lanes cover the
      // tile's 32 pixels = one 128-byte run of that channel's plane (two runs where
      // the tile straddles two images)
      int* t32 = reinterpret_cast<int*>(stage);
#pragma unroll
      for (int mi = 0; mi < MI; ++mi) {
#pragma unroll
        for (int ni = 0; ni < NI; ++ni) {
#pragma unroll
          for (int vq = 0; vq < 4; ++vq)
#pragma unroll
            for (int i = 0; i < 4; ++i)
              t32[(8 * vq + 4 * lgrp + i) * Scratch::kPitch32 + lrow] = acc[mi][ni][4 * vq + i];
          asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
          __builtin_amdgcn_wave_barrier();
          if ((e.plane & 3) == 0) {
            // 4 | plane: 4 | pix and a lane's four pixels lie in one image
            const int c = lane >> 3, p4 = (lane & 7) * 4;
            v4i col[4];
#pragma unroll
            for (int it = 0; it < 4; ++it)
              col[it] = *reinterpret_cast<const v4i*>(t32 + (it * 8 + c) * Scratch::kPitch32 + p4);
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            __builtin_amdgcn_wave_barrier();
            const int m0 = m_base + mi * 32 + p4;
            const int img = m0 / e.plane, pix = m0 - img * e.plane;
#pragma unroll
            for (int it = 0; it < 4; ++it) {
              const int n = n_base + ni * 32 + it * 8 + c;
              if (n < N && m0 < M)
                *reinterpret_cast<v4i*>(e.out32 + (static_cast<size_t>(img) * N + n) * e.plane +
                                        pix) = col[it];
            }
          } else {
            // any other plane (7 x 7): a lane takes one pixel of the tile's 32, a store
            // instruction two channels, so that it still writes runs of up to 128 bytes
            // (broken only where the tile passes from one image to the next)
            const int p = lane & 31, c2 = lane >> 5;
            int col[16];
#pragma unroll
            for (int it = 0; it < 16; ++it) col[it] = t32[(it * 2 + c2) * Scratch::kPitch32 + p];
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            __builtin_amdgcn_wave_barrier();
            const int m = m_base + mi * 32 + p;
            const int img = m / e.plane, pix = m - img * e.plane;
#pragma unroll
            for (int it = 0; it < 16; ++it) {
              const int n = n_base + ni * 32 + it * 2 + c2;
              if (n < N && m < M)
                e.out32[(static_cast<size_t>(img) * N + n) * e.plane + pix] = col[it];
            }
          }
        }
      }
    } else {
#pragma unroll
      for (int ni = 0; ni < NI; ++ni)
#pragma unroll
        for (int vq = 0; vq < 4; ++vq)
#pragma unroll
          for (int mi = 0; mi < MI; ++mi) {
            const int m = m_base + mi * 32 + lrow, n = n_base + ni * 32 + 8 * vq + 4 * lgrp;
            if (m < M && n < N) {
              const v4i w = acc_quad(mi, ni, vq);
              const int img = m / e.plane, pix = m - img * e.plane;
#pragma unroll
              for (int i = 0; i < 4; ++i)  // N % 4 == 0 on this path
                e.out32[(static_cast<size_t>(img) * N + (n + i)) * e.plane + pix] = w[i];
            }
          }
    }
  }

  // the requantized result as float: requantize, then the int8 dequantize over the
  // calibrated range, element by element in registers
  if (MODE == kEpiF32 && e.outf != nullptr) {
    auto dequantized_tile = [&](auto relu) {
      store_rows32(reinterpret_cast<int*>(e.outf), [&](int mi, int ni, int vq) {
        v4i w;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int q = decltype(relu)::value ? epi_requant_relu(acc[mi][ni][4 * vq + i], s)
                                              : epi_requant(acc[mi][ni][4 * vq + i], s, -127.0f);
          w[i] = epi_dequant_bits(q, s);
        }
        return w;
      });
    };
    if (e.relu)
      dequantized_tile(std::true_type());
    else
      dequantized_tile(std::false_type());
  }

  if (e.out8 != nullptr) {
    // the staged tile leaves in 16-byte pieces in row-major order, 64 per store instruction
    // (a wave tile of 96 columns has 6 pieces per row: the last instruction is then partial)
    constexpr int kPieces = TM * LPR;
    constexpr int kIters = (kPieces + 63) / 64;
    // the residual operand's pieces are fetched now, behind the requantization's arithmetic
    v4i resv[MODE == kEpiSum ? kIters : 1];
    if constexpr (MODE == kEpiSum) {
      if (e.res != nullptr) {
#pragma unroll
        for (int it = 0; it < kIters; ++it) {
          const int piece = it * 64 + lane;
          const int rr = (64 % LPR == 0) ? it * RPI + lane / LPR : piece / LPR;
          const int c16 = (64 % LPR == 0) ? lane % LPR : piece - rr * LPR;
          const int m = m_base + rr, n = n_base + c16 * 16;
          resv[it] = v4i{0, 0, 0, 0};
          if ((kPieces % 64 == 0 || piece < kPieces) && m < M && n < N)
            resv[it] = __builtin_nontemporal_load(
                reinterpret_cast<const v4i*>(e.res + static_cast<size_t>(m) * ldo + n));
        }
      }
    }
    auto requantize_tile = [&](auto relu) {
#pragma unroll
      for (int ni = 0; ni < NI; ++ni)
#pragma unroll
        for (int vq = 0; vq < 4; ++vq)
#pragma unroll
          for (int mi = 0; mi < MI; ++mi) {
            const int nl = ni * 32 + 8 * vq + 4 * lgrp, ml = mi * 32 + lrow;
            *reinterpret_cast<uint32_t*>(stage + ml * LD + nl) =
                epi_requant_pack<decltype(relu)::value>(acc[mi][ni][4 * vq], acc[mi][ni][4 * vq + 1],
                                                        acc[mi][ni][4 * vq + 2],
                                                        acc[mi][ni][4 * vq + 3], s);
          }
    };
    if (e.relu)
      requantize_tile(std::true_type());
    else
      requantize_tile(std::false_type());
    // the wave reads back what its own lanes wrote: LDS executes a wave's
    // instructions in order, the wait makes the writes complete first
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_wave_barrier();
    auto store_tile = [&](auto stream, auto sum_mode) {
      constexpr int SM = decltype(sum_mode)::value;  // 0 no sum, 1 sum, 2 sum + relu
#pragma unroll
      for (int it = 0; it < kIters; ++it) {
        const int piece = it * 64 + lane;
        const int rr = (64 % LPR == 0) ? it * RPI + lane / LPR : piece / LPR;
        const int c16 = (64 % LPR == 0) ? lane % LPR : piece - rr * LPR;
        if (kPieces % 64 != 0 && piece >= kPieces) continue;
        v4i val = *reinterpret_cast<const v4i*>(stage + rr * LD + c16 * 16);
        if constexpr (SM != 0) {
#pragma unroll
          for (int w = 0; w < 4; ++w)
            val[w] = static_cast<int>(sum4<SM == 2, true>(
                static_cast<uint32_t>(val[w]), static_cast<uint32_t>(resv[it][w]), rule));
        }
        const int m = m_base + rr, n = n_base + c16 * 16;
        if (m < M && n < N)
          epi_store16<decltype(stream)::value>(val, e.out8 + static_cast<size_t>(m) * ldo + n);
      }
    };
    if constexpr (MODE == kEpiSum) {
      if (e.res != nullptr) {
        if (e.stream8) {
          if (e.sum_relu)
            store_tile(std::true_type(), std::integral_constant<int, 2>());
          else
            store_tile(std::true_type(), std::integral_constant<int, 1>());
        } else {
          if (e.sum_relu)
            store_tile(std::false_type(), std::integral_constant<int, 2>());
          else
            store_tile(std::false_type(), std::integral_constant<int, 1>());
        }
        return;
      }
    }
    if (e.stream8)
      store_tile(std::true_type(), std::integral_constant<int, 0>());
    else
      store_tile(std::false_type(), std::integral_constant<int, 0>());
  }
}

// ---- split-K -------------------------------------------------------------------------
// Shapes with few output tiles and a long reduction leave most CUs idle.  There `splits`
// work-groups share one output tile, each reducing a slice of kt_per_split K stages.  Integer
// accumulation is associative, so the sum of the slices is the unsplit result bit for bit.
// Every work-group of a tile leaves its accumulators in the workspace (in lane order: the
// work-group that reads them back has the same thread -> output mapping, so both sides
// move whole 1 KiB runs per wave instruction and nothing is transposed), then takes a
// ticket from the tile's counter; the one that draws the last ticket adds the other
// slices to its own registers and runs the ordinary epilogue, the others exit.  No
// work-group waits for another.
//
// Visibility across the XCDs' L2s without a fence: partials are written and read with
// device-scope accesses (sc1: written through to, and read from, the level all XCDs
// share), a work-group's stores have completed (vmcnt(0) on every lane, then the
// barrier) before its thread 0 takes the ticket with a device-scope atomic, and the last
// work-group issues its loads only after the atomic has returned.
struct SplitK {
  int splits;          // work-groups per output tile; 1 = no split
  int kt_per_split;    // K stages per work-group
  unsigned* counters;  // [tiles], zero when the kernel starts
  int* partials;       // [tiles][splits][BM * BN]
};

inline size_t splitk_counter_bytes(long tiles) {
  return (static_cast<size_t>(tiles) * 4 + 255) / 256 * 256;
}
inline size_t splitk_workspace_bytes(long tiles, int splits, int bm, int bn) {
  if (splits <= 1) return 0;
  return splitk_counter_bytes(tiles) + static_cast<size_t>(tiles) * splits * bm * bn * 4;
}

// (a template only so that every file including this header may define it)
template <int kBlock>
__global__ void splitk_zero_kernel(unsigned* counters, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) counters[i] = 0u;
}

// Host side: turns the requested split count into the kernel's SplitK (never more slices
// than K stages, no empty slice), carves the workspace and clears the counters on `s`.
template <class Cfg>
inline void splitk_setup(hipStream_t s, SplitK& sk, long tiles, int K, int splits, void* ws,
                         size_t ws_bytes) {
  const int KT = (K + Cfg::BK - 1) / Cfg::BK;
  if (splits > KT) splits = KT;
  if (splits < 1) splits = 1;
  sk.kt_per_split = (KT + splits - 1) / splits;
  if (sk.kt_per_split < 1) sk.kt_per_split = 1;
  sk.splits = KT > 0 ? (KT + sk.kt_per_split - 1) / sk.kt_per_split : 1;
  sk.counters = nullptr;
  sk.partials = nullptr;
  if (sk.splits <= 1) {
    sk.splits = 1;
    return;
  }
  const size_t need = splitk_workspace_bytes(tiles, sk.splits, Cfg::BM, Cfg::BN);
  MXQ_CHECK(ws != nullptr && aligned16(ws), "split-K needs a 16-byte aligned workspace");
  MXQ_CHECK(ws_bytes >= need, "split-K workspace too small: " << ws_bytes << " < " << need);
  MXQ_CHECK(tiles * sk.splits < (1L << 30), "split-K grid too large");
  sk.counters = static_cast<unsigned*>(ws);
  sk.partials = reinterpret_cast<int*>(static_cast<char*>(ws) + splitk_counter_bytes(tiles));
  hipLaunchKernelGGL(splitk_zero_kernel<256>, dim3(static_cast<unsigned>((tiles + 255) / 256)),
                     dim3(256), 0, s, sk.counters, static_cast<int>(tiles));
  MXQ_LAUNCH_CHECK();
}

// Device side, after the K loop of a split work-group.  Returns true in the work-group
// that arrived last: its accumulators then hold the sum over all slices.
template <class Cfg>
__device__ __forceinline__ bool splitk_gather(v16i (&acc)[Cfg::MI][Cfg::NI], const SplitK& sk,
                                              int tile, int z) {
  constexpr int MI = Cfg::MI, NI = Cfg::NI, QUADS = MI * NI * 4;
  constexpr int kTileInts = Cfg::BM * Cfg::BN;
  static_assert(QUADS * 4 * Cfg::kThreads == kTileInts, "lane-order layout covers the tile");
  constexpr int kDeviceScope = 16;  // sc1 in the buffer instructions' cache policy
  constexpr int kRsrcFlags = 0x00020000;
  const int tid = threadIdx.x;
  __shared__ unsigned s_ticket;
  int* tile_base = sk.partials + static_cast<size_t>(tile) * sk.splits * kTileInts;
  {
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
        tile_base + static_cast<size_t>(z) * kTileInts, 0, kTileInts * 4, kRsrcFlags);
#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
      for (int ni = 0; ni < NI; ++ni)
#pragma unroll
        for (int vq = 0; vq < 4; ++vq) {
          const v4i w = {acc[mi][ni][4 * vq], acc[mi][ni][4 * vq + 1], acc[mi][ni][4 * vq + 2],
                         acc[mi][ni][4 * vq + 3]};
          const int q = (mi * NI + ni) * 4 + vq;
          __builtin_amdgcn_raw_buffer_store_b128(w, rs, (q * Cfg::kThreads + tid) * 16, 0,
                                                 kDeviceScope);
        }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  if (tid == 0)
    s_ticket = __hip_atomic_fetch_add(sk.counters + tile, 1u, __ATOMIC_RELAXED,
                                      __HIP_MEMORY_SCOPE_AGENT);
  __syncthreads();
  if (s_ticket != static_cast<unsigned>(sk.splits - 1)) return false;
  for (int zz = 0; zz < sk.splits; ++zz) {
    if (zz == z) continue;
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
        tile_base + static_cast<size_t>(zz) * kTileInts, 0, kTileInts * 4, kRsrcFlags);
#pragma unroll
    for (int mi = 0; mi < MI; ++mi) {
      v4i w[NI * 4];
#pragma unroll
      for (int j = 0; j < NI * 4; ++j)
        w[j] = __builtin_amdgcn_raw_buffer_load_b128(
            rs, ((mi * NI * 4 + j) * Cfg::kThreads + tid) * 16, 0, kDeviceScope);
#pragma unroll
      for (int ni = 0; ni < NI; ++ni)
#pragma unroll
        for (int vq = 0; vq < 4; ++vq)
#pragma unroll
          for (int i = 0; i < 4; ++i)
            acc[mi][ni][4 * vq + i] =
                static_cast<int>(static_cast<uint32_t>(acc[mi][ni][4 * vq + i]) +
                                 static_cast<uint32_t>(w[ni * 4 + vq][i]));
    }
  }
  return true;
}

// Range scalars, written once per launch.
// MODE as for the epilogues: only a kernel built for the residual sum looks at its fields
// (three more scalar registers, which some of the tiled kernels do not have to spare).
template <int MODE = kEpiPlain>
__device__ __forceinline__ void epilogue_ranges(const Epilogue& e) {
  const EpiScalars s = epi_scalars(e);
  *e.omin = -s.max_out;
  *e.omax = s.max_out;
  // also for an output without elements, whose buffer pointer may be null
  if (e.rmin != nullptr && e.rmax != nullptr) {
    if (MODE == kEpiSum && e.with_sum) {  // the sum's calibrated range, as quantized_elemwise_add reports it
      *e.rmin = e.sum_min_calib;
      *e.rmax = e.sum_max_calib;
    } else {
      *e.rmin = -e.real_range;
      *e.rmax = e.real_range;
    }
  }
}

}  // namespace mxq
#endif  // MXQ_GEMM_H_
