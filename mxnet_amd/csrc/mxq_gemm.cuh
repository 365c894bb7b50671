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
#ifndef MXQ_GEMM_CUH_
#define MXQ_GEMM_CUH_

#include <hip/hip_runtime.h>

#include <cstdint>

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
  float* omin;             // int32 output range
  float* omax;
  float* rmin;             // requantized range (only with out8)
  float* rmax;
  int relu;
  float real_range;        // MaxAbs(min_calib, max_calib), host-computed
};

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
  return s;
}

__device__ __forceinline__ int epi_bias32(const Epilogue& e, const EpiScalars& s, int n) {
  if (e.bias == nullptr || s.foq == 0.0f) return 0;
  float p = static_cast<float>(static_cast<int>(e.bias[n])) * s.fbq;
  return static_cast<int>(p / s.foq);
}

// FloatToQuantized<int8>(float(acc) * in_scale) with the sign applied through
// the float before the truncating convert (trunc is odd; |v| >= 0.5 rounds a
// zero input to 0 either way).
__device__ __forceinline__ int epi_requant(int acc, const EpiScalars& s) {
  float f = static_cast<float>(acc) * s.in_scale;
  float t = fabsf(f) * s.qscale;
  float u = t + 0.5f;
  float v = (127.0f < u) ? 127.0f : u;
  int iv = static_cast<int>(v);
  return (f < 0.0f) ? -iv : ((f > 0.0f) ? iv : 0);
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
  if (CH == 8) return (r ^ (r >> 3)) & 7;
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
  static_assert(BM % (32 * WM) == 0 && BN % (32 * WN) == 0, "wave tile");
  static_assert((BM * CH) % kThreads == 0 && (BN * CH) % kThreads == 0, "loader");
  static_assert(kThreads % CH == 0, "loader rows");
};

// Work-group -> tile mapping.  Hardware hands consecutive work-group ids to the
// 8 XCDs round-robin; remap so that each XCD (own L2) owns a contiguous run of
// logical tile ids, and order logical ids in bands of GROUP tile-rows so the run
// is a compact rectangle that shares activation rows and weight rows in L2.
__device__ __forceinline__ void tile_coords(int bid, int tiles_m, int tiles_n, int& tm,
                                            int& tn) {
  const int total = tiles_m * tiles_n;
  int lid = bid;
  if ((total & 7) == 0) lid = (bid & 7) * (total >> 3) + (bid >> 3);
  constexpr int GROUP = 4;
  const int band = GROUP * tiles_n;
  const int g = lid / band;
  const int first_m = g * GROUP;
  const int rows = (tiles_m - first_m) < GROUP ? (tiles_m - first_m) : GROUP;
  const int in_band = lid - g * band;
  tm = first_m + in_band % rows;
  tn = in_band / rows;
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

// Stores one wave's accumulators.  m_base/n_base: origin of the wave tile.
template <class Cfg>
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
        if (e.out32 != nullptr) {
          if (full) {
            v4i w = {v[0], v[1], v[2], v[3]};
            *reinterpret_cast<v4i*>(e.out32 + off) = w;
          } else {
#pragma unroll
            for (int i = 0; i < 4; ++i)
              if (n + i < N) e.out32[off + i] = v[i];
          }
        }
        if (e.out8 != nullptr) {
          int q[4];
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            q[i] = epi_requant(v[i], s);
            if (e.relu) q[i] = q[i] > 0 ? q[i] : 0;
          }
          if (full) {
            uint32_t w = (uint32_t(q[0]) & 0xffu) | ((uint32_t(q[1]) & 0xffu) << 8) |
                         ((uint32_t(q[2]) & 0xffu) << 16) | (uint32_t(q[3]) << 24);
            *reinterpret_cast<uint32_t*>(e.out8 + off) = w;
          } else {
#pragma unroll
            for (int i = 0; i < 4; ++i)
              if (n + i < N) e.out8[off + i] = static_cast<int8_t>(q[i]);
          }
        }
      }
    }
  }
}

// Range scalars, written once per launch.
__device__ __forceinline__ void epilogue_ranges(const Epilogue& e) {
  const EpiScalars s = epi_scalars(e);
  *e.omin = -s.max_out;
  *e.omax = s.max_out;
  if (e.out8 != nullptr && e.rmin != nullptr) {
    *e.rmin = -e.real_range;
    *e.rmax = e.real_range;
  }
}

}  // namespace mxq
#endif  // MXQ_GEMM_CUH_
