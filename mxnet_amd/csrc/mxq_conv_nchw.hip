// _contrib_quantized_conv on the operator's own tensors: NCHW int8 data, OIHW int8
// weights, NCHW int32 output (src/operator/quantization/quantized_conv.cc:38-45).  The
// reference's GPU operator brings both operands to NHWC with two TransposeImpl calls,
// runs cuDNN, and transposes the result back (quantized_conv.cu:145-148,183).  Here a
// 1 x 1 convolution, which is most of a bottleneck network, never leaves NCHW:
//
//   out[n][o][p] = bias32[o] + sum_c W[o][c] * X[n][c][p]        p = pixel of the plane
//
// per image is a GEMM whose activation operand lies "K-major" in memory: channel rows of
// contiguous pixels.  A work-group stages [BK channels] x [BP pixels] slabs of the plane
// straight into LDS (buffer_load ... lds, 16 bytes of one channel row per lane) and reads
// the MFMA fragments out of them with the transposing LDS load of gfx950
// (ds_read_b64_tr_b8): 16 lanes that point at 8 channel rows x 16 pixels get back, per
// lane, one pixel's 8 consecutive channels, which is the operand layout
// v_mfma_i32_32x32x32_i8 wants.  The weights [O][C] are already K-contiguous (OIHW of a
// 1 x 1 window is OHWI) and take the same path as in the fully-connected kernel.  In the
// result a lane holds one pixel and registers hold channels, so every store instruction
// writes two 128-byte runs of two channel planes: the int32 output goes to its NCHW place
// straight from the accumulators.  No adapter launch, no second copy of any tensor.
//
// Unit-stride planes of 4 | P bytes that are no multiple of 16 (14 x 14) take the same direct
// loads: 16 bytes from a dword mark, over columns padded to a multiple of 16 per image (a
// plane's last piece runs into the next channel's first pixels; those columns are never
// stored) and pixel tiles that run across image boundaries.  Strided 1 x 1 convolutions run
// in the same kernel with a gathering loader: a thread fetches the four pixels of its LDS
// dword from wherever the stride puts them (one 8-byte load and a v_perm for stride 2 over
// rows of 4 | OW pixels, two dwords for 2 | OW, bytes otherwise) and the operand becomes the
// matrix [C][N * OH * OW].  No workspace, no pre-pass: a strided layer reads only the cache
// lines it uses.  Where that loader would have to fetch single bytes (odd rows, 7 x 7
// planes), and for strided layers with a large weight matrix, a pre-pass gathers the pixels
// into one row per channel in the caller's workspace first and the kernel reads that with
// its 16-byte loads.  Everything else (3 x 3, padded 1 x 1, C % 16 != 0) takes the NHWC
// kernels of mxq_conv.hip behind the layout adapters.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>

#include "../../include/mxq.h"
#include "mxq_common.h"
#include "mxq_gemm.h"
#include "mxq_tiles.h"

namespace mxq {

// mxq_conv.hip: both operand transposes of the adapter route (w_out == nullptr: data only)
void nchw_to_nhwc_pair(hipStream_t s, const int8_t* data, int8_t* d_out, int N, int C, int H,
                       int W, int Cp, const int8_t* weight, int8_t* w_out, int O, int KH, int KW);

namespace {

// The activation operand as rows of one channel each.  GM == 0 (native): image n, channel
// c, pixel p at data[n * img_stride + c * row_stride + p], planes of 16 | P bytes read as they
// lie, pixel tiles inside one image.  GM != 0 (gathered): the operand is the matrix
// [C][N * P] whose column n * P + oh * OW + ow is input pixel (oh * sh, ow * sw) of image n --
// what a strided layer reads, or a plane whose size is no multiple of 16 -- and pixel tiles
// run over the columns regardless of where one image ends.
struct PlaneArgs {
  const int8_t* data;
  const int8_t* weight;  // [O][C]
  int N, C, P, O;        // P = output pixels per image
  int img_stride, row_stride;   // native
  int pitch;             // native, 0: pixel tiles inside one image.  > 0 (a multiple of 16):
                         // pixel tiles over the columns of the whole batch, image n's P pixels
                         // at columns n * pitch ... -- either a pre-gathered operand
                         // (gather_planes_kernel: one row per channel, img_stride == pitch) or
                         // the tensor itself read in 16-byte pieces from dword marks (planes of
                         // 4 | P bytes: img_stride = C * P, row_stride = P; a plane's last piece
                         // runs into the next channel's pixels, whose columns are never stored)
  int H, W, OW, sh, sw;         // gathered: input plane, output row length, strides
  uint32_t data_bytes;   // extent of the activation tensor
  int tiles_p, tiles_o;  // pixel tiles (per image if native, per matrix if gathered), channel tiles
  int stream32;          // the int32 planes leave with non-temporal stores
  Epilogue epi;          // bias, input ranges, out32 ([N][O][P]), omin / omax
};

// Tile of BP pixels x BO output channels; BK channels per stage.  The names CH / BK /
// kThreads are what DmaLane and RowIssuerBuffer (mxq_gemm.h) read for the weight operand.
template <int BP_, int BO_, int BK_, int WP_, int WO_>
struct PlaneCfg {
  static constexpr int BP = BP_, BO = BO_, BK = BK_, WP = WP_, WO = WO_;
  static constexpr int NW = WP * WO, kThreads = 64 * NW;
  static constexpr int CHP = BP / 16;      // 16-byte pixel chunks per channel row
  static constexpr int CH = BK / 16;       // 16-byte chunks per weight row
  static constexpr int TP = BP / WP, TO = BO / WO;
  static constexpr int MI = TP / 32, NI = TO / 32, KS = BK / 32;
  static constexpr int A_SLOTS = BK * CHP, B_SLOTS = BO * CH;
  static constexpr int STAGE_SLOTS = A_SLOTS + B_SLOTS;
  static constexpr int A_INSTR = A_SLOTS / (64 * NW), B_INSTR = B_SLOTS / (64 * NW);
  // gathered operand: a thread owns one group of 4 consecutive pixels (one LDS dword per
  // channel) and every TPG-th channel of a stage
  static constexpr int GROUPS = BP / 4, TPG = kThreads / GROUPS, CPS = BK / TPG;
  static_assert(BP % (32 * WP) == 0 && BO % (32 * WO) == 0, "wave tile");
  static_assert(A_SLOTS % (64 * NW) == 0 && B_SLOTS % (64 * NW) == 0, "loader");
  static_assert(CHP == 4 || CHP == 8 || CHP == 16, "pixel-chunk swizzle");
  static_assert(CH == 4 || CH == 8 || CH == 16, "fragment addressing of the weight operand");
  static_assert(kThreads % GROUPS == 0 && BK % TPG == 0 && TPG % 8 == 0,
                "gathering loader: a thread's channels share their low three bits");
};

// Where pixel chunk pc of channel row c sits in its row: pc ^ plane_swz(c).  A transposing
// read touches, per 16 lanes, one 16-byte chunk of 8 consecutive rows, and two such groups
// (chunks pc and pc + 1, pc even) go through the LDS together: the XOR makes those 16
// pieces hit 16 different bank groups.  Rows of 128 bytes: the row's low three bits; rows
// of 64 bytes (four rows per 256 bytes of banks): bit 2 of the row moves the chunk by two;
// rows of 256 bytes (every row on the same banks): twice the row's low three bits, so that
// one group takes the even and the other the odd chunks.
template <int CHP>
__device__ __forceinline__ int plane_swz(int c) {
  return CHP == 8 ? (c & 7) : (CHP == 16 ? 2 * (c & 7) : ((c >> 1) & 2));
}

typedef int v2i __attribute__((ext_vector_type(2)));

__device__ __forceinline__ v2i lds_read_tr8(const char* p) {
  return __builtin_amdgcn_ds_read_tr8_b64_v2i32(
      (v2i __attribute__((address_space(3)))*)(p));
}

// How a gathered operand's four pixels of a group are fetched.
constexpr int kNative = 0;      // not gathered: 16-byte direct-to-LDS loads
// (1 was a dword-gathering loader for unit-stride planes of 4 | P bytes; the direct loads read
// those now)
constexpr int kGatherPair = 2;  // sw == 2, 4 | OW, rows on 8-byte marks: 8 bytes and a v_perm
constexpr int kGatherBytes = 3; // anything else: byte by byte
constexpr int kGatherPair2 = 4; // sw == 2, 2 | OW, rows on dword marks: two dwords (two pixels
                                // each, a pair never leaves its row) and a v_perm

// Lab builds (-DMXQ_STAMPS) record, for every work-group's first lane, the shader clock and
// the 100 MHz real-time counter at four points of the kernel (entry, first stage issued,
// K loop done, last store issued); mxq_dbg_read_plane_stamps copies them out.  The product
// build compiles none of it.
#ifdef MXQ_STAMPS
__device__ long long mxq_dbg_plane_stamps[8 * 16384];
#define PLANE_STAMP(k)                                                                   \
  do {                                                                                   \
    if (threadIdx.x == 0 && blockIdx.x < 16384) {                                        \
      mxq_dbg_plane_stamps[blockIdx.x * 8 + (k)] = __builtin_readcyclecounter();         \
      mxq_dbg_plane_stamps[blockIdx.x * 8 + 4 + (k)] = __builtin_amdgcn_s_memrealtime(); \
    }                                                                                    \
  } while (0)
#else
#define PLANE_STAMP(k)
#endif

template <class Cfg, int NS, int GM>
__global__ __launch_bounds__(Cfg::kThreads, 2) void conv1x1_planes_kernel(PlaneArgs p) {
  PLANE_STAMP(0);
  constexpr int BP = Cfg::BP, BK = Cfg::BK, CHP = Cfg::CHP, CH = Cfg::CH, NW = Cfg::NW;
  constexpr int MI = Cfg::MI, NI = Cfg::NI, KS = Cfg::KS;
  constexpr int AI = GM == kNative ? Cfg::A_INSTR : 0, BI = Cfg::B_INSTR, CPT = AI + BI;
  constexpr int STAGE_BYTES = Cfg::STAGE_SLOTS * 16, A_BYTES = Cfg::A_SLOTS * 16;
  static_assert((NS - 2) * CPT < 64, "vmcnt range");
  static_assert(GM == kNative || NS == 2, "the gathering loader works one stage ahead");
  __shared__ __attribute__((aligned(16))) v4i lds[NS * Cfg::STAGE_SLOTS];
  __shared__ __attribute__((aligned(16))) int sbias[Cfg::BO];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wp = wave / Cfg::WO, wo = wave % Cfg::WO;

  // tile order: the output-channel tiles of one pixel slab are neighbours, and the
  // round-robin of work-group ids over the XCDs is undone so that they meet in one L2
  constexpr bool gathered = GM != kNative;
  const bool flat = gathered || p.pitch != 0;   // pixel tiles run over the whole batch
  const int pitch = gathered ? p.P : p.pitch;   // columns per image then
  const int images = flat ? 1 : p.N;
  const int total = images * p.tiles_p * p.tiles_o;
  const int lid = xcd_remap(blockIdx.x, total);
  const int to = lid % p.tiles_o;
  const int rest = lid / p.tiles_o;
  const int tp = rest % p.tiles_p, n = rest / p.tiles_p;
  const int p0 = tp * BP, o0 = to * Cfg::BO;
  const int KT = (p.C + BK - 1) / BK;
  const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds));

  // native activation loads: slot q of a stage (16 bytes) = channel row q / CHP, chunk q % CHP
  const v4i arsrc = make_rsrc(p.data, p.data_bytes);
  uint32_t a_off[AI > 0 ? AI : 1];
  int a_c[AI > 0 ? AI : 1];
  if constexpr (!gathered) {
#pragma unroll
    for (int j = 0; j < AI; ++j) {
      const int q = (j * NW + wave) * 64 + lane;
      const int c = q / CHP, pc = (q % CHP) ^ plane_swz<CHP>(c);
      a_c[j] = c;
      if (p.pitch != 0) {
        // columns over the whole batch, `pitch` (a multiple of 16) per image: the chunk's image
        const int v = p0 + pc * 16, img = v / p.pitch;
        a_off[j] = img < p.N ? static_cast<uint32_t>(img) * p.img_stride + (v - img * p.pitch) +
                                   static_cast<uint32_t>(c) * p.row_stride
                             : kOutOfRange;
      } else {
        a_off[j] = static_cast<uint32_t>(n) * p.img_stride +
                   static_cast<uint32_t>(c) * p.row_stride + p0 + pc * 16;
      }
    }
  }
  RowIssuerBuffer<Cfg, BI> bi;
  bi.init(p.weight, o0, p.O, p.C, wave, lane, 0);
  // direct-to-LDS loads of a stage: the weights, and the native activation slab
  auto issue = [&](int stage) {
    if (stage >= KT) return;
    const uint32_t sb = lds0 + static_cast<uint32_t>(stage % NS) * STAGE_BYTES;
#pragma unroll
    for (int j = 0; j < AI; ++j) {
      const int c = stage * BK + a_c[j];
      const uint32_t off =
          c < p.C ? a_off[j] + static_cast<uint32_t>(stage * BK) * p.row_stride : kOutOfRange;
      dma_buffer(sb + (j * NW + wave) * 1024, off, arsrc);
    }
#pragma unroll
    for (int j = 0; j < BI; ++j) bi.issue(j, stage, sb + A_BYTES + (j * NW + wave) * 1024);
  };

  // gathered activation loads: this thread's pixel group and first channel of a stage
  constexpr int CPS = Cfg::CPS, TPG = Cfg::TPG;
  const int grp = tid % Cfg::GROUPS, cs = tid / Cfg::GROUPS;
  const int plane_in = p.H * p.W;
  int goff[4] = {0, 0, 0, 0};   // byte offsets of the group's pixels in channel 0 of the tensor
  if constexpr (gathered) {
    const long long V = 1LL * p.N * p.P;
#pragma unroll
    for (int j = 0; j < ((GM == kGatherBytes || GM == kGatherPair2) ? 4 : 1); ++j) {
      const long long v = 1LL * p0 + 4 * grp + j;
      const int vv = v < V ? static_cast<int>(v) : 0;   // columns past the end read pixel 0
      const int img = vv / p.P, px = vv - img * p.P;
      const int oh = px / p.OW, ow = px - oh * p.OW;
      goff[j] = img * p.C * plane_in + oh * p.sh * p.W + ow * p.sw;
    }
  }
  uint32_t areg[gathered ? CPS : 1];
  auto gather = [&](int stage) {
    if constexpr (gathered) {
#pragma unroll
      for (int i = 0; i < CPS; ++i) {
        int c = stage * BK + cs + TPG * i;
        c = c < p.C ? c : p.C - 1;   // the weights' zero K tail cancels whatever these rows hold
        const int8_t* row = p.data + static_cast<size_t>(c) * plane_in;
        if (GM == kGatherPair) {
          typedef uint32_t u2 __attribute__((ext_vector_type(2)));
          const u2 w = *reinterpret_cast<const u2*>(row + goff[0]);
          areg[i] = __builtin_amdgcn_perm(w.y, w.x, 0x06040200u);
        } else if (GM == kGatherPair2) {
          const uint32_t w0 = *reinterpret_cast<const uint32_t*>(row + goff[0]);
          const uint32_t w1 = *reinterpret_cast<const uint32_t*>(row + goff[2]);
          areg[i] = __builtin_amdgcn_perm(w1, w0, 0x06040200u);
        } else {
          const uint32_t b0 = static_cast<uint8_t>(row[goff[0]]);
          const uint32_t b1 = static_cast<uint8_t>(row[goff[1]]);
          const uint32_t b2 = static_cast<uint8_t>(row[goff[2]]);
          const uint32_t b3 = static_cast<uint8_t>(row[goff[3]]);
          areg[i] = b0 | (b1 << 8) | (b2 << 16) | (b3 << 24);
        }
      }
    }
  };
  // LDS dword of (channel row cs + TPG * i, pixel group grp): TPG is a multiple of 8, so the
  // row's swizzle is that of cs for every i
  const int gslot = cs * BP + ((((grp >> 2) ^ plane_swz<CHP>(cs))) << 4) + ((grp & 3) << 2);
  auto stash = [&](int stage) {
    if constexpr (gathered) {
      char* sa = reinterpret_cast<char*>(lds) + (stage % NS) * STAGE_BYTES;
#pragma unroll
      for (int i = 0; i < CPS; ++i)
        *reinterpret_cast<uint32_t*>(sa + gslot + TPG * i * BP) = areg[i];
    }
  };

  // fragment addresses.  Activation: lane = 16 * G + s reads 8 bytes of channel row
  // 16 * (G / 2) + s / 2 (+ 32 * ks + 8 * t) at pixel 16 * (G % 2) + 8 * (s % 2) of MFMA
  // tile mi; the transposing load hands lane l the 8 channels of pixel l % 32, and two
  // such loads (t = 0, 1) make the 16 bytes of k-group l / 32.
  const int G = lane >> 4, s16 = lane & 15;
  const int crow = 16 * (G >> 1) + (s16 >> 1);
  int a_frag[MI];
#pragma unroll
  for (int mi = 0; mi < MI; ++mi) {
    const int pc = (wp * Cfg::TP + 32 * mi) / 16 + (G & 1);
    a_frag[mi] = crow * BP + ((pc ^ plane_swz<CHP>(crow)) << 4) + 8 * (s16 & 1);
  }
  const int frow = lane & 31, fgrp = lane >> 5;
  const int rb = wo * Cfg::TO + frow;
  int fb0[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) fb0[ks] = rb * CH + ((ks * 2 + fgrp) ^ swz<CH>(rb));

  v16i acc[MI][NI];
#pragma unroll
  for (int mi = 0; mi < MI; ++mi)
#pragma unroll
    for (int ni = 0; ni < NI; ++ni)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[mi][ni][v] = 0;

  auto compute = [&](int kt) {
    const char* sa = reinterpret_cast<const char*>(lds) + (kt % NS) * STAGE_BYTES;
    const v4i* sbw = reinterpret_cast<const v4i*>(sa + A_BYTES);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      v4i fa[MI], fb[NI];
#pragma unroll
      for (int mi = 0; mi < MI; ++mi) {
        const v2i lo = lds_read_tr8(sa + a_frag[mi] + (32 * ks) * BP);
        const v2i hi = lds_read_tr8(sa + a_frag[mi] + (32 * ks + 8) * BP);
        fa[mi] = v4i{lo.x, lo.y, hi.x, hi.y};
      }
#pragma unroll
      for (int ni = 0; ni < NI; ++ni) fb[ni] = sbw[fb0[ks] + ni * 32 * CH];
#pragma unroll
      for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int ni = 0; ni < NI; ++ni)
          acc[mi][ni] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[ni], fa[mi], acc[mi][ni], 0, 0, 0);
    }
  };

  if constexpr (!gathered) {
#pragma unroll
    for (int st = 0; st < NS - 1; ++st) issue(st);
  } else {
    gather(0);
    issue(0);
  }
  // what the epilogue needs, behind the first operand fetch
  const EpiScalars es = epi_scalars(p.epi);
  if (tid < Cfg::BO) sbias[tid] = (o0 + tid < p.O) ? epi_bias32(p.epi, es, o0 + tid) : 0;

  PLANE_STAMP(1);
  if constexpr (!gathered) {
    for (int kt = 0; kt < KT; ++kt) {
      const int newest = (kt + NS - 2) < (KT - 1) ? (kt + NS - 2) : (KT - 1);
      wait_ahead<CPT, NS - 2>(newest - kt);
      __builtin_amdgcn_s_barrier();
      issue(kt + NS - 1);
      compute(kt);
    }
  } else {
    // one stage ahead: the registers and the weights' direct loads of stage kt + 1 are on
    // their way while stage kt is multiplied; both have landed (vmcnt counts them together)
    // before the registers go to LDS and the barrier publishes the stage
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    stash(0);
    __syncthreads();
    for (int kt = 0; kt < KT; ++kt) {
      if (kt + 1 < KT) {
        gather(kt + 1);
        issue(kt + 1);
      }
      compute(kt);
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      if (kt + 1 < KT) stash(kt + 1);
      __syncthreads();
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  PLANE_STAMP(2);
  if (blockIdx.x == 0 && tid == 0) epilogue_ranges(p.epi);
  __syncthreads();  // sbias

  // In the accumulators a lane holds one pixel and registers hold channels
  // (8 * (v / 4) + 4 * (lane / 32) + v % 4 of the MFMA tile).
  if ((p.P & 3) == 0 && (reinterpret_cast<uintptr_t>(p.epi.out32) & 15u) == 0) {
    // Planes of whole 16-byte runs: the wave's tile goes through its share of the (now free)
    // stage ring, channel-major, and leaves with 16 bytes per lane along the pixels, so a
    // store instruction writes runs of 4 * TP bytes of 256 / TP channel planes instead of two
    // runs of 128 bytes (measured on store-only kernels of this shape: 2.9 -> 4.8 TB/s for
    // 14 x 14 planes, 4.2 -> 5.0 for 28 x 28).  A group of four pixels never straddles two
    // images because 4 | P.  The stores are plain ones except for the very largest outputs
    // (`stream32`, set by the launcher): with the non-temporal hint that pays for the int8
    // tiles of the NHWC kernels on every layer, the 19 ResNet-50 layers through this entry
    // point took 517.8 us instead of 500.0 (same box, same command).
    constexpr int TP = Cfg::TP, LP = TP + 8;   // row pitch in dwords: lanes 32-63 write four
                                               // rows further down, 32 banks away
    constexpr int RING = NS * STAGE_BYTES;
    constexpr int CHB = (32 * LP * 4 * NW <= RING) ? 32 : ((16 * LP * 4 * NW <= RING) ? 16 : 8);
    static_assert(CHB * LP * 4 * NW <= RING, "stage ring too small for the epilogue's tile");
    constexpr int LPR = TP / 4, RPI = 64 / LPR;   // lanes per channel row, rows per instruction
    int* t32 = reinterpret_cast<int*>(lds) + wave * (CHB * LP);
    const int px4 = (lane % LPR) * 4, r0 = lane / LPR;
    const int v = p0 + wp * TP + px4;
    int img = n, px = v;
    if (flat) {
      img = v / pitch;
      px = v - img * pitch;
    }
    const bool ok = img < p.N && px < p.P;
    int32_t* obase = p.epi.out32 + static_cast<size_t>(img) * p.O * p.P + px;
#pragma unroll
    for (int ni = 0; ni < NI; ++ni) {
#pragma unroll
      for (int part = 0; part < 32 / CHB; ++part) {
#pragma unroll
        for (int vq = 0; vq < 4; ++vq) {
          if ((8 * vq) / CHB != part) continue;
          const int ol = wo * Cfg::TO + ni * 32 + 8 * vq + 4 * fgrp;  // channel inside the tile
          const v4i b = *reinterpret_cast<const v4i*>(sbias + ol);
#pragma unroll
          for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int mi = 0; mi < MI; ++mi)
              t32[((8 * vq) % CHB + 4 * fgrp + i) * LP + 32 * mi + frow] =
                  static_cast<int>(static_cast<uint32_t>(acc[mi][ni][4 * vq + i]) +
                                   static_cast<uint32_t>(b[i]));
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_wave_barrier();
        v4i back[CHB / RPI];
#pragma unroll
        for (int it = 0; it < CHB / RPI; ++it)
          back[it] = *reinterpret_cast<const v4i*>(t32 + (it * RPI + r0) * LP + px4);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_wave_barrier();
        if (p.stream32) {
#pragma unroll
          for (int it = 0; it < CHB / RPI; ++it) {
            const int o = o0 + wo * Cfg::TO + ni * 32 + part * CHB + it * RPI + r0;
            if (ok && o < p.O)
              __builtin_nontemporal_store(
                  back[it], reinterpret_cast<v4i*>(obase + static_cast<size_t>(o) * p.P));
          }
        } else {
#pragma unroll
          for (int it = 0; it < CHB / RPI; ++it) {
            const int o = o0 + wo * Cfg::TO + ni * 32 + part * CHB + it * RPI + r0;
            if (ok && o < p.O)
              *reinterpret_cast<v4i*>(obase + static_cast<size_t>(o) * p.P) = back[it];
          }
        }
      }
    }
    PLANE_STAMP(3);
    return;
  }
  // Any other plane (7 x 7): dword stores straight from the accumulators, a store
  // instruction writes 32 consecutive int32 of two channel planes (fewer where a tile
  // passes from one image to the next)
  size_t obase[MI];   // offset of (image, channel 0, pixel) in out32
  bool ovalid[MI];
#pragma unroll
  for (int mi = 0; mi < MI; ++mi) {
    const int v = p0 + wp * Cfg::TP + 32 * mi + frow;
    int img = n, px = v;
    if (flat) {
      img = v / pitch;
      px = v - img * pitch;
    }
    ovalid[mi] = img < p.N && px < p.P;
    obase[mi] = static_cast<size_t>(img) * p.O * p.P + px;
  }
#pragma unroll
  for (int ni = 0; ni < NI; ++ni) {
#pragma unroll
    for (int vq = 0; vq < 4; ++vq) {
      const int ol = wo * Cfg::TO + ni * 32 + 8 * vq + 4 * fgrp;  // channel inside the tile
      const v4i b = *reinterpret_cast<const v4i*>(sbias + ol);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int o = o0 + ol + i;
        if (o < p.O) {
          int32_t* plane = p.epi.out32 + static_cast<size_t>(o) * p.P;
#pragma unroll
          for (int mi = 0; mi < MI; ++mi) {
            if (ovalid[mi])
              plane[obase[mi]] = static_cast<int>(static_cast<uint32_t>(acc[mi][ni][4 * vq + i]) +
                                                  static_cast<uint32_t>(b[i]));
          }
        }
      }
    }
  }
  PLANE_STAMP(3);
}

// ---- pre-pass for gathered operands that would need byte loads --------------------------
// out[c][n * pitch + oh * OW + ow] = in[n][c][oh * sh][ow * sw]: the pixels a 1 x 1
// convolution without padding reads, as one row of `row_stride` bytes per channel over the
// whole batch (columns past a plane's OH * OW pixels are not written).  Used where the
// kernel's own gathering loader would have to fetch single bytes (odd rows, 7 x 7 planes):
// the pre-pass costs one launch and the kernel then reads 16-byte pieces through its ring.
// Work is cut into pieces "2^lg consecutive dwords of one plane" (2^lg = the power of two
// that covers a plane's dwords, at most 64); a group of 2^lg lanes walks `run` consecutive
// pieces, so the divisions that find its first plane are paid once per thread and every
// later piece is found by counting.  kGatherItems pieces are requested before any is stored,
// and every load is unconditional (a lane past the plane or past the run reads the plane's
// first bytes and drops them): loads inside branches are waited for one by one.  One piece
// per thread with its divisions took 22 us for the 51 MB of a 64 x 256 x 56 x 56 input, a
// plane per wave 11-15 us for the 6-13 MB tensors of 14 x 14 and 7 x 7 planes (65 K to
// 131 K short waves); this form 8 us.  ow_magic = ceil(2^32 / OW) finds a pixel's row,
// exact below 2^16.
constexpr int kGatherItems = 4;

struct GatherArgs {
  const uint8_t* in;
  uint8_t* out;
  int C, H, W, OW, P, sh, sw, pitch, row_stride;
  unsigned planes;
  int lg;              // lanes per group = 1 << lg
  int pieces;          // pieces per plane = ceil(pitch / 4 / lanes per group)
  unsigned run;        // consecutive pieces per group
  unsigned total;      // planes * pieces
  uint32_t ow_magic;
};

__global__ __launch_bounds__(256) void gather_planes_kernel(GatherArgs a) {
  const unsigned slot = blockIdx.x * 256u + threadIdx.x;
  const unsigned group = slot >> a.lg, lane = slot & ((1u << a.lg) - 1u);
  unsigned q = group * a.run;
  if (q >= a.total) return;
  const unsigned q_end = (q + a.run < a.total) ? q + a.run : a.total;
  // position of the first piece
  unsigned b = q / static_cast<unsigned>(a.pieces);
  int piece = static_cast<int>(q - b * a.pieces);
  unsigned n = b / static_cast<unsigned>(a.C);
  int c = static_cast<int>(b - n * a.C);
  const int per = a.pitch >> 2, plane_in = a.H * a.W;
  const uint8_t* src = a.in + static_cast<size_t>(b) * plane_in;
  while (q < q_end) {
    uint32_t v[kGatherItems];
    uint8_t* to[kGatherItems];
    bool ok[kGatherItems];
#pragma unroll
    for (int u = 0; u < kGatherItems; ++u) {
      const int dd = (piece << a.lg) + static_cast<int>(lane);
      ok[u] = q < q_end && dd < per && 4 * dd < a.P;
      to[u] = a.out + static_cast<size_t>(c) * a.row_stride + static_cast<size_t>(n) * a.pitch +
              4 * dd;
      const int p4 = ok[u] ? 4 * dd : 0;
      // (rows of one pixel: ceil(2^32 / 1) does not fit the magic's 32 bits)
      int oh = a.OW == 1 ? p4 : static_cast<int>(__umulhi(static_cast<uint32_t>(p4), a.ow_magic));
      int ow = p4 - oh * a.OW;
      uint32_t bytes[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const bool in_plane = p4 + j < a.P;
        bytes[j] = src[in_plane ? oh * a.sh * a.W + ow * a.sw : 0];
        bytes[j] = in_plane ? bytes[j] : 0u;
        if (++ow == a.OW) {
          ow = 0;
          ++oh;
        }
      }
      v[u] = bytes[0] | (bytes[1] << 8) | (bytes[2] << 16) | (bytes[3] << 24);
      // the next piece (the pointer only moves while q < q_end, so it stays in the tensor)
      ++q;
      if (q < q_end) {
        if (++piece == a.pieces) {
          piece = 0;
          src += plane_in;
          if (++c == a.C) {
            c = 0;
            ++n;
          }
        }
      }
    }
#pragma unroll
    for (int u = 0; u < kGatherItems; ++u)
      if (ok[u]) *reinterpret_cast<uint32_t*>(to[u]) = v[u];
  }
}

constexpr int kGatherMaxPlane = 1 << 16;  // pixels per gathered plane (the row division)

void launch_gather(hipStream_t s, const int8_t* in, int8_t* out, int N, int C, int H, int W,
                   int OH, int OW, int sh, int sw, int pitch, int row_stride) {
  const long long planes = 1LL * N * C;
  if (planes == 0 || pitch == 0) return;
  MXQ_CHECK(OH * OW < kGatherMaxPlane, "plane too large for the gather");
  GatherArgs a;
  a.in = reinterpret_cast<const uint8_t*>(in);
  a.out = reinterpret_cast<uint8_t*>(out);
  a.C = C; a.H = H; a.W = W; a.OW = OW; a.P = OH * OW; a.sh = sh; a.sw = sw;
  a.pitch = pitch; a.row_stride = row_stride;
  a.planes = static_cast<unsigned>(planes);
  a.lg = 0;
  while (a.lg < 6 && (1 << a.lg) < pitch / 4) ++a.lg;
  a.pieces = (pitch / 4 + (1 << a.lg) - 1) >> a.lg;
  const long long total = planes * a.pieces;
  MXQ_CHECK(total < (1LL << 31), "too many planes");
  a.total = static_cast<unsigned>(total);
  // groups: about 16 waves per CU, each group with at least 2 * kGatherItems pieces
  const long long groups_per_wave = 64 >> a.lg;
  long long groups = 16LL * num_cus() * groups_per_wave;
  long long run = (total + groups - 1) / groups;
  if (run < 2 * kGatherItems) run = 2 * kGatherItems;
  a.run = static_cast<unsigned>(run);
  groups = (total + run - 1) / run;
  a.ow_magic = static_cast<uint32_t>(((1ULL << 32) + OW - 1) / OW);
  const unsigned grid = static_cast<unsigned>(((groups << a.lg) + 255) / 256);
  hipLaunchKernelGGL(gather_planes_kernel, dim3(grid), dim3(256), 0, s, a);
  MXQ_LAUNCH_CHECK();
}

typedef PlaneCfg<128, 128, 64, 2, 2> PlaneM;   // 4 waves, wave tile 64 pixels x 64 channels
typedef PlaneCfg<128, 64, 64, 2, 2> PlaneN64;  // 4 waves, wave tile 64 x 32
typedef PlaneCfg<64, 128, 64, 2, 2> PlaneP64;  // 4 waves, wave tile 32 x 64
typedef PlaneCfg<64, 64, 64, 2, 2> PlaneS;     // 4 waves, wave tile 32 x 32
typedef PlaneCfg<128, 256, 64, 2, 4> PlaneW;   // 8 waves, wave tile 64 x 64
typedef PlaneCfg<256, 128, 64, 4, 2> PlaneH;   // 8 waves, wave tile 64 x 64
typedef PlaneCfg<256, 256, 64, 2, 4> PlaneL;   // 8 waves, wave tile 128 x 64
// 128-byte stages: half as many K steps.  Measured inside the ResNet-50 pass on every
// gathered and every small-plane layer in five tile shapes: ahead only for the loader-gathered
// 1024 -> 256 layer at 14 x 14 (-2.2 us), level or behind elsewhere (+0.3 ... +9.4 us).
typedef PlaneCfg<64, 128, 128, 2, 2> PlaneP64k2;

template <class Cfg>
void launch_planes(hipStream_t s, PlaneArgs a, int gm) {
  const bool flat = gm != kNative || a.pitch != 0;
  const long long cols = gm != kNative ? 1LL * a.N * a.P : (flat ? 1LL * a.N * a.pitch : a.P);
  a.tiles_p = static_cast<int>((cols + Cfg::BP - 1) / Cfg::BP);
  a.tiles_o = (a.O + Cfg::BO - 1) / Cfg::BO;
  const long long total = 1LL * (flat ? 1 : a.N) * a.tiles_p * a.tiles_o;
  MXQ_CHECK(total < (1LL << 31), "grid too large");
  const dim3 grid(static_cast<unsigned>(total)), block(Cfg::kThreads);
  if (gm == kGatherPair) {
    hipLaunchKernelGGL((conv1x1_planes_kernel<Cfg, 2, kGatherPair>), grid, block, 0, s, a);
  } else if (gm == kGatherBytes) {
    hipLaunchKernelGGL((conv1x1_planes_kernel<Cfg, 2, kGatherBytes>), grid, block, 0, s, a);
  } else if (gm == kGatherPair2) {
    hipLaunchKernelGGL((conv1x1_planes_kernel<Cfg, 2, kGatherPair2>), grid, block, 0, s, a);
  } else {
    // two ring stages whatever the reduction length: four (48 to 128 KiB of LDS) leave room
    // for fewer work-groups per CU and measured level or behind on every ResNet-50 layer
    // (512 -> 1024 / 2 at 28 x 28: 30.5 us with two stages, 34.9 with four)
    hipLaunchKernelGGL((conv1x1_planes_kernel<Cfg, 2, kNative>), grid, block, 0, s, a);
  }
  MXQ_LAUNCH_CHECK();
}

// The route a convolution takes.
enum class Route {
  kPlanes,        // 1 x 1, unit stride, 16 | plane: the NCHW kernel on the operator's own tensors
  kPlanesGather,  // any other unpadded 1 x 1: the same kernel, its loader gathering the pixels
                  // the layer reads
  kPlanesPrepass, // ... or, where that loader would fetch single bytes, after a pre-pass that
                  // gathers them into one row per channel
  kSpaceToDepth,  // few-channel stride-2 stem through mxq_nchw_to_s2d_nhwc_i8
  kAdapters       // NHWC copies of both operands, NHWC kernel writing NCHW planes
};

int padded_channels(int C) { return (C + 15) / 16 * 16; }
size_t up256(size_t x) { return (x + 255) / 256 * 256; }

struct NchwPlan {
  Route route;
  int OH, OW;
  // kSpaceToDepth
  int off_h, off_w, H2, W2, K2h, K2w, pad2_h, pad2_w;
  // NHWC view of the adapter routes
  int vC;
  int gather_mode;         // kPlanesGather: how the loader fetches a group's four pixels
  int pitch, row_stride;   // kPlanesPrepass: columns per image and bytes per channel row
  bool weight_in_place;    // 1 x 1 window over C % 16 == 0 channels: OIHW is OHWI already
  size_t d_bytes, w_bytes, split_bytes;
};

NchwPlan plan_nchw(int N, int C, int H, int W, int O, int KH, int KW, int sh, int sw, int ph,
                   int pw, int dh, int dw, bool operands_aligned) {
  MXQ_CHECK(N >= 0 && C > 0 && H > 0 && W > 0 && O > 0 && KH > 0 && KW > 0, "bad shape");
  MXQ_CHECK(sh > 0 && sw > 0 && dh > 0 && dw > 0 && ph >= 0 && pw >= 0, "bad stride/dilate/pad");
  const int eh = dh * (KH - 1) + 1, ew = dw * (KW - 1) + 1;
  MXQ_CHECK(H + 2 * ph >= eh && W + 2 * pw >= ew, "kernel larger than padded input");
  NchwPlan pl = {};
  pl.OH = (H + 2 * ph - eh) / sh + 1;
  pl.OW = (W + 2 * pw - ew) / sw + 1;
  const long long P = 1LL * pl.OH * pl.OW;
  const bool one = KH == 1 && KW == 1 && ph == 0 && pw == 0;
  const bool small = 1LL * N * C * P < (1LL << 31) && 1LL * O * C < (1LL << 31) &&
                     1LL * N * C * H * W < (1LL << 31);
  if (one && operands_aligned && C % 16 == 0 && small) {
    if (sh == 1 && sw == 1 && P % 16 == 0) {
      pl.route = Route::kPlanes;
      return pl;
    }
    // planes of 4 | P bytes (14 x 14): the same direct loads, 16 bytes from dword marks, over
    // columns padded to a multiple of 16 per image
    if (sh == 1 && sw == 1 && P % 4 == 0 &&
        1LL * N * ((P + 15) / 16 * 16) < (1LL << 31)) {
      pl.route = Route::kPlanes;
      pl.pitch = static_cast<int>((P + 15) / 16 * 16);
      return pl;
    }
    // The gathering loader works one stage ahead out of registers; the pre-pass costs a launch
    // and a copy of what the layer reads but feeds the kernel's direct-to-LDS ring.  Measured
    // on the ResNet-50 layers at batch 64: the loader wins while the weight matrix is small
    // (256 -> 128 / 2: 34 -> 28 us, 1024 -> 256 at 14 x 14: 24 -> 20 us), the ring once the
    // layer is a real GEMM (512 -> 1024 / 2 at 28 x 28: 38 us against 53 us).
    const int plane_in = H * W;
    const long long pitch = (P + 3) / 4 * 4, row = (1LL * N * pitch + 15) / 16 * 16;
    const bool prepass_ok = P < kGatherMaxPlane && 1LL * C * row < (1LL << 31);
    const bool light = 1LL * O * C <= 256 * 1024 || !prepass_ok;
    int mode = kGatherBytes;
    if (sw == 2 && pl.OW % 4 == 0 && (sh * W) % 8 == 0 && plane_in % 8 == 0 && 2 * pl.OW <= W)
      mode = kGatherPair;
    else if (sw == 2 && pl.OW % 2 == 0 && (sh * W) % 4 == 0 && plane_in % 4 == 0 && 2 * pl.OW <= W)
      mode = kGatherPair2;
    if ((mode != kGatherBytes && light) || !prepass_ok) {
      pl.route = Route::kPlanesGather;
      pl.gather_mode = mode;
      return pl;
    }
    // (a pre-pass in front of a very long reduction over few pixels loses to the adapters,
    // whose kernel has the deeper stages: 2048 -> 512 at 7 x 7 24.8 against 21.6 us)
    if (!(C >= 2048 && 1LL * N * P <= 4096)) {
      pl.route = Route::kPlanesPrepass;
      pl.pitch = static_cast<int>(pitch);
      pl.row_stride = static_cast<int>(row);
      pl.d_bytes = up256(static_cast<size_t>(C) * row);
      return pl;
    }
  }
  // a stride-2 convolution over at most 4 channels (an image stem) runs as the unit-stride
  // convolution over the space-to-depth form of its operands: 4 * C real channels out of 16
  // instead of C out of 16
  if (C <= 4 && sh == 2 && sw == 2 && dh == 1 && dw == 1 && KH >= 2 && KW >= 2) {
    pl.off_h = ph & 1;
    pl.off_w = pw & 1;
    pl.H2 = (H + pl.off_h + 1) / 2;
    pl.W2 = (W + pl.off_w + 1) / 2;
    pl.K2h = (KH + 1) / 2;
    pl.K2w = (KW + 1) / 2;
    pl.pad2_h = (ph - pl.off_h) / 2;
    pl.pad2_w = (pw - pl.off_w) / 2;
    // only when the transformed problem gives exactly the operator's output extent
    if (pl.H2 + 2 * pl.pad2_h - pl.K2h + 1 == pl.OH && pl.W2 + 2 * pl.pad2_w - pl.K2w + 1 == pl.OW) {
      pl.route = Route::kSpaceToDepth;
      pl.vC = padded_channels(4 * C);
      pl.d_bytes = up256(static_cast<size_t>(N) * pl.H2 * pl.W2 * pl.vC);
      pl.w_bytes = up256(static_cast<size_t>(O) * pl.K2h * pl.K2w * pl.vC);
      pl.split_bytes = mxq_quantized_conv_workspace(N, pl.H2, pl.W2, pl.vC, O, pl.K2h, pl.K2w, 1,
                                                    1, pl.pad2_h, pl.pad2_w, 1, 1, 0);
      return pl;
    }
  }
  pl.route = Route::kAdapters;
  pl.vC = padded_channels(C);
  pl.weight_in_place = KH == 1 && KW == 1 && C % 16 == 0 && operands_aligned;
  pl.d_bytes = up256(static_cast<size_t>(N) * H * W * pl.vC);
  pl.w_bytes = pl.weight_in_place ? 0 : up256(static_cast<size_t>(O) * KH * KW * pl.vC);
  pl.split_bytes =
      mxq_quantized_conv_workspace(N, H, W, pl.vC, O, KH, KW, sh, sw, ph, pw, dh, dw, 0);
  return pl;
}

// The entry points of the adapter routes are this library's own C functions: their error
// text is already on the thread when they fail.
#define MXQ_FORWARD(call)                                      \
  do {                                                         \
    if ((call) != 0) throw ::mxq::Error(mxq_last_error());     \
  } while (0)

void conv_nchw(void* stream, const int8_t* data, const int8_t* weight, const int8_t* bias, int N,
               int C, int H, int W, int O, int KH, int KW, int sh, int sw, int ph, int pw, int dh,
               int dw, const float* min_data, const float* max_data, const float* min_weight,
               const float* max_weight, const float* min_bias, const float* max_bias,
               int32_t* out32, float* omin, float* omax, void* workspace, size_t workspace_bytes,
               int cfg) {
  MXQ_CHECK(min_data && max_data && min_weight && max_weight, "null input range pointer");
  MXQ_CHECK(omin && omax, "null output range pointer");
  MXQ_CHECK(bias == nullptr || (min_bias && max_bias), "bias given without its range");
  MXQ_CHECK(N == 0 || (data != nullptr && weight != nullptr && out32 != nullptr),
            "null tensor pointer");
  if (N == 0) {
    // no output elements: the range scalars alone
    MXQ_FORWARD(mxq_quantized_conv_nhwc(stream, data, weight, bias, 0, H, W, C, O, KH, KW, sh, sw,
                                        ph, pw, dh, dw, min_data, max_data, min_weight,
                                        max_weight, min_bias, max_bias, out32, omin, omax,
                                        nullptr, nullptr, nullptr, 0, 0.f, 0.f, nullptr, 0));
    return;
  }
  // cfg 1 pins the adapter route; 71.. pin a tile of the NCHW kernel
  const bool aligned = aligned16(data) && aligned16(weight) && cfg != 1;
  NchwPlan pl = plan_nchw(N, C, H, W, O, KH, KW, sh, sw, ph, pw, dh, dw, aligned);
  const bool planes_route = pl.route == Route::kPlanes || pl.route == Route::kPlanesGather ||
                            pl.route == Route::kPlanesPrepass;
  MXQ_CHECK(cfg < 70 || planes_route,
            "shape does not qualify for the NCHW 1x1 kernel");
  hipStream_t s = static_cast<hipStream_t>(stream);
  char* ws = static_cast<char*>(workspace);
  const size_t need = pl.d_bytes + pl.w_bytes;
  MXQ_CHECK(need == 0 || (ws != nullptr && aligned16(ws) && workspace_bytes >= need),
            "workspace too small: " << workspace_bytes << " < " << need
                                    << " (see mxq_quantized_conv_nchw_workspace)");

  if (planes_route) {
    PlaneArgs a = {};
    a.N = N; a.C = C; a.P = pl.OH * pl.OW; a.O = O;
    a.data = data;
    a.weight = weight;
    a.data_bytes = static_cast<uint32_t>(N) * C * H * W;
    int gm = kNative;
    if (pl.route == Route::kPlanesGather) {
      a.H = H; a.W = W; a.OW = pl.OW; a.sh = sh; a.sw = sw;
      gm = pl.gather_mode;
    } else if (pl.route == Route::kPlanesPrepass) {
      launch_gather(s, data, reinterpret_cast<int8_t*>(ws), N, C, H, W, pl.OH, pl.OW, sh, sw,
                    pl.pitch, pl.row_stride);
      a.data = reinterpret_cast<const int8_t*>(ws);
      a.img_stride = pl.pitch;
      a.row_stride = pl.row_stride;
      a.pitch = pl.pitch;
      a.data_bytes = static_cast<uint32_t>(C) * pl.row_stride;
    } else {
      a.img_stride = C * a.P;
      a.row_stride = a.P;
      a.pitch = pl.pitch;   // 0: whole 16-byte planes, tiles inside an image
    }
    Epilogue& e = a.epi;
    e = Epilogue();
    e.bias = bias;
    e.min_data = min_data; e.max_data = max_data;
    e.min_weight = min_weight; e.max_weight = max_weight;
    e.min_bias = min_bias; e.max_bias = max_bias;
    e.out32 = out32;
    e.omin = omin; e.omax = omax;
    // Non-temporal stores only for an output of large planes that no cache level will hold
    // (56 x 56, 64 -> 256 at batch 64: 205 MB, the pass 2.5 us shorter); on every other
    // ResNet-50 layer the hint measured level or behind inside the pass (+0.1 ... +10 us,
    // worst on 14 x 14 and 28 x 28 planes)
    a.stream32 = (a.P >= 2048 && 4LL * N * O * a.P >= (128LL << 20)) ? 1 : 0;
    int pick = cfg;
    if (pick < 70) {
      const long cus = num_cus();
      // columns a pixel tile may run over: a gathered operand is one long row per channel
      const bool flat = gm != kNative || a.pitch != 0;
      const long long cols = gm != kNative ? 1LL * N * a.P : (flat ? 1LL * N * a.pitch : a.P);
      const long long rows = flat ? 1 : N;
      auto tiles = [&](int bp, int bo) {
        return rows * ((cols + bp - 1) / bp) * ((O + bo - 1) / bo);
      };
      auto padded = [&](int bp) { return rows * ((cols + bp - 1) / bp * bp); };
      // From per-layer sweeps of every tile on the ResNet-50 layers at batch 64 (operands
      // rotated): 64 output channels take the 128 x 64 tile; a layer with a long reduction
      // whose 256 x 128 tiles cover three quarters of the chip takes those (256 -> 128 / 2:
      // 19.8 us against 20.9; 512 -> 2048 at 7 x 7: 19.6 against 22); everything else
      // 128 x 128, shrunk to 64 pixels and then 64 channels while there is less than one
      // tile per CU (1024 -> 512 at 7 x 7: 16.3 us on 64 x 64 against 19.2).  The 256-column
      // tiles never measured ahead by more than the run-to-run spread.
      if (O <= 64) {
        pick = (tiles(128, 64) >= cus || cols > 64) ? 72 : 74;
      } else if (C >= 256 && 100 * padded(256) <= 104 * padded(128) &&
                 4 * tiles(256, 128) >= 3 * cus) {
        pick = 77;
      } else {
        int bp = 128, bo = 128;
        if (tiles(bp, bo) < cus) bp = 64;
        if (tiles(bp, bo) < cus) bo = 64;
        pick = bp == 128 ? 71 : (bo == 128 ? 73 : 74);
        // a long reduction over 14 x 14 planes: 128-byte stages halve its K steps (-2.2 us
        // inside the ResNet-50 pass)
        if (pick == 73 && C >= 1024 && pl.route == Route::kPlanes && a.pitch != 0) pick = 84;
      }
    }
    switch (pick) {
      case 71: launch_planes<PlaneM>(s, a, gm); break;
      case 72: launch_planes<PlaneN64>(s, a, gm); break;
      case 73: launch_planes<PlaneP64>(s, a, gm); break;
      case 74: launch_planes<PlaneS>(s, a, gm); break;
      case 75: launch_planes<PlaneW>(s, a, gm); break;
      case 77: launch_planes<PlaneH>(s, a, gm); break;
      case 78: launch_planes<PlaneL>(s, a, gm); break;
      case 84: launch_planes<PlaneP64k2>(s, a, gm); break;
      default: MXQ_CHECK(false, "unknown NCHW tile configuration " << pick);
    }
    return;
  }

  int8_t* d_nhwc = reinterpret_cast<int8_t*>(ws);
  int8_t* w_ohwi = reinterpret_cast<int8_t*>(ws + pl.d_bytes);
  const size_t split_room = workspace_bytes - need;
  void* split_ws = split_room != 0 ? ws + need : nullptr;
  if (pl.route == Route::kSpaceToDepth) {
    MXQ_FORWARD(mxq_nchw_to_s2d_nhwc_i8(stream, data, d_nhwc, N, C, H, W, pl.off_h, pl.off_w,
                                        pl.vC));
    MXQ_FORWARD(mxq_nchw_to_s2d_nhwc_i8(stream, weight, w_ohwi, O, C, KH, KW, 0, 0, pl.vC));
    MXQ_FORWARD(mxq_quantized_conv_nhwc_out_nchw(
        stream, d_nhwc, w_ohwi, bias, N, pl.H2, pl.W2, pl.vC, O, pl.K2h, pl.K2w, 1, 1, pl.pad2_h,
        pl.pad2_w, 1, 1, min_data, max_data, min_weight, max_weight, min_bias, max_bias, out32,
        omin, omax, split_ws, split_room));
    return;
  }
  const int8_t* wk = pl.weight_in_place ? weight : w_ohwi;
  nchw_to_nhwc_pair(s, data, d_nhwc, N, C, H, W, pl.vC, weight,
                    pl.weight_in_place ? nullptr : w_ohwi, O, KH, KW);
  MXQ_FORWARD(mxq_quantized_conv_nhwc_out_nchw(
      stream, d_nhwc, wk, bias, N, H, W, pl.vC, O, KH, KW, sh, sw, ph, pw, dh, dw, min_data,
      max_data, min_weight, max_weight, min_bias, max_bias, out32, omin, omax, split_ws,
      split_room));
}

}  // namespace
}  // namespace mxq

using namespace mxq;

extern "C" {

size_t mxq_quantized_conv_nchw_workspace(int N, int C, int H, int W, int O, int KH, int KW,
                                         int stride_h, int stride_w, int pad_h, int pad_w,
                                         int dilate_h, int dilate_w, int operands_aligned16) {
  try {
    if (N <= 0) return 0;
    const NchwPlan b = plan_nchw(N, C, H, W, O, KH, KW, stride_h, stride_w, pad_h, pad_w,
                                 dilate_h, dilate_w, false);
    const size_t nb = b.d_bytes + b.w_bytes + b.split_bytes;
    const NchwPlan a = plan_nchw(N, C, H, W, O, KH, KW, stride_h, stride_w, pad_h, pad_w,
                                 dilate_h, dilate_w, true);
    const size_t na = a.d_bytes + a.w_bytes + a.split_bytes;
    // without the promise: enough for either route
    if (operands_aligned16 == 0) return na > nb ? na : nb;
    return na;
  } catch (...) {
    return 0;
  }
}

int mxq_quantized_conv_nchw(void* stream, const int8_t* data, const int8_t* weight,
                            const int8_t* bias, int N, int C, int H, int W, int O, int KH, int KW,
                            int stride_h, int stride_w, int pad_h, int pad_w, int dilate_h,
                            int dilate_w, const float* min_data, const float* max_data,
                            const float* min_weight, const float* max_weight,
                            const float* min_bias, const float* max_bias, int32_t* out32,
                            float* omin, float* omax, void* workspace, size_t workspace_bytes) {
  MXQ_API_BEGIN();
  conv_nchw(stream, data, weight, bias, N, C, H, W, O, KH, KW, stride_h, stride_w, pad_h, pad_w,
            dilate_h, dilate_w, min_data, max_data, min_weight, max_weight, min_bias, max_bias,
            out32, omin, omax, workspace, workspace_bytes, 0);
  MXQ_API_END();
}

#ifdef MXQ_STAMPS
int mxq_dbg_read_plane_stamps(long long* host, int count) {
  return hipMemcpyFromSymbol(host, HIP_SYMBOL(mxq_dbg_plane_stamps),
                             sizeof(long long) * count) == hipSuccess ? 0 : -1;
}
#endif

#ifdef MXQ_TEST_HOOKS
// Test-only twin (declared in tests/mxq_test_hooks.h): cfg 1 pins the route through the
// layout adapters, 71 ... 84 a tile of the NCHW kernel, 0 leaves the choice to the launcher.
int mxq_test_quantized_conv_nchw(void* stream, const int8_t* data, const int8_t* weight,
                                 const int8_t* bias, int N, int C, int H, int W, int O, int KH,
                                 int KW, int stride_h, int stride_w, int pad_h, int pad_w,
                                 int dilate_h, int dilate_w, const float* min_data,
                                 const float* max_data, const float* min_weight,
                                 const float* max_weight, const float* min_bias,
                                 const float* max_bias, int32_t* out32, float* omin, float* omax,
                                 void* workspace, size_t workspace_bytes, int cfg) {
  MXQ_API_BEGIN();
  conv_nchw(stream, data, weight, bias, N, C, H, W, O, KH, KW, stride_h, stride_w, pad_h, pad_w,
            dilate_h, dilate_w, min_data, max_data, min_weight, max_weight, min_bias, max_bias,
            out32, omin, omax, workspace, workspace_bytes, cfg);
  MXQ_API_END();
}
#endif  // MXQ_TEST_HOOKS

}  // extern "C"
