// Byte movers of the quantized graph for gfx950: the operators that rearrange int8 / uint8
// data without touching its values and pass the range scalars through.
//   _contrib_quantized_embedding  src/operator/quantization/quantized_indexing_op.cc:103-122
//                                 (rows taken by TakeZeroAxisCPU<clip>,
//                                 src/operator/tensor/indexing_op.cc:30-61)
//   _contrib_quantized_transpose  src/operator/quantization/quantized_transpose.cc:49-104,
//                                 dnnl/dnnl_quantized_transpose.cc (cpu only in the reference)
// Both are bound by HBM.  Rows (embedding vectors, or the runs of a transpose whose
// innermost axis stays innermost) are copied by groups of 1..64 lanes, 16 bytes per lane
// where addresses allow; a transpose that moves the innermost axis goes through a
// 64 x 64-byte LDS tile so that both the reads and the writes are contiguous runs.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "../../include/mxq.h"
#include "mxq_common.h"
#include "mxq_thin_transpose.h"

namespace mxq {

namespace {

constexpr int kThreads = 256;
constexpr int kMaxDims = 8;

typedef uint32_t u4 __attribute__((ext_vector_type(4)));

// Lanes that share one row: the smallest power of two that covers its `units` pieces,
// at most a wave.
int group_lanes(size_t units) {
  int g = 1;
  while (g < 64 && static_cast<size_t>(g) < units) g <<= 1;
  return g;
}

int grid_for_rows(size_t rows, int group) {
  const size_t rows_per_block = kThreads / group;
  size_t want = (rows + rows_per_block - 1) / rows_per_block;
  const size_t cap = static_cast<size_t>(num_cus()) * 8;
  if (want < 1) want = 1;
  return static_cast<int>(want < cap ? want : cap);
}

// Copies one row of `bytes` bytes with the `group` lanes that share it (lane g of them).
template <bool VEC>
__device__ __forceinline__ void copy_row(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst,
                                         size_t bytes, int g, int group) {
  if (VEC) {
    const u4* s16 = reinterpret_cast<const u4*>(src);
    u4* d16 = reinterpret_cast<u4*>(dst);
    const size_t n16 = bytes >> 4;
    for (size_t c = g; c < n16; c += group) d16[c] = s16[c];
  } else {
    for (size_t c = g; c < bytes; c += group) dst[c] = src[c];
  }
}

// ---- embedding ------------------------------------------------------------------------

// static_cast<int64_t>(idx[i]) clipped to [0, K - 1] (indexing_op.cc:44-49)
template <typename IT>
__device__ __forceinline__ int64_t clipped_index(const void* idx, size_t i, int64_t K) {
  int64_t j = static_cast<int64_t>(static_cast<const IT*>(idx)[i]);
  if (j <= 0) return 0;
  return j >= K ? K - 1 : j;
}

struct EmbedArgs {
  const void* idx;
  const uint8_t* weight;
  uint8_t* out;
  const float* wmin;
  const float* wmax;
  float* omin;
  float* omax;
  size_t n;        // indices
  int64_t K;       // rows of the table
  size_t D;        // bytes per row
  int group, shift;
};

template <typename IT, bool VEC>
__global__ __launch_bounds__(kThreads) void embedding_kernel(EmbedArgs a) {
  const int g = threadIdx.x & (a.group - 1);
  const size_t rows_per_block = kThreads >> a.shift;
  size_t row = size_t(blockIdx.x) * rows_per_block + (threadIdx.x >> a.shift);
  const size_t step = size_t(gridDim.x) * rows_per_block;
  for (; row < a.n; row += step) {
    const int64_t j = clipped_index<IT>(a.idx, row, a.K);
    copy_row<VEC>(a.weight + static_cast<size_t>(j) * a.D, a.out + row * a.D, a.D, g, a.group);
  }
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    *a.omin = *a.wmin;
    *a.omax = *a.wmax;
  }
}

template <typename IT>
void launch_embedding(hipStream_t s, const EmbedArgs& a, bool vec) {
  const int grid = grid_for_rows(a.n, a.group);
  if (vec)
    hipLaunchKernelGGL((embedding_kernel<IT, true>), dim3(grid), dim3(kThreads), 0, s, a);
  else
    hipLaunchKernelGGL((embedding_kernel<IT, false>), dim3(grid), dim3(kThreads), 0, s, a);
  MXQ_LAUNCH_CHECK();
}

// ---- transpose ------------------------------------------------------------------------

// A permutation after merging axes that stay adjacent: out axis d is in axis perm[d].
struct Perm {
  int nd;
  int64_t out_extent[kMaxDims];
  int64_t in_stride[kMaxDims];  // stride in the input of out axis d, in elements (= bytes)
};

struct RowsArgs {
  const uint8_t* in;
  uint8_t* out;
  const float* imin;
  const float* imax;
  float* omin;
  float* omax;
  Perm p;        // the axes before the innermost one (nd of them)
  size_t rows;   // product of p.out_extent
  size_t L;      // bytes of the innermost run
  int group, shift;
};

__device__ __forceinline__ void pass_range(const float* imin, const float* imax, float* omin,
                                           float* omax) {
  if (blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) {
    *omin = *imin;
    *omax = *imax;
  }
}

// Input offset of output row `row`: its coordinates along the outer axes times their
// input strides.  32-bit arithmetic where the row count allows.
template <typename UI>
__device__ __forceinline__ size_t permuted_offset(const Perm& p, UI row) {
  size_t off = 0;
  for (int d = p.nd - 1; d >= 0; --d) {
    const UI e = static_cast<UI>(p.out_extent[d]);
    const UI q = row / e;
    off += static_cast<size_t>(row - q * e) * static_cast<size_t>(p.in_stride[d]);
    row = q;
  }
  return off;
}

// The innermost axis stays innermost: every output row is a contiguous run of the input.
template <typename UI, bool VEC>
__global__ __launch_bounds__(kThreads) void permute_rows_kernel(RowsArgs a) {
  const int g = threadIdx.x & (a.group - 1);
  const size_t rows_per_block = kThreads >> a.shift;
  size_t row = size_t(blockIdx.x) * rows_per_block + (threadIdx.x >> a.shift);
  const size_t step = size_t(gridDim.x) * rows_per_block;
  for (; row < a.rows; row += step)
    copy_row<VEC>(a.in + permuted_offset<UI>(a.p, static_cast<UI>(row)), a.out + row * a.L, a.L, g,
                  a.group);
  pass_range(a.imin, a.imax, a.omin, a.omax);
}

constexpr int kTile = 64;

struct TileArgs {
  const uint8_t* in;
  uint8_t* out;
  const float* imin;
  const float* imax;
  float* omin;
  float* omax;
  Perm p;             // the axes other than A and B, outermost first (nd of them)
  int64_t p_out_stride[kMaxDims];
  int64_t A, B;       // extents: A is innermost in the input, B innermost in the output
  int64_t a_out_stride, b_in_stride;
  int64_t batches;    // product of p.out_extent
  unsigned tiles_a;   // tiles along A
  // permute_tile16_kernel only: when per_xcd != 0 the grid is one-dimensional, tiles and
  // batches in one sequence (A fastest) of which every XCD owns a contiguous range
  unsigned tiles_ab = 0, xcd_total = 0, per_xcd = 0;
};

// The innermost axis moves: 64 (B) x 64 (A) bytes per tile through LDS.  Reads run along A,
// writes along B.  blockIdx.x = tile (A fastest), blockIdx.y walks the other axes.
__global__ __launch_bounds__(kThreads) void permute_tile_kernel(TileArgs a) {
  __shared__ __attribute__((aligned(16))) uint8_t tile[kTile][kTile + 4];
  const int t = threadIdx.x;
  const int64_t tb = blockIdx.x / a.tiles_a, ta = blockIdx.x - tb * a.tiles_a;
  const int64_t a0 = ta * kTile, b0 = tb * kTile;
  const int r = t >> 4, c4 = (t & 15) * 4;
  for (int64_t z = blockIdx.y; z < a.batches; z += gridDim.y) {
    size_t in_off = 0, out_off = 0;
    {
      int64_t rem = z;
      for (int d = a.p.nd - 1; d >= 0; --d) {
        const int64_t q = rem / a.p.out_extent[d], i = rem - q * a.p.out_extent[d];
        in_off += static_cast<size_t>(i * a.p.in_stride[d]);
        out_off += static_cast<size_t>(i * a.p_out_stride[d]);
        rem = q;
      }
    }
    const uint8_t* src = a.in + in_off;
    uint8_t* dst = a.out + out_off;
    // in: rows along B (stride b_in_stride), 64 bytes along A each
#pragma unroll
    for (int pass = 0; pass < 4; ++pass) {
      const int br = pass * 16 + r;
      const int64_t b = b0 + br, aa = a0 + c4;
      if (b < a.B) {
        const uint8_t* p = src + static_cast<size_t>(b * a.b_in_stride + aa);
        if (aa + 3 < a.A && (reinterpret_cast<uintptr_t>(p) & 3u) == 0) {
          *reinterpret_cast<uint32_t*>(&tile[br][c4]) = *reinterpret_cast<const uint32_t*>(p);
        } else {
#pragma unroll
          for (int k = 0; k < 4; ++k)
            if (aa + k < a.A) tile[br][c4 + k] = p[k];
        }
      }
    }
    __syncthreads();
    // out: rows along A (stride a_out_stride), 64 bytes along B each
#pragma unroll
    for (int pass = 0; pass < 4; ++pass) {
      const int ar = pass * 16 + r;
      const int64_t aa = a0 + ar, b = b0 + c4;
      if (aa < a.A) {
        uint8_t* p = dst + static_cast<size_t>(aa * a.a_out_stride + b);
        if (b + 3 < a.B && (reinterpret_cast<uintptr_t>(p) & 3u) == 0) {
          const uint32_t w = uint32_t(tile[c4][ar]) | (uint32_t(tile[c4 + 1][ar]) << 8) |
                             (uint32_t(tile[c4 + 2][ar]) << 16) |
                             (uint32_t(tile[c4 + 3][ar]) << 24);
          *reinterpret_cast<uint32_t*>(p) = w;
        } else {
#pragma unroll
          for (int k = 0; k < 4; ++k)
            if (b + k < a.B) p[k] = tile[c4 + k][ar];
        }
      }
    }
    __syncthreads();
  }
  pass_range(a.imin, a.imax, a.omin, a.omax);
}

// Offsets of batch z along the axes other than A and B.
__device__ __forceinline__ void batch_offsets(const TileArgs& a, int64_t z, size_t& in_off,
                                              size_t& out_off) {
  in_off = 0;
  out_off = 0;
  for (int d = a.p.nd - 1; d >= 0; --d) {
    const int64_t q = z / a.p.out_extent[d], i = z - q * a.p.out_extent[d];
    in_off += static_cast<size_t>(i * a.p.in_stride[d]);
    out_off += static_cast<size_t>(i * a.p_out_stride[d]);
    z = q;
  }
}

// The same for friendly strides (A % 4 == 0 and every input stride a multiple of 4; B % 16
// == 0 and every output stride a multiple of 16; aligned pointers): TB (B) x 128 (A) bytes
// per tile, every thread loads dwords along A (a wave reads whole 128-byte runs), transposes
// 4 x 4 bytes in registers with v_perm and parks the result in LDS, from where 16-byte
// pieces of the output rows leave.  TB = 128 makes the output runs whole cache lines too.
template <int TB>
__global__ __launch_bounds__(kThreads) void permute_tile4_kernel(TileArgs a) {
  constexpr int kPitch = TB / 4 + 1;  // dwords per transposed row: TB bytes + 4 of padding
  constexpr int kPasses = TB / 32;
  __shared__ uint32_t tile[128 * kPitch];
  const int t = threadIdx.x;
  const int64_t tb = blockIdx.x / a.tiles_a, ta = blockIdx.x - tb * a.tiles_a;
  const int64_t a0 = ta * 128, b0 = tb * TB;
  const int sq = t & 31;
  for (int64_t z = blockIdx.y; z < a.batches; z += gridDim.y) {
    size_t in_off, out_off;
    batch_offsets(a, z, in_off, out_off);
    const uint8_t* src = a.in + in_off;
    uint8_t* dst = a.out + out_off;
    const int64_t aa = a0 + 4 * sq;
    // every dword of the thread first, then the byte transposes and the LDS writes
    uint32_t w[kPasses][4];
#pragma unroll
    for (int pass = 0; pass < kPasses; ++pass)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int64_t b = b0 + 4 * ((t >> 5) + 8 * pass) + j;
        w[pass][j] = (b < a.B && aa < a.A)
                         ? __builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(
                               src + static_cast<size_t>(b * a.b_in_stride + aa)))
                         : 0u;
      }
#pragma unroll
    for (int pass = 0; pass < kPasses; ++pass) {
      const int rq = (t >> 5) + 8 * pass;
      // x[i] = byte i of w[0..3]
      const uint32_t t0 = __builtin_amdgcn_perm(w[pass][1], w[pass][0], 0x05010400u);
      const uint32_t t1 = __builtin_amdgcn_perm(w[pass][1], w[pass][0], 0x07030602u);
      const uint32_t t2 = __builtin_amdgcn_perm(w[pass][3], w[pass][2], 0x05010400u);
      const uint32_t t3 = __builtin_amdgcn_perm(w[pass][3], w[pass][2], 0x07030602u);
      tile[(4 * sq + 0) * kPitch + rq] = __builtin_amdgcn_perm(t2, t0, 0x05040100u);
      tile[(4 * sq + 1) * kPitch + rq] = __builtin_amdgcn_perm(t2, t0, 0x07060302u);
      tile[(4 * sq + 2) * kPitch + rq] = __builtin_amdgcn_perm(t3, t1, 0x05040100u);
      tile[(4 * sq + 3) * kPitch + rq] = __builtin_amdgcn_perm(t3, t1, 0x07060302u);
    }
    __syncthreads();
    const int64_t left = a.B - b0;
    const int nb = left < TB ? static_cast<int>(left) : TB;  // bytes per output row (16 | nb)
    const int per_row = nb >> 4;                              // 16-byte pieces per row
    const int pieces = 128 * per_row;
    for (int c = t; c < pieces; c += kThreads) {
      const int sl = per_row == TB / 16 ? c / (TB / 16) : c / per_row;
      const int k = c - sl * per_row;
      if (a0 + sl < a.A) {
        u4 v;
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = tile[sl * kPitch + 4 * k + i];
        __builtin_nontemporal_store(
            v, reinterpret_cast<u4*>(dst + static_cast<size_t>((a0 + sl) * a.a_out_stride + b0 + 16 * k)));
      }
    }
    __syncthreads();
  }
  pass_range(a.imin, a.imax, a.omin, a.omax);
}

// The same with 16-byte loads (A % 16 == 0 and every input stride a multiple of 16 as well):
// a thread takes 16 bytes along A of four consecutive B rows, so the 128 x 128-byte tile
// costs it four load instructions instead of sixteen; 8 lanes cover a row's 128 bytes.
template <int PIECE>
__global__ __launch_bounds__(kThreads) void permute_tile16_kernel(TileArgs a) {
  constexpr int kPitch = 33;  // dwords per transposed row: 128 bytes + 4 of padding
  __shared__ uint32_t tile[128 * kPitch];
  const int t = threadIdx.x;
  unsigned tile_id = blockIdx.x;
  int64_t z0 = blockIdx.y, z_step = gridDim.y;
  if (a.per_xcd != 0) {
    // work-group ids go round the 8 XCDs: undone, so that tiles which share input cache
    // lines (rows of A that miss the 128-byte marks) meet in one L2
    const unsigned item = (blockIdx.x & 7u) * a.per_xcd + (blockIdx.x >> 3);
    if (item >= a.xcd_total) return;  // (work-group 0 is item 0: the range is still passed on)
    z0 = item / a.tiles_ab;
    tile_id = item - static_cast<unsigned>(z0) * a.tiles_ab;
    z_step = a.batches;
  }
  const int64_t tb = tile_id / a.tiles_a, ta = tile_id - tb * a.tiles_a;
  const int64_t a0 = ta * 128, b0 = tb * 128;
  const int sq = t & 7, rq = t >> 3;
  for (int64_t z = z0; z < a.batches; z += z_step) {
    size_t in_off, out_off;
    batch_offsets(a, z, in_off, out_off);
    const uint8_t* src = a.in + in_off;
    uint8_t* dst = a.out + out_off;
    const int64_t aa = a0 + 16 * sq;
    u4 w[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int64_t b = b0 + 4 * rq + j;
      w[j] = (b < a.B && aa < a.A)
                 ? __builtin_nontemporal_load(reinterpret_cast<const u4*>(
                       src + static_cast<size_t>(b * a.b_in_stride + aa)))
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
    const int64_t left = a.B - b0;
    const int nb = left < 128 ? static_cast<int>(left) : 128;  // bytes per output row (PIECE | nb)
    const int per_row = nb / PIECE;
    const int pieces = 128 * per_row;
    for (int c = t; c < pieces; c += kThreads) {
      const int sl = per_row == 128 / PIECE ? c / (128 / PIECE) : c / per_row;
      const int k = c - sl * per_row;
      if (a0 + sl < a.A) {
        uint8_t* to = dst + static_cast<size_t>((a0 + sl) * a.a_out_stride + b0 + PIECE * k);
        if (PIECE == 16) {
          u4 v;
#pragma unroll
          for (int i = 0; i < 4; ++i) v[i] = tile[sl * kPitch + 4 * k + i];
          __builtin_nontemporal_store(v, reinterpret_cast<u4*>(to));
        } else {
          // output rows of 4 | B bytes (14 x 14 planes): dword pieces
          __builtin_nontemporal_store(tile[sl * kPitch + k], reinterpret_cast<uint32_t*>(to));
        }
      }
    }
    __syncthreads();
  }
  pass_range(a.imin, a.imax, a.omin, a.omax);
}

// The innermost axis moves and one of the two extents is thin (at most 64 bytes, e.g. planes
// of 7 x 7) while the other is a multiple of 128, both matrices dense ([B][A] in, [A][B] out):
// see thin_transpose_tile.  Batches along blockIdx.y.
template <bool THIN_IN>
__global__ __launch_bounds__(kThreads) void permute_thin_kernel(TileArgs a) {
  __shared__ __attribute__((aligned(16))) uint8_t flat[128 * 64];
  const int L = static_cast<int>(THIN_IN ? a.B : a.A), T = static_cast<int>(THIN_IN ? a.A : a.B);
  for (int64_t z = blockIdx.y; z < a.batches; z += gridDim.y) {
    size_t in_off, out_off;
    batch_offsets(a, z, in_off, out_off);
    thin_transpose_tile<THIN_IN>(a.in + in_off, a.out + out_off, L, T, blockIdx.x * 128, flat);
    __syncthreads();
  }
  pass_range(a.imin, a.imax, a.omin, a.omax);
}

// The innermost run of E bytes (16 | E, E <= 256) stays whole but the two axes around it
// swap neighbours (attention's (batch, seq, heads, E) <-> (batch, heads, seq, E)): rows of
// such short runs copied one by one touch half cache lines on one side.  Here T x T runs
// go through LDS: reads are T runs along A (contiguous in the input), writes T runs along
// B (contiguous in the output); the LDS row pitch of T * E + E bytes keeps the read-back
// of a wave on distinct banks.
constexpr int kElemLdsBytes = 17408;  // max over E of T * (T + 1) * E with T = min(16, 1024 / E)

struct ElemArgs {
  TileArgs t;     // A / B count runs; a_out_stride / b_in_stride are in bytes
  int E, T;
};

__global__ __launch_bounds__(kThreads) void permute_elem_kernel(ElemArgs e) {
  __shared__ __attribute__((aligned(16))) uint8_t tile[kElemLdsBytes];
  const TileArgs& a = e.t;
  const int E = e.E, T = e.T;
  const int run16 = (T * E) >> 4;          // 16-byte pieces per tile row
  const int pitch = T * E + E;
  const int pieces = T * run16;
  const int64_t tb = blockIdx.x / a.tiles_a, ta = blockIdx.x - tb * a.tiles_a;
  const int64_t a0 = ta * T, b0 = tb * T;
  for (int64_t z = blockIdx.y; z < a.batches; z += gridDim.y) {
    size_t in_off, out_off;
    batch_offsets(a, z, in_off, out_off);
    const uint8_t* src = a.in + in_off;
    uint8_t* dst = a.out + out_off;
    // at most 4 pieces per thread (T * T * E / 16 <= 1024): all loads first, unconditional
    // (a piece outside the tensor reads the batch's first bytes and is dropped), then the
    // LDS writes; the same for the way out
    u4 v[4];
    int slot[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int c = threadIdx.x + j * kThreads;
      const int b = c / run16, off = (c - b * run16) << 4;
      const bool ok = c < pieces && b0 + b < a.B && a0 + off / E < a.A;
      slot[j] = ok ? b * pitch + off : -1;
      const size_t at = ok ? static_cast<size_t>((b0 + b) * a.b_in_stride + a0 * E + off) : 0;
      v[j] = *reinterpret_cast<const u4*>(src + at);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (slot[j] >= 0) *reinterpret_cast<u4*>(tile + slot[j]) = v[j];
    __syncthreads();
    size_t to[4];
    bool put[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int c = threadIdx.x + j * kThreads;
      const int ar = c / run16, off = (c - ar * run16) << 4;
      const int b = off / E, within = off - b * E;
      put[j] = c < pieces && a0 + ar < a.A && b0 + b < a.B;
      to[j] = static_cast<size_t>((a0 + ar) * a.a_out_stride + b0 * E + off);
      v[j] = *reinterpret_cast<const u4*>(tile + (c < pieces ? b * pitch + ar * E + within : 0));
    }
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (put[j]) *reinterpret_cast<u4*>(dst + to[j]) = v[j];
    __syncthreads();
  }
  pass_range(a.imin, a.imax, a.omin, a.omax);
}

// The same swap for runs of 16, 32, 64, 128 or 256 bytes without LDS: the 64 lanes of a wave
// are (16-byte piece of the run) x (2^sa_shift runs along A) x (2^sb_shift runs along B), so
// one load instruction reads 2^sa_shift consecutive runs of the input for each of its B
// positions and one store instruction writes 2^sb_shift consecutive runs of the output for
// each of its A positions: at least 128 contiguous bytes on both sides.  A lane moves
// kElemDirectPieces pieces that follow one another along B; one wave per tile, no loop.
constexpr int kElemDirectPieces = 2;

struct ElemDirectArgs {
  TileArgs t;  // A / B count runs; a_out_stride / b_in_stride in bytes; tiles_a = tiles along A
  unsigned tiles_b;
  int e16_shift, sa_shift, sb_shift;
};

__global__ __launch_bounds__(kThreads) void permute_elem_direct_kernel(ElemDirectArgs e) {
  const TileArgs& a = e.t;
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t within = lane & ((1u << e.e16_shift) - 1u);
  const uint32_t asub = (lane >> e.e16_shift) & ((1u << e.sa_shift) - 1u);
  const uint32_t bsub = lane >> (e.e16_shift + e.sa_shift);
  const uint64_t per_batch = uint64_t(a.tiles_a) * e.tiles_b;
  const uint64_t wave = uint64_t(blockIdx.x) * (kThreads / 64) +
                        __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  if (wave < per_batch * static_cast<uint64_t>(a.batches)) {
    const uint64_t z = wave / per_batch, rem = wave - z * per_batch;
    const uint64_t tb = rem / a.tiles_a, ta = rem - tb * a.tiles_a;
    size_t in_off, out_off;
    batch_offsets(a, static_cast<int64_t>(z), in_off, out_off);
    const int64_t ai = static_cast<int64_t>(ta << e.sa_shift) + asub;
    const int64_t b0 = static_cast<int64_t>((tb * kElemDirectPieces) << e.sb_shift) + bsub;
    const int E = 16 << e.e16_shift;
    const uint8_t* src = a.in + in_off + static_cast<size_t>(ai) * E + 16 * within;
    uint8_t* dst = a.out + out_off + static_cast<size_t>(ai * a.a_out_stride) + 16 * within;
    u4 v[kElemDirectPieces];
#pragma unroll
    for (int j = 0; j < kElemDirectPieces; ++j) {
      const int64_t b = b0 + (int64_t(j) << e.sb_shift);
      v[j] = (ai < a.A && b < a.B)
                 ? __builtin_nontemporal_load(
                       reinterpret_cast<const u4*>(src + static_cast<size_t>(b * a.b_in_stride)))
                 : u4{0, 0, 0, 0};
    }
#pragma unroll
    for (int j = 0; j < kElemDirectPieces; ++j) {
      const int64_t b = b0 + (int64_t(j) << e.sb_shift);
      if (ai < a.A && b < a.B)
        __builtin_nontemporal_store(v[j], reinterpret_cast<u4*>(dst + static_cast<size_t>(b) * E));
    }
  }
  pass_range(a.imin, a.imax, a.omin, a.omax);
}

__global__ void range_only_kernel(const float* imin, const float* imax, float* omin, float* omax) {
  *omin = *imin;
  *omax = *imax;
}

}  // namespace
}  // namespace mxq

using namespace mxq;

extern "C" {

int mxq_quantized_embedding(void* stream, const void* indices, int index_type,
                            const int8_t* weight, const float* min_weight,
                            const float* max_weight, int8_t* out, float* omin, float* omax,
                            size_t n_indices, int64_t input_dim, int64_t output_dim) {
  MXQ_API_BEGIN();
  MXQ_CHECK(input_dim > 0 && output_dim > 0, "empty embedding table");
  MXQ_CHECK(min_weight != nullptr && max_weight != nullptr && omin != nullptr && omax != nullptr,
            "null range pointer");
  MXQ_CHECK(weight != nullptr, "null weight pointer");
  MXQ_CHECK(n_indices == 0 || (indices != nullptr && out != nullptr), "null data pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  EmbedArgs a;
  a.idx = indices;
  a.weight = reinterpret_cast<const uint8_t*>(weight);
  a.out = reinterpret_cast<uint8_t*>(out);
  a.wmin = min_weight; a.wmax = max_weight; a.omin = omin; a.omax = omax;
  a.n = n_indices;
  a.K = input_dim;
  a.D = static_cast<size_t>(output_dim);
  const bool vec = (a.D % 16 == 0) && aligned16(weight) && aligned16(out);
  a.group = group_lanes(vec ? a.D / 16 : a.D);
  a.shift = __builtin_ctz(a.group);
  switch (index_type) {
    case MXQ_FLOAT32: launch_embedding<float>(s, a, vec); break;
    case MXQ_FLOAT64: launch_embedding<double>(s, a, vec); break;
    case MXQ_UINT8: launch_embedding<uint8_t>(s, a, vec); break;
    case MXQ_INT32: launch_embedding<int32_t>(s, a, vec); break;
    case MXQ_INT8: launch_embedding<int8_t>(s, a, vec); break;
    case MXQ_INT64: launch_embedding<int64_t>(s, a, vec); break;
    default: MXQ_CHECK(false, "unsupported index type " << index_type);
  }
  MXQ_API_END();
}

int mxq_quantized_transpose(void* stream, const void* in, const float* imin, const float* imax,
                            void* out, float* omin, float* omax, int ndim,
                            const int64_t* in_shape, const int* axes) {
  MXQ_API_BEGIN();
  MXQ_CHECK(ndim >= 0 && ndim <= kMaxDims, "at most " << kMaxDims << " axes, got " << ndim);
  MXQ_CHECK(imin != nullptr && imax != nullptr && omin != nullptr && omax != nullptr,
            "null range pointer");
  MXQ_CHECK(ndim == 0 || in_shape != nullptr, "null shape pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  // axes == nullptr reverses the axes (TransposeParam's default, matrix_op-inl.h)
  int perm[kMaxDims];
  bool seen[kMaxDims] = {false};
  for (int d = 0; d < ndim; ++d) {
    int ax = axes ? axes[d] : ndim - 1 - d;
    if (ax < 0) ax += ndim;
    MXQ_CHECK(ax >= 0 && ax < ndim && !seen[ax], "axes is not a permutation");
    seen[ax] = true;
    perm[d] = ax;
  }
  int64_t in_stride[kMaxDims];
  size_t total = 1;
  for (int d = ndim - 1; d >= 0; --d) {
    MXQ_CHECK(in_shape[d] >= 0, "negative extent");
    in_stride[d] = static_cast<int64_t>(total);
    total *= static_cast<size_t>(in_shape[d]);
  }
  if (total == 0) {
    hipLaunchKernelGGL(range_only_kernel, dim3(1), dim3(1), 0, s, imin, imax, omin, omax);
    MXQ_LAUNCH_CHECK();
    return 0;
  }
  MXQ_CHECK(in != nullptr && out != nullptr, "null data pointer");
  // drop axes of extent 1, merge out axes that are adjacent in the input as well
  int64_t oe[kMaxDims], os[kMaxDims];
  int nd = 0;
  for (int d = 0; d < ndim; ++d) {
    const int64_t e = in_shape[perm[d]], st = in_stride[perm[d]];
    if (e == 1) continue;
    if (nd > 0 && os[nd - 1] == st * e) {
      oe[nd - 1] *= e;
      os[nd - 1] = st;
    } else {
      oe[nd] = e;
      os[nd] = st;
      ++nd;
    }
  }
  if (nd == 0) {
    oe[0] = 1;
    os[0] = 1;
    nd = 1;
  }
  if (os[nd - 1] == 1) {
    // innermost axis unchanged: rows of L contiguous bytes
    RowsArgs a;
    a.in = static_cast<const uint8_t*>(in);
    a.out = static_cast<uint8_t*>(out);
    a.imin = imin; a.imax = imax; a.omin = omin; a.omax = omax;
    a.L = static_cast<size_t>(oe[nd - 1]);
    a.p.nd = nd - 1;
    a.rows = 1;
    bool strides16 = true;
    for (int d = 0; d < nd - 1; ++d) {
      a.p.out_extent[d] = oe[d];
      a.p.in_stride[d] = os[d];
      a.rows *= static_cast<size_t>(oe[d]);
      strides16 = strides16 && (os[d] % 16 == 0);
    }
    // few long rows: cut them into pieces (one more outer axis) so that a group of lanes
    // never owns megabytes while most of the chip idles
    if (a.L >= 8192 && a.p.nd < kMaxDims) {
      size_t seg = 2048;
      while (seg > 128 && a.L % seg != 0) seg >>= 1;
      if (a.L % seg == 0) {
        a.p.out_extent[a.p.nd] = static_cast<int64_t>(a.L / seg);
        a.p.in_stride[a.p.nd] = static_cast<int64_t>(seg);
        ++a.p.nd;
        a.rows *= a.L / seg;
        a.L = seg;
      }
    }
    const bool vec = (a.L % 16 == 0) && strides16 && aligned16(in) && aligned16(out);
    if (vec && a.L <= 256 && nd >= 3) {
      // short runs between two axes that swap neighbours: T x T runs through LDS
      const int db = nd - 2;
      int da = -1;
      for (int d = 0; d < nd - 1; ++d)
        if (os[d] == static_cast<int64_t>(a.L)) da = d;
      // worth it only when both axes fill a good part of a tile (3 x 1000 runs of 16 bytes
      // take 87 us this way and 48 us row by row)
      if (da >= 0 && da != db && oe[da] >= 8 && oe[db] >= 8) {
        ElemArgs e;
        TileArgs& t = e.t;
        t.in = a.in; t.out = a.out;
        t.imin = imin; t.imax = imax; t.omin = omin; t.omax = omax;
        e.E = static_cast<int>(a.L);
        e.T = 1024 / e.E < 16 ? 1024 / e.E : 16;
        int64_t out_stride[kMaxDims];
        int64_t acc = static_cast<int64_t>(a.L);
        for (int d = nd - 2; d >= 0; --d) {
          out_stride[d] = acc;
          acc *= oe[d];
        }
        t.A = oe[da];
        t.B = oe[db];
        t.a_out_stride = out_stride[da];
        t.b_in_stride = os[db];
        t.p.nd = 0;
        t.batches = 1;
        for (int d = 0; d < nd - 1; ++d) {
          if (d == da || d == db) continue;
          t.p.out_extent[t.p.nd] = oe[d];
          t.p.in_stride[t.p.nd] = os[d];
          t.p_out_stride[t.p.nd] = out_stride[d];
          t.batches *= oe[d];
          ++t.p.nd;
        }
        const int e16 = e.E >> 4;
        if ((e16 & (e16 - 1)) == 0 && e16 <= 16) {
          // power-of-two runs: straight through registers
          ElemDirectArgs d;
          d.t = t;
          d.e16_shift = __builtin_ctz(e16);
          const int run_shift = 6 - d.e16_shift;  // runs per wave instruction
          d.sa_shift = (run_shift + 1) / 2;
          d.sb_shift = run_shift - d.sa_shift;
          const int64_t da_tiles = (t.A + (int64_t(1) << d.sa_shift) - 1) >> d.sa_shift;
          const int64_t per_b = int64_t(kElemDirectPieces) << d.sb_shift;
          const int64_t db_tiles = (t.B + per_b - 1) / per_b;
          const int64_t waves_per_group = kThreads / 64;
          if (da_tiles < (int64_t(1) << 31) && db_tiles < (int64_t(1) << 31) &&
              t.batches < (int64_t(1) << 40) / (da_tiles * db_tiles + 1)) {
            const int64_t groups = (da_tiles * db_tiles * t.batches + waves_per_group - 1) / waves_per_group;
            if (groups < (int64_t(1) << 31)) {
              d.t.tiles_a = static_cast<unsigned>(da_tiles);
              d.tiles_b = static_cast<unsigned>(db_tiles);
              hipLaunchKernelGGL(permute_elem_direct_kernel, dim3(static_cast<unsigned>(groups)),
                                 dim3(kThreads), 0, s, d);
              MXQ_LAUNCH_CHECK();
              return 0;
            }
          }
        }
        const int64_t ta = (t.A + e.T - 1) / e.T, tb = (t.B + e.T - 1) / e.T;
        if (ta * tb < (int64_t(1) << 31)) {
          t.tiles_a = static_cast<unsigned>(ta);
          const int64_t gy = t.batches < 65535 ? t.batches : 65535;
          hipLaunchKernelGGL(permute_elem_kernel,
                             dim3(static_cast<unsigned>(ta * tb), static_cast<unsigned>(gy)),
                             dim3(kThreads), 0, s, e);
          MXQ_LAUNCH_CHECK();
          return 0;
        }
      }
    }
    size_t units = vec ? a.L / 16 : a.L;
    a.group = group_lanes(units);
    a.shift = __builtin_ctz(a.group);
    const bool narrow = a.rows < (size_t(1) << 32);
    const int grid = grid_for_rows(a.rows, a.group);
#define MXQ_ROWS(UI, V) \
  hipLaunchKernelGGL((permute_rows_kernel<UI, V>), dim3(grid), dim3(kThreads), 0, s, a)
    if (narrow) { if (vec) MXQ_ROWS(uint32_t, true); else MXQ_ROWS(uint32_t, false); }
    else        { if (vec) MXQ_ROWS(uint64_t, true); else MXQ_ROWS(uint64_t, false); }
#undef MXQ_ROWS
    MXQ_LAUNCH_CHECK();
    return 0;
  }
  // innermost axis moves: A = the out axis with input stride 1, B = the innermost out axis
  int64_t out_stride[kMaxDims];
  {
    int64_t acc = 1;
    for (int d = nd - 1; d >= 0; --d) {
      out_stride[d] = acc;
      acc *= oe[d];
    }
  }
  int da = -1;
  for (int d = 0; d < nd; ++d)
    if (os[d] == 1) da = d;
  MXQ_CHECK(da >= 0 && da != nd - 1, "internal: no unit-stride axis");
  TileArgs a;
  a.in = static_cast<const uint8_t*>(in);
  a.out = static_cast<uint8_t*>(out);
  a.imin = imin; a.imax = imax; a.omin = omin; a.omax = omax;
  a.A = oe[da];
  a.B = oe[nd - 1];
  a.a_out_stride = out_stride[da];
  a.b_in_stride = os[nd - 1];
  a.p.nd = 0;
  a.batches = 1;
  for (int d = 0; d < nd - 1; ++d) {
    if (d == da) continue;
    a.p.out_extent[a.p.nd] = oe[d];
    a.p.in_stride[a.p.nd] = os[d];
    a.p_out_stride[a.p.nd] = out_stride[d];
    a.batches *= oe[d];
    ++a.p.nd;
  }
  bool friendly = (a.A % 4 == 0) && (a.B % 16 == 0) && (a.b_in_stride % 4 == 0) &&
                  (a.a_out_stride % 16 == 0) && aligned16(in) && aligned16(out);
  for (int d = 0; d < a.p.nd; ++d)
    friendly = friendly && (a.p.in_stride[d] % 4 == 0) && (a.p_out_stride[d] % 16 == 0);
  {
    // a thin extent beside a long one, dense matrices, every batch on a 16-byte mark
    bool marks = aligned16(in) && aligned16(out) && a.b_in_stride == a.A && a.a_out_stride == a.B;
    for (int d = 0; d < a.p.nd; ++d)
      marks = marks && (a.p.in_stride[d] % 16 == 0) && (a.p_out_stride[d] % 16 == 0);
    const bool thin_in = a.A <= 64 && a.B % 128 == 0;   // input [B][A], A thin
    const bool thin_out = a.B <= 64 && a.A % 128 == 0;  // input [B][A], B thin
    const int64_t longer = thin_in ? a.B : a.A;
    if (!friendly && marks && (thin_in || thin_out) && longer < (int64_t(1) << 31)) {
      const int64_t gy = a.batches < 65535 ? a.batches : 65535;
      const dim3 grid(static_cast<unsigned>(longer / 128), static_cast<unsigned>(gy));
      if (thin_in)
        hipLaunchKernelGGL(permute_thin_kernel<true>, grid, dim3(kThreads), 0, s, a);
      else
        hipLaunchKernelGGL(permute_thin_kernel<false>, grid, dim3(kThreads), 0, s, a);
      MXQ_LAUNCH_CHECK();
      return 0;
    }
  }
  {
    // 16-byte loads with dword stores: output rows and strides that are multiples of 4 only
    bool in16 = (a.A % 16 == 0) && (a.b_in_stride % 16 == 0) && aligned16(in);
    bool out4 = (a.B % 4 == 0) && (a.a_out_stride % 4 == 0) &&
                (reinterpret_cast<uintptr_t>(out) & 3u) == 0;
    for (int d = 0; d < a.p.nd; ++d) {
      in16 = in16 && (a.p.in_stride[d] % 16 == 0);
      out4 = out4 && (a.p_out_stride[d] % 4 == 0);
    }
    const int64_t fa = (a.A + 127) / 128, fb = (a.B + 127) / 128;
    if (!friendly && in16 && out4 && a.A >= 128 && a.B >= 128 && fa * fb < (int64_t(1) << 31)) {
      a.tiles_a = static_cast<unsigned>(fa);
      const int64_t fy = a.batches < 65535 ? a.batches : 65535;
      hipLaunchKernelGGL(permute_tile16_kernel<4>,
                         dim3(static_cast<unsigned>(fa * fb), static_cast<unsigned>(fy)),
                         dim3(kThreads), 0, s, a);
      MXQ_LAUNCH_CHECK();
      return 0;
    }
  }
  if (friendly) {
    // output rows of 128 bytes per tile (whole cache lines on both sides) where B has them
    // and A fills the tile's 128 columns (with 64 the larger tile idles half its lanes)
    const int tile_b = (a.B >= 128 && a.A >= 128) ? 128 : 64;
    const int64_t fa = (a.A + 127) / 128, fb = (a.B + tile_b - 1) / tile_b;
    if (fa * fb < (int64_t(1) << 31)) {
      a.tiles_a = static_cast<unsigned>(fa);
      const int64_t fy = a.batches < 65535 ? a.batches : 65535;
      const dim3 grid(static_cast<unsigned>(fa * fb), static_cast<unsigned>(fy));
      bool friendly16 = (a.A % 16 == 0) && (a.b_in_stride % 16 == 0);
      for (int d = 0; d < a.p.nd; ++d) friendly16 = friendly16 && (a.p.in_stride[d] % 16 == 0);
      if (tile_b == 128 && friendly16 && a.A % 128 != 0 && a.batches <= 65535 &&
          fa * fb * a.batches < (int64_t(1) << 31) - 8) {
        // rows of A that miss the 128-byte marks (56 x 56, 28 x 28 planes): XCD-aware order,
        // measured on the convolution's adapters (22.6 -> 21.1 us, 14.3 -> 12.1 us); rows on
        // the marks lose 10 % with it and keep the plain grid
        a.tiles_ab = static_cast<unsigned>(fa * fb);
        a.xcd_total = static_cast<unsigned>(fa * fb * a.batches);
        a.per_xcd = (a.xcd_total + 7u) / 8u;
        hipLaunchKernelGGL(permute_tile16_kernel<16>, dim3(a.per_xcd * 8u), dim3(kThreads), 0, s, a);
      } else if (tile_b == 128 && friendly16)
        hipLaunchKernelGGL(permute_tile16_kernel<16>, grid, dim3(kThreads), 0, s, a);
      else if (tile_b == 128)
        hipLaunchKernelGGL(permute_tile4_kernel<128>, grid, dim3(kThreads), 0, s, a);
      else
        hipLaunchKernelGGL(permute_tile4_kernel<64>, grid, dim3(kThreads), 0, s, a);
      MXQ_LAUNCH_CHECK();
      return 0;
    }
  }
  const int64_t ta = (a.A + kTile - 1) / kTile, tb = (a.B + kTile - 1) / kTile;
  MXQ_CHECK(ta * tb < (int64_t(1) << 31), "tensor too large for the tile grid");
  a.tiles_a = static_cast<unsigned>(ta);
  const int64_t gy = a.batches < 65535 ? a.batches : 65535;
  hipLaunchKernelGGL(permute_tile_kernel,
                     dim3(static_cast<unsigned>(ta * tb), static_cast<unsigned>(gy)),
                     dim3(kThreads), 0, s, a);
  MXQ_LAUNCH_CHECK();
  MXQ_API_END();
}

}  // extern "C"
