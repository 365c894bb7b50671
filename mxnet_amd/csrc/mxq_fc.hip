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
#include "mxq_fc_args.h"
#include "mxq_gemm.h"
#include "mxq_tiles.h"

namespace mxq {

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
  }
  if (cfg >= 21 && cfg < 61)
    MXQ_CHECK(buf_ok, "shape does not qualify for the buffer-load DMA kernels");
  if (cfg < 11) MXQ_CHECK(plan.splits <= 1, "the register-staged kernels have no split-K form");
  const FcLaunch how = {cfg, plan.splits, plan.stream_groups, aligned};
  switch (epi_mode(a.epi)) {
    case kEpiF32: fc_launch_f32(s, a, how, ws); break;
    case kEpiSum: fc_launch_sum(s, a, how, ws); break;
    default: fc_launch_plain(s, a, how, ws);
  }
}

// Scratch bytes with which launch_fc takes its fastest route for this shape (0 when it
// would not split).  Assumes 16-byte aligned operands.  The residual-sum form plans its tile
// on its own (plan_fc's `sum`), so the figure is the larger of the two plans: a workspace
// sized by this query serves mxq_quantized_fc and mxq_quantized_fc_sum alike.
size_t fc_workspace_bytes(int M, int N, int K, bool fused8) {
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  const size_t plain =
      fc_plan_workspace(plan_fc(M, N, K, K % 16 == 0, fused8, GemmForce(), false), M, N);
  if (!fused8) return plain;
  const size_t sum =
      fc_plan_workspace(plan_fc(M, N, K, K % 16 == 0, true, GemmForce(), true), M, N);
  return plain > sum ? plain : sum;
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

#ifdef MXQ_TEST_HOOKS
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
#endif  // MXQ_TEST_HOOKS

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

#ifdef MXQ_TEST_HOOKS
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
#endif  // MXQ_TEST_HOOKS

#ifdef MXQ_TEST_HOOKS
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
#endif  // MXQ_TEST_HOOKS

}  // extern "C"
