// What the fully-connected launcher hands to its kernels, and the three entry points of the
// kernel translation units: the kernels are built once per epilogue mode (mxq_gemm.h:
// kEpiPlain / kEpiF32 / kEpiSum), each mode in a file of its own so that they compile side
// by side.
#ifndef MXQ_FC_ARGS_H_
#define MXQ_FC_ARGS_H_

#include <hip/hip_runtime.h>

#include <cstdint>

#include "mxq_common.h"
#include "mxq_gemm.h"
#include "mxq_tiles.h"

namespace mxq {

struct FcArgs {
  const int8_t* data;    // [M][K]
  const int8_t* weight;  // [N][K]
  int M, N, K;
  int ldo;               // output row pitch in elements (N for the FC)
  Epilogue epi;
  SplitK sk;
};

// What launch_fc decided: the tile configuration (mxq_fc.hip lists them), the split-K
// factor and, for the short-K streaming kernel, its work-groups per CU.
struct FcLaunch {
  int cfg;
  int splits;
  int stream_groups;
  bool aligned;  // K % 16 == 0 and 16-byte aligned operands
};

// Launch the kernel of `how.cfg` built for the mode (mxq_fc_plain.hip, mxq_fc_f32.hip,
// mxq_fc_sum.hip).  The caller has checked that the shape qualifies for the configuration.
void fc_launch_plain(hipStream_t s, const FcArgs& a, const FcLaunch& how, const Workspace& ws);
void fc_launch_f32(hipStream_t s, const FcArgs& a, const FcLaunch& how, const Workspace& ws);
void fc_launch_sum(hipStream_t s, const FcArgs& a, const FcLaunch& how, const Workspace& ws);

}  // namespace mxq
#endif  // MXQ_FC_ARGS_H_
