// The fully-connected kernels built for the float output (mxq_quantized_fc_f32).
#include "mxq_fc_kernels.h"

namespace mxq {

void fc_launch_f32(hipStream_t s, const FcArgs& a, const FcLaunch& how, const Workspace& ws) {
  fc_launch_mode<kEpiF32>(s, a, how, ws);
}

}  // namespace mxq
