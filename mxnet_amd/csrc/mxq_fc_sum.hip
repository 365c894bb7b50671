// The fully-connected kernels built for the residual sum in the epilogue (mxq_quantized_fc_sum).
#include "mxq_fc_kernels.h"

namespace mxq {

void fc_launch_sum(hipStream_t s, const FcArgs& a, const FcLaunch& how, const Workspace& ws) {
  fc_launch_mode<kEpiSum>(s, a, how, ws);
}

}  // namespace mxq
