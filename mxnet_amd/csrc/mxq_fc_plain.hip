// The fully-connected kernels built for the int32 and int8 outputs.
#include "mxq_fc_kernels.h"

namespace mxq {

void fc_launch_plain(hipStream_t s, const FcArgs& a, const FcLaunch& how, const Workspace& ws) {
  fc_launch_mode<kEpiPlain>(s, a, how, ws);
}

}  // namespace mxq
