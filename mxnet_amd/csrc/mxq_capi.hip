// Error string, version and device query shared by the launchers of libmxq_hip.so.
#include <string>

#include "../../include/mxq.h"
#include "mxq_common.h"

namespace mxq {

static thread_local std::string tl_last_error;

void set_last_error(const std::string& msg) { tl_last_error = msg; }

int num_cus() {
  int dev = 0;
  MXQ_HIP(hipGetDevice(&dev));
  static thread_local int cached_dev = -1, cached_cus = 0;
  if (cached_dev != dev) {
    MXQ_HIP(hipDeviceGetAttribute(&cached_cus, hipDeviceAttributeMultiprocessorCount, dev));
    cached_dev = dev;
  }
  return cached_cus;
}

}  // namespace mxq

extern "C" {

const char* mxq_last_error(void) { return mxq::tl_last_error.c_str(); }

int mxq_abi_version(void) { return MXQ_ABI_VERSION; }

}  // extern "C"
