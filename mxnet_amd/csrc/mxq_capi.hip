// Error string, version and tuning knobs of libmxq_hip.so.
#include <cstring>
#include <string>

#include "../../include/mxq.h"
#include "mxq_common.h"

namespace mxq {

extern int g_cast_blocks_per_cu;
extern int g_fc_config;
extern int g_fc_stream_groups;
extern int g_conv_config;

static thread_local std::string tl_last_error;

void set_last_error(const std::string& msg) { tl_last_error = msg; }

}  // namespace mxq

extern "C" {

const char* mxq_last_error(void) { return mxq::tl_last_error.c_str(); }

int mxq_abi_version(void) { return MXQ_ABI_VERSION; }

// Development knobs (not part of the operator contract): returns 0 if the key is known.
int mxq_set_tuning(const char* key, int value) {
  if (std::strcmp(key, "cast_blocks_per_cu") == 0) {
    if (value < 1 || value > 64) return -1;
    mxq::g_cast_blocks_per_cu = value;
    return 0;
  }
  if (std::strcmp(key, "fc_config") == 0) {
    mxq::g_fc_config = value;
    return 0;
  }
  if (std::strcmp(key, "fc_stream_groups") == 0) {
    if (value < 1 || value > 16) return -1;
    mxq::g_fc_stream_groups = value;
    return 0;
  }
  if (std::strcmp(key, "conv_config") == 0) {
    mxq::g_conv_config = value;
    return 0;
  }
  return -1;
}

}  // extern "C"
