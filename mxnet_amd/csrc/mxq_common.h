// Shared host-side helpers of libmxq_hip.so: thread-local error string and the
// exception -> return-code fence every C-ABI entry point goes through.
#ifndef MXQ_COMMON_H_
#define MXQ_COMMON_H_

#include <hip/hip_runtime.h>

#include <cstdint>
#include <sstream>
#include <stdexcept>
#include <string>

namespace mxq {

void set_last_error(const std::string& msg);

struct Error : public std::runtime_error {
  explicit Error(const std::string& m) : std::runtime_error(m) {}
};

#define MXQ_CHECK(cond, msg)                                   \
  do {                                                         \
    if (!(cond)) {                                             \
      std::ostringstream os_;                                  \
      os_ << __func__ << ": check failed: " #cond ": " << msg; \
      throw ::mxq::Error(os_.str());                           \
    }                                                          \
  } while (0)

#define MXQ_HIP(call)                                                       \
  do {                                                                      \
    hipError_t e_ = (call);                                                 \
    if (e_ != hipSuccess) {                                                 \
      std::ostringstream os_;                                               \
      os_ << __func__ << ": " #call " failed: " << hipGetErrorString(e_);   \
      throw ::mxq::Error(os_.str());                                        \
    }                                                                       \
  } while (0)

// Checks the launch itself (bad configuration, missing code object); does not
// synchronise.
#define MXQ_LAUNCH_CHECK() MXQ_HIP(hipGetLastError())

#define MXQ_API_BEGIN() try {
#define MXQ_API_END()                        \
  }                                          \
  catch (const std::exception& e) {          \
    ::mxq::set_last_error(e.what());         \
    return -1;                               \
  }                                          \
  catch (...) {                              \
    ::mxq::set_last_error("unknown error");  \
    return -1;                               \
  }                                          \
  return 0;

// Compute units of the calling thread's current device (cached per thread and device).
int num_cus();

// Work-groups of 256 threads per CU the streaming kernels are launched with at most:
// more resident waves lower the HBM bandwidth they reach (8 waves per CU: 6.0 TB/s,
// 16: 5.5, 32 and more: 5.4 on a 256 MB cast).
constexpr int kCastBlocksPerCu = 2;

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace mxq

#endif  // MXQ_COMMON_H_
