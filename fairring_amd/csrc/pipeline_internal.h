// Shared by the files that implement the pipeline (pipeline.cc and the
// schedule_*.cc files, one per kind of operation); not part of its interface.
#pragma once

#include <stdexcept>
#include <string>

#include <hip/hip_runtime.h>

namespace frg {

struct HipFailure : std::runtime_error {
  using std::runtime_error::runtime_error;
};
struct ContractFailure : std::runtime_error {
  int code;
  ContractFailure(int c, const std::string& m) : std::runtime_error(m), code(c) {}
};

// Throws on failure, like the reference's CUDA_CHECK (fairring/utils.h:35-45).
#define FRG_HIP_CHECK(op)                                                        \
  do {                                                                           \
    hipError_t res_ = (op);                                                      \
    if (res_ != hipSuccess) {                                                    \
      (void)hipGetLastError();                                                   \
      throw HipFailure(std::string("HIP error at ") + __FILE__ + ":" +           \
                       std::to_string(__LINE__) + ": " + hipGetErrorString(res_)); \
    }                                                                            \
  } while (0)

// Makes `device` current for the scope and restores the caller's device.
class DeviceGuard {
 public:
  explicit DeviceGuard(int device) {
    FRG_HIP_CHECK(hipGetDevice(&prev_));
    if (prev_ != device) {
      FRG_HIP_CHECK(hipSetDevice(device));
      changed_ = true;
    }
  }
  ~DeviceGuard() {
    if (changed_) (void)hipSetDevice(prev_);
  }

 private:
  int prev_ = 0;
  bool changed_ = false;
};

}  // namespace frg
