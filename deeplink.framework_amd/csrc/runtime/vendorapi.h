// Vendor typedefs for the AMD (HIP) backend: the counterpart of
// dipu/torch_dipu/csrc_dipu/vendor/cuda/vendorapi.h:37-49 for gfx950.
#pragma once

// Inside a DIPU tree the vendor directory's own vendorapi.h (TORCH_CHECK-based) has already declared everything below.
#ifndef DIPU_CALLHIP

#include <hip/hip_runtime_api.h>

#include <stdexcept>
#include <string>

namespace dipu {

// Throws like TORCH_CHECK does in a DIPU build: every HIP failure becomes a C++
// exception carrying the expression and HIP's own error text.
#define DIPU_CALLHIP(Expr)                                                                           \
  {                                                                                                  \
    hipError_t ret_ = (Expr);                                                                        \
    if (ret_ != hipSuccess) {                                                                        \
      (void)hipGetLastError(); /* the exception carries the failure; leave no sticky error behind */  \
      throw std::runtime_error(std::string("call hip error, expr = " #Expr ", ret = ") +             \
                               std::to_string(static_cast<int>(ret_)) + " (" + hipGetErrorString(ret_) + ")"); \
    }                                                                                                \
  }

using deviceStream_t = hipStream_t;
#define deviceDefaultStreamLiteral nullptr
using deviceEvent_t = hipEvent_t;

// Single-GPU backend: the collective types exist only so the 12 link-required
// dicl symbols (dipu/torch_dipu/csrc_dipu/runtime/device/diclapis.h:23-82) can be declared.
using diclComm_t = void*;
struct commUniqueId {
  char internal[128];
};

}  // namespace dipu

#endif  // DIPU_CALLHIP
