// common.h -- error plumbing shared by the translation units of libcswap_hip.so
#pragma once
#include <hip/hip_runtime.h>
#include "../../include/cswap_hip.h"

namespace cswap {

// hipError_t of the most recent failure on this thread (0 = none)
int& last_hip_error();

inline int hip_fail(hipError_t e)
{
  last_hip_error() = (int)e;
  return CSWAP_E_HIP;
}

// compute units of the current device (0 if the query fails), looked up once per device
int device_compute_units();

// to be called right after a kernel launch: picks up launch-configuration errors
inline int check_launch()
{
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? CSWAP_OK : hip_fail(e);
}

#define CSWAP_HIP_TRY(expr)                                   \
  do {                                                        \
    hipError_t e_ = (expr);                                   \
    if (e_ != hipSuccess) return ::cswap::hip_fail(e_);       \
  } while (0)

}  // namespace cswap
