// common.cpp -- error strings and ABI version
#include "common.h"

#include <atomic>

namespace cswap {
int device_compute_units()
{
  static std::atomic<int> cus[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
  int v = cus[dev].load(std::memory_order_relaxed);
  if (!v) {
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
    cus[dev].store(v, std::memory_order_relaxed);
  }
  return v;
}

int& last_hip_error()
{
  static thread_local int e = 0;
  return e;
}
}  // namespace cswap

extern "C" const char* cswap_strerror(int code)
{
  switch (code) {
    case CSWAP_OK: return "ok";
    case CSWAP_E_ARG: return "invalid argument";
    case CSWAP_E_UNSUPPORTED: return "not supported by this build";
    case CSWAP_E_HIP: return "HIP runtime error";
    case CSWAP_E_NOMEM: return "buffer or pool too small";
    case CSWAP_E_STATE: return "call out of order";
    default: return "unknown error";
  }
}

extern "C" int cswap_last_hip_error(void) { return cswap::last_hip_error(); }
extern "C" int cswap_abi_version(void) { return 1; }
