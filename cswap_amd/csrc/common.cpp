// common.cpp -- error strings and ABI version
#include "common.h"

namespace cswap {
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
