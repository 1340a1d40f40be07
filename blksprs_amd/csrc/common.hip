// Error reporting of the C ABI.
#include "common.h"

namespace bsa {

char *error_buffer() {
  static thread_local char buf[512] = {0};
  return buf;
}

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(error_buffer(), 512, fmt, ap);
  va_end(ap);
  return code;
}

}  // namespace bsa

extern "C" int bsa_abi_version(void) { return BSA_ABI_VERSION; }

extern "C" const char *bsa_last_error(void) { return bsa::error_buffer(); }

#ifndef BSA_BUILD_INFO
#define BSA_BUILD_INFO "hipcc: unknown (built without blksprs_amd/csrc/build.py)"
#endif
extern "C" const char *bsa_build_info(void) { return BSA_BUILD_INFO; }
