#include "common.h"

#include <stdarg.h>
#include <stdio.h>

#include "api.h"

namespace bc4g {

static thread_local char g_error[512] = "";

int fail(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return 1;
}

int check_launch(const char* what) {
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail("%s: launch failed: %s", what, hipGetErrorString(e));
  return 0;
}

int compute_units() {
  static int cus[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (cus[dev] == 0) {
    int v = 0;
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0) v = 256;
    cus[dev] = v;
  }
  return cus[dev];
}

}  // namespace bc4g

#ifndef BC4G_SOURCES_DIGEST
#define BC4G_SOURCES_DIGEST "unknown"
#endif

extern "C" const char* bc4g_last_error() { return bc4g::g_error; }
extern "C" int bc4g_version() { return 2; }
// The digest of the kernel sources and compiler flags this library was built from (the build passes it
// in): whoever loads the library compares it with the sources beside it, so that signatures declared
// for new sources are never bound to an old binary.
// (behind a marker, so that it can also be found in the file without loading it)
static const char kSourcesDigest[] = "bc4g-sources-digest:" BC4G_SOURCES_DIGEST;
extern "C" const char* bc4g_sources_digest() { return kSourcesDigest + sizeof("bc4g-sources-digest:") - 1; }
