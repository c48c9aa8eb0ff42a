// Library-level entry points: the thread-local error message, the ABI version, the device check.

#include <string>

#include "tf_common.h"

namespace tf {

static thread_local std::string g_error;

void set_error(const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  g_error = buf;
}

void clear_error() { g_error.clear(); }

}  // namespace tf

extern "C" const char* tf_last_error(void) { return tf::g_error.c_str(); }

extern "C" int tf_version(void) { return 3; }

// A digest of the sources and flags this library was built from, given by the build (tensorfold_amd/build.py); the
// loader compares it with the sources it sees and rebuilds or refuses a library that is out of date.
#ifndef TF_BUILD_ID
#define TF_BUILD_ID "unknown"
#endif
extern "C" const char* tf_build_id(void) {
  static const char id[] = "TFMI_BUILD_ID=" TF_BUILD_ID;
  return id + sizeof("TFMI_BUILD_ID=") - 1;
}

extern "C" int tf_check_device(void) {
  tf::clear_error();
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) {
    tf::set_error("libtfmi needs an AMD Instinct MI355X (gfx950); no HIP device is available");
    return 1;
  }
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, dev) != hipSuccess) {
    tf::set_error("libtfmi: hipGetDeviceProperties failed for device %d", dev);
    return 1;
  }
  const std::string arch(prop.gcnArchName);
  if (arch.rfind("gfx950", 0) != 0) {
    tf::set_error("libtfmi's kernels are built for gfx950 (MI355X) only; this GPU (%s) is %s", prop.name,
                  prop.gcnArchName);
    return 1;
  }
  return 0;
}
