// Host-side plumbing shared by every entry point: error string, version, device check.
#include "fmoba_common.h"

#include <string.h>

namespace fmoba {
static thread_local char g_err[512] = "";
void set_error(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}
}  // namespace fmoba

extern "C" int fmoba_version(void) { return 100; }
extern "C" const char *fmoba_last_error(void) { return fmoba::g_err; }

extern "C" int fmoba_check_device(void) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) {
    fmoba::set_error("no HIP device is current");
    return 1;
  }
  hipDeviceProp_t p;
  if (hipGetDeviceProperties(&p, dev) != hipSuccess) {
    fmoba::set_error("hipGetDeviceProperties failed");
    return 1;
  }
  if (strncmp(p.gcnArchName, "gfx950", 6) != 0) {
    fmoba::set_error("FlashMoBA-HIP only supports gfx950 (MI350X/MI355X); found %s", p.gcnArchName);
    return 1;
  }
  return 0;
}
