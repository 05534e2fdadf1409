// Process-wide pieces of the kernel library: the error text of the last refused call
// (per host thread) and a description of the device the kernels were built for.
#include "common.h"

#include <string.h>

thread_local char pylon_error_text[512] = "";

extern "C" const char* pylon_last_error() { return pylon_error_text; }

extern "C" int pylon_abi_version() { return 1; }

// 0 if the current device can run this library's code objects (gfx950), else 1 with
// the device's architecture name in the error text.
extern "C" int pylon_check_device() {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) PYLON_REFUSE("no HIP device: %s", hipGetErrorString(e));
  hipDeviceProp_t prop;
  e = hipGetDeviceProperties(&prop, dev);
  if (e != hipSuccess) PYLON_REFUSE("hipGetDeviceProperties failed: %s", hipGetErrorString(e));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    PYLON_REFUSE("these kernels are built for gfx950; the device is %s", prop.gcnArchName);
  return 0;
}
