// Entry points of libaops that are not operators: version, error text, device summary.
#include <stdio.h>
#include <string.h>

#include "aops_common.h"

namespace aops {

static thread_local int g_last_hip_error = 0;

int record_launch_status(hipError_t e) {
  if (e == hipSuccess) return AOPS_OK;
  g_last_hip_error = (int)e;
  return AOPS_ERR_LAUNCH;
}

}  // namespace aops

extern "C" int aops_version(void) { return 100; }

extern "C" const char* aops_strerror(int code) {
  switch (code) {
    case AOPS_OK:
      return "success";
    case AOPS_ERR_INVALID_ARGUMENT:
      return "invalid argument (null pointer, negative size or unsupported size)";
    case AOPS_ERR_WORKSPACE:
      return "workspace missing or too small";
    case AOPS_ERR_LAUNCH:
      return "HIP kernel launch failed";
    default:
      return "unknown error code";
  }
}

extern "C" int aops_last_hip_error(void) { return aops::g_last_hip_error; }

extern "C" int aops_device_info(int device, char* buf, size_t buf_len) {
  if (!buf || buf_len == 0) return AOPS_ERR_INVALID_ARGUMENT;
  hipDeviceProp_t p;
  hipError_t e = hipGetDeviceProperties(&p, device);
  if (e != hipSuccess) return aops::record_launch_status(e);
  int n = snprintf(buf, buf_len,
                   "device %d: %s (%s)\n"
                   "  compute units        : %d\n"
                   "  wavefront size       : %d\n"
                   "  LDS per workgroup    : %zu KiB\n"
                   "  L2 cache             : %d KiB\n"
                   "  device memory        : %.1f GiB\n"
                   "  memory bus / clock   : %d bit / %d MHz\n"
                   "  engine clock         : %d MHz\n",
                   device, p.name, p.gcnArchName, p.multiProcessorCount, p.warpSize,
                   p.sharedMemPerBlock / 1024, p.l2CacheSize / 1024,
                   (double)p.totalGlobalMem / (1024.0 * 1024.0 * 1024.0), p.memoryBusWidth,
                   p.memoryClockRate / 1000, p.clockRate / 1000);
  if (n < 0) return AOPS_ERR_INVALID_ARGUMENT;
  return n < (int)buf_len ? n : (int)buf_len - 1;
}
