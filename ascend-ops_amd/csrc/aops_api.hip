// Entry points of libaops that are not operators: version, error text, device summary.
#include <stdio.h>

#include <atomic>
#include <string.h>

#include "aops_common.h"

namespace aops {

static thread_local int g_last_hip_error = 0;

int record_launch_status(hipError_t e) {
  if (e == hipSuccess) return AOPS_OK;
  g_last_hip_error = (int)e;
  return AOPS_ERR_LAUNCH;
}

int device_cu_count() {
  constexpr int kMaxDevices = 64;
  constexpr int kDefault = 256;
  static std::atomic<int> cus[kMaxDevices];  // 0 = not asked yet; every writer stores the same value
  // "No device to ask" (a workspace query on a machine without a GPU) answers with an MI355X's count; any
  // other failure of the runtime is kept for aops_last_hip_error() instead of being swallowed.
  auto fallback = [](hipError_t e) {
    (void)hipGetLastError();
    if (e != hipErrorNoDevice && e != hipErrorInvalidDevice && e != hipErrorInsufficientDriver &&
        e != hipErrorNotInitialized)
      (void)record_launch_status(e);
    return kDefault;
  };
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fallback(e);
  if (dev < 0 || dev >= kMaxDevices) return kDefault;
  int v = cus[dev].load(std::memory_order_relaxed);
  if (v == 0) {
    e = hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev);
    if (e != hipSuccess) return fallback(e);
    if (v <= 0) v = kDefault;
    cus[dev].store(v, std::memory_order_relaxed);
  }
  return v;
}

hipError_t allow_dynamic_lds(const void* kernel, int bytes, std::atomic<uint64_t>& done) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) dev = -1;
  const bool tracked = dev >= 0 && dev < 64;
  if (tracked && (done.load(std::memory_order_relaxed) >> dev & 1)) return hipSuccess;
  const hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e == hipSuccess && tracked) done.fetch_or(uint64_t(1) << dev, std::memory_order_relaxed);
  return e;
}

}  // namespace aops

extern "C" int aops_version(void) { return 200; }

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
    case AOPS_ERR_SCRATCH_LIMIT:
      return "problem needs more scratch than the fixed maximum of the entry point that allocates nothing";
    default:
      return "unknown error code";
  }
}

extern "C" int aops_last_hip_error(void) { return aops::g_last_hip_error; }

namespace aops {
__global__ void empty_kernel() {}
}  // namespace aops

extern "C" int aops_empty_launch(int64_t workgroups, int threads, void* stream) {
  if (workgroups <= 0 || workgroups > 0x7fffffff || threads <= 0 || threads > 1024)
    return AOPS_ERR_INVALID_ARGUMENT;
  aops::empty_kernel<<<(unsigned)workgroups, (unsigned)threads, 0, static_cast<hipStream_t>(stream)>>>();
  return aops::record_launch_status(hipGetLastError());
}

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
