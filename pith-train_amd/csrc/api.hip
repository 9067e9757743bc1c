// Error reporting and version entry points of libpith_hip.so.
#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstring>

#include "pith_common.h"

namespace pith {
namespace {
thread_local char g_last_error[512] = "";
}

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
  return code;
}

int compute_units() {
  constexpr int kMaxDevices = 64;
  static std::atomic<int> cached[kMaxDevices];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 0;
  int n = cached[dev].load(std::memory_order_relaxed);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n < 0) n = 0;
    cached[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}

// Work split of the direct-load kernels: 256-row workgroups (one per compute unit at a time) unless
// they would leave the device badly used; then 128-row workgroups, twice as many, each about a
// fifth less efficient. Under the causal mask the heaviest workgroup carries twice the average
// work, so a launch needs about four rounds of workgroups before the light ones fill the gaps;
// without a mask only the fill of the last round matters.
bool prefer_half_rows(int64_t Sq, int64_t Hq, int64_t B, bool causal) {
  const int64_t cus = compute_units_or_default();
  const int64_t wgs = ((Sq + 255) / 256) * Hq * B;
  if (causal) return wgs < 4 * cus;
  const int64_t rounds = (wgs + cus - 1) / cus;
  return wgs * 4 < rounds * cus * 3;  // less than 3/4 of the slots of its rounds
}

void begin_launch() { (void)hipGetLastError(); }

int check_launch(const char* what) {
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(PITH_ERR_LAUNCH, "%s: launch failed: %s", what, hipGetErrorString(e));
  return PITH_OK;
}
}  // namespace pith

extern "C" int pith_version(void) { return 100; /* 0.1.0 */ }

extern "C" const char* pith_last_error(void) { return pith::g_last_error; }

extern "C" const char* pith_error_name(int code) {
  switch (code) {
    case PITH_OK: return "PITH_OK";
    case PITH_ERR_NULL_POINTER: return "PITH_ERR_NULL_POINTER";
    case PITH_ERR_BAD_SHAPE: return "PITH_ERR_BAD_SHAPE";
    case PITH_ERR_BAD_DTYPE: return "PITH_ERR_BAD_DTYPE";
    case PITH_ERR_UNSUPPORTED: return "PITH_ERR_UNSUPPORTED";
    case PITH_ERR_MISALIGNED: return "PITH_ERR_MISALIGNED";
    case PITH_ERR_LAUNCH: return "PITH_ERR_LAUNCH";
    default: return "PITH_ERR_UNKNOWN";
  }
}

extern "C" int pith_device_info(int device, pith_device_info_t* info) {
  if (!info) return pith::fail(PITH_ERR_NULL_POINTER, "pith_device_info: info is NULL");
  hipDeviceProp_t prop;
  const hipError_t e = hipGetDeviceProperties(&prop, device);
  if (e != hipSuccess) return pith::fail(PITH_ERR_LAUNCH, "pith_device_info: device %d: %s", device, hipGetErrorString(e));
  std::memset(info, 0, sizeof(*info));
  std::strncpy(info->arch_name, prop.gcnArchName, sizeof(info->arch_name) - 1);
  info->compute_units = prop.multiProcessorCount;
  info->lds_bytes_per_workgroup = (int32_t)prop.sharedMemPerBlock;
  info->clock_khz = prop.clockRate;
  info->supported = std::strncmp(prop.gcnArchName, "gfx950", 6) == 0;
  info->hbm_bytes = (int64_t)prop.totalGlobalMem;
  return PITH_OK;
}
