// Device selection, error text and table-memory helpers of libgearhip.so.
#include <string.h>

#include "common.hpp"

namespace gearhip {

int env_int(const char *name, int dflt) {
  const char *v = getenv(name);
  if (v == nullptr || *v == '\0') return dflt;
  char *end = nullptr;
  long x = strtol(v, &end, 10);
  if (end == v) return dflt;
  return (int)x;
}

}  // namespace gearhip

using namespace gearhip;

extern "C" int gear_hip_abi_version(void) { return GEAR_HIP_ABI_VERSION; }

extern "C" int gear_hip_set_device(int device_id) {
  if (device_id < 0) return GEAR_HIP_EINVAL;
  int current = -1;
  GEARHIP_CHECK(hipGetDevice(&current));
  if (current != device_id) GEARHIP_CHECK(hipSetDevice(device_id));
  // Warm-up of the allocation-free prefix sum (address of its static array, its ordering event):
  // best effort -- a failure here must not fail device selection for callers that never use
  // that entry point, which reports the error itself when it is called.
  if (scan_static_init() != 0) (void)hipGetLastError();
  return 0;
}

extern "C" int gear_hip_device_count(int *count) {
  if (count == nullptr) return GEAR_HIP_EINVAL;
  *count = 0;
  hipError_t e = hipGetDeviceCount(count);
  if (e == hipErrorNoDevice) {
    *count = 0;
    return 0;
  }
  return (int)e;
}

extern "C" const char *gear_hip_error_string(int code) {
  switch (code) {
    case 0: return "success";
    case GEAR_HIP_EINVAL: return "gear_hip: invalid argument";
    case GEAR_HIP_EWORKSPACE: return "gear_hip: workspace missing or too small";
    case GEAR_HIP_ERANGE: return "gear_hip: size out of the supported range";
    case GEAR_HIP_EALIGN: return "gear_hip: pointer is not sufficiently aligned";
    case GEAR_HIP_ENOTREADY: return "gear_hip: set-up for this call has not run and cannot run now";
    default: break;
  }
  if (code > 0) return hipGetErrorString((hipError_t)code);
  return "gear_hip: unknown error code";
}

extern "C" int gear_hip_host_alloc(size_t bytes, void **host_ptr, void **dev_ptr) {
  if (host_ptr == nullptr) return GEAR_HIP_EINVAL;
  *host_ptr = nullptr;
  if (dev_ptr) *dev_ptr = nullptr;
  if (bytes == 0) return GEAR_HIP_EINVAL;
  void *h = nullptr;
  GEARHIP_CHECK(hipHostMalloc(&h, bytes, hipHostMallocMapped | hipHostMallocPortable));
  void *d = nullptr;
  hipError_t e = hipHostGetDevicePointer(&d, h, 0);
  if (e != hipSuccess) {
    (void)hipHostFree(h);
    return (int)e;
  }
  *host_ptr = h;
  if (dev_ptr) *dev_ptr = d;
  return 0;
}

extern "C" int gear_hip_host_free(void *host_ptr) {
  if (host_ptr == nullptr) return GEAR_HIP_EINVAL;
  GEARHIP_CHECK(hipHostFree(host_ptr));
  return 0;
}

extern "C" int gear_hip_device_alloc(size_t bytes, void **dev_ptr) {
  if (dev_ptr == nullptr || bytes == 0) return GEAR_HIP_EINVAL;
  *dev_ptr = nullptr;
  GEARHIP_CHECK(hipMalloc(dev_ptr, bytes));
  return 0;
}

extern "C" int gear_hip_device_free(void *dev_ptr) {
  if (dev_ptr == nullptr) return GEAR_HIP_EINVAL;
  GEARHIP_CHECK(hipFree(dev_ptr));
  return 0;
}

extern "C" int gear_hip_memcpy(void *dst, const void *src, size_t bytes) {
  if (bytes == 0) return 0;
  if (dst == nullptr || src == nullptr) return GEAR_HIP_EINVAL;
  GEARHIP_CHECK(hipMemcpy(dst, src, bytes, hipMemcpyDefault));
  return 0;
}

extern "C" int gear_hip_host_register(void *host_ptr, size_t bytes, void **dev_ptr) {
  if (host_ptr == nullptr || bytes == 0) return GEAR_HIP_EINVAL;
  if (dev_ptr) *dev_ptr = nullptr;
  hipError_t e = hipHostRegister(host_ptr, bytes, hipHostRegisterMapped | hipHostRegisterPortable);
  if (e != hipSuccess) {
    (void)hipGetLastError();  // do not leave the refusal behind for the next call to report
    return (int)e;
  }
  void *d = nullptr;
  e = hipHostGetDevicePointer(&d, host_ptr, 0);
  if (e != hipSuccess) {
    (void)hipHostUnregister(host_ptr);
    (void)hipGetLastError();
    return (int)e;
  }
  if (dev_ptr) *dev_ptr = d;
  return 0;
}

extern "C" int gear_hip_host_unregister(void *host_ptr) {
  if (host_ptr == nullptr) return GEAR_HIP_EINVAL;
  GEARHIP_CHECK(hipHostUnregister(host_ptr));
  return 0;
}
