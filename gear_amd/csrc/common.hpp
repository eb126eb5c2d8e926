// Shared declarations for the HIP sources of libgearhip.so (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>

#include "gear_hip.h"

namespace gearhip {

constexpr int kWave = 64;  // CDNA4 wavefront width

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
// 16-byte vector that may start at any byte address.  gfx950 runs with unaligned global access
// enabled, so this still compiles to one global_load_dwordx4.
struct __attribute__((packed, aligned(1))) u32x4_any {
  u32x4 v;
};
typedef uint32_t u32x4_a1 __attribute__((ext_vector_type(4), aligned(1)));

inline hipStream_t as_stream(void *s) { return reinterpret_cast<hipStream_t>(s); }

// Tunables that can be overridden from the environment for experiments (read once).
int env_int(const char *name, int dflt);

#define GEARHIP_RETURN_IF_LAUNCH_FAILED()        \
  do {                                           \
    hipError_t e__ = hipGetLastError();          \
    if (e__ != hipSuccess) return (int)e__;      \
  } while (0)

#define GEARHIP_CHECK(expr)                      \
  do {                                           \
    hipError_t e__ = (expr);                     \
    if (e__ != hipSuccess) return (int)e__;      \
  } while (0)

__host__ __device__ inline int64_t ceil_div64(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Looks up, for the current device, the address of the static device array behind
// gear_hip_scan_f32_f64_static (scan.hip); called by gear_hip_set_device so that the lookup
// happens at set-up rather than inside the first hot-path call.
int scan_static_init();

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

}  // namespace gearhip
