// Priority update weights[idx[j]] = values[j] with "last occurrence wins" for repeated indices.
//
// With unique indices this is one scatter.  Otherwise the (index, position) pairs go through the
// stable LSD radix sort on the index; inside each run of equal indices positions stay ascending,
// so the last element of a run is the last update of that index and it alone is written.
#include "radix_sort.hpp"

namespace gearhip {
namespace {

constexpr int kBlock = 256;

template <typename T>
__global__ __launch_bounds__(kBlock) void scatter_unique_kernel(T *__restrict__ w, int64_t n,
                                                                const int64_t *__restrict__ idx,
                                                                const T *__restrict__ v,
                                                                int64_t num) {
  const int64_t j = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (j >= num) return;
  const int64_t i = idx[j];
  if (i >= 0 && i < n) w[i] = v[j];
}

__global__ __launch_bounds__(kBlock) void scatter_prepare_kernel(const int64_t *__restrict__ idx,
                                                                 int64_t n, int64_t num,
                                                                 uint64_t *__restrict__ keys,
                                                                 uint32_t *__restrict__ pos) {
  const int64_t j = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (j >= num) return;
  const int64_t i = idx[j];
  keys[j] = (i >= 0 && i < n) ? (uint64_t)i : (uint64_t)n;  // n = "ignore", sorts last
  pos[j] = (uint32_t)j;
}

template <typename T>
__global__ __launch_bounds__(kBlock) void scatter_winners_kernel(T *__restrict__ w, int64_t n,
                                                                 const uint64_t *__restrict__ keys,
                                                                 const uint32_t *__restrict__ pos,
                                                                 const T *__restrict__ v,
                                                                 int64_t num) {
  const int64_t j = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (j >= num) return;
  const uint64_t key = keys[j];
  if (key >= (uint64_t)n) return;
  if (j + 1 < num && keys[j + 1] == key) return;  // a later update of the same index exists
  w[key] = v[pos[j]];
}

struct Layout {
  size_t kin, vin, kout, vout, ktmp, vtmp, hist, total;
};
Layout layout(int64_t num) {
  Layout l;
  const size_t m = num > 0 ? (size_t)num : 1;
  const size_t k8 = align_up(m * 8, 256), v4 = align_up(m * 4, 256);
  size_t o = 0;
  l.kin = o;  o += k8;
  l.kout = o; o += k8;
  l.ktmp = o; o += k8;
  l.vin = o;  o += v4;
  l.vout = o; o += v4;
  l.vtmp = o; o += v4;
  l.hist = o; o += radix::hist_bytes(num);
  l.total = o;
  return l;
}

}  // namespace
}  // namespace gearhip

using namespace gearhip;

extern "C" size_t gear_hip_scatter_workspace_bytes(int64_t num) { return layout(num).total; }

namespace {
template <typename T>
int scatter_any(T *weights, int64_t n, const int64_t *idx, const T *values, int64_t num,
                int unique_indices, void *workspace, size_t workspace_bytes, void *stream) {
  if (n < 0 || num < 0) return GEAR_HIP_EINVAL;
  if (num == 0 || n == 0) return 0;
  if (!weights || !idx || !values) return GEAR_HIP_EINVAL;
  if (num >= (1ll << 32)) return GEAR_HIP_ERANGE;
  hipStream_t st = as_stream(stream);
  const dim3 grid((unsigned)ceil_div64(num, kBlock)), block(kBlock);
  if (unique_indices) {
    scatter_unique_kernel<T><<<grid, block, 0, st>>>(weights, n, idx, values, num);
    GEARHIP_RETURN_IF_LAUNCH_FAILED();
    return 0;
  }
  const Layout l = layout(num);
  if (!workspace || workspace_bytes < l.total || (reinterpret_cast<uintptr_t>(workspace) & 7))
    return GEAR_HIP_EWORKSPACE;
  char *ws = static_cast<char *>(workspace);
  uint64_t *kin = reinterpret_cast<uint64_t *>(ws + l.kin);
  uint64_t *kout = reinterpret_cast<uint64_t *>(ws + l.kout);
  uint32_t *vin = reinterpret_cast<uint32_t *>(ws + l.vin);
  uint32_t *vout = reinterpret_cast<uint32_t *>(ws + l.vout);
  scatter_prepare_kernel<<<grid, block, 0, st>>>(idx, n, num, kin, vin);
  GEARHIP_RETURN_IF_LAUNCH_FAILED();
  int bits = 0;
  while (bits < 64 && ((uint64_t)n >> bits) != 0) ++bits;  // keys are in [0, n]
  int rc = radix::sort_pairs<uint64_t, uint32_t>(
      kin, kout, vin, vout, reinterpret_cast<uint64_t *>(ws + l.ktmp),
      reinterpret_cast<uint32_t *>(ws + l.vtmp), num, 0, bits,
      reinterpret_cast<uint32_t *>(ws + l.hist), st);
  if (rc) return rc;
  scatter_winners_kernel<T><<<grid, block, 0, st>>>(weights, n, kout, vout, values, num);
  GEARHIP_RETURN_IF_LAUNCH_FAILED();
  return 0;
}
}  // namespace

extern "C" int gear_hip_scatter_f32(float *weights, int64_t n, const int64_t *idx,
                                    const float *values, int64_t num, int unique_indices,
                                    void *workspace, size_t workspace_bytes, void *stream) {
  return scatter_any<float>(weights, n, idx, values, num, unique_indices, workspace,
                            workspace_bytes, stream);
}

extern "C" int gear_hip_scatter_i64(int64_t *table, int64_t n, const int64_t *idx,
                                    const int64_t *values, int64_t num, int unique_indices,
                                    void *workspace, size_t workspace_bytes, void *stream) {
  return scatter_any<int64_t>(table, n, idx, values, num, unique_indices, workspace,
                              workspace_bytes, stream);
}
