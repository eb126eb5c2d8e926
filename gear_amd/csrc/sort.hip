// gear_hip_sort_i64: ascending stable sort of non-negative int64 keys with optional payload.
#include "radix_sort.hpp"

using namespace gearhip;

namespace {
struct SortWs {
  size_t ktmp, vtmp, hist, total;
};
SortWs sort_ws(int64_t num) {
  SortWs w;
  const size_t n = num > 0 ? (size_t)num : 1;
  w.ktmp = 0;
  w.vtmp = align_up(n * 8, 256);
  w.hist = w.vtmp + align_up(n * 8, 256);
  w.total = w.hist + radix::hist_bytes(num);
  return w;
}
}  // namespace

extern "C" size_t gear_hip_sort_workspace_bytes(int64_t num) { return sort_ws(num).total; }

extern "C" int gear_hip_sort_i64(const int64_t *keys_in, int64_t *keys_out, const int64_t *vals_in,
                                 int64_t *vals_out, int64_t num, int key_bits, void *workspace,
                                 size_t workspace_bytes, void *stream) {
  if (num < 0 || key_bits < 0 || key_bits > 64) return GEAR_HIP_EINVAL;
  if (num == 0) return 0;
  if (!keys_in || !keys_out || ((vals_in == nullptr) != (vals_out == nullptr)))
    return GEAR_HIP_EINVAL;
  if (keys_in == keys_out || (vals_in && vals_in == vals_out)) return GEAR_HIP_EINVAL;
  const SortWs w = sort_ws(num);
  if (!workspace || workspace_bytes < w.total || (reinterpret_cast<uintptr_t>(workspace) & 7))
    return GEAR_HIP_EWORKSPACE;
  char *ws = static_cast<char *>(workspace);
  return radix::sort_pairs<uint64_t, uint64_t>(
      reinterpret_cast<const uint64_t *>(keys_in), reinterpret_cast<uint64_t *>(keys_out),
      reinterpret_cast<const uint64_t *>(vals_in), reinterpret_cast<uint64_t *>(vals_out),
      reinterpret_cast<uint64_t *>(ws + w.ktmp), reinterpret_cast<uint64_t *>(ws + w.vtmp), num, 0,
      key_bits, reinterpret_cast<uint32_t *>(ws + w.hist), as_stream(stream));
}
