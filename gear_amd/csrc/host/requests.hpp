// Pending priority updates and inference requests of the online path, host side
// (reference include/index/request.h, src/index/request.cc).
//
// WeightUpdateRequestArray keeps at most one pending (timestep, weight) per trajectory index:
// a later update of the same index replaces the earlier one, and the index keeps the position of
// its first appearance (request.cc:41-51).  continuous() packs the pending updates into dense
// arrays -- indices, then timesteps `capacity` entries further in the same int64 array, weights --
// and clears the pending set (request.cc:53-75).  The dense arrays are what the device scatter
// kernels consume; the staging arrays live in pinned memory so the GPU can read them in place.
#pragma once
#include <cstdint>
#include <memory>
#include <stdexcept>
#include <vector>

#include "memory.hpp"

namespace gearhost {

inline std::unique_ptr<MemoryBlock> staging_block(size_t bytes) {
  auto b = std::make_unique<MemoryBlock>(bytes ? bytes : 64,
                                         hip_device_visible() ? Placement::kPinned : Placement::kHost);
  if (b->alloc() < 0) throw std::runtime_error("cannot allocate request staging memory");
  return b;
}

struct InferenceRequestArray {
  size_t count = 0, capacity;
  std::unique_ptr<MemoryBlock> src_blk, idx_blk;
  int32_t *srcs;
  int64_t *idxs, *tss;
  explicit InferenceRequestArray(int64_t cap)
      : capacity((size_t)cap), src_blk(staging_block(capacity * 4)),
        idx_blk(staging_block(2 * capacity * 8)) {
    srcs = static_cast<int32_t *>(src_blk->host());
    idxs = static_cast<int64_t *>(idx_blk->host());
    tss = idxs + capacity;
  }
  void insert(size_t sim, int64_t index, int64_t timestep) {
    if (count >= capacity) throw std::runtime_error("inference request array is full");
    srcs[count] = (int32_t)sim;
    idxs[count] = index;
    tss[count] = timestep;
    ++count;
  }
  void clear() { count = 0; }
};

struct WeightUpdateRequestArray {
  size_t count = 0, capacity;
  std::vector<size_t> list;
  std::vector<uint8_t> updated;
  std::unique_ptr<MemoryBlock> ts_blk, w_blk;
  int64_t *timesteps;
  float *weights;
  explicit WeightUpdateRequestArray(int64_t cap)
      : capacity((size_t)cap), updated(capacity, 0), ts_blk(staging_block(capacity * 8)),
        w_blk(staging_block(capacity * 4)) {
    timesteps = static_cast<int64_t *>(ts_blk->host());
    weights = static_cast<float *>(w_blk->host());
  }
  void update(size_t index, int64_t timestep, float weight) {
    if (index >= capacity) throw std::out_of_range("trajectory index outside the request array");
    if (!updated[index]) {
      ++count;
      updated[index] = 1;
      list.push_back(index);
    }
    timesteps[index] = timestep;
    weights[index] = weight;
  }
  // idxs: int64[>= 2*capacity] (indices at [0,num), timesteps at [capacity, capacity+num)),
  // w: float[>= num].  Returns num.
  int64_t continuous(int64_t *idxs, int64_t idxs_size, float *w, int64_t w_size) {
    const int64_t num = (int64_t)count;
    if (idxs_size < (int64_t)capacity + num || idxs_size < 2 * num)
      throw std::runtime_error(
          "Index output array for continuous weight update array has less space than required");
    if (w_size < num)
      throw std::runtime_error(
          "Weights output array for continuous weight update array has less space than required");
    for (int64_t i = 0; i < num; ++i) {
      const size_t idx = list[(size_t)i];
      idxs[i] = (int64_t)idx;
      idxs[capacity + i] = timesteps[idx];
      w[i] = weights[idx];
      updated[idx] = 0;
    }
    count = 0;
    list.clear();
    return num;
  }
};

struct CachedRequest {
  size_t capacity;
  InferenceRequestArray iarr;
  WeightUpdateRequestArray warr;
  explicit CachedRequest(int64_t cap) : capacity((size_t)cap), iarr(cap), warr(cap) {}
};

}  // namespace gearhost
