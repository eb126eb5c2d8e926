// Per-shard index arrays: trajectory lengths ("timesteps", int64) and priorities ("weights",
// fp32) in one block; weights start at the next multiple of 128 bytes after the timesteps
// (reference include/index/set.h:20-29,35-69).  The block is pinned host memory (or a SysV
// segment when shared), so the CPU writes priorities in place and the GPU can read them.
#pragma once
#include <chrono>
#include <cstring>
#include <memory>
#include <stdexcept>
#include <thread>
#include <vector>

#include "memory.hpp"

namespace gearhost {

inline size_t round_up_128(size_t bytes) { return (bytes + 127) / 128 * 128; }

// Serialised form: timesteps int64[n] immediately followed by weights fp32[n]
// (set.h:153-165, index/pybind.cc:15-50).
struct IndexsetState {
  size_t global_capacity, local_capacity, index_offset;
  std::vector<uint8_t> bytes;
  IndexsetState(size_t g, size_t l, size_t o, const int64_t *ts, const float *w)
      : global_capacity(g), local_capacity(l), index_offset(o), bytes(l * 12) {
    if (l) {
      std::memcpy(bytes.data(), ts, l * 8);
      std::memcpy(bytes.data() + l * 8, w, l * 4);
    }
  }
  const int64_t *timesteps() const { return reinterpret_cast<const int64_t *>(bytes.data()); }
  const float *weights() const {
    return reinterpret_cast<const float *>(bytes.data() + local_capacity * 8);
  }
};

class Indexset {
 public:
  Indexset(size_t global_capacity, size_t local_capacity, size_t index_offset, bool shared = false,
           key_t key = 0, bool create = false)
      : global_(global_capacity), local_(local_capacity), offset_(index_offset), shared_(shared) {
    const size_t bytes = round_up_128(local_ * 8) + round_up_128(local_ * 4);
    Placement p = shared ? Placement::kShm
                         : (hip_device_visible() ? Placement::kPinned : Placement::kHost);
    block_ = std::make_unique<MemoryBlock>(bytes ? bytes : 128, p, key, create);
    // a client may start before the creator: poll like set.h:53-62 (at most 1000 x 100 ms)
    int tries = 0;
    while (block_->alloc() < 0 && tries < (shared && !create ? 1000 : 1)) {
      std::this_thread::sleep_for(std::chrono::milliseconds(100));
      ++tries;
    }
    if (block_->host() == nullptr) throw std::runtime_error("Error allocate status table memory!");
  }
  Indexset(const IndexsetState &s, bool shared = false, key_t key = 0, bool create = false)
      : Indexset(s.global_capacity, s.local_capacity, s.index_offset, shared, key, create) {
    if (local_) {
      std::memcpy(timesteps(), s.timesteps(), local_ * 8);
      std::memcpy(weights(), s.weights(), local_ * 4);
    }
  }
  int64_t *timesteps() { return static_cast<int64_t *>(block_->host()); }
  float *weights() {
    return reinterpret_cast<float *>(static_cast<char *>(block_->host()) + round_up_128(local_ * 8));
  }
  // GPU-visible aliases (nullptr when the block is plain host memory)
  const float *device_weights() const {
    return block_->device() ? reinterpret_cast<const float *>(static_cast<char *>(block_->device()) +
                                                              round_up_128(local_ * 8))
                            : nullptr;
  }
  size_t global_capacity() const { return global_; }
  size_t local_capacity() const { return local_; }
  size_t index_offset() const { return offset_; }
  bool is_sharing() const { return shared_; }
  key_t shm_key() const { return block_->key(); }
  IndexsetState get_state() { return IndexsetState(global_, local_, offset_, timesteps(), weights()); }
  void set_timestep(size_t i, int64_t ts) { check(i); timesteps()[i] = ts; }
  void set_weight(size_t i, float w) { check(i); weights()[i] = w; }

 private:
  void check(size_t i) const {
    if (i >= local_) throw std::out_of_range("index outside the local shard");
  }
  size_t global_, local_, offset_;
  bool shared_;
  std::unique_ptr<MemoryBlock> block_;
};

}  // namespace gearhost
