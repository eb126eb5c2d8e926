// Table / index memory: where the bytes live and which address the GPU uses for them.
//
// Stands in for the reference's gear::memory classes (include/memory/*.h, src/memory/*.cc):
//   kHost    calloc                                     Memory        (memory.cc:36-50)
//   kShm     SysV shared memory, optionally pinned      SharedMemory  (shared_memory.cc:35-82)
//   kPinned  hipHostMalloc(mapped|portable), zero-copy  CudaUVMemory  (cuda_uvm.cc:10-54)
//   kDevice  hipMalloc, HBM resident                    CudaMemory    (cuda_memory.cc:6-28)
#pragma once
#include <sys/types.h>

#include <cstddef>
#include <cstdint>
#include <string>

namespace gearhost {

enum class Placement : int { kHost = 0, kPinned = 1, kShm = 2, kDevice = 3 };

const char *placement_name(Placement p);
// "host" | "pinned" | "shm" | "device" | "auto"; auto = pinned when a HIP device is visible,
// shm otherwise.  Throws std::runtime_error on anything else.
Placement parse_placement(const std::string &name);
bool hip_device_visible();

class MemoryBlock {
 public:
  MemoryBlock(size_t size, Placement placement, key_t key = 0, bool create = true);
  ~MemoryBlock();
  MemoryBlock(const MemoryBlock &) = delete;
  MemoryBlock &operator=(const MemoryBlock &) = delete;

  // Returns the size on success or when already allocated, -1 on failure (never throws for a
  // missing shared segment: callers poll, cf. shared_dataset.py:72-74).
  ssize_t alloc();
  ssize_t free();

  void *host() const { return host_; }      // CPU-visible address (nullptr for kDevice)
  void *device() const { return device_; }  // GPU-visible address (nullptr when the GPU cannot see it)
  void *any() const { return host_ ? host_ : device_; }
  size_t size() const { return size_; }
  Placement placement() const { return placement_; }
  key_t key() const { return key_; }
  bool create() const { return create_; }
  int shmid() const { return shmid_; }
  bool registered() const { return registered_; }
  std::string to_string() const;

  // memcpy that also works when this block lives in HBM
  void write(size_t offset, const void *src, size_t bytes);
  void read(size_t offset, void *dst, size_t bytes) const;

 private:
  size_t size_;
  Placement placement_;
  key_t key_;
  bool create_;
  int shmid_ = -1;
  bool registered_ = false;
  void *host_ = nullptr;
  void *device_ = nullptr;
};

}  // namespace gearhost
