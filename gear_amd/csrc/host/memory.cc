#include "memory.hpp"

#include <sys/ipc.h>
#include <sys/shm.h>

#include <cerrno>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <sstream>
#include <stdexcept>

#include "gear_hip.h"

namespace gearhost {

const char *placement_name(Placement p) {
  switch (p) {
    case Placement::kHost: return "host";
    case Placement::kPinned: return "pinned";
    case Placement::kShm: return "shm";
    case Placement::kDevice: return "device";
  }
  return "?";
}

bool hip_device_visible() {
  int n = 0;
  return gear_hip_device_count(&n) == 0 && n > 0;
}

Placement parse_placement(const std::string &name) {
  if (name == "host") return Placement::kHost;
  if (name == "pinned" || name == "uvm") return Placement::kPinned;
  if (name == "shm" || name == "shared") return Placement::kShm;
  if (name == "device" || name == "hbm") return Placement::kDevice;
  if (name == "auto" || name.empty()) return hip_device_visible() ? Placement::kPinned : Placement::kShm;
  throw std::runtime_error("unknown table placement '" + name +
                           "' (expected auto, host, pinned, shm or device)");
}

MemoryBlock::MemoryBlock(size_t size, Placement placement, key_t key, bool create)
    : size_(size), placement_(placement), key_(key), create_(create) {}

MemoryBlock::~MemoryBlock() { this->free(); }

std::string MemoryBlock::to_string() const {
  std::stringstream ss;
  ss << "<GearMemory, addr: " << any() << ", size: " << size_
     << ", memory type: " << placement_name(placement_) << ">";
  return ss.str();
}

ssize_t MemoryBlock::alloc() {
  if (host_ != nullptr || device_ != nullptr) return (ssize_t)size_;
  if (size_ == 0) return -1;
  switch (placement_) {
    case Placement::kHost:
      host_ = calloc(size_, 1);
      return host_ ? (ssize_t)size_ : -1;
    case Placement::kPinned: {
      void *h = nullptr, *d = nullptr;
      int rc = gear_hip_host_alloc(size_, &h, &d);
      if (rc != 0) {
        fprintf(stderr, "gear: pinned allocation of %zu bytes failed: %s\n", size_,
                gear_hip_error_string(rc));
        return -1;
      }
      memset(h, 0, size_);
      host_ = h;
      device_ = d;
      return (ssize_t)size_;
    }
    case Placement::kDevice: {
      void *d = nullptr;
      int rc = gear_hip_device_alloc(size_, &d);
      if (rc != 0) {
        fprintf(stderr, "gear: device allocation of %zu bytes failed: %s\n", size_,
                gear_hip_error_string(rc));
        return -1;
      }
      device_ = d;
      return (ssize_t)size_;
    }
    case Placement::kShm: {
      // shared_memory.cc:40-57: creator uses IPC_CREAT|0777, clients attach with 0666
      shmid_ = create_ ? shmget(key_, size_, IPC_CREAT | 0777) : shmget(key_, size_, 0666);
      if (shmid_ == -1) return -1;
      void *p = shmat(shmid_, nullptr, 0);
      if (p == reinterpret_cast<void *>(-1)) {
        shmid_ = -1;
        return -1;
      }
      host_ = p;
      // Pinning an existing segment is what the reference does next (shared_memory.cc:59-61).
      // Some ROCm hosts refuse it, so it is only tried on request; without it the segment is a
      // CPU-side table and the gather entry points refuse it with a clear message.
      const char *want = getenv("GEAR_HIP_HOST_REGISTER");
      if (want && want[0] == '1') {
        void *d = nullptr;
        if (gear_hip_host_register(host_, size_, &d) == 0) {
          device_ = d;
          registered_ = true;
        }
      }
      return (ssize_t)size_;
    }
  }
  return -1;
}

ssize_t MemoryBlock::free() {
  if (host_ == nullptr && device_ == nullptr) return -1;
  switch (placement_) {
    case Placement::kHost: ::free(host_); break;
    case Placement::kPinned: gear_hip_host_free(host_); break;
    case Placement::kDevice: gear_hip_device_free(device_); break;
    case Placement::kShm:
      if (registered_) gear_hip_host_unregister(host_);
      shmdt(host_);
      if (create_ && shmid_ != -1) shmctl(shmid_, IPC_RMID, nullptr);  // shared_memory.cc:76-80
      break;
  }
  host_ = device_ = nullptr;
  registered_ = false;
  return (ssize_t)size_;
}

void MemoryBlock::write(size_t offset, const void *src, size_t bytes) {
  if (offset + bytes > size_) throw std::runtime_error("write past the end of a memory block");
  if (bytes == 0) return;
  if (host_) {
    memcpy(static_cast<char *>(host_) + offset, src, bytes);
  } else if (device_) {
    int rc = gear_hip_memcpy(static_cast<char *>(device_) + offset, src, bytes);
    if (rc) throw std::runtime_error(std::string("copy to device table failed: ") + gear_hip_error_string(rc));
  } else {
    throw std::runtime_error("memory block is not allocated");
  }
}

void MemoryBlock::read(size_t offset, void *dst, size_t bytes) const {
  if (offset + bytes > size_) throw std::runtime_error("read past the end of a memory block");
  if (bytes == 0) return;
  if (host_) {
    memcpy(dst, static_cast<const char *>(host_) + offset, bytes);
  } else if (device_) {
    int rc = gear_hip_memcpy(dst, static_cast<const char *>(device_) + offset, bytes);
    if (rc) throw std::runtime_error(std::string("copy from device table failed: ") + gear_hip_error_string(rc));
  } else {
    throw std::runtime_error("memory block is not allocated");
  }
}

}  // namespace gearhost
