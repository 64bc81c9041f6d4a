// Caller-provided device memory as a sized, non-owning view (reference
// src/matrix_ops/workspace.h).  All sizes are kept in bytes; size<T>() converts.
#pragma once
#include <gpu-api.h>

#include <cstddef>
#include <stdexcept>

namespace rtat {

class Workspace {
 public:
  Workspace() = default;
  template <typename T>
  Workspace(T* base, size_t count) : bytes(count * sizeof(T)), base((char*)base) {}
  virtual ~Workspace() = default;

  // Sub-view of `other`: `offset` and `count` are BYTES (reference workspace.h:24-30, where
  // an overflow prints and terminates; here it throws).
  Workspace(Workspace& other, size_t offset, size_t count)
      : bytes(count), base(other.base + offset) {
    if (offset + count > other.bytes) throw std::out_of_range("Workspace sub-view exceeds parent");
  }

  // Split `n` elements of T off the front and keep the rest (reference workspace.h:32-40).
  template <typename T>
  Workspace peel(size_t n) {
    const size_t take = n * sizeof(T);
    if (take > bytes) throw std::out_of_range("Workspace::peel beyond the end");
    Workspace front(base, take);
    base += take;
    bytes -= take;
    return front;
  }

  template <typename T>
  operator T*() const { return (T*)base; }

  template <typename T>
  size_t size() const { return bytes / sizeof(T); }

 protected:
  size_t bytes = 0;
  char* base = nullptr;
};

// Owns one device allocation (reference workspace.h:49-66).
class ManagedWorkspace : public Workspace {
 public:
  explicit ManagedWorkspace(size_t nbytes) { allocate(nbytes); }
  ~ManagedWorkspace() override { release(); }
  ManagedWorkspace(const ManagedWorkspace&) = delete;
  ManagedWorkspace& operator=(const ManagedWorkspace&) = delete;

  // Re-allocate (contents are NOT kept) when fewer than `count` elements of T fit.  Waits
  // for the device first: queued work may still be using the old block.
  template <typename T>
  void grow_to_fit(size_t count) {
    if (size<T>() >= count) return;
    gpuAssert(gpu::DeviceSynchronize());
    release();
    allocate(count * sizeof(T));
  }

 private:
  void allocate(size_t nbytes) {
    base = nullptr;
    bytes = 0;
    if (nbytes == 0) return;
    if (gpu::Malloc(&base, nbytes) != gpu::Success) throw std::bad_alloc();
    bytes = nbytes;
  }
  void release() {
    if (base) gpuAssert(gpu::Free(base));
    base = nullptr;
    bytes = 0;
  }
};

}  // namespace rtat
