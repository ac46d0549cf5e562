// Thin HIP runtime layer under the C ABI: device selection, one stream, owned device buffers,
// a grow-only bump arena for activations and transform workspaces, pinned staging buffers.
// The reference has no counterpart (its object runs in host memory); the only device code it
// contains are cudaMalloc/cudaFree wrappers (src/nncv/vm/cuda/vm_alloc_cuda.cu:6-10).
#pragma once
#include <memory>
#include <mutex>
#include <vector>

#include "common.hpp"

namespace nncv_hip {

class DeviceBuffer {
 public:
  DeviceBuffer() = default;
  explicit DeviceBuffer(size_t bytes) { reset(bytes); }
  DeviceBuffer(const DeviceBuffer&) = delete;
  DeviceBuffer& operator=(const DeviceBuffer&) = delete;
  DeviceBuffer(DeviceBuffer&& o) noexcept : p_(o.p_), n_(o.n_) { o.p_ = nullptr; o.n_ = 0; }
  DeviceBuffer& operator=(DeviceBuffer&& o) noexcept {
    if (this != &o) { release(); p_ = o.p_; n_ = o.n_; o.p_ = nullptr; o.n_ = 0; }
    return *this;
  }
  ~DeviceBuffer() { release(); }
  void reset(size_t bytes) {
    release();
    if (bytes) NNCV_HIP_CHECK(hipMalloc(&p_, bytes));
    n_ = bytes;
  }
  void release() {
    if (p_) (void)hipFree(p_);
    p_ = nullptr;
    n_ = 0;
  }
  void* get() const { return p_; }
  template <typename T> T* as() const { return static_cast<T*>(p_); }
  size_t bytes() const { return n_; }

 private:
  void* p_ = nullptr;
  size_t n_ = 0;
};

class PinnedBuffer {
 public:
  ~PinnedBuffer() { if (p_) (void)hipHostFree(p_); }
  void* ensure(size_t bytes) {
    if (bytes > n_) {
      if (p_) (void)hipHostFree(p_);
      p_ = nullptr;
      NNCV_HIP_CHECK(hipHostMalloc(&p_, bytes, hipHostMallocDefault));
      n_ = bytes;
    }
    return p_;
  }

 private:
  void* p_ = nullptr;
  size_t n_ = 0;
};

// Bump allocator over one device allocation.  `plan` first (no memory touched), then `reserve`
// grows the backing store if the plan does not fit; pointers are handed out 256-byte aligned.
class Arena {
 public:
  // true when the backing store was replaced (pointers handed out before are gone)
  bool reserve(size_t bytes, hipStream_t s) {
    bool grown = false;
    if (bytes > buf_.bytes()) {
      NNCV_HIP_CHECK(hipStreamSynchronize(s));  // nobody may still be using the old block
      buf_.reset(bytes + bytes / 8);
      grown = true;
    }
    off_ = 0;
    return grown;
  }
  void* take(size_t bytes) {
    const size_t a = (off_ + 255) & ~size_t(255);
    NNCV_REQUIRE(a + bytes <= buf_.bytes(), "arena overflow: workspace plan and use disagree");
    off_ = a + bytes;
    return static_cast<char*>(buf_.get()) + a;
  }
  size_t capacity() const { return buf_.bytes(); }

 private:
  DeviceBuffer buf_;
  size_t off_ = 0;
};

inline size_t align256(size_t b) { return (b + 255) & ~size_t(255); }

// The device array behind nncv_hip_conv_forward_noalloc (noalloc.hip): 1 KiB of ticket counters, then the
// workspace.  noalloc_scratch() is its address on the current device (resolved once per device).
constexpr size_t kNoAllocCounterBytes = 1024;
constexpr size_t kNoAllocWorkspaceBytes = size_t(4) << 20;
constexpr size_t kNoAllocScratchBytes = kNoAllocCounterBytes + kNoAllocWorkspaceBytes;
void* noalloc_scratch();
void launch_clear_words(void* p, int n_words, hipStream_t s);

// stream_probe.hip: up to `want` library-owned streams, the first *found of which were measured to overlap pairwise
std::vector<hipStream_t> pick_streams(int want, int* found);

// Process-wide state.  All public entry points serialise on `mu`.
class Context {
 public:
  static Context& get();
  void init(int device);  // idempotent; device < 0 keeps the current one
  hipStream_t stream() const { return stream_; }
  int device() const { return device_; }
  const std::string& arch() const { return arch_; }
  Arena arena;
  PinnedBuffer pin_in, pin_out;
  std::recursive_mutex mu;
  // Cross-stream ordering of consecutive calls (they share the arena): see Sync in capi.cpp.
  void order_after_previous(hipStream_t s);
  void note_stream(hipStream_t s, bool pending);

 private:
  bool ready_ = false;
  int device_ = -1;
  hipStream_t stream_ = nullptr;
  hipStream_t tail_stream_ = nullptr;  // stream of the previous call; tail_pending_: it was left with work in flight
  hipEvent_t tail_event_ = nullptr;
  bool tail_pending_ = false;
  std::string arch_;
};

}  // namespace nncv_hip
