#include "hostcopy.hpp"

#include <algorithm>
#include <condition_variable>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <thread>
#include <vector>

namespace nncv_hip {

namespace {

class CopyPool {
 public:
  static CopyPool& get() {
    static CopyPool* p = new CopyPool();  // never destroyed: its threads may outlive static destruction order
    return *p;
  }
  void run(char* dst, const char* src, size_t bytes) {
    const int parts = (int)workers_.size() + 1;
    if (parts == 1 || bytes < (size_t(256) << 10)) {
      memcpy(dst, src, bytes);
      return;
    }
    const size_t piece = ((bytes + parts - 1) / parts + 4095) & ~size_t(4095);
    {
      std::lock_guard<std::mutex> lk(mu_);
      dst_ = dst; src_ = src; bytes_ = bytes; piece_ = piece;
      pending_ = parts - 1;
      ++generation_;
    }
    wake_.notify_all();
    copy_part(0);
    std::unique_lock<std::mutex> lk(mu_);
    done_.wait(lk, [&] { return pending_ == 0; });
  }

 private:
  CopyPool() {
    const char* e = getenv("NNCV_HIP_COPY_THREADS");
    int n = e ? atoi(e) : 4;
    const int hw = (int)std::thread::hardware_concurrency();
    if (hw > 0) n = std::min(n, hw);
    n = std::max(1, std::min(n, 16));
    for (int i = 1; i < n; ++i) workers_.emplace_back([this, i] { loop(i); });
    for (auto& t : workers_) t.detach();
  }
  void copy_part(int i) {
    const size_t lo = std::min(bytes_, piece_ * (size_t)i), hi = std::min(bytes_, lo + piece_);
    if (hi > lo) memcpy(dst_ + lo, src_ + lo, hi - lo);
  }
  void loop(int i) {
    unsigned long long seen = 0;
    for (;;) {
      {
        std::unique_lock<std::mutex> lk(mu_);
        wake_.wait(lk, [&] { return generation_ != seen; });
        seen = generation_;
      }
      copy_part(i);
      {
        std::lock_guard<std::mutex> lk(mu_);
        --pending_;
      }
      done_.notify_one();
    }
  }
  std::vector<std::thread> workers_;
  std::mutex mu_;
  std::condition_variable wake_, done_;
  char* dst_ = nullptr;
  const char* src_ = nullptr;
  size_t bytes_ = 0, piece_ = 0;
  int pending_ = 0;
  unsigned long long generation_ = 0;
};

}  // namespace

void parallel_copy(void* dst, const void* src, size_t bytes) {
  CopyPool::get().run(static_cast<char*>(dst), static_cast<const char*>(src), bytes);
}

}  // namespace nncv_hip
