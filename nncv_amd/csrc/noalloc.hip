// The scratch memory of the one entry point that allocates nothing (nncv_hip_conv_forward_noalloc): callers that
// cannot call hipMalloc -- code under HIP graph capture, serving loops, harnesses that forbid it -- still need the
// partial-sum workspace and the ticket counters of the K split that fp32 3x3 layers use
// (conv3x3_patch.hip, tile_reduce_store_splitk).  Here that workspace is a file-scope device array: each GPU the
// library runs on holds its own copy at its own address until the process ends.
//
// In host code the array's name is a stand-in, not a device address; the address on the current device comes
// from hipGetSymbolAddress, once per device, and everything else uses that pointer.
#include <mutex>

#include "runtime.hpp"

namespace nncv_hip {

namespace {

constexpr int kMaxDevices = 64;

static __device__ __align__(256) unsigned char scratch[kNoAllocScratchBytes];

std::mutex g_mu;
void* g_ptr[kMaxDevices] = {};

__global__ void clear_words_kernel(unsigned* p, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0u;
}

}  // namespace

void* noalloc_scratch() {
  int dev = -1;
  NNCV_HIP_CHECK(hipGetDevice(&dev));
  NNCV_REQUIRE(dev >= 0 && dev < kMaxDevices, "device index out of range");
  std::lock_guard<std::mutex> lk(g_mu);
  if (!g_ptr[dev]) {
    void* p = nullptr;
    NNCV_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    NNCV_REQUIRE(p != nullptr, "hipGetSymbolAddress returned no address for the scratch array");
    g_ptr[dev] = p;
  }
  return g_ptr[dev];
}

// A fill kernel, not hipMemsetAsync: a caller may be capturing the stream into a graph.
void launch_clear_words(void* p, int n_words, hipStream_t s) {
  hipLaunchKernelGGL(clear_words_kernel, dim3((n_words + 255) / 256), dim3(256), 0, s, static_cast<unsigned*>(p), n_words);
  NNCV_HIP_CHECK(hipGetLastError());
}

}  // namespace nncv_hip
