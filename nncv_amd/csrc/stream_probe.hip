// Which HIP streams of this process run their work side by side (nncv_hip_pick_streams).
//
// A process gets GPU_MAX_HW_QUEUES hardware queues (4 unless the environment says otherwise); streams beyond them share
// queues, the command processor serves queue q from pipe q mod 4, and the runtime does not deal streams to queues evenly.
// Measured on this chip with chains of 35 us kernels: two streams on one queue gain nothing over one stream, two queues
// on one pipe 1.14x, two pipes 1.99x, four pipes 3.95x.  Which queue a stream got cannot be asked, so it is measured:
// a chain of short single-workgroup kernels on a candidate next to the same chain on every stream already taken.
// The reference has no counterpart (its compiled forward is one synchronous CPU call, examples/Res18/main.cpp:95-99).
#include <chrono>
#include <vector>

#include "runtime.hpp"

namespace nncv_hip {

namespace {

// a bounded chain of dependent multiply-adds: `iters` steps of about four clocks each, one wave
__global__ __launch_bounds__(64) void probe_spin_kernel(int iters, float* sink) {
  float x = (float)threadIdx.x * 1e-3f;
  for (int i = 0; i < iters; ++i) x = __builtin_fmaf(x, 0.999f, 0.001f);
  if (x == 123456.0f) sink[threadIdx.x] = x;  // never true: keeps the loop
}

constexpr int kChain = 8;       // kernels per chain
constexpr int kSpin = 12000;    // about 25 us per kernel

void enqueue_chain(hipStream_t s, float* sink) {
  for (int k = 0; k < kChain; ++k) hipLaunchKernelGGL(probe_spin_kernel, dim3(1), dim3(64), 0, s, kSpin, sink);
  NNCV_HIP_CHECK(hipGetLastError());
}

// seconds for `reps` rounds of one chain on `a` (and one on `b` when given), all of them waited for
double cost(hipStream_t a, hipStream_t b, float* sink, int reps) {
  const auto t0 = std::chrono::steady_clock::now();
  for (int r = 0; r < reps; ++r) {
    enqueue_chain(a, sink);
    if (b) enqueue_chain(b, sink);
  }
  NNCV_HIP_CHECK(hipStreamSynchronize(a));
  if (b) NNCV_HIP_CHECK(hipStreamSynchronize(b));
  return std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count() / reps;
}

}  // namespace

// Streams (default priority, non-blocking, owned by the library until the process ends) of which the first `*found`
// overlap pairwise; the rest of the `want` fill the list up from the candidates that did not.
std::vector<hipStream_t> pick_streams(int want, int* found) {
  static std::vector<hipStream_t> taken, spare;
  static int n_overlapping = 0;
  static bool probed = false;
  if (!probed) {
    constexpr int kCandidates = 8;
    DeviceBuffer sink(64 * sizeof(float));
    std::vector<hipStream_t> cand(kCandidates);
    for (auto& s : cand) NNCV_HIP_CHECK(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    // clocks up, code object loaded
    const auto t0 = std::chrono::steady_clock::now();
    while (std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count() < 0.03) (void)cost(cand[0], nullptr, sink.as<float>(), 4);
    const double alone = cost(cand[0], nullptr, sink.as<float>(), 8);
    taken.push_back(cand[0]);
    for (int c = 1; c < kCandidates; ++c) {
      bool ok = true;
      for (hipStream_t t : taken)
        if (cost(t, cand[c], sink.as<float>(), 8) >= 1.5 * alone) {
          ok = false;
          break;
        }
      (ok ? taken : spare).push_back(cand[c]);
    }
    n_overlapping = (int)taken.size();
    probed = true;
  }
  std::vector<hipStream_t> out;
  for (hipStream_t s : taken)
    if ((int)out.size() < want) out.push_back(s);
  if (found) *found = (int)out.size() < n_overlapping ? (int)out.size() : n_overlapping;
  for (hipStream_t s : spare)
    if ((int)out.size() < want) out.push_back(s);
  return out;
}

}  // namespace nncv_hip
