// extern "C" surface of libnncv_hip.so (declared in include/nncv_hip.h).
#include <cstring>
#include <functional>
#include <memory>
#include <mutex>
#include <vector>

#include "../../include/nncv_hip.h"
#include "arena_plan.hpp"
#include "graph.hpp"
#include "hostcopy.hpp"
#include "model.hpp"

using namespace nncv_hip;

namespace nncv_hip {

Context& Context::get() {
  static Context c;
  return c;
}

void Context::init(int device) {
  if (ready_ && (device < 0 || device == device_)) return;
  int count = 0;
  NNCV_HIP_CHECK(hipGetDeviceCount(&count));
  NNCV_REQUIRE(count > 0, "no HIP device visible");
  if (device < 0) NNCV_HIP_CHECK(hipGetDevice(&device));
  NNCV_REQUIRE(device < count, "device index out of range");
  NNCV_REQUIRE(!ready_ || device == device_, "nncv_hip is already initialised on another device");
  NNCV_HIP_CHECK(hipSetDevice(device));
  hipDeviceProp_t prop;
  NNCV_HIP_CHECK(hipGetDeviceProperties(&prop, device));
  arch_ = prop.gcnArchName;
  // the code objects in this library exist for gfx950 only; anything else cannot run them
  NNCV_REQUIRE(arch_.rfind("gfx950", 0) == 0, "this library is built for gfx950 (MI355X); found " + arch_);
  NNCV_HIP_CHECK(hipStreamCreate(&stream_));  // default priority
  NNCV_HIP_CHECK(hipEventCreateWithFlags(&tail_event_, hipEventDisableTiming));
  device_ = device;
  ready_ = true;
  (void)noalloc_scratch();  // the scratch array's address on this device, resolved with the device current
}

// The event is recorded by the call that leaves work pending, on its own (then certainly live) stream; a later call on
// another stream only waits for the event, so a caller stream destroyed in between is never touched again.
void Context::order_after_previous(hipStream_t s) {
  if (!tail_pending_ || tail_stream_ == s) return;
  NNCV_HIP_CHECK(hipStreamWaitEvent(s, tail_event_, 0));
  tail_pending_ = false;
}

void Context::note_stream(hipStream_t s, bool pending) {
  tail_stream_ = s;
  tail_pending_ = pending;
  if (pending) NNCV_HIP_CHECK(hipEventRecord(tail_event_, s));
}

}  // namespace nncv_hip

namespace {

thread_local std::string g_last_error;

// int-returning entry points: 0 / -1 + message.
int guarded(const std::function<void()>& fn) {
  try {
    std::lock_guard<std::recursive_mutex> lk(Context::get().mu);
    fn();
    return 0;
  } catch (const std::exception& e) {
    g_last_error = e.what();
    return -1;
  }
}

// void entry points of the reference ABI: report like the reference does, then abort.
void guarded_abort(const char* what, const std::function<void()>& fn) {
  try {
    std::lock_guard<std::recursive_mutex> lk(Context::get().mu);
    fn();
  } catch (const std::exception& e) {
    fprintf(stderr, "[ Erro ] %s: %s\n", what, e.what());
    fflush(stderr);
    abort();
  }
}

// NULL stream -> library stream + synchronise on exit.  Workspace (one arena), split-K tickets and the
// pinned staging buffers are shared by every call, and the mutex only serialises the enqueueing: work
// left pending on one caller stream must not overlap work enqueued next on another.  So a call that
// arrives on a different stream than the previous one first makes its stream wait for everything the
// previous stream was given (an event recorded there now: the mutex is held, so that is exactly the
// earlier calls' work).  Calls that stay on one stream pay nothing.
// A caller stream that is being captured into a HIP graph takes neither the wait nor the event: both would reach
// outside the capture and end it.  The captured launches then run whenever the caller's graph does, and ordering
// them against other users of the library's shared workspace is the caller's business, as for the graph itself.
bool stream_is_capturing(hipStream_t s) {
  hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(s, &st) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  return st == hipStreamCaptureStatusActive;
}

struct Sync {
  hipStream_t s;
  bool own;
  bool capturing;
  explicit Sync(void* user) : s(user ? static_cast<hipStream_t>(user) : Context::get().stream()), own(user == nullptr) {
    capturing = !own && stream_is_capturing(s);
    if (!capturing) Context::get().order_after_previous(s);
  }
  bool done = false;
  void finish() {
    if (own) NNCV_HIP_CHECK(hipStreamSynchronize(s));
    if (!capturing) Context::get().note_stream(s, /*pending=*/!own);
    done = true;
  }
  ~Sync() {  // left early by an exception: whatever was enqueued may still be running
    if (!done && !capturing) {
      try {
        Context::get().note_stream(s, true);
      } catch (...) {
      }
    }
  }
};

// A network handle (nncv_hip_resnet18 / nncv_hip_graph) owns its workspace, so passes of DIFFERENT handles on
// different streams run concurrently: two passes in flight fill each other's launch gaps, prologues and tails
// (ResNet-18 at batch 32: 0.18-0.19 ms per pass against 0.24 one after the other).  Calls on ONE handle share that
// workspace (and the K-split tickets of its layers), so a call that arrives on another stream than the handle's
// previous one first makes its stream wait for that one, as Sync does for the library-wide arena.
struct HandleState {
  Arena arena;
  hipStream_t tail = nullptr;
  bool pending = false;
  hipEvent_t ev = nullptr;
  ~HandleState() {
    if (ev) (void)hipEventDestroy(ev);
  }
};

struct HandleSync {
  HandleState& h;
  hipStream_t s;
  bool own;
  bool done = false;
  HandleSync(HandleState& hs, void* user) : h(hs), s(user ? static_cast<hipStream_t>(user) : Context::get().stream()), own(user == nullptr) {
    // the event was recorded when the previous call ended, on its stream: that stream is not touched again here
    if (h.pending && h.tail != s) {
      NNCV_HIP_CHECK(hipStreamWaitEvent(s, h.ev, 0));
      h.pending = false;
    }
  }
  void leave(bool pending) {
    h.tail = s;
    h.pending = pending;
    if (pending) {
      if (!h.ev) NNCV_HIP_CHECK(hipEventCreateWithFlags(&h.ev, hipEventDisableTiming));
      NNCV_HIP_CHECK(hipEventRecord(h.ev, s));
    }
  }
  void finish() {
    if (own) NNCV_HIP_CHECK(hipStreamSynchronize(s));
    leave(!own);
    done = true;
  }
  ~HandleSync() {  // left early by an exception: whatever was enqueued may still be running
    if (!done) {
      try {
        leave(true);
      } catch (...) {
      }
    }
  }
};

// ---- host memref helpers ----------------------------------------------------------------
template <int R>
bool contiguous(const intptr_t* sizes, const intptr_t* strides) {
  intptr_t expect = 1;
  for (int i = R - 1; i >= 0; --i) {
    if (sizes[i] != 1 && strides[i] != expect) return false;
    expect *= sizes[i];
  }
  return true;
}

// copy a strided rank-R host tensor of `es`-byte elements to/from a dense buffer
template <int R>
void strided_copy(char* base, intptr_t offset, const intptr_t* sizes, const intptr_t* strides, size_t es, char* dense,
                  bool to_dense) {
  intptr_t idx[R] = {0};
  long long total = 1;
  for (int i = 0; i < R; ++i) total *= sizes[i];
  for (long long lin = 0; lin < total; ++lin) {
    intptr_t off = offset;
    for (int i = 0; i < R; ++i) off += idx[i] * strides[i];
    if (to_dense) memcpy(dense + lin * es, base + off * es, es);
    else memcpy(base + off * es, dense + lin * es, es);
    for (int i = R - 1; i >= 0; --i) {
      if (++idx[i] < sizes[i]) break;
      idx[i] = 0;
    }
  }
}

// upload a host memref to `dev` (dense, row-major)
template <int R>
void upload(const void* aligned, intptr_t offset, const intptr_t* sizes, const intptr_t* strides, size_t es, void* dev,
            PinnedBuffer& pin, hipStream_t s) {
  long long total = 1;
  for (int i = 0; i < R; ++i) total *= sizes[i];
  char* base = static_cast<char*>(const_cast<void*>(aligned));
  if (contiguous<R>(sizes, strides)) {
    NNCV_HIP_CHECK(hipMemcpyAsync(dev, base + offset * es, total * es, hipMemcpyHostToDevice, s));
  } else {
    char* p = static_cast<char*>(pin.ensure(total * es));
    strided_copy<R>(base, offset, sizes, strides, es, p, true);
    NNCV_HIP_CHECK(hipMemcpyAsync(dev, p, total * es, hipMemcpyHostToDevice, s));
  }
  NNCV_HIP_CHECK(hipStreamSynchronize(s));  // the pinned buffer / caller memory may be reused at once
}

template <int R>
void download(void* aligned, intptr_t offset, const intptr_t* sizes, const intptr_t* strides, size_t es, const void* dev,
              PinnedBuffer& pin, hipStream_t s) {
  long long total = 1;
  for (int i = 0; i < R; ++i) total *= sizes[i];
  char* base = static_cast<char*>(aligned);
  if (contiguous<R>(sizes, strides)) {
    NNCV_HIP_CHECK(hipMemcpyAsync(base + offset * es, dev, total * es, hipMemcpyDeviceToHost, s));
    NNCV_HIP_CHECK(hipStreamSynchronize(s));
  } else {
    char* p = static_cast<char*>(pin.ensure(total * es));
    NNCV_HIP_CHECK(hipMemcpyAsync(p, dev, total * es, hipMemcpyDeviceToHost, s));
    NNCV_HIP_CHECK(hipStreamSynchronize(s));
    strided_copy<R>(base, offset, sizes, strides, es, p, false);
  }
}

// ---- model cache for the handle-less reference ABI ---------------------------------------
struct CachedModel {
  const void* host_ptr;
  long long n;
  int dt;
  uint64_t fingerprint;
  std::unique_ptr<ResNet18> model;
};
std::vector<CachedModel>& model_cache() {
  static std::vector<CachedModel> c;
  return c;
}

void drop_graphs_of(const void* m);

// cheap change detector for a parameter blob that lives at the same address: 4096 strided samples.  A caller written
// against the reference (whose compiled forward re-reads the blob on every call) and rewriting parameters in place
// between the samples would go unnoticed: NNCV_HIP_PARAMS_HASH=full hashes every byte instead (about 5 ms per call
// for ResNet-18's 47 MB).
uint64_t fingerprint(const void* p, long long n, size_t es) {
  NNCV_REQUIRE(p && n > 0, "params: empty memref");
  const unsigned char* b = static_cast<const unsigned char*>(p);
  uint64_t h = 1469598103934665603ull ^ (uint64_t)n;
  static const bool full = [] {
    const char* e = getenv("NNCV_HIP_PARAMS_HASH");
    return e && !strcmp(e, "full");
  }();
  if (full) {
    const size_t bytes = (size_t)n * es, words = bytes / 8;
    uint64_t h2 = 0x9e3779b97f4a7c15ull;
    for (size_t i = 0; i + 1 < words; i += 2) {  // two independent chains: the multiplies overlap
      uint64_t a, c;
      memcpy(&a, b + i * 8, 8);
      memcpy(&c, b + i * 8 + 8, 8);
      h = (h ^ a) * 1099511628211ull;
      h2 = (h2 ^ c) * 0x100000001b3ull + 0x632be59bd9b4e019ull;
    }
    for (size_t k = (words & ~size_t(1)) * 8; k < bytes; ++k) h = (h ^ b[k]) * 1099511628211ull;
    return h ^ (h2 * 0xff51afd7ed558ccdull);
  }
  const long long step = std::max<long long>(1, n / 4096);
  for (long long i = 0; i < n; i += step)
    for (size_t k = 0; k < es; ++k) h = (h ^ b[i * es + k]) * 1099511628211ull;
  for (size_t k = 0; k < es; ++k) h = (h ^ b[(n - 1) * es + k]) * 1099511628211ull;
  return h;
}

std::unique_ptr<ResNet18> build_model(const void* host, long long n, int dt, int algo, hipStream_t s) {
  DeviceBuffer blob((size_t)n * dtype_size(dt));
  NNCV_HIP_CHECK(hipMemcpyAsync(blob.get(), host, blob.bytes(), hipMemcpyHostToDevice, s));
  auto m = std::make_unique<ResNet18>(blob.get(), n, dt, algo, s);
  NNCV_HIP_CHECK(hipStreamSynchronize(s));  // the staging blob dies here
  return m;
}

ResNet18& cached_model(const void* host, long long n, int dt, hipStream_t s) {
  const uint64_t fp = fingerprint(host, n, dtype_size(dt));
  auto& cache = model_cache();
  for (auto& e : cache)
    if (e.host_ptr == host && e.n == n && e.dt == dt) {
      if (e.fingerprint != fp) {  // same address, new contents: rebuild
        e.model.reset();
        e.model = build_model(host, n, dt, kAlgoAuto, s);
        e.fingerprint = fp;
      }
      return *e.model;
    }
  if (cache.size() >= 4) cache.erase(cache.begin());
  cache.push_back(CachedModel{host, n, dt, fp, build_model(host, n, dt, kAlgoAuto, s)});
  return *cache.back().model;
}

// ---- HIP-graph replay of the forward pass --------------------------------------------------
// A forward pass is 18-73 kernel launches on one stream with fixed arguments for a given (model,
// input pointer, output pointer, shape, workspace).  The second call with the same combination captures
// the launches into a graph and every later call replays it: one submission instead of 18-73.  That is
// what batch-1 latency is made of (MobileNetV3 at batch 1: 0.308 ms against 0.323), and it is what lets
// the host keep two passes in flight on two streams (ResNet-18 at batch 32: 0.184 ms per pass replayed
// against 0.196 with plain launches; MobileNetV3 at batch 32: 0.269 against 0.326).  With one pass at a
// time and a large batch a replay costs about 4 us that queued plain launches do not (0.264 against
// 0.260 ms): NNCV_HIP_GRAPH=size replays only launch-bound passes (up to two / four 224x224 images),
// NNCV_HIP_GRAPH=0 none.  The pass contains no memset nodes; the event profiler bypasses replay.
struct GraphEntry {
  const void* m;  // the handle (its HandleState) the pass was captured for: clones of one model capture their own
  const void* src;
  const float* logits;
  int N, H, W;
  void* ws;
  hipStream_t s;
  hipGraph_t graph;
  hipGraphExec_t exec;
};
std::vector<GraphEntry>& graph_cache() {
  static std::vector<GraphEntry> c;
  return c;
}
void drop_graph(GraphEntry& e) {
  if (e.exec) (void)hipGraphExecDestroy(e.exec);
  if (e.graph) (void)hipGraphDestroy(e.graph);
  e.exec = nullptr;
  e.graph = nullptr;
}
void drop_graphs_of(const void* m) {
  auto& c = graph_cache();
  for (size_t i = 0; i < c.size();) {
    if (c[i].m == m) {
      drop_graph(c[i]);
      c.erase(c.begin() + i);
    } else {
      ++i;
    }
  }
}

// `run` enqueues the whole pass on `s`; `owner` identifies the handle it belongs to.
void replay(const void* owner, const std::function<void()>& run, const void* src, int N, int H, int W, const float* logits, void* ws,
            hipStream_t s, bool launch_bound) {
  static const int mode = [] {  // -1 by size, 0 never, 1 always (the default)
    const char* e = getenv("NNCV_HIP_GRAPH");
    return !e ? 1 : (!strcmp(e, "size") ? -1 : (atoi(e) != 0 ? 1 : 0));
  }();
  const bool use = mode == 1 || (mode == -1 && launch_bound);
  if (!use || profiler_enabled()) {
    run();
    return;
  }
  auto& cache = graph_cache();
  GraphEntry* hit = nullptr;
  for (auto& e : cache)
    if (e.m == owner && e.src == src && e.logits == logits && e.N == N && e.H == H && e.W == W && e.ws == ws && e.s == s) hit = &e;
  if (!hit) {  // first sighting: run eagerly (this also performs every one-time kernel attribute set-up)
    if (cache.size() >= 32) {
      // the oldest entry goes; its last replay may still be running on another stream
      (void)hipDeviceSynchronize();
      drop_graph(cache.front());
      cache.erase(cache.begin());
    }
    cache.push_back(GraphEntry{owner, src, logits, N, H, W, ws, s, nullptr, nullptr});
    run();
    return;
  }
  if (!hit->exec) {  // second sighting: capture
    NNCV_HIP_CHECK(hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal));
    try {
      run();
    } catch (...) {
      hipGraph_t g = nullptr;
      (void)hipStreamEndCapture(s, &g);
      if (g) (void)hipGraphDestroy(g);
      throw;
    }
    NNCV_HIP_CHECK(hipStreamEndCapture(s, &hit->graph));
    NNCV_HIP_CHECK(hipGraphInstantiate(&hit->exec, hit->graph, nullptr, nullptr, 0));
  }
  NNCV_HIP_CHECK(hipGraphLaunch(hit->exec, s));
}

void forward_replay(const void* owner, const ResNet18& m, const void* src, int N, int H, int W, float* logits, void* ws, hipStream_t s) {
  // 18 launches: launch-bound up to about two 224x224 images
  replay(owner, [&] { m.forward(src, N, H, W, logits, ws, s); }, src, N, H, W, logits, ws, s, (long long)N * H * W <= 2ll * 224 * 224);
}

// ---- the MobileNetV3 object behind the handle-less reference ABI ----------------------------
struct CachedGraph {
  const void* host_ptr;
  long long n;
  int dt;
  uint64_t fingerprint;
  std::unique_ptr<Graph> graph;
};
std::vector<CachedGraph>& graph_model_cache() {
  static std::vector<CachedGraph> c;
  return c;
}
long long mobilenetv3_elems() {
  static const long long n = [] {
    long long k = 0;
    (void)mobilenetv3_small_ops(&k);
    return k;
  }();
  return n;
}
std::unique_ptr<Graph> build_graph(const GraphOp* ops, int n_ops, int c_in, const void* host, long long n, int dt, hipStream_t s) {
  DeviceBuffer blob((size_t)n * dtype_size(dt));
  NNCV_HIP_CHECK(hipMemcpyAsync(blob.get(), host, blob.bytes(), hipMemcpyHostToDevice, s));
  auto g = std::make_unique<Graph>(ops, n_ops, c_in, blob.get(), n, dt, s);
  NNCV_HIP_CHECK(hipStreamSynchronize(s));  // the staging blob dies here
  return g;
}
Graph& cached_mobilenetv3(const void* host, long long n, int dt, hipStream_t s) {
  const uint64_t fp = fingerprint(host, n, dtype_size(dt));
  auto& cache = graph_model_cache();
  auto make = [&] {
    long long k = 0;
    const std::vector<GraphOp> ops = mobilenetv3_small_ops(&k);
    return build_graph(ops.data(), (int)ops.size(), 3, host, n, dt, s);
  };
  for (auto& e : cache)
    if (e.host_ptr == host && e.n == n && e.dt == dt) {
      if (e.fingerprint != fp) {
        e.graph.reset();
        e.graph = make();
        e.fingerprint = fp;
      }
      return *e.graph;
    }
  if (cache.size() >= 4) cache.erase(cache.begin());
  cache.push_back(CachedGraph{host, n, dt, fp, make()});
  return *cache.back().graph;
}

// ---- the host-buffer call: the upload of a large dense input ---------------------------------------------------------
// _mlir_ciface_forward hands over pageable host memory (examples/Res18/main.cpp:79-99).  The DMA engine moves config 4's
// 9.6 MB in 0.23 ms from pinned memory; through the runtime's own staging of pageable memory the same copy takes 0.34 ms.
// So the input goes to pinned staging memory in pieces, each copied by a few host threads while the DMA engine moves the
// piece before it; a caller buffer that is pinned already is handed to the DMA engine as it is.
// Tried and not kept: cutting the batch into two halves (or a quarter, a quarter and a half) whose forward passes start
// as soon as their bytes have landed, on streams and workspaces of their own.  The passes of 8-16 images are launch-bound
// (8 + 8 + 16 images one after the other: 0.41 ms against 0.26 for the 32 at once), submitting a pass costs the host
// 50-100 us during which the DMA queue ran dry, and the call measured 0.63-0.77 ms against 0.68 before and 0.59 for this
// form with a pinned buffer.
bool host_pointer_is_pinned(const void* p) {
  hipPointerAttribute_t at;
  if (hipPointerGetAttributes(&at, p) != hipSuccess) {
    (void)hipGetLastError();  // plain malloc memory is unknown to the runtime: an error, not a fault
    return false;
  }
  return at.type == hipMemoryTypeHost;
}

void upload_dense(const char* hsrc, size_t bytes, void* dev, PinnedBuffer& pin, hipStream_t s) {
  static const bool plain = getenv("NNCV_HIP_NO_STAGED_UPLOAD") != nullptr;
  if (plain || bytes < (size_t(1) << 20) || host_pointer_is_pinned(hsrc)) {
    NNCV_HIP_CHECK(hipMemcpyAsync(dev, hsrc, bytes, hipMemcpyHostToDevice, s));
    return;
  }
  char* stage = static_cast<char*>(pin.ensure(bytes));
  const size_t piece = size_t(2) << 20;
  for (size_t off = 0; off < bytes; off += piece) {
    const size_t n = std::min(piece, bytes - off);
    parallel_copy(stage + off, hsrc + off, n);
    NNCV_HIP_CHECK(hipMemcpyAsync(static_cast<char*>(dev) + off, stage + off, n, hipMemcpyHostToDevice, s));
  }
}

void forward_abi(nncv_memref2d* dst, nncv_memref4d* src, void* params, int dt) {
  NNCV_REQUIRE(dst && src && params, "null descriptor");
  Context& ctx = Context::get();
  ctx.init(-1);
  hipStream_t s = ctx.stream();
  ctx.order_after_previous(s);
  const size_t es = dtype_size(dt);
  const nncv_memref1d* p = static_cast<const nncv_memref1d*>(params);
  NNCV_REQUIRE(p->aligned && p->strides[0] == 1, "params must be a dense rank-1 memref");
  const int N = (int)src->sizes[0], C = (int)src->sizes[1], H = (int)src->sizes[2], W = (int)src->sizes[3];
  NNCV_REQUIRE(C == 3, "forward: input must be [N,3,H,W]");
  const char* blob = static_cast<const char*>(p->aligned) + p->offset * (intptr_t)es;
  // Which network the object is follows from the size of its parameter array: ResNet-18
  // (tests/Nets/Res18.mlir) or MobileNetV3-small (tests/Nets/MobileNetV3.mlir); both map
  // [N,3,H,W] to [N,1000].
  const bool mobilenet = p->sizes[0] == mobilenetv3_elems();
  ResNet18* model = mobilenet ? nullptr : &cached_model(blob, p->sizes[0], dt, s);
  Graph* graph = mobilenet ? &cached_mobilenetv3(blob, p->sizes[0], dt, s) : nullptr;

  const size_t in_bytes = align256((size_t)N * 3 * H * W * es), out_bytes = align256((size_t)N * 1000 * 4);
  const size_t ws_bytes = mobilenet ? graph->workspace_bytes(N, H, W) : model->workspace_bytes(N, H, W);
  ctx.arena.reserve(in_bytes + 2 * out_bytes + ws_bytes + 2048, s);
  void* d_in = ctx.arena.take(in_bytes);
  float* d_out = static_cast<float*>(ctx.arena.take(out_bytes));
  void* ws = ctx.arena.take(ws_bytes);
  // The reference object assumes identity layout and would misread a strided input
  // (DnnModelLowering.cpp:107-108); strides are honoured here instead.
  if (contiguous<4>(src->sizes, src->strides))
    upload_dense(static_cast<const char*>(src->aligned) + src->offset * (intptr_t)es, (size_t)N * 3 * H * W * es, d_in, ctx.pin_in, s);
  else
    upload<4>(src->aligned, src->offset, src->sizes, src->strides, es, d_in, ctx.pin_in, s);
  if (mobilenet) graph->forward(d_in, N, H, W, d_out, ws, s);
  else model->forward(d_in, N, H, W, d_out, ws, s);

  // MLIR C-interface convention: the callee allocates the result and overwrites *dst.
  void* result = nullptr;
  NNCV_REQUIRE(posix_memalign(&result, 64, std::max<size_t>(64, (size_t)N * 1000 * es)) == 0, "out of host memory");
  if (dt == kF32) {
    NNCV_HIP_CHECK(hipMemcpyAsync(result, d_out, (size_t)N * 1000 * 4, hipMemcpyDeviceToHost, s));
    NNCV_HIP_CHECK(hipStreamSynchronize(s));
  } else {
    // rounded to half on the device (one round-to-nearest-even conversion, what the host's would be): half the bytes over
    // the bus and no conversion loop on the host
    void* d_half = ctx.arena.take(align256((size_t)N * 1000 * 2));
    launch_cast(d_out, kF32, d_half, kF16, (long long)N * 1000, s);
    void* tmp = ctx.pin_out.ensure((size_t)N * 1000 * 2);
    NNCV_HIP_CHECK(hipMemcpyAsync(tmp, d_half, (size_t)N * 1000 * 2, hipMemcpyDeviceToHost, s));
    NNCV_HIP_CHECK(hipStreamSynchronize(s));
    memcpy(result, tmp, (size_t)N * 1000 * 2);
  }
  dst->allocated = result;
  dst->aligned = result;
  dst->offset = 0;
  dst->sizes[0] = N;
  dst->sizes[1] = 1000;
  dst->strides[0] = 1000;
  dst->strides[1] = 1;
}

struct nncv_hip_model_impl {
  std::shared_ptr<ResNet18> m;  // shared with the handle's clones
  HandleState st;
  int passes = 0;  // forward passes the caller keeps in flight next to this handle's; 0 = the process-wide default
};
struct nncv_hip_conv_impl {
  std::unique_ptr<ConvLayer> c;
};
struct nncv_hip_graph_impl {
  std::unique_ptr<Graph> g;
  HandleState st;
};

}  // namespace

struct nncv_hip_model : nncv_hip_model_impl {};
struct nncv_hip_conv : nncv_hip_conv_impl {};
struct nncv_hip_graph : nncv_hip_graph_impl {};

extern "C" {

// ---------------------------------------------------------------------------------------------
// Part 1 — reference ABI
// ---------------------------------------------------------------------------------------------
void _mlir_ciface_forward(nncv_memref2d* dst, nncv_memref4d* src, void* params) {
  guarded_abort("_mlir_ciface_forward", [&] { forward_abi(dst, src, params, kF32); });
}

void _mlir_ciface_forward_f16(nncv_memref2d* dst, nncv_memref4d* src, void* params) {
  guarded_abort("_mlir_ciface_forward_f16", [&] { forward_abi(dst, src, params, kF16); });
}

void _mlir_ciface_matmul(nncv_memref2d* res, nncv_memref2d* a, nncv_memref2d* b, nncv_memref2d* c) {
  guarded_abort("_mlir_ciface_matmul", [&] {
    NNCV_REQUIRE(res && a && b && c, "null descriptor");
    Context& ctx = Context::get();
    ctx.init(-1);
    hipStream_t s = ctx.stream();
    ctx.order_after_previous(s);
    const int M = (int)a->sizes[0], K = (int)a->sizes[1], N = (int)b->sizes[1];
    NNCV_REQUIRE(b->sizes[0] == K && c->sizes[0] == M && c->sizes[1] == N, "matmul: shapes do not agree");
    const size_t ab = align256((size_t)M * K * 4), bb = align256((size_t)K * N * 4), cb = align256((size_t)M * N * 4);
    ctx.arena.reserve(ab + bb + cb + 1024, s);
    float* dA = static_cast<float*>(ctx.arena.take(ab));
    float* dB = static_cast<float*>(ctx.arena.take(bb));
    float* dC = static_cast<float*>(ctx.arena.take(cb));
    upload<2>(a->aligned, a->offset, a->sizes, a->strides, 4, dA, ctx.pin_in, s);
    upload<2>(b->aligned, b->offset, b->sizes, b->strides, 4, dB, ctx.pin_in, s);
    upload<2>(c->aligned, c->offset, c->sizes, c->strides, 4, dC, ctx.pin_in, s);
    launch_gemm_nn_f32(dA, dB, dC, M, N, K, s);
    download<2>(c->aligned, c->offset, c->sizes, c->strides, 4, dC, ctx.pin_out, s);
    *res = *c;  // in-place bufferization: the result aliases `outs`
  });
}

void _mlir_ciface_batch_nchw_conv(nncv_memref4d* res, nncv_memref4d* in, nncv_memref4d* filter, nncv_memref4d* out) {
  guarded_abort("_mlir_ciface_batch_nchw_conv", [&] {
    NNCV_REQUIRE(res && in && filter && out, "null descriptor");
    Context& ctx = Context::get();
    ctx.init(-1);
    hipStream_t s = ctx.stream();
    ctx.order_after_previous(s);
    const int N = (int)in->sizes[0], C = (int)in->sizes[1], H = (int)in->sizes[2], W = (int)in->sizes[3];
    const int F = (int)filter->sizes[0], R = (int)filter->sizes[2], S = (int)filter->sizes[3];
    const int OH = (int)out->sizes[2], OW = (int)out->sizes[3];
    NNCV_REQUIRE(filter->sizes[1] == C && out->sizes[0] == N && out->sizes[1] == F, "conv: shapes do not agree");
    NNCV_REQUIRE(H >= R && W >= S && OH >= 1 && OW >= 1, "conv: filter larger than input");
    // stride is an attribute of the compiled op in the reference; recover it from the shapes
    int stride = 1;
    if (OH > 1) stride = (H - R) / (OH - 1);
    else if (OW > 1) stride = (W - S) / (OW - 1);
    NNCV_REQUIRE(stride >= 1 && (H - R) / stride + 1 == OH && (W - S) / stride + 1 == OW,
                 "conv: output shape is not (in - filter)/stride + 1 for any stride");
    const size_t ib = align256((size_t)N * C * H * W * 4), fb = align256((size_t)F * C * R * S * 4),
                 ob = align256((size_t)N * F * OH * OW * 4);
    ConvLayer::Desc d;
    d.dt = kF32; d.C = C; d.F = F; d.R = R; d.S = S; d.stride = stride; d.pad = 0; d.relu = kActNone; d.algo = kAlgoAuto;
    DeviceBuffer dF(fb);
    upload<4>(filter->aligned, filter->offset, filter->sizes, filter->strides, 4, dF.get(), ctx.pin_in, s);
    ConvLayer layer(d, dF.get(), nullptr, nullptr, nullptr, nullptr, s);
    const size_t wsb = layer.workspace_bytes(N, H, W, true);
    ctx.arena.reserve(ib + ob + wsb + 1024, s);
    void* dI = ctx.arena.take(ib);
    void* dO = ctx.arena.take(ob);
    void* ws = ctx.arena.take(wsb);
    upload<4>(in->aligned, in->offset, in->sizes, in->strides, 4, dI, ctx.pin_in, s);
    upload<4>(out->aligned, out->offset, out->sizes, out->strides, 4, dO, ctx.pin_in, s);
    layer.forward_strided(dI, strides_of(kNCHW, C, H, W), N, H, W, nullptr, dO, strides_of(kNCHW, F, OH, OW), true, ws, s);
    download<4>(out->aligned, out->offset, out->sizes, out->strides, 4, dO, ctx.pin_out, s);
    *res = *out;
  });
}

// ---------------------------------------------------------------------------------------------
// Part 2 — device-resident forms
// ---------------------------------------------------------------------------------------------
int nncv_hip_init(int device) {
  return guarded([&] { Context::get().init(device); });
}

const char* nncv_hip_last_error(void) { return g_last_error.c_str(); }

void nncv_hip_profile_enable(int on) {
  guarded([&] { profiler_enable(on != 0); });
}

int nncv_hip_conv3x3_patch_plan(int stride, int N, int OH, int OW, int F, int slabs, int* plan) {
  if (!plan) return 1;
  return conv3x3_patch_plan(stride, N, OH, OW, F, slabs, plan) ? 0 : 1;
}

int nncv_hip_set_overlap_hint(int passes) {
  return guarded([&] {
    const int want = passes < 1 ? 1 : passes;
    if (want == overlap_default()) return;
    // captured passes hold the launch shapes and workspace offsets of the old setting
    (void)hipDeviceSynchronize();
    auto& gc = graph_cache();
    for (auto& e : gc) drop_graph(e);
    gc.clear();
    set_overlap_hint(want);
  });
}

int nncv_hip_params_invalidate(const void* params) {
  return guarded([&] {
    std::lock_guard<std::recursive_mutex> lk(Context::get().mu);
    auto& mc = model_cache();
    for (size_t i = 0; i < mc.size();)
      if (!params || mc[i].host_ptr == params) {
        mc.erase(mc.begin() + i);
      } else {
        ++i;
      }
    auto& gc = graph_model_cache();
    for (size_t i = 0; i < gc.size();)
      if (!params || gc[i].host_ptr == params) {
        gc.erase(gc.begin() + i);
      } else {
        ++i;
      }
  });
}

int nncv_hip_conv3x3_stream_plan(int N, int H, int W, int C, int F, int* plan) {
  if (!plan) return 1;
  return conv3x3_stream_plan(N, H, W, C, F, plan) ? 0 : 1;
}

size_t nncv_hip_profile_report(char* buf, size_t cap) {
  std::string r;
  if (guarded([&] { r = profiler_report(); }) != 0) r = "{}";
  if (buf && cap) {
    const size_t n = std::min(cap - 1, r.size());
    memcpy(buf, r.data(), n);
    buf[n] = 0;
  }
  return r.size() + 1;
}

const char* nncv_hip_device_arch(void) {
  if (guarded([&] { Context::get().init(-1); }) != 0) return "";
  return Context::get().arch().c_str();
}

nncv_hip_model* nncv_hip_resnet18_create(const void* params, int64_t n_elems, int dtype, int algo3x3) {
  return nncv_hip_resnet18_create_ex(params, n_elems, dtype, algo3x3, 0);
}

nncv_hip_model* nncv_hip_resnet18_create_ex(const void* params, int64_t n_elems, int dtype, int algo3x3, int passes_in_flight) {
  nncv_hip_model* h = nullptr;
  const int rc = guarded([&] {
    NNCV_REQUIRE(params, "null params");
    NNCV_REQUIRE(dtype == kF32 || dtype == kF16, "dtype must be 1 (fp32) or 2 (fp16)");
    NNCV_REQUIRE(passes_in_flight >= 0 && passes_in_flight <= 64, "passes_in_flight must be 0 (the default) .. 64");
    Context& ctx = Context::get();
    ctx.init(-1);
    h = new nncv_hip_model();
    h->passes = passes_in_flight;
    try {
      h->m = build_model(params, n_elems, dtype, algo3x3, ctx.stream());
    } catch (...) {
      delete h;
      h = nullptr;
      throw;
    }
  });
  return rc == 0 ? h : nullptr;
}

nncv_hip_model* nncv_hip_resnet18_clone(nncv_hip_model* m) {
  nncv_hip_model* h = nullptr;
  const int rc = guarded([&] {
    NNCV_REQUIRE(m && m->m, "null argument");
    NNCV_REQUIRE(m->m->dtype() == kF16, "clone: fp16 models only (an fp32 model's K-split tickets belong to its layers)");
    h = new nncv_hip_model();
    h->m = m->m;
    h->passes = m->passes;
  });
  return rc == 0 ? h : nullptr;
}

int nncv_hip_resnet18_passes_in_flight(const nncv_hip_model* m) { return m ? (m->passes > 0 ? m->passes : overlap_default()) : -1; }

int nncv_hip_pick_streams(int want, void** streams, int* overlapping) {
  return guarded([&] {
    NNCV_REQUIRE(streams && want >= 1 && want <= 8, "pick_streams: want must be 1..8 and streams non-null");
    Context::get().init(-1);
    int found = 0;
    const std::vector<hipStream_t> v = pick_streams(want, &found);
    NNCV_REQUIRE((int)v.size() == want, "pick_streams: fewer streams than asked for");
    for (int i = 0; i < want; ++i) streams[i] = v[i];
    if (overlapping) *overlapping = found;
  });
}

void nncv_hip_resnet18_destroy(nncv_hip_model* m) {
  if (!m) return;
  guarded([&] {
    (void)hipDeviceSynchronize();
    drop_graphs_of(&m->st);  // this handle's captured passes only: clones keep theirs
    delete m;
  });
}

int nncv_hip_resnet18_forward(nncv_hip_model* m, const void* src, int N, int H, int W, float* logits, void* stream) {
  return guarded([&] {
    NNCV_REQUIRE(m && m->m && src && logits, "null argument");
    HandleSync sy(m->st, stream);
    OverlapScope hint(m->passes);
    const size_t wsb = m->m->workspace_bytes(N, H, W);
    if (m->st.arena.reserve(wsb + 1024, sy.s)) drop_graphs_of(&m->st);  // captured against the old workspace
    forward_replay(&m->st, *m->m, src, N, H, W, logits, m->st.arena.take(wsb), sy.s);
    sy.finish();
  });
}

int nncv_hip_preprocess_u8(const void* hwc_u8, int N, int H, int W, int channels, int dtype, void* nchw_out, void* stream) {
  return guarded([&] {
    NNCV_REQUIRE(hwc_u8 && nchw_out, "null argument");
    NNCV_REQUIRE(dtype == kF32 || dtype == kF16, "dtype must be 1 (fp32) or 2 (fp16)");
    Context::get().init(-1);
    Sync sy(stream);
    launch_preprocess_u8(hwc_u8, nchw_out, dtype, N, H, W, channels, sy.s);
    sy.finish();
  });
}

int nncv_hip_argmax(const float* logits, int N, int F, int* top1, void* stream) {
  return guarded([&] {
    NNCV_REQUIRE(logits && top1, "null argument");
    Context::get().init(-1);
    Sync sy(stream);
    launch_argmax_rows(logits, top1, N, F, sy.s);
    sy.finish();
  });
}

int nncv_hip_resnet18_classify_u8(nncv_hip_model* m, const void* hwc_u8, int N, int H, int W, int channels, float* logits,
                                  int* top1, void* stream) {
  return guarded([&] {
    NNCV_REQUIRE(m && m->m && hwc_u8 && logits && top1, "null argument");
    HandleSync sy(m->st, stream);
    OverlapScope hint(m->passes);
    const int dt = m->m->dtype();
    const size_t in_b = align256((size_t)N * 3 * H * W * dtype_size(dt));
    const size_t wsb = m->m->workspace_bytes(N, H, W);
    m->st.arena.reserve(in_b + wsb + 2048, sy.s);
    void* x = m->st.arena.take(in_b);
    launch_preprocess_u8(hwc_u8, x, dt, N, H, W, channels, sy.s);
    m->m->forward(x, N, H, W, logits, m->st.arena.take(wsb), sy.s);
    launch_argmax_rows(logits, top1, N, 1000, sy.s);
    sy.finish();
  });
}

int nncv_hip_resnet18_forward_tap(nncv_hip_model* m, const void* src, int N, int H, int W, float* logits, int stage,
                                  void* tap, void* stream) {
  return guarded([&] {
    NNCV_REQUIRE(m && m->m && src && logits && tap, "null argument");
    NNCV_REQUIRE(stage >= 0 && stage <= 4, "stage must be 0..4");
    HandleSync sy(m->st, stream);
    OverlapScope hint(m->passes);
    const size_t wsb = m->m->workspace_bytes(N, H, W);
    m->st.arena.reserve(wsb + 1024, sy.s);
    m->m->forward(src, N, H, W, logits, m->st.arena.take(wsb), sy.s, stage, tap);
    sy.finish();
  });
}

nncv_hip_conv* nncv_hip_conv_create(int dtype, const void* weights, int F, int C, int R, int S, int stride, int pad,
                                    const void* gamma, const void* beta, const void* mean, const void* var, int relu,
                                    int algo) {
  nncv_hip_conv* h = nullptr;
  const int rc = guarded([&] {
    NNCV_REQUIRE(weights, "null weights");
    NNCV_REQUIRE(dtype == kF32 || dtype == kF16, "dtype must be 1 (fp32) or 2 (fp16)");
    NNCV_REQUIRE(F > 0 && C > 0 && R > 0 && S > 0, "conv: bad geometry");
    Context& ctx = Context::get();
    ctx.init(-1);
    hipStream_t s = ctx.stream();
    const size_t es = dtype_size(dtype);
    DeviceBuffer w((size_t)F * C * R * S * es), bn;
    NNCV_HIP_CHECK(hipMemcpyAsync(w.get(), weights, w.bytes(), hipMemcpyHostToDevice, s));
    const char* g = nullptr;
    if (gamma) {
      NNCV_REQUIRE(beta && mean && var, "conv: BN needs gamma, beta, mean and var");
      bn.reset((size_t)4 * F * es);
      const void* srcs[4] = {gamma, beta, mean, var};
      for (int i = 0; i < 4; ++i)
        NNCV_HIP_CHECK(hipMemcpyAsync(bn.as<char>() + (size_t)i * F * es, srcs[i], (size_t)F * es, hipMemcpyHostToDevice, s));
      g = bn.as<char>();
    }
    ConvLayer::Desc d;
    d.dt = dtype; d.C = C; d.F = F; d.R = R; d.S = S; d.stride = stride; d.pad = pad; d.relu = relu; d.algo = algo;
    h = new nncv_hip_conv();
    try {
      h->c = std::make_unique<ConvLayer>(d, w.get(), g, g ? g + (size_t)F * es : nullptr, g ? g + (size_t)2 * F * es : nullptr,
                                         g ? g + (size_t)3 * F * es : nullptr, s);
      NNCV_HIP_CHECK(hipStreamSynchronize(s));
    } catch (...) {
      delete h;
      h = nullptr;
      throw;
    }
  });
  return rc == 0 ? h : nullptr;
}

void nncv_hip_conv_destroy(nncv_hip_conv* c) {
  if (!c) return;
  guarded([&] {
    (void)hipDeviceSynchronize();
    delete c;
  });
}

int nncv_hip_conv_algo(const nncv_hip_conv* c) { return (c && c->c) ? c->c->algo() : -1; }

int nncv_hip_conv_forward(nncv_hip_conv* c, const void* in, int N, int H, int W, int layout, const void* residual, void* out,
                          void* stream) {
  return guarded([&] {
    NNCV_REQUIRE(c && c->c && in && out, "null argument");
    NNCV_REQUIRE(layout == kNCHW || layout == kNHWC, "layout must be 0 (NCHW) or 1 (NHWC)");
    Context& ctx = Context::get();
    Sync sy(stream);
    const ConvLayer& L = *c->c;
    const size_t wsb = L.workspace_bytes(N, H, W, layout == kNCHW);
    ctx.arena.reserve(wsb + 1024, sy.s);
    void* ws = ctx.arena.take(wsb);
    if (layout == kNHWC) {
      L.forward(in, N, H, W, residual, out, ws, sy.s);
    } else {
      const int OH = L.out_h(H), OW = L.out_w(W);
      L.forward_strided(in, strides_of(kNCHW, L.desc().C, H, W), N, H, W, residual, out, strides_of(kNCHW, L.desc().F, OH, OW),
                        false, ws, sy.s);
    }
    sy.finish();
  });
}

int nncv_hip_conv_forward_noalloc(nncv_hip_conv* c, const void* in, int N, int H, int W, const void* residual, void* out,
                                  void* stream) {
  return guarded([&] {
    NNCV_REQUIRE(c && c->c && in && out, "null argument");
    const ConvLayer& L = *c->c;
    const size_t wsb = L.workspace_bytes(N, H, W, false);
    NNCV_REQUIRE(wsb <= kNoAllocWorkspaceBytes,
                 "nncv_hip_conv_forward_noalloc: this layer and shape need " + std::to_string(wsb) + " bytes of workspace, the "
                 "scratch array holds " + std::to_string(kNoAllocWorkspaceBytes) + "; use nncv_hip_conv_forward");
    static_assert(ConvLayer::kSplitKCounterInts * sizeof(int) <= kNoAllocCounterBytes, "ticket counters outgrow their slot");
    Sync sy(stream);
    char* scratch = static_cast<char*>(noalloc_scratch());
    // the array keeps the previous call's contents: the tickets must start at zero (the workspace is written before it is read)
    launch_clear_words(scratch, ConvLayer::kSplitKCounterInts, sy.s);
    L.forward(in, N, H, W, residual, out, scratch + kNoAllocCounterBytes, sy.s, reinterpret_cast<int*>(scratch));
    sy.finish();
  });
}

int nncv_hip_conv_time(nncv_hip_conv* c, const void* in, int N, int H, int W, const void* residual, void* out, int reps,
                       void* stream, float* avg_us) {
  return guarded([&] {
    NNCV_REQUIRE(c && c->c && in && out && avg_us && reps > 0, "null argument");
    Context& ctx = Context::get();
    Sync sy(stream);
    const ConvLayer& L = *c->c;
    const size_t wsb = L.workspace_bytes(N, H, W, false);
    ctx.arena.reserve(wsb + 1024, sy.s);
    void* ws = ctx.arena.take(wsb);
    hipEvent_t e0, e1;
    NNCV_HIP_CHECK(hipEventCreate(&e0));
    NNCV_HIP_CHECK(hipEventCreate(&e1));
    for (int i = 0; i < 5; ++i) L.forward(in, N, H, W, residual, out, ws, sy.s);
    NNCV_HIP_CHECK(hipEventRecord(e0, sy.s));
    for (int i = 0; i < reps; ++i) L.forward(in, N, H, W, residual, out, ws, sy.s);
    NNCV_HIP_CHECK(hipEventRecord(e1, sy.s));
    NNCV_HIP_CHECK(hipEventSynchronize(e1));
    float ms = 0.0f;
    NNCV_HIP_CHECK(hipEventElapsedTime(&ms, e0, e1));
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    *avg_us = ms * 1000.0f / (float)reps;
    sy.finish();
  });
}

unsigned long long nncv_hip_plan_arena(int n, const int* first_op, const int* last_op, const unsigned long long* bytes,
                                       unsigned long long align, unsigned long long* offsets) {
  unsigned long long total = 0;
  const int rc = guarded([&] {
    NNCV_REQUIRE(n >= 0 && (n == 0 || (first_op && last_op && bytes && offsets)), "null argument");
    NNCV_REQUIRE(align >= 1 && (align & (align - 1)) == 0, "align must be a power of two");
    std::vector<TensorLife> t((size_t)n);
    for (int i = 0; i < n; ++i) {
      NNCV_REQUIRE(first_op[i] <= last_op[i], "a tensor's first operator must not come after its last");
      t[i] = TensorLife{first_op[i], last_op[i], (size_t)bytes[i], 0};
    }
    total = plan_offsets(t, (size_t)align);
    for (int i = 0; i < n; ++i) offsets[i] = t[i].offset;
  });
  return rc == 0 ? total : ~0ull;
}

int nncv_hip_matmul_time(const float* A, const float* B, float* C, int M, int N, int K, int reps, void* stream, float* avg_us) {
  return guarded([&] {
    NNCV_REQUIRE(A && B && C && avg_us && reps > 0, "null argument");
    Context::get().init(-1);
    Sync sy(stream);
    hipEvent_t e0, e1;
    NNCV_HIP_CHECK(hipEventCreate(&e0));
    NNCV_HIP_CHECK(hipEventCreate(&e1));
    for (int i = 0; i < 5; ++i) launch_gemm_nn_f32(A, B, C, M, N, K, sy.s);
    NNCV_HIP_CHECK(hipEventRecord(e0, sy.s));
    for (int i = 0; i < reps; ++i) launch_gemm_nn_f32(A, B, C, M, N, K, sy.s);
    NNCV_HIP_CHECK(hipEventRecord(e1, sy.s));
    NNCV_HIP_CHECK(hipEventSynchronize(e1));
    float ms = 0.0f;
    NNCV_HIP_CHECK(hipEventElapsedTime(&ms, e0, e1));
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    *avg_us = ms * 1000.0f / (float)reps;
    sy.finish();
  });
}

int nncv_hip_matmul_f32(const float* A, const float* B, float* C, int M, int N, int K, void* stream) {
  return guarded([&] {
    NNCV_REQUIRE(A && B && C, "null argument");
    Context::get().init(-1);
    Sync sy(stream);
    launch_gemm_nn_f32(A, B, C, M, N, K, sy.s);
    sy.finish();
  });
}

int nncv_hip_wino43_filter(int dtype, const void* w, void* U, int F, int C, void* stream) {
  return guarded([&] {
    NNCV_REQUIRE(w && U, "null argument");
    Context::get().init(-1);
    Sync sy(stream);
    launch_wino43_filter(w, dtype, U, dtype, F, C, sy.s);
    sy.finish();
  });
}

int nncv_hip_wino43_input(int dtype, const void* in, int layout, void* V, int N, int C, int H, int W, int pad, void* stream) {
  return guarded([&] {
    NNCV_REQUIRE(in && V, "null argument");
    Context::get().init(-1);
    Sync sy(stream);
    launch_wino43_input(in, dtype, strides_of(layout, C, H, W), V, dtype, N, C, H, W, pad, sy.s);
    sy.finish();
  });
}

int nncv_hip_wino43_gemm(int dtype, const void* V, const void* U, void* M, int64_t tiles, int C, int F, void* stream) {
  return guarded([&] {
    NNCV_REQUIRE(V && U && M, "null argument");
    NNCV_REQUIRE(tiles > 0 && tiles < (1ll << 31), "tiles out of range");
    Context::get().init(-1);
    Sync sy(stream);
    IgemmArgs a{};
    a.in = V; a.wt = U; a.out = M;
    a.N = (int)tiles; a.H = 1; a.W = 1; a.C = C; a.F = F; a.R = 1; a.S = 1; a.OH = 1; a.OW = 1;
    a.stride_h = a.stride_w = 1; a.ldo = F; a.batch = 36;
    a.in_bs = tiles * C; a.wt_bs = (long long)F * C; a.out_bs = tiles * F;
    launch_igemm(a, dtype, dtype, sy.s);
    sy.finish();
  });
}

int nncv_hip_wino43_output(int dtype, const void* M, void* out, int layout, int N, int F, int OH, int OW, const float* scale,
                           const float* shift, const void* residual, int relu, void* stream) {
  return guarded([&] {
    NNCV_REQUIRE(M && out, "null argument");
    Context::get().init(-1);
    Sync sy(stream);
    WinoOutArgs o{};
    o.M = M; o.out = out; o.residual = residual; o.scale = scale; o.shift = shift;
    o.st = strides_of(layout, F, OH, OW); o.N = N; o.F = F; o.OH = OH; o.OW = OW; o.relu = relu; o.accumulate = 0;
    launch_wino43_output(o, dtype, dtype, sy.s);
    sy.finish();
  });
}

int nncv_hip_maxpool3x3s2(int dtype, const void* in, void* out, int N, int H, int W, int C, void* stream) {
  return guarded([&] {
    NNCV_REQUIRE(in && out, "null argument");
    Context::get().init(-1);
    Sync sy(stream);
    launch_maxpool3x3s2_nhwc(in, out, dtype, N, H, W, C, sy.s);
    sy.finish();
  });
}

int nncv_hip_global_avgpool(int dtype, const void* in, void* out, int N, int H, int W, int C, void* stream) {
  return guarded([&] {
    NNCV_REQUIRE(in && out, "null argument");
    Context::get().init(-1);
    Sync sy(stream);
    launch_global_avgpool_nhwc(in, out, dtype, N, H * W, C, sy.s);
    sy.finish();
  });
}

// ---------------------------------------------------------------------------------------------
// Network graphs and their single operators
// ---------------------------------------------------------------------------------------------
nncv_hip_graph* nncv_hip_graph_create(const nncv_hip_graph_op* ops, int n_ops, int in_channels, const void* params,
                                      int64_t n_elems, int dtype) {
  nncv_hip_graph* h = nullptr;
  const int rc = guarded([&] {
    NNCV_REQUIRE(ops && params && n_ops > 0 && n_elems > 0, "null or empty argument");
    NNCV_REQUIRE(dtype == kF32 || dtype == kF16, "dtype must be 1 (fp32) or 2 (fp16)");
    Context& ctx = Context::get();
    ctx.init(-1);
    h = new nncv_hip_graph();
    try {
      h->g = build_graph(ops, n_ops, in_channels, params, n_elems, dtype, ctx.stream());
    } catch (...) {
      delete h;
      h = nullptr;
      throw;
    }
  });
  return rc == 0 ? h : nullptr;
}

void nncv_hip_graph_destroy(nncv_hip_graph* g) {
  if (!g) return;
  guarded([&] {
    (void)hipDeviceSynchronize();
    drop_graphs_of(&g->st);
    delete g;
  });
}

int nncv_hip_graph_output_shape(const nncv_hip_graph* g, int H, int W, int* shape) {
  return guarded([&] {
    NNCV_REQUIRE(g && g->g && shape, "null argument");
    g->g->output_shape(H, W, &shape[0], &shape[1], &shape[2]);
  });
}

int nncv_hip_graph_forward(nncv_hip_graph* g, const void* src, int N, int H, int W, float* out, int64_t out_elems, void* stream) {
  return guarded([&] {
    NNCV_REQUIRE(g && g->g && src && out, "null argument");
    HandleSync sy(g->st, stream);
    const Graph& gr = *g->g;
    int C, OH, OW;
    gr.output_shape(H, W, &C, &OH, &OW);
    NNCV_REQUIRE(out_elems == (int64_t)N * C * OH * OW, "graph: out_elems does not match the output shape");
    const size_t wsb = gr.workspace_bytes(N, H, W);
    if (g->st.arena.reserve(wsb + 1024, sy.s)) drop_graphs_of(&g->st);  // captured against the old workspace
    void* ws = g->st.arena.take(wsb);
    // 49-73 launches: launch-bound up to about four 224x224 images
    replay(&g->st, [&] { gr.forward(src, N, H, W, out, ws, sy.s); }, src, N, H, W, out, ws, sy.s, (long long)N * H * W <= 4ll * 224 * 224);
    sy.finish();
  });
}

int64_t nncv_hip_graph_plan(const nncv_hip_graph_op* ops, int n_ops, int in_channels, int dtype, int N, int H, int W,
                            int64_t* tensor_info, int tensor_cap, int32_t* launch_dst) {
  int64_t total = -1;
  const int rc = guarded([&] {
    NNCV_REQUIRE(ops && n_ops > 0 && tensor_info && launch_dst, "null or empty argument");
    const Graph g(ops, n_ops, in_channels, nullptr, 0, dtype, nullptr);  // structure only: no device work
    NNCV_REQUIRE(g.num_tensors() <= tensor_cap, "graph_plan: tensor_info holds fewer tensors than the graph has");
    std::vector<long long> info((size_t)4 * g.num_tensors());
    std::vector<int> dst((size_t)n_ops);
    total = (int64_t)g.describe_plan(N, H, W, info.data(), dst.data());
    for (size_t k = 0; k < info.size(); ++k) tensor_info[k] = info[k];
    for (int i = 0; i < n_ops; ++i) launch_dst[i] = dst[i];
  });
  return rc == 0 ? total : -1;
}

int nncv_hip_mobilenetv3_small_ops(nncv_hip_graph_op* ops, int cap, int64_t* n_elems) {
  long long n = 0;
  const std::vector<GraphOp> v = mobilenetv3_small_ops(&n);
  if (n_elems) *n_elems = n;
  if (ops)
    for (int i = 0; i < cap && i < (int)v.size(); ++i) ops[i] = v[i];
  return (int)v.size();
}

int nncv_hip_dwconv(int dtype, const void* in, const void* w, const float* scale, const float* shift, void* out, int N, int H,
                    int W, int C, int K, int stride, int pad, int act, void* stream) {
  return guarded([&] {
    NNCV_REQUIRE(in && w && out, "null argument");
    NNCV_REQUIRE(dtype == kF32 || dtype == kF16, "dtype must be 1 (fp32) or 2 (fp16)");
    NNCV_REQUIRE(K == 3 || K == 5, "dwconv: kernel size must be 3 or 5");
    NNCV_REQUIRE(N >= 1 && H >= 1 && W >= 1 && C >= 1 && stride >= 1 && pad >= 0 && H + 2 * pad >= K && W + 2 * pad >= K,
                 "dwconv: bad geometry");
    Context::get().init(-1);
    Sync sy(stream);
    DeviceBuffer wt((size_t)C * K * K * dtype_size(dtype));
    launch_weight_dw(w, dtype, wt.get(), dtype, C, K, sy.s);
    DwConvArgs a{};
    a.in = in; a.wt = wt.get(); a.out = out; a.scale = scale; a.shift = shift;
    a.N = N; a.H = H; a.W = W; a.C = C; a.K = K; a.stride = stride; a.pad = pad;
    a.OH = (H + 2 * pad - K) / stride + 1; a.OW = (W + 2 * pad - K) / stride + 1; a.act = act;
    launch_dwconv(a, dtype, sy.s);
    NNCV_HIP_CHECK(hipStreamSynchronize(sy.s));  // the re-laid filter dies here
  });
}

int nncv_hip_scale_channels(int dtype, const void* x, const void* gate, void* out, int N, int HW, int C, void* stream) {
  return guarded([&] {
    NNCV_REQUIRE(x && gate && out, "null argument");
    Context::get().init(-1);
    Sync sy(stream);
    launch_scale_channels(x, gate, out, dtype, N, HW, C, sy.s);
    sy.finish();
  });
}

int nncv_hip_eltwise(int dtype, const void* a, const void* b, void* out, int64_t n, int act, void* stream) {
  return guarded([&] {
    NNCV_REQUIRE(a && out && n >= 0, "null argument");
    NNCV_REQUIRE(act >= kActNone && act <= kActSigmoid, "unknown activation");
    Context::get().init(-1);
    Sync sy(stream);
    launch_eltwise(a, b, out, dtype, n, act, sy.s);
    sy.finish();
  });
}

int nncv_hip_concat_slice(int dtype, const void* x, void* out, int64_t P, int C, int ldo, int c0, void* stream) {
  return guarded([&] {
    NNCV_REQUIRE(x && out && P >= 0, "null argument");
    Context::get().init(-1);
    Sync sy(stream);
    launch_concat_slice(x, out, dtype, P, C, ldo, c0, sy.s);
    sy.finish();
  });
}

int nncv_hip_upsample2x(int dtype, const void* x, void* out, int N, int H, int W, int C, int ldo, int c0, void* stream) {
  return guarded([&] {
    NNCV_REQUIRE(x && out, "null argument");
    Context::get().init(-1);
    Sync sy(stream);
    launch_upsample2x(x, out, dtype, N, H, W, C, ldo, c0, sy.s);
    sy.finish();
  });
}

int nncv_hip_maxpool(int dtype, const void* in, void* out, int N, int H, int W, int C, int K, int stride, int pad, void* stream) {
  return guarded([&] {
    NNCV_REQUIRE(in && out, "null argument");
    Context::get().init(-1);
    Sync sy(stream);
    launch_maxpool_nhwc(in, out, dtype, N, H, W, C, K, stride, pad, sy.s);
    sy.finish();
  });
}

}  // extern "C"
