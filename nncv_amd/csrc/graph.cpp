#include "graph.hpp"

#include <algorithm>

#include "arena_plan.hpp"

namespace nncv_hip {

namespace {

int round_up(int v, int m) { return (v + m - 1) / m * m; }

// shift[c] = (shift ? shift[c] : 0) + (scale ? scale[c] : 1) * bias[c]:  BN(conv + bias) folded
// into one scale/shift pair, or a plain bias turned into the epilogue's fp32 shift.
template <typename T>
__global__ void fold_bias_kernel(const T* __restrict__ bias, const float* __restrict__ scale, float* __restrict__ shift, int has_shift,
                                 int F) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= F) return;
  const float b = (float)bias[c];
  shift[c] = (has_shift ? shift[c] : 0.0f) + (scale ? scale[c] : 1.0f) * b;
}

const char* kind_name(int k) {
  switch (k) {
    case NNCV_HIP_OP_CONV: return "conv";
    case NNCV_HIP_OP_DWCONV: return "dwconv";
    case NNCV_HIP_OP_MAXPOOL: return "maxpool";
    case NNCV_HIP_OP_GAVGPOOL: return "gavgpool";
    case NNCV_HIP_OP_SCALE: return "scale";
    case NNCV_HIP_OP_ADD: return "add";
    case NNCV_HIP_OP_ACT: return "act";
    case NNCV_HIP_OP_CONCAT: return "concat";
    case NNCV_HIP_OP_UPSAMPLE2X: return "upsample2x";
    case NNCV_HIP_OP_YOLO_DETECT: return "yolo_detect";
    default: return "?";
  }
}

int n_inputs(int kind) {
  switch (kind) {
    case NNCV_HIP_OP_SCALE:
    case NNCV_HIP_OP_ADD: return 2;
    case NNCV_HIP_OP_CONCAT: return 4;
    case NNCV_HIP_OP_YOLO_DETECT: return 3;
    case NNCV_HIP_OP_CONV: return 2;  // second one (residual) optional
    default: return 1;
  }
}

}  // namespace

Graph::Graph(const GraphOp* ops, int n, int in_channels, const void* params, long long n_elems, int dt, hipStream_t s)
    : dt_(dt), c_in_(in_channels), dry_(params == nullptr) {
  NNCV_REQUIRE(dt == kF32 || dt == kF16, "graph: dtype must be 1 (fp32) or 2 (fp16)");
  NNCV_REQUIRE(ops && n > 0 && in_channels > 0, "graph: empty operator list");
  const int vn = dt == kF16 ? 8 : 4;
  const size_t es = dtype_size(dt);
  const char* blob = static_cast<const char*>(params);

  int max_id = 0;
  for (int i = 0; i < n; ++i) max_id = std::max(max_id, ops[i].out);
  NNCV_REQUIRE(max_id >= 1 && max_id <= 4 * n + 4, "graph: tensor ids out of range");
  n_tensors_ = max_id + 1;
  channels_.assign(n_tensors_, 0);
  logical_.assign(n_tensors_, 0);
  last_use_.assign(n_tensors_, -1);
  channels_[0] = round_up(in_channels, vn);
  logical_[0] = in_channels;
  nodes_.resize(n);

  auto param = [&](long long off, long long count, const std::string& what) -> const void* {
    NNCV_REQUIRE(off >= 0 && (dry_ || off + count <= n_elems), "graph: " + what + " lies outside the parameter blob");
    return blob + (size_t)off * es;
  };

  for (int i = 0; i < n; ++i) {
    const GraphOp& op = ops[i];
    const std::string where = "graph: operator " + std::to_string(i) + " (" + kind_name(op.kind) + "): ";
    Node& nd = nodes_[i];
    nd.op = op;
    NNCV_REQUIRE(op.kind >= NNCV_HIP_OP_CONV && op.kind <= NNCV_HIP_OP_YOLO_DETECT, where + "unknown kind");
    NNCV_REQUIRE(op.kind != NNCV_HIP_OP_YOLO_DETECT || i == n - 1, where + "must be the last operator");
    NNCV_REQUIRE(op.out >= 1 && op.out < n_tensors_ && channels_[op.out] == 0, where + "`out` must be a new tensor id");
    NNCV_REQUIRE(op.act >= kActNone && op.act <= kActSigmoid, where + "unknown activation");
    const int ni = n_inputs(op.kind);
    for (int k = 0; k < 4; ++k) {
      const int t = op.in[k];
      if (k >= ni) {
        NNCV_REQUIRE(t < 0, where + "too many inputs");
        continue;
      }
      const bool optional =
          k > 0 && (op.kind == NNCV_HIP_OP_CONV || op.kind == NNCV_HIP_OP_CONCAT || op.kind == NNCV_HIP_OP_YOLO_DETECT);
      if (t < 0 && optional) continue;
      NNCV_REQUIRE(t >= 0 && t < n_tensors_ && channels_[t] > 0, where + "input is not a tensor defined earlier");
      last_use_[t] = i;
    }
    const int C = channels_[op.in[0]];
    nd.C = C;
    int Cout = C;       // logical channels of the result
    int Cstored = -1;   // stored channels when they differ
    // Only convolutions (which know the real count from their filters), the Detect decode and the
    // network output may read a tensor that is stored with padding channels.
    if (op.kind != NNCV_HIP_OP_CONV && op.kind != NNCV_HIP_OP_YOLO_DETECT)
      for (int k = 0; k < ni; ++k)
        if (op.in[k] >= 0)
          NNCV_REQUIRE(logical_[op.in[k]] == channels_[op.in[k]],
                       where + "channel count of an input must be a multiple of the 16-byte vector");
    switch (op.kind) {
      case NNCV_HIP_OP_CONV: {
        NNCV_REQUIRE(op.F > 0, where + "F must be positive");
        NNCV_REQUIRE(op.K >= 1 && op.K <= 11 && op.stride >= 1 && op.pad >= 0, where + "bad geometry");
        NNCV_REQUIRE(op.in[1] < 0 || logical_[op.in[1]] == op.F, where + "residual has another channel count");
        Cout = op.F;
        Cstored = round_up(op.F, vn);
        const int Cl = logical_[op.in[0]];  // channels the filters really have
        const void* w = param(op.w, (long long)op.F * Cl * op.K * op.K, where + "w");
        if (dry_) break;
        nd.wt.reset((size_t)Cstored * op.K * op.K * C * es);
        NNCV_HIP_CHECK(hipMemsetAsync(nd.wt.get(), 0, nd.wt.bytes(), s));
        launch_weight_frsc(w, dt, nd.wt.get(), dt, op.F, Cl, op.K, op.K, C, s);
        if (op.K == 3 && (op.stride == 1 || op.stride == 2) && op.pad == 1 && Cl == C && Cstored == op.F && C % (128 / (int)es) == 0) {
          nd.wfrag.reset((size_t)((op.F + 63) / 64) * 64 * 9 * C * es);
          launch_weight_frag3x3(w, dt, nd.wfrag.get(), dt, op.F, C, s);
          if (dt == kF16 && op.stride == 1 && C % 64 == 0 && op.F % 32 == 0) {
            nd.wfrag32.reset(weight_frag32_bytes(op.F, C));
            launch_weight_frag32(w, dt, nd.wfrag32.get(), op.F, C, s);
          }
        }
        break;
      }
      case NNCV_HIP_OP_DWCONV: {
        NNCV_REQUIRE(op.K == 3 || op.K == 5, where + "K must be 3 or 5");
        NNCV_REQUIRE(op.stride >= 1 && op.pad >= 0, where + "bad geometry");
        const void* w = param(op.w, (long long)C * op.K * op.K, where + "w");
        if (dry_) break;
        nd.wt.reset((size_t)C * op.K * op.K * es);
        launch_weight_dw(w, dt, nd.wt.get(), dt, C, op.K, s);
        break;
      }
      case NNCV_HIP_OP_MAXPOOL:
        NNCV_REQUIRE(op.K >= 1 && op.stride >= 1 && op.pad >= 0 && 2 * op.pad <= op.K, where + "bad geometry");
        break;
      case NNCV_HIP_OP_SCALE:
      case NNCV_HIP_OP_ADD:
        NNCV_REQUIRE(channels_[op.in[1]] == C, where + "operands have different channel counts");
        break;
      case NNCV_HIP_OP_CONCAT:
        for (int k = 1; k < 4; ++k)
          if (op.in[k] >= 0) Cout += channels_[op.in[k]];
        break;
      case NNCV_HIP_OP_YOLO_DETECT: {
        NNCV_REQUIRE(op.K >= 1 && op.K <= 4 && op.F >= 5, where + "K anchors (1..4) of F >= 5 values each");
        int levels = 0;
        for (int k = 0; k < 3; ++k)
          if (op.in[k] >= 0) {
            NNCV_REQUIRE(k == levels, where + "levels must be in[0], in[1], ... without gaps");
            NNCV_REQUIRE(logical_[op.in[k]] == op.K * op.F, where + "a head must have K * F channels");
            ++levels;
          }
        // anchors and strides are tiny and needed as kernel arguments: read them back once
        const void* an = param(op.w, (long long)levels * op.K * 2, where + "anchors");
        const void* st = param(op.bias, levels, where + "strides");
        std::vector<float> anchors((size_t)levels * op.K * 2), strides(levels);
        Cout = op.F;
        Cstored = op.F;
        if (dry_) break;
        DeviceBuffer tmp((anchors.size() + strides.size()) * 4);
        launch_cast(an, dt, tmp.get(), kF32, (long long)anchors.size(), s);
        launch_cast(st, dt, tmp.as<float>() + anchors.size(), kF32, levels, s);
        NNCV_HIP_CHECK(hipMemcpyAsync(anchors.data(), tmp.get(), anchors.size() * 4, hipMemcpyDeviceToHost, s));
        NNCV_HIP_CHECK(hipMemcpyAsync(strides.data(), tmp.as<float>() + anchors.size(), strides.size() * 4, hipMemcpyDeviceToHost, s));
        NNCV_HIP_CHECK(hipStreamSynchronize(s));
        detect_stride_ = strides;
        detect_anchor_wh_.resize(anchors.size());
        for (int l = 0; l < levels; ++l)
          for (int q = 0; q < op.K * 2; ++q) detect_anchor_wh_[l * op.K * 2 + q] = anchors[l * op.K * 2 + q] * strides[l];
        break;
      }
      default: break;
    }
    if (!dry_ && (op.kind == NNCV_HIP_OP_CONV || op.kind == NNCV_HIP_OP_DWCONV)) {
      const int F = Cout, Fs = Cstored > 0 ? Cstored : Cout;
      if (op.gamma >= 0) {
        NNCV_REQUIRE(op.beta >= 0 && op.mean >= 0 && op.var >= 0, where + "BatchNorm needs gamma, beta, mean and var");
        nd.scale.reset((size_t)Fs * 4);
        nd.shift.reset((size_t)Fs * 4);
        launch_fill_f32(nd.scale.as<float>(), 0.0f, Fs, s);
        launch_fill_f32(nd.shift.as<float>(), 0.0f, Fs, s);
        launch_bn_fold(param(op.gamma, F, where + "gamma"), param(op.beta, F, where + "beta"), param(op.mean, F, where + "mean"),
                       param(op.var, F, where + "var"), dt, nd.scale.as<float>(), nd.shift.as<float>(), F, s, op.eps);
      }
      if (op.bias >= 0) {
        const void* b = param(op.bias, F, where + "bias");
        const bool had = nd.shift.get() != nullptr;
        if (!had) {
          nd.shift.reset((size_t)Fs * 4);
          launch_fill_f32(nd.shift.as<float>(), 0.0f, Fs, s);
        }
        const unsigned grid = (unsigned)((F + 255) / 256);
        if (dt == kF16)
          hipLaunchKernelGGL((fold_bias_kernel<half_t>), dim3(grid), dim3(256), 0, s, (const half_t*)b, nd.scale.as<float>(),
                             nd.shift.as<float>(), had ? 1 : 0, F);
        else
          hipLaunchKernelGGL((fold_bias_kernel<float>), dim3(grid), dim3(256), 0, s, (const float*)b, nd.scale.as<float>(),
                             nd.shift.as<float>(), had ? 1 : 0, F);
        NNCV_HIP_CHECK(hipGetLastError());
      }
    }
    if (Cstored < 0) Cstored = Cout;
    NNCV_REQUIRE(Cstored % vn == 0 || op.kind == NNCV_HIP_OP_YOLO_DETECT,
                 where + "channel count must be a multiple of the 16-byte vector");
    channels_[op.out] = Cstored;
    logical_[op.out] = Cout;
  }
  for (int t = 1; t < n_tensors_; ++t) NNCV_REQUIRE(channels_[t] > 0, "graph: tensor " + std::to_string(t) + " is never produced");

  // squeeze-excitation blocks
  static const bool no_se = getenv("NNCV_HIP_NO_SE_FUSION") != nullptr;
  std::vector<int> readers(n_tensors_, 0);
  for (int i = 0; i < n; ++i)
    for (int k = 0; k < 4; ++k)
      if (ops[i].in[k] >= 0) ++readers[ops[i].in[k]];
  auto plain_fc = [&](const GraphOp& o, int in) {
    return o.kind == NNCV_HIP_OP_CONV && o.K == 1 && o.stride == 1 && o.pad == 0 && o.in[0] == in && o.in[1] < 0 && o.bias >= 0 &&
           o.gamma < 0 && readers[in] == 1;
  };
  for (int i = 0; !no_se && i + 3 < n; ++i) {
    const GraphOp &p0 = ops[i], &f1 = ops[i + 1], &f2 = ops[i + 2], &sc = ops[i + 3];
    if (p0.kind != NNCV_HIP_OP_GAVGPOOL || p0.in[0] == 0 || !plain_fc(f1, p0.out) || !plain_fc(f2, f1.out)) continue;
    if (sc.kind != NNCV_HIP_OP_SCALE || sc.in[0] != p0.in[0] || sc.in[1] != f2.out || readers[f2.out] != 1) continue;
    if (f2.F != channels_[p0.in[0]] || !se_block_applicable(dt, 1, f2.F, f1.F)) continue;
    nodes_[i].se_head = true;
    nodes_[i + 1].skip = nodes_[i + 2].skip = nodes_[i + 3].skip = true;
    i += 3;
  }

  // an image convolution (fp16, <= 4 channels, stride 2) that is the only reader of the input
  static const bool no_pairs = getenv("NNCV_HIP_NO_PAIR_STEM") != nullptr;
  if (!no_pairs && dt == kF16 && c_in_ <= 4 && readers[0] == 1)
    for (int i = 0; i < n; ++i)
      if (ops[i].kind == NNCV_HIP_OP_CONV && ops[i].in[0] == 0 && ops[i].stride == 2 && ops[i].in[1] < 0) {
        const GraphOp& o = ops[i];
        const int Fp = channels_[o.out], S2 = (o.K + (o.pad & 1) + 1) / 2;
        pair_stem_ = i;
        if (dry_) continue;
        nodes_[i].wt_pairs.reset((size_t)Fp * o.K * S2 * 8 * es);
        launch_weight_pairs(param(o.w, (long long)o.F * c_in_ * o.K * o.K, "pair stem w"), dt, nodes_[i].wt_pairs.get(), o.F, Fp, c_in_,
                            o.K, o.pad, s);
      }

  // x + act(conv(.)): the ADD rides in the convolution's epilogue
  static const bool no_add = getenv("NNCV_HIP_NO_ADD_FUSION") != nullptr;
  for (int i = 0; !no_add && i + 1 < n; ++i) {
    const GraphOp &cv = ops[i], &ad = ops[i + 1];
    if (cv.kind != NNCV_HIP_OP_CONV || cv.in[1] >= 0 || ad.kind != NNCV_HIP_OP_ADD || ad.act != kActNone) continue;
    if (readers[cv.out] != 1 || logical_[cv.out] != channels_[cv.out]) continue;
    const int other = ad.in[0] == cv.out ? ad.in[1] : (ad.in[1] == cv.out ? ad.in[0] : -1);
    if (other < 0 || other == cv.out) continue;
    nodes_[i].add_res = other;
    nodes_[i].add_out = ad.out;
    nodes_[i + 1].skip = true;
  }

  // concatenation views
  view_of_.assign(n_tensors_, -1);
  view_c0_.assign(n_tensors_, 0);
  static const bool no_views = getenv("NNCV_HIP_NO_CONCAT_VIEWS") != nullptr;
  if (!no_views) {
    std::vector<int> producer(n_tensors_, -1), cat_uses(n_tensors_, 0);
    for (int i = 0; i < n; ++i) {
      producer[nodes_[i].add_out >= 0 ? nodes_[i].add_out : ops[i].out] = i;
      if (ops[i].kind == NNCV_HIP_OP_CONCAT)
        for (int k = 0; k < 4; ++k)
          if (ops[i].in[k] >= 0) ++cat_uses[ops[i].in[k]];
    }
    // may operator i read tensor t at a pitch / write its result at a pitch?
    auto reads_pitched = [&](int i, int t) {
      const GraphOp& o = ops[i];
      if (nodes_[i].skip)  // merged into its predecessor: the residual of a conv + ADD pair shares the result's pitch
        return i > 0 && nodes_[i - 1].add_out >= 0 && nodes_[i - 1].add_res != t;
      switch (o.kind) {
        case NNCV_HIP_OP_CONV: return o.in[1] != t;  // not as the residual
        case NNCV_HIP_OP_MAXPOOL:
        case NNCV_HIP_OP_UPSAMPLE2X:
        case NNCV_HIP_OP_ADD:
        case NNCV_HIP_OP_ACT:
        case NNCV_HIP_OP_CONCAT:
        case NNCV_HIP_OP_YOLO_DETECT: return true;
        default: return false;
      }
    };
    auto writes_pitched = [&](int i) {
      const GraphOp& o = ops[i];
      if (nodes_[i].se_head || nodes_[i].skip) return false;
      switch (o.kind) {
        case NNCV_HIP_OP_CONV: return o.in[1] < 0 && nodes_[i].add_res < 0;  // residual and result share one pitch
        case NNCV_HIP_OP_MAXPOOL:
        case NNCV_HIP_OP_UPSAMPLE2X:
        case NNCV_HIP_OP_ADD:
        case NNCV_HIP_OP_ACT:
        case NNCV_HIP_OP_CONCAT: return true;
        default: return false;
      }
    };
    for (int i = 0; i < n; ++i) {
      if (ops[i].kind != NNCV_HIP_OP_CONCAT) continue;
      int c0 = 0;
      for (int k = 0; k < 4; ++k) {
        const int t = ops[i].in[k];
        if (t < 0) continue;
        bool ok = t != 0 && cat_uses[t] == 1 && producer[t] >= 0 && writes_pitched(producer[t]) && logical_[t] == channels_[t];
        for (int j = 0; ok && j < n; ++j)
          for (int q = 0; q < 4; ++q)
            if (ops[j].in[q] == t && !reads_pitched(j, t)) ok = false;
        if (ok) {
          view_of_[t] = ops[i].out;
          view_c0_[t] = c0;
        }
        c0 += channels_[t];
      }
    }
  }
}

void Graph::root_of(int t, int* root, int* c0) const {
  int off = 0;
  while (view_of_[t] >= 0) {
    off += view_c0_[t];
    t = view_of_[t];
  }
  *root = t;
  *c0 = off;
}

const Graph::Plan& Graph::plan_of(int N, int H, int W) const {
  for (const Plan& p : plans_)
    if (p.N == N && p.H == H && p.W == W) return p;
  NNCV_REQUIRE(N >= 1 && H >= 1 && W >= 1, "graph: empty input");
  Plan p;
  p.N = N; p.H = H; p.W = W;
  p.dims.assign(n_tensors_, Dims{0, 0, 0});
  p.dims[0] = Dims{channels_[0], H, W};
  const int n = (int)nodes_.size();
  for (int i = 0; i < n; ++i) {
    const GraphOp& op = nodes_[i].op;
    const std::string where = "graph: operator " + std::to_string(i) + " (" + kind_name(op.kind) + "): ";
    const Dims a = p.dims[op.in[0]];
    Dims o{channels_[op.out], a.H, a.W};
    switch (op.kind) {
      case NNCV_HIP_OP_CONV:
      case NNCV_HIP_OP_DWCONV:
      case NNCV_HIP_OP_MAXPOOL:
        NNCV_REQUIRE(a.H + 2 * op.pad >= op.K && a.W + 2 * op.pad >= op.K, where + "image smaller than the window");
        o.H = (a.H + 2 * op.pad - op.K) / op.stride + 1;
        o.W = (a.W + 2 * op.pad - op.K) / op.stride + 1;
        if (op.kind == NNCV_HIP_OP_CONV && op.in[1] >= 0)
          NNCV_REQUIRE(p.dims[op.in[1]].H == o.H && p.dims[op.in[1]].W == o.W, where + "residual has another size");
        break;
      case NNCV_HIP_OP_GAVGPOOL: o.H = o.W = 1; break;
      case NNCV_HIP_OP_SCALE:
        NNCV_REQUIRE(p.dims[op.in[1]].H == 1 && p.dims[op.in[1]].W == 1, where + "the gate must be [N,C,1,1]");
        break;
      case NNCV_HIP_OP_ADD:
        NNCV_REQUIRE(p.dims[op.in[1]].H == a.H && p.dims[op.in[1]].W == a.W, where + "operands have different sizes");
        break;
      case NNCV_HIP_OP_CONCAT:
        for (int k = 1; k < 4; ++k)
          if (op.in[k] >= 0)
            NNCV_REQUIRE(p.dims[op.in[k]].H == a.H && p.dims[op.in[k]].W == a.W, where + "operands have different sizes");
        break;
      case NNCV_HIP_OP_UPSAMPLE2X: o.H = 2 * a.H; o.W = 2 * a.W; break;
      case NNCV_HIP_OP_YOLO_DETECT: {  // [N, boxes, F]: reported as channels = boxes, height = F, width = 1
        long long boxes = 0;
        for (int k = 0; k < 3; ++k)
          if (op.in[k] >= 0) boxes += (long long)op.K * p.dims[op.in[k]].H * p.dims[op.in[k]].W;
        NNCV_REQUIRE(boxes * op.F * N < (1ll << 31), where + "tensor too large");
        o.C = (int)boxes; o.H = op.F; o.W = 1;
        break;
      }
      default: break;
    }
    NNCV_REQUIRE((long long)N * o.H * o.W * o.C < (1ll << 31), where + "tensor too large");
    p.dims[op.out] = o;
  }
  // Lifetimes in operator steps: step 0 lays the input out as NHWC, step i + 1 is operator i,
  // step n + 1 converts the output.  A tensor is live from the step that writes it to the last
  // step that reads it, so an operator's output never shares memory with any of its inputs.
  std::vector<TensorLife> life(n_tensors_);
  const size_t es = dtype_size(dt_);
  life[0] = TensorLife{0, std::max(0, last_use_[0] + 1), (size_t)N * H * W * channels_[0] * es, 0};
  for (int i = 0; i < n; ++i) {
    const int t = nodes_[i].op.out;
    const Dims d = p.dims[t];
    life[t] = TensorLife{i + 1, std::max(i + 1, last_use_[t] + 1), (size_t)N * d.H * d.W * d.C * es, 0};
    if (nodes_[i].op.kind == NNCV_HIP_OP_YOLO_DETECT) life[t].bytes = 256;  // written straight to the caller's buffer
  }
  // Operators that were merged into an earlier launch write their result at that launch's step, so the
  // result is live from there: the tail of a squeeze-excitation block (written by the block's one launch
  // at the pooling operator's step), the ADD of a convolution + ADD pair (written by the convolution),
  // the later two of three chained 5x5 stride-1 pad-2 max-pools (one launch writes all three results).
  // Without this the planner sees the merged result and an input of the earlier launch as disjoint in
  // time and may lay one over the other.
  for (int i = 0; i < n; ++i) {
    if (nodes_[i].se_head && i + 3 < n) life[nodes_[i + 3].op.out].first_op = i + 1;
    if (nodes_[i].add_out >= 0) life[nodes_[i].add_out].first_op = std::min(life[nodes_[i].add_out].first_op, i + 1);
  }
  {
    auto pool5 = [&](int k, int in) {
      return k < n && !nodes_[k].skip && nodes_[k].op.kind == NNCV_HIP_OP_MAXPOOL && nodes_[k].op.K == 5 && nodes_[k].op.stride == 1 &&
             nodes_[k].op.pad == 2 && (in < 0 || nodes_[k].op.in[0] == in);
    };
    for (int i = 0; i + 2 < n; ++i)
      if (pool5(i, -1) && pool5(i + 1, nodes_[i].op.out) && pool5(i + 2, nodes_[i + 1].op.out)) {
        life[nodes_[i + 1].op.out].first_op = i + 1;
        life[nodes_[i + 2].op.out].first_op = i + 1;
      }
  }
  life[nodes_[n - 1].op.out].last_op = n + 1;
  // a tensor that lives inside a concatenated one has no memory of its own; the concatenated
  // tensor is live from its first such input to the last reader of any of them
  for (int t = 1; t < n_tensors_; ++t) {
    if (view_of_[t] < 0) continue;
    int root, c0;
    root_of(t, &root, &c0);
    life[root].first_op = std::min(life[root].first_op, life[t].first_op);
    life[root].last_op = std::max(life[root].last_op, life[t].last_op);
  }
  for (int t = 1; t < n_tensors_; ++t)
    if (view_of_[t] >= 0) life[t] = TensorLife{life[t].first_op, life[t].first_op, 0, 0};
  for (int i = 0; i < n; ++i)  // the output of a convolution that was merged with its ADD is never stored
    if (nodes_[i].add_out >= 0) life[nodes_[i].op.out] = TensorLife{i + 1, i + 1, 0, 0};
  // memory is handed on a few launches after its last reader, not at once (arena_plan.hpp)
  for (int t = 0; t < n_tensors_; ++t)
    if (life[t].bytes > 0) life[t].last_op = std::min(n + 1, life[t].last_op + arena_linger());
  p.total = plan_offsets(life, 256);
  p.offset.resize(n_tensors_);
  p.root_bytes.resize(n_tensors_);
  for (int t = 0; t < n_tensors_; ++t) {
    int root, c0;
    root_of(t, &root, &c0);
    p.offset[t] = life[root].offset + (size_t)c0 * es;
    p.root_bytes[t] = life[root].bytes;
  }
  check_plan(p);
  if (plans_.size() >= 8) plans_.erase(plans_.begin());
  plans_.push_back(std::move(p));
  return plans_.back();
}

// The tensors one launch of forward() touches: what it writes and what it reads.
void Graph::launch_io(int i, std::vector<int>* writes, std::vector<int>* reads) const {
  writes->clear();
  reads->clear();
  const int n = (int)nodes_.size();
  const Node& nd = nodes_[i];
  const GraphOp& op = nd.op;
  if (nd.skip) return;
  if (nd.se_head) {
    reads->push_back(op.in[0]);
    writes->push_back(nodes_[i + 3].op.out);
    return;
  }
  for (int k = 0; k < 4; ++k)  // inputs of a CONCAT that already live in its result are not copied
    if (op.in[k] >= 0 && !(op.kind == NNCV_HIP_OP_CONCAT && view_of_[op.in[k]] == op.out)) reads->push_back(op.in[k]);
  if (nd.add_res >= 0) reads->push_back(nd.add_res);
  if (op.kind == NNCV_HIP_OP_YOLO_DETECT) return;  // writes the caller's buffer
  writes->push_back(nd.add_out >= 0 ? nd.add_out : op.out);
  auto pool5 = [&](int k, int in) {
    return k < n && !nodes_[k].skip && nodes_[k].op.kind == NNCV_HIP_OP_MAXPOOL && nodes_[k].op.K == 5 && nodes_[k].op.stride == 1 &&
           nodes_[k].op.pad == 2 && (in < 0 || nodes_[k].op.in[0] == in);
  };
  if (pool5(i, -1) && pool5(i + 1, op.out) && pool5(i + 2, nodes_[i + 1].op.out)) {
    writes->push_back(nodes_[i + 1].op.out);
    writes->push_back(nodes_[i + 2].op.out);
  }
}

// No launch may write memory that it also reads (a 3x3 convolution in place is a race between
// workgroups on the halo rows) or that another tensor it writes occupies.  Two tensors inside the same
// concatenated tensor are channel slices of the same rows and must not share channels; everything
// else is compared as whole byte ranges.
void Graph::check_plan(const Plan& p) const {
  const size_t es = dtype_size(dt_);
  auto clash = [&](int a, int b) {
    int ra, ca, rb, cb;
    root_of(a, &ra, &ca);
    root_of(b, &rb, &cb);
    if (ra == rb) return a == b || (ca < cb + channels_[b] && cb < ca + channels_[a]);
    const size_t a0 = p.offset[a] - (size_t)ca * es, b0 = p.offset[b] - (size_t)cb * es;
    return p.root_bytes[a] > 0 && p.root_bytes[b] > 0 && a0 < b0 + p.root_bytes[b] && b0 < a0 + p.root_bytes[a];
  };
  std::vector<int> w, r;
  for (int i = 0; i < (int)nodes_.size(); ++i) {
    launch_io(i, &w, &r);
    for (size_t x = 0; x < w.size(); ++x) {
      for (int t : r)
        NNCV_REQUIRE(!clash(w[x], t), "graph: workspace plan lays the result of operator " + std::to_string(i) + " (tensor " +
                                          std::to_string(w[x]) + ") over its input tensor " + std::to_string(t));
      for (size_t y = x + 1; y < w.size(); ++y)
        NNCV_REQUIRE(!clash(w[x], w[y]), "graph: workspace plan lays two results of operator " + std::to_string(i) + " over each other");
    }
  }
}

size_t Graph::describe_plan(int N, int H, int W, long long* tensor_info, int* launch_dst) const {
  const Plan& p = plan_of(N, H, W);
  for (int t = 0; t < n_tensors_; ++t) {
    int root, c0;
    root_of(t, &root, &c0);
    tensor_info[4 * t + 0] = root;
    tensor_info[4 * t + 1] = (long long)p.offset[t];
    tensor_info[4 * t + 2] = (long long)p.root_bytes[t];
    tensor_info[4 * t + 3] = c0;
  }
  std::vector<int> w, r;
  for (int i = 0; i < (int)nodes_.size(); ++i) {
    launch_io(i, &w, &r);
    launch_dst[i] = w.empty() ? -1 : w[0];
  }
  return p.total;
}

void Graph::output_shape(int H, int W, int* C, int* OH, int* OW) const {
  const Plan& p = plan_of(1, H, W);
  const int t = nodes_.back().op.out;
  const Dims d = p.dims[t];
  *C = nodes_.back().op.kind == NNCV_HIP_OP_YOLO_DETECT ? d.C : logical_[t];
  *OH = d.H; *OW = d.W;
}

size_t Graph::workspace_bytes(int N, int H, int W) const { return plan_of(N, H, W).total; }

void Graph::forward(const void* src, int N, int H, int W, float* out, void* ws, hipStream_t s) const {
  const Plan& p = plan_of(N, H, W);
  char* base = static_cast<char*>(ws);
  auto at = [&](int t) -> void* { return base + p.offset[t]; };
  // elements between consecutive pixels of tensor t: its own channel count, or that of the
  // concatenated tensor it lives in
  auto pitch = [&](int t) {
    int root, c0;
    root_of(t, &root, &c0);
    return channels_[root];
  };
  const bool pairs = pair_stem_ >= 0 && W % 2 == 0;
  if (pairs)
    launch_image_to_nhwc(src, at(0), dt_, N, c_in_, H, W, s, 4);
  else if (image_to_nhwc_applicable(dt_, c_in_))
    launch_image_to_nhwc(src, at(0), dt_, N, c_in_, H, W, s);
  else
    launch_relayout(src, dt_, strides_of(kNCHW, c_in_, H, W), at(0), dt_, strides_of(kNHWC, channels_[0], H, W), N, c_in_,
                    channels_[0], H, W, false, s);
  for (size_t i = 0; i < nodes_.size(); ++i) {
    const Node& nd = nodes_[i];
    const GraphOp& op = nd.op;
    const Dims a = p.dims[op.in[0]], o = p.dims[op.out];
    if (nd.skip) continue;
    if (nd.se_head) {
      const Node &f1 = nodes_[i + 1], &f2 = nodes_[i + 2];
      SeArgs e{};
      e.x = at(op.in[0]); e.w1 = f1.wt.get(); e.b1 = f1.shift.as<float>(); e.w2 = f2.wt.get(); e.b2 = f2.shift.as<float>();
      e.out = at(nodes_[i + 3].op.out);
      e.N = N; e.HW = a.H * a.W; e.C = a.C; e.SQ = f1.op.F; e.act1 = f1.op.act; e.act2 = f2.op.act;
      launch_se_block(e, dt_, s);
      continue;
    }
    switch (op.kind) {
      case NNCV_HIP_OP_CONV: {
        IgemmArgs g{};
        const int dst = nd.add_out >= 0 ? nd.add_out : op.out;
        g.in = at(op.in[0]); g.wt = nd.wt.get(); g.wt_frag = nd.wfrag.get(); g.wt_frag32 = nd.wfrag32.get(); g.out = at(dst);
        g.scale = nd.scale.as<float>(); g.shift = nd.shift.as<float>();
        g.residual = nd.add_res >= 0 ? at(nd.add_res) : (op.in[1] >= 0 ? at(op.in[1]) : nullptr);
        // padding filters (zero rows, zero scale/shift) are computed like any other: o.C >= op.F
        g.N = N; g.H = a.H; g.W = a.W; g.C = a.C; g.F = o.C; g.R = g.S = op.K; g.OH = o.H; g.OW = o.W;
        g.stride_h = g.stride_w = op.stride; g.pad_h = g.pad_w = op.pad;
        g.relu = nd.add_res >= 0 ? (op.act | kActResidualAfter) : op.act;
        g.ldo = pitch(dst); g.batch = 1;
        if (pairs && (int)i == pair_stem_) {  // the image as [N][H][W/2][2 pixels x 4 channels]
          g.wt = nd.wt_pairs.get();
          g.W = a.W / 2; g.C = 8; g.S = (op.K + (op.pad & 1) + 1) / 2;
          g.stride_w = 1; g.pad_w = (op.pad + 1) / 2;
        }
        if (pitch(op.in[0]) != a.C) {  // the input is a slice of a wider tensor
          g.pix_stride = pitch(op.in[0]);
          const unsigned long long span = (unsigned long long)N * a.H * a.W * g.pix_stride * dtype_size(dt_);
          g.in_bytes = span < 0xffffffffull ? (unsigned)span : 0xffffffffu;
        }
        g.alg_flops = 2.0 * N * o.H * o.W * op.F * (double)op.K * op.K * logical_[op.in[0]];
        launch_igemm(g, dt_, dt_, s);
        break;
      }
      case NNCV_HIP_OP_DWCONV: {
        DwConvArgs d{};
        d.in = at(op.in[0]); d.wt = nd.wt.get(); d.out = at(op.out);
        d.scale = nd.scale.as<float>(); d.shift = nd.shift.as<float>();
        d.N = N; d.H = a.H; d.W = a.W; d.C = a.C; d.K = op.K; d.stride = op.stride; d.pad = op.pad; d.OH = o.H; d.OW = o.W;
        d.act = op.act;
        launch_dwconv(d, dt_, s);
        break;
      }
      case NNCV_HIP_OP_MAXPOOL: {
        // three 5x5 stride-1 pad-2 pools in a row (SPPF): one launch that keeps all three results
        auto pool5 = [&](size_t k, int in) {
          return k < nodes_.size() && !nodes_[k].skip && nodes_[k].op.kind == NNCV_HIP_OP_MAXPOOL && nodes_[k].op.K == 5 &&
                 nodes_[k].op.stride == 1 && nodes_[k].op.pad == 2 && (in < 0 || nodes_[k].op.in[0] == in);
        };
        if (pool5(i, -1) && pool5(i + 1, op.out) && pool5(i + 2, nodes_[i + 1].op.out) && maxpool5_chain3_applicable(dt_, a.H, a.W, a.C)) {
          const int t2 = nodes_[i + 1].op.out, t3 = nodes_[i + 2].op.out;
          launch_maxpool5_chain3(at(op.in[0]), at(op.out), at(t2), at(t3), dt_, N, a.H, a.W, a.C, pitch(op.in[0]), pitch(op.out),
                                 pitch(t2), pitch(t3), s);
          i += 2;
          break;
        }
        launch_maxpool_nhwc(at(op.in[0]), at(op.out), dt_, N, a.H, a.W, a.C, op.K, op.stride, op.pad, s, pitch(op.in[0]),
                            pitch(op.out));
        break;
      }
      case NNCV_HIP_OP_GAVGPOOL:
        launch_global_avgpool_nhwc(at(op.in[0]), at(op.out), dt_, N, a.H * a.W, a.C, s);
        break;
      case NNCV_HIP_OP_SCALE:
        launch_scale_channels(at(op.in[0]), at(op.in[1]), at(op.out), dt_, N, a.H * a.W, a.C, s);
        break;
      case NNCV_HIP_OP_ADD:
        launch_eltwise_pitched(at(op.in[0]), pitch(op.in[0]), at(op.in[1]), pitch(op.in[1]), at(op.out), pitch(op.out), dt_,
                               (long long)N * a.H * a.W, a.C, op.act, s);
        break;
      case NNCV_HIP_OP_ACT:
        launch_eltwise_pitched(at(op.in[0]), pitch(op.in[0]), nullptr, pitch(op.in[0]), at(op.out), pitch(op.out), dt_,
                               (long long)N * a.H * a.W, a.C, op.act, s);
        break;
      case NNCV_HIP_OP_CONCAT: {
        int c0 = 0;
        for (int k = 0; k < 4; ++k) {
          if (op.in[k] < 0) continue;
          const int Ck = p.dims[op.in[k]].C;
          // inputs that live in this tensor already are in place; the others are copied into their slice
          if (view_of_[op.in[k]] != op.out)
            launch_concat_slice(at(op.in[k]), static_cast<char*>(at(op.out)) + (size_t)c0 * dtype_size(dt_), dt_,
                                (long long)N * o.H * o.W, Ck, pitch(op.out), 0, s, pitch(op.in[k]));
          c0 += Ck;
        }
        break;
      }
      case NNCV_HIP_OP_UPSAMPLE2X:
        launch_upsample2x(at(op.in[0]), at(op.out), dt_, N, a.H, a.W, a.C, pitch(op.out), 0, s, pitch(op.in[0]));
        break;
      case NNCV_HIP_OP_YOLO_DETECT: {
        long long box0 = 0;
        for (int k = 0; k < 3 && op.in[k] >= 0; ++k) {
          const Dims h = p.dims[op.in[k]];
          DetectArgs d{};
          d.head = at(op.in[k]); d.out = out; d.N = N; d.H = h.H; d.W = h.W; d.A = op.K; d.F = op.F; d.ldc = pitch(op.in[k]);
          d.box0 = box0; d.boxes_total = o.C; d.stride = detect_stride_[k];
          for (int q = 0; q < op.K * 2; ++q) d.anchor_wh[q] = detect_anchor_wh_[k * op.K * 2 + q];
          launch_yolo_detect(d, dt_, s);
          box0 += (long long)op.K * h.H * h.W;
        }
        break;
      }
      default: fail("graph: unknown operator kind");
    }
  }
  if (nodes_.back().op.kind == NNCV_HIP_OP_YOLO_DETECT) return;  // already in the caller's buffer, fp32
  const int t = nodes_.back().op.out;
  const Dims d = p.dims[t];
  const int Cl = logical_[t];
  launch_relayout(at(t), dt_, strides_of(kNHWC, d.C, d.H, d.W), out, kF32, strides_of(kNCHW, Cl, d.H, d.W), N, Cl, Cl, d.H, d.W,
                  false, s);
}

// ---------------------------------------------------------------------------------------------
// MobileNetV3-small, the network of tests/Nets/MobileNetV3.mlir (torchvision's mobilenet_v3_small:
// 52 convolutions of which 11 depthwise, 9 squeeze-excitation blocks, BatchNorm epsilon 1e-3,
// two Linear layers).  Parameter order = state_dict order without num_batches_tracked:
//   conv weight, then BN weight / bias / running_mean / running_var; SE fc1 weight, bias, fc2
//   weight, bias; classifier weight, bias.
// ---------------------------------------------------------------------------------------------
std::vector<GraphOp> mobilenetv3_small_ops(long long* n_elems) {
  std::vector<GraphOp> ops;
  long long off = 0;
  int next = 1;
  const float eps = 1e-3f;
  auto blank = [](int kind) {
    GraphOp o{};
    o.kind = kind;
    o.in[0] = o.in[1] = o.in[2] = o.in[3] = -1;
    o.w = o.bias = o.gamma = o.beta = o.mean = o.var = -1;
    return o;
  };
  // conv / dwconv followed by BatchNorm
  auto conv_bn = [&](int in, int C, int F, int K, int stride, bool depthwise, int act, int residual) {
    GraphOp o = blank(depthwise ? NNCV_HIP_OP_DWCONV : NNCV_HIP_OP_CONV);
    o.in[0] = in; o.in[1] = residual; o.out = next++;
    o.F = F; o.K = K; o.stride = stride; o.pad = (K - 1) / 2; o.act = act; o.eps = eps;
    o.w = off; off += (long long)F * (depthwise ? 1 : C) * K * K;
    o.gamma = off; off += F;
    o.beta = off; off += F;
    o.mean = off; off += F;
    o.var = off; off += F;
    ops.push_back(o);
    return o.out;
  };
  // 1x1 convolution / Linear with bias
  auto fc = [&](int in, int C, int F, int act) {
    GraphOp o = blank(NNCV_HIP_OP_CONV);
    o.in[0] = in; o.out = next++;
    o.F = F; o.K = 1; o.stride = 1; o.pad = 0; o.act = act;
    o.w = off; off += (long long)F * C;
    o.bias = off; off += F;
    ops.push_back(o);
    return o.out;
  };
  auto simple = [&](int kind, int a, int b) {
    GraphOp o = blank(kind);
    o.in[0] = a; o.in[1] = b; o.out = next++;
    ops.push_back(o);
    return o.out;
  };
  auto make_divisible8 = [](int v) {  // torchvision _make_divisible(v, 8)
    int nv = std::max(8, (v + 4) / 8 * 8);
    if (nv * 10 < 9 * v) nv += 8;
    return nv;
  };

  int x = conv_bn(0, 3, 16, 3, 2, false, kActHardSwish, -1);
  struct Cfg { int cin, k, exp, cout, se, hs, stride; };
  const Cfg cfgs[11] = {{16, 3, 16, 16, 1, 0, 2},  {16, 3, 72, 24, 0, 0, 2},  {24, 3, 88, 24, 0, 0, 1},  {24, 5, 96, 40, 1, 1, 2},
                        {40, 5, 240, 40, 1, 1, 1}, {40, 5, 240, 40, 1, 1, 1}, {40, 5, 120, 48, 1, 1, 1}, {48, 5, 144, 48, 1, 1, 1},
                        {48, 5, 288, 96, 1, 1, 2}, {96, 5, 576, 96, 1, 1, 1}, {96, 5, 576, 96, 1, 1, 1}};
  for (const Cfg& c : cfgs) {
    const int act = c.hs ? kActHardSwish : kActRelu;
    const int block_in = x;
    int y = x;
    if (c.exp != c.cin) y = conv_bn(y, c.cin, c.exp, 1, 1, false, act, -1);
    y = conv_bn(y, c.exp, c.exp, c.k, c.stride, true, act, -1);
    if (c.se) {
      const int sq = make_divisible8(c.exp / 4);
      int g = simple(NNCV_HIP_OP_GAVGPOOL, y, -1);
      g = fc(g, c.exp, sq, kActRelu);
      g = fc(g, sq, c.exp, kActHardSigmoid);
      y = simple(NNCV_HIP_OP_SCALE, y, g);
    }
    const bool res = c.stride == 1 && c.cin == c.cout;
    x = conv_bn(y, c.exp, c.cout, 1, 1, false, kActNone, res ? block_in : -1);
  }
  x = conv_bn(x, 96, 576, 1, 1, false, kActHardSwish, -1);
  x = simple(NNCV_HIP_OP_GAVGPOOL, x, -1);
  x = fc(x, 576, 1024, kActHardSwish);
  x = fc(x, 1024, 1000, kActNone);
  if (n_elems) *n_elems = off;
  return ops;
}

}  // namespace nncv_hip
