#include "model.hpp"

#include "arena_plan.hpp"

#include <cstring>

namespace nncv_hip {

static int env_algo3x3() {
  const char* e = getenv("NNCV_HIP_CONV3X3");
  if (!e) return kAlgoAuto;
  if (!strcmp(e, "winograd")) return kAlgoWinograd;
  if (!strcmp(e, "igemm")) return kAlgoIgemm;
  return kAlgoAuto;
}

static int round_up(int v, int m) { return (v + m - 1) / m * m; }

// scratch of the patch kernel's K split: at most 256 workgroups' 64x64 fp32 partial tiles
constexpr size_t kSplitKWsBytes = 256 * 4096 * sizeof(float);
constexpr int kSplitKCounters = ConvLayer::kSplitKCounterInts;

ConvLayer::ConvLayer(const Desc& d, const void* w, const void* gamma, const void* beta, const void* mean, const void* var,
                     hipStream_t s)
    : d_(d) {
  NNCV_REQUIRE(d.dt == kF32 || d.dt == kF16, "conv: dtype must be f32 or f16");
  NNCV_REQUIRE(d.C > 0 && d.F > 0 && d.R > 0 && d.S > 0 && d.stride > 0 && d.pad >= 0, "conv: bad geometry");
  NNCV_REQUIRE(d.relu >= kActNone && d.relu <= kActSigmoid, "conv: unknown activation");
  const int ce = d.dt == kF16 ? 8 : 4;
  const size_t es = dtype_size(d.dt);
  const bool wino_ok = !d.stem && d.relu <= kActRelu && d.R == 3 && d.S == 3 && d.stride == 1 && d.C % ce == 0 && d.F % 4 == 0;
  int algo = d.algo;
  if (algo == kAlgoAuto) algo = env_algo3x3();
  // default: the direct form for both types.  In fp16 F(4,3) costs about 10x the rounding error;
  // in fp32 it is exact enough, but its three extra passes over 2.25x larger tensors cost more
  // than the 2.25x fewer multiplies save at every ResNet-18 size measured (batch 1..32).
  if (algo == kAlgoAuto) algo = kAlgoIgemm;
  if (algo == kAlgoWinograd && !wino_ok) algo = kAlgoIgemm;
  // F(4x4,3x3) with half-precision V, U and M loses about ten times the direct form's rounding error per
  // layer (2.5-3e-3 relative L2, up to 3e-2 on some shapes): outside the 1e-2 / identical-top-1 bar this
  // library holds fp16 results to.  A request for it is therefore served by the direct form, and says so
  // once.  (The four stages stay available as fp16 operators, nncv_hip_wino43_*.)
  if (algo == kAlgoWinograd && d.dt == kF16) {
    static bool told = false;
    if (!told) {
      fprintf(stderr, "[ Warn ] nncv_hip: fp16 Winograd F(4x4,3x3) does not hold the fp16 accuracy bar; 3x3 layers use the direct form\n");
      told = true;
    }
    algo = kAlgoIgemm;
  }
  algo_ = algo;

  if (d.stem) {
    NNCV_REQUIRE(d.C == 3 && d.R == 7 && d.S == 7 && d.stride == 2 && d.pad == 3, "stem: must be 7x7 s2 p3 over 3 channels");
    NNCV_REQUIRE(d.F % 4 == 0, "stem: F must be a multiple of 4");
    wt_.reset((size_t)d.F * 224 * es);
    launch_stem_weight(w, d.dt, wt_.get(), d.dt, d.F, 0, s);
    wt_shift_.reset((size_t)d.F * 224 * es);  // pairs start one column further left (fused stem)
    launch_stem_weight(w, d.dt, wt_shift_.get(), d.dt, d.F, 1, s);
  } else if (algo_ == kAlgoWinograd) {
    U_.reset((size_t)36 * d.F * d.C * es);
    launch_wino43_filter(w, d.dt, U_.get(), d.dt, d.F, d.C, s);
  } else {
    const int Cp = round_up(d.C, ce), Fp = round_up(d.F, 4);
    wt_.reset((size_t)Fp * d.R * d.S * Cp * es);
    NNCV_HIP_CHECK(hipMemsetAsync(wt_.get(), 0, wt_.bytes(), s));
    launch_weight_frsc(w, d.dt, wt_.get(), d.dt, d.F, d.C, d.R, d.S, Cp, s);
    if (d.R == 3 && d.S == 3 && (d.stride == 1 || d.stride == 2) && d.pad == 1 && d.C % (128 / (int)es) == 0) {
      wfrag_.reset((size_t)((d.F + 63) / 64) * 64 * 9 * d.C * es);
      launch_weight_frag3x3(w, d.dt, wfrag_.get(), d.dt, d.F, d.C, s);
      if (d.dt == kF16 && d.stride == 1 && d.C % 64 == 0 && d.F % 32 == 0) {
        wfrag32_.reset(weight_frag32_bytes(d.F, d.C));
        launch_weight_frag32(w, d.dt, wfrag32_.get(), d.F, d.C, s);
      }
      if (d.dt == kF32) {
        splitk_counters_.reset(kSplitKCounters * sizeof(int));
        NNCV_HIP_CHECK(hipMemsetAsync(splitk_counters_.get(), 0, splitk_counters_.bytes(), s));
      }
    }
  }
  if (gamma) {
    NNCV_REQUIRE(beta && mean && var, "conv: BN needs gamma, beta, mean and var");
    const int Fp = round_up(d.F, 4);
    scale_.reset((size_t)Fp * 4);
    shift_.reset((size_t)Fp * 4);
    launch_fill_f32(scale_.as<float>(), 0.0f, Fp, s);
    launch_fill_f32(shift_.as<float>(), 0.0f, Fp, s);
    launch_bn_fold(gamma, beta, mean, var, d.dt, scale_.as<float>(), shift_.as<float>(), d.F, s);
  }
}

size_t ConvLayer::workspace_bytes(int N, int H, int W, bool strided) const {
  const size_t es = dtype_size(d_.dt);
  const int ce = d_.dt == kF16 ? 8 : 4;
  const int OH = out_h(H), OW = out_w(W);
  size_t b = 0;
  if (d_.stem) b += align256((size_t)N * (H + 6) * ((W + 9) / 2) * 8 * es);
  if (algo_ == kAlgoWinograd) {
    const size_t tiles = (size_t)N * ((OH + 3) / 4) * ((OW + 3) / 4);
    b += align256(36 * tiles * d_.C * es) + align256(36 * tiles * d_.F * es);
  }
  // strided (operator-level) form of the igemm path stages NHWC copies of input and output
  if (strided && !d_.stem && algo_ == kAlgoIgemm)
    b += align256((size_t)N * H * W * round_up(d_.C, ce) * es) + 2 * align256((size_t)N * OH * OW * round_up(d_.F, 4) * es);
  if (!strided && splitk_counters_.get()) b += kSplitKWsBytes;
  return b;
}

void ConvLayer::forward(const void* in, int N, int H, int W, const void* residual, void* out, void* ws, hipStream_t s,
                        int* counters) const {
  const int OH = out_h(H), OW = out_w(W);
  NNCV_REQUIRE(N > 0 && OH > 0 && OW > 0, "conv: empty tensor");
  const size_t es = dtype_size(d_.dt);
  char* wsp = static_cast<char*>(ws);
  if (d_.stem) {
    const int HP = H + 6, WP = (W + 9) / 2;
    launch_stem_pack(in, d_.dt, wsp, d_.dt, N, H, W, s);
    IgemmArgs a{};
    a.in = wsp; a.wt = wt_.get(); a.out = out;
    a.scale = scale_.as<float>(); a.shift = shift_.as<float>(); a.residual = residual;
    // a filter row is 4 consecutive pixel pairs = 32 contiguous elements: one K step
    a.N = N; a.H = HP; a.W = WP; a.C = 32; a.pix_stride = 8; a.F = d_.F; a.R = 7; a.S = 1; a.OH = OH; a.OW = OW;
    a.stride_h = 2; a.stride_w = 1; a.pad_h = 0; a.pad_w = 0;
    a.relu = d_.relu; a.ldo = d_.F; a.batch = 1;
    a.alg_flops = 2.0 * N * OH * OW * d_.F * 147.0;  // the 7x7x3 filter, not its padded 7x8x4 packing
    launch_igemm(a, d_.dt, d_.dt, s);
    return;
  }
  if (algo_ == kAlgoWinograd) {
    forward_strided(in, strides_of(kNHWC, d_.C, H, W), N, H, W, residual, out, strides_of(kNHWC, d_.F, OH, OW), false, ws, s);
    return;
  }
  NNCV_REQUIRE(d_.C % (16 / (int)es) == 0 && d_.F % 4 == 0, "conv: NHWC igemm needs C %% chunk == 0 and F %% 4 == 0");
  IgemmArgs a{};
  a.in = in; a.wt = wt_.get(); a.wt_frag = wfrag_.get(); a.wt_frag32 = wfrag32_.get(); a.out = out;
  a.scale = scale_.as<float>(); a.shift = shift_.as<float>(); a.residual = residual;
  a.N = N; a.H = H; a.W = W; a.C = d_.C; a.F = d_.F; a.R = d_.R; a.S = d_.S; a.OH = OH; a.OW = OW;
  a.stride_h = a.stride_w = d_.stride; a.pad_h = a.pad_w = d_.pad;
  a.relu = d_.relu; a.ldo = d_.F; a.batch = 1;
  if (ws && splitk_counters_.get()) {
    a.splitk_ws = ws; a.splitk_ws_bytes = kSplitKWsBytes;
    a.splitk_counters = counters ? counters : splitk_counters_.as<int>(); a.splitk_counters_n = kSplitKCounters;
  }
  launch_igemm(a, d_.dt, d_.dt, s);
}

bool ConvLayer::forward_stem_pool(const void* in, int N, int H, int W, void* pooled_out, hipStream_t s) const {
  if (!d_.stem || d_.relu != kActRelu || !stem_pool_applicable(d_.dt, N, H, W, d_.F)) return false;
  launch_stem_pool(in, wt_shift_.get(), scale_.as<float>(), shift_.as<float>(), pooled_out, N, H, W, s);
  return true;
}

bool ConvLayer::fuse_shortcut(const ConvLayer& ds, hipStream_t s) {
  const Desc& q = ds.d_;
  const size_t es = dtype_size(d_.dt);
  const int ce = d_.dt == kF16 ? 8 : 4;
  if (d_.stem || algo_ != kAlgoIgemm || ds.algo_ != kAlgoIgemm || q.dt != d_.dt || q.C != d_.C || q.stride != d_.stride ||
      d_.R != 3 || d_.S != 3 || d_.pad != 1 || q.R != 1 || q.S != 1 || q.pad != 0 || d_.F % 128 != 0 || q.F % 8 != 0 ||
      d_.C % ce != 0 || !scale_.get() || !ds.scale_.get())
    return false;
  const size_t row = (size_t)9 * d_.C * es;
  wt_cat_.reset((size_t)(d_.F + q.F) * row);
  NNCV_HIP_CHECK(hipMemsetAsync(wt_cat_.get(), 0, wt_cat_.bytes(), s));
  NNCV_HIP_CHECK(hipMemcpyAsync(wt_cat_.get(), wt_.get(), (size_t)d_.F * row, hipMemcpyDeviceToDevice, s));
  // the shortcut's [F][C] rows become the centre tap (r = s = 1) of otherwise zero 3x3 filters
  NNCV_HIP_CHECK(hipMemcpy2DAsync(wt_cat_.as<char>() + (size_t)d_.F * row + (size_t)4 * d_.C * es, row, ds.wt_.get(),
                                  (size_t)d_.C * es, (size_t)d_.C * es, q.F, hipMemcpyDeviceToDevice, s));
  scale_cat_.reset((size_t)(d_.F + q.F) * 4);
  shift_cat_.reset((size_t)(d_.F + q.F) * 4);
  NNCV_HIP_CHECK(hipMemcpyAsync(scale_cat_.get(), scale_.get(), (size_t)d_.F * 4, hipMemcpyDeviceToDevice, s));
  NNCV_HIP_CHECK(hipMemcpyAsync(shift_cat_.get(), shift_.get(), (size_t)d_.F * 4, hipMemcpyDeviceToDevice, s));
  NNCV_HIP_CHECK(hipMemcpyAsync(scale_cat_.as<float>() + d_.F, ds.scale_.get(), (size_t)q.F * 4, hipMemcpyDeviceToDevice, s));
  NNCV_HIP_CHECK(hipMemcpyAsync(shift_cat_.as<float>() + d_.F, ds.shift_.get(), (size_t)q.F * 4, hipMemcpyDeviceToDevice, s));
  if (wfrag_.get() && d_.C % (128 / (int)es) == 0) {
    aux_wfrag_.reset((size_t)((q.F + 63) / 64) * 64 * d_.C * es);
    launch_weight_frag1x1(ds.wt_.get(), d_.dt, aux_wfrag_.get(), d_.dt, q.F, d_.C, s);  // [F][1][1][C] rows
  }
  aux_F_ = q.F;
  aux_relu_ = q.relu;
  aux_flops_per_pixel_ = 2.0 * q.F * q.C;
  return true;
}

void ConvLayer::forward_with_shortcut(const void* in, int N, int H, int W, void* out, void* shortcut_out, void* ws,
                                      hipStream_t s) const {
  NNCV_REQUIRE(aux_F_ > 0, "conv: no fused shortcut");
  const int OH = out_h(H), OW = out_w(W);
  NNCV_REQUIRE(N > 0 && OH > 0 && OW > 0, "conv: empty tensor");
  IgemmArgs a{};
  a.in = in; a.wt = wt_cat_.get(); a.wt_frag = wfrag_.get(); a.aux_wt_frag = aux_wfrag_.get(); a.out = out;
  a.scale = scale_cat_.as<float>(); a.shift = shift_cat_.as<float>();
  a.N = N; a.H = H; a.W = W; a.C = d_.C; a.F = d_.F + aux_F_; a.R = 3; a.S = 3; a.OH = OH; a.OW = OW;
  a.stride_h = a.stride_w = d_.stride; a.pad_h = a.pad_w = 1;
  a.relu = d_.relu; a.ldo = d_.F; a.batch = 1;
  a.aux_f0 = d_.F; a.aux_tap = 4; a.aux_relu = aux_relu_; a.aux_ldo = aux_F_; a.aux_out = shortcut_out;
  a.alg_flops = (2.0 * d_.F * 9.0 * d_.C + aux_flops_per_pixel_) * N * OH * OW;
  if (ws && splitk_counters_.get()) {
    a.splitk_ws = ws; a.splitk_ws_bytes = kSplitKWsBytes;
    a.splitk_counters = splitk_counters_.as<int>(); a.splitk_counters_n = kSplitKCounters;
  }
  launch_igemm(a, d_.dt, d_.dt, s);
}

void ConvLayer::forward_strided(const void* in, Strides4 in_st, int N, int H, int W, const void* residual, void* out,
                                Strides4 out_st, bool accumulate, void* ws, hipStream_t s) const {
  NNCV_REQUIRE(!d_.stem, "conv: the stem has no strided form");
  const int OH = out_h(H), OW = out_w(W);
  NNCV_REQUIRE(N > 0 && OH > 0 && OW > 0, "conv: empty tensor");
  const size_t es = dtype_size(d_.dt);
  const int ce = d_.dt == kF16 ? 8 : 4;
  char* wsp = static_cast<char*>(ws);
  if (algo_ == kAlgoWinograd) {
    const int TH = (OH + 3) / 4, TW = (OW + 3) / 4;
    const long long tiles = (long long)N * TH * TW;
    void* V = wsp;
    void* M = wsp + align256((size_t)36 * tiles * d_.C * es);
    launch_wino43_input(in, d_.dt, in_st, V, d_.dt, N, d_.C, H, W, d_.pad, s);
    IgemmArgs a{};
    a.in = V; a.wt = U_.get(); a.out = M;
    NNCV_REQUIRE(tiles < (1ll << 31), "conv: too many Winograd tiles");
    a.N = (int)tiles; a.H = 1; a.W = 1; a.C = d_.C; a.F = d_.F; a.R = 1; a.S = 1; a.OH = 1; a.OW = 1;
    a.stride_h = a.stride_w = 1; a.ldo = d_.F; a.batch = 36;
    a.in_bs = tiles * d_.C; a.wt_bs = (long long)d_.F * d_.C; a.out_bs = tiles * d_.F;
    launch_igemm(a, d_.dt, d_.dt, s);
    WinoOutArgs o{};
    o.M = M; o.out = out; o.residual = residual; o.scale = scale_.as<float>(); o.shift = shift_.as<float>();
    o.st = out_st; o.N = N; o.F = d_.F; o.OH = OH; o.OW = OW; o.relu = d_.relu; o.accumulate = accumulate;
    launch_wino43_output(o, d_.dt, d_.dt, s);
    return;
  }
  // implicit GEMM through NHWC staging copies (operator-level forms only; the network itself is
  // NHWC end to end and never comes here)
  const int Cp = round_up(d_.C, ce), Fp = round_up(d_.F, 4);
  const size_t in_b = align256((size_t)N * H * W * Cp * es), out_b = align256((size_t)N * OH * OW * Fp * es);
  void* xin = wsp;
  void* yout = wsp + in_b;
  void* rin = residual ? wsp + in_b + out_b : nullptr;
  launch_relayout(in, d_.dt, in_st, xin, d_.dt, strides_of(kNHWC, Cp, H, W), N, d_.C, Cp, H, W, false, s);
  if (residual)
    launch_relayout(residual, d_.dt, out_st, rin, d_.dt, strides_of(kNHWC, Fp, OH, OW), N, d_.F, Fp, OH, OW, false, s);
  IgemmArgs a{};
  a.in = xin; a.wt = wt_.get(); a.out = yout; a.residual = rin;
  a.scale = scale_.as<float>(); a.shift = shift_.as<float>();
  a.N = N; a.H = H; a.W = W; a.C = Cp; a.F = Fp; a.R = d_.R; a.S = d_.S; a.OH = OH; a.OW = OW;
  a.stride_h = a.stride_w = d_.stride; a.pad_h = a.pad_w = d_.pad;
  a.relu = d_.relu; a.ldo = Fp; a.batch = 1;
  NNCV_REQUIRE(!(accumulate && (d_.relu || residual)), "conv: accumulate form has no epilogue");
  launch_igemm(a, d_.dt, d_.dt, s);
  // out (+)= y : y is NHWC with Fp channels; only the first F are copied
  launch_relayout(yout, d_.dt, strides_of(kNHWC, Fp, OH, OW), out, d_.dt, out_st, N, d_.F, d_.F, OH, OW, accumulate, s);
}

// ---------------------------------------------------------------------------------------------

ResNet18::ResNet18(const void* params, long long n_elems, int dt, int algo3x3, hipStream_t s) : dt_(dt) {
  NNCV_REQUIRE(n_elems == kResNet18Elems,
               "ResNet-18 params: expected 11699112 elements in the canonical model.bin order, got " + std::to_string(n_elems));
  const size_t es = dtype_size(dt);
  const char* p = static_cast<const char*>(params);
  auto take = [&](long long n) { const void* r = p; p += n * es; return r; };
  auto make = [&](int C, int F, int R, int stride, int pad, bool relu, bool stem) {
    ConvLayer::Desc d;
    d.dt = dt; d.C = C; d.F = F; d.R = d.S = R; d.stride = stride; d.pad = pad; d.relu = relu; d.stem = stem;
    d.algo = (R == 3 && stride == 1) ? algo3x3 : kAlgoIgemm;
    const void* w = take((long long)F * C * R * R);
    const void* g = take(F); const void* b = take(F); const void* m = take(F); const void* v = take(F);
    return std::make_unique<ConvLayer>(d, w, g, b, m, v, s);
  };
  stem_ = make(3, 64, 7, 2, 3, true, true);
  int cin = 64;
  const int widths[4] = {64, 128, 256, 512};
  for (int L = 0; L < 4; ++L)
    for (int blk = 0; blk < 2; ++blk) {
      const int F = widths[L], stride = (L > 0 && blk == 0) ? 2 : 1;
      Block b;
      b.c1 = make(cin, F, 3, stride, 1, true, false);
      b.c2 = make(F, F, 3, 1, 1, true, false);  // ReLU after the residual add
      if (stride != 1 || cin != F) {
        b.ds = make(cin, F, 1, stride, 0, false, false);
        static const bool no_fuse = getenv("NNCV_HIP_NO_SHORTCUT_FUSION") != nullptr;
        if (!no_fuse) b.c1->fuse_shortcut(*b.ds, s);
      }
      blocks_.push_back(std::move(b));
      cin = F;
    }
  const void* fw = take(1000 * 512);
  const void* fb = take(1000);
  fc_w_.reset((size_t)1000 * 512 * es);
  NNCV_HIP_CHECK(hipMemcpyAsync(fc_w_.get(), fw, fc_w_.bytes(), hipMemcpyDeviceToDevice, s));
  fc_b_.reset(1000 * 4);
  launch_cast(fb, dt, fc_b_.get(), kF32, 1000, s);
  NNCV_REQUIRE((p - static_cast<const char*>(params)) == (long long)(kResNet18Elems * es), "ResNet-18 params: table walk mismatch");
}

namespace {
// Workspace layout of one forward pass, planned with plan_offsets (arena_plan.hpp) from the
// tensors' sizes and the operator range over which each one is live.  Operator numbering: 0 stem
// convolution, 1 max-pool, then per BasicBlock k: 2+3k conv1, 3+3k shortcut conv, 4+3k conv2,
// 26 average pool, 27 FC.
struct Plan {
  int h1, w1, h2, w2;            // after stem, after maxpool
  size_t stem_out, pooled, cws;  // offsets
  size_t x[9];                   // x[k] = input of block k; x[8] = network body output
  size_t y1[8], idn[8];
  size_t total;
};
}  // namespace

static Plan make_plan(const ConvLayer& stem, const std::vector<const ConvLayer*>& c1s, const std::vector<const ConvLayer*>& c2s,
                      const std::vector<const ConvLayer*>& dss, int dt, int N, int H, int W) {
  Plan p{};
  const size_t es = dtype_size(dt);
  p.h1 = stem.out_h(H); p.w1 = stem.out_w(W);
  p.h2 = (p.h1 + 2 - 3) / 2 + 1; p.w2 = (p.w1 + 2 - 3) / 2 + 1;
  std::vector<TensorLife> t;
  auto add = [&](int first, int last, size_t bytes) { t.push_back(TensorLife{first, last, bytes, 0}); return (int)t.size() - 1; };
  // the fused stem kernel writes the pooled tensor directly: no stem output, no packed image
  const bool fused_stem = stem.desc().relu == kActRelu && stem_pool_applicable(dt, N, H, W, stem.desc().F);
  const int i_stem = add(0, 1, fused_stem ? 0 : (size_t)N * p.h1 * p.w1 * 64 * es);
  size_t cws = fused_stem ? 0 : stem.workspace_bytes(N, H, W);
  int h = p.h2, w = p.w2, ch = 64;
  int ix[9], iy1[8], iidn[8];
  ix[0] = add(1, 0, 0);  // last use filled in below
  const int nb = (int)c1s.size();
  for (int k = 0; k < nb; ++k) {
    const int o = 2 + 3 * k;
    const int oh = c1s[k]->out_h(h), ow = c1s[k]->out_w(w), f = c2s[k]->desc().F;
    cws = std::max(cws, c1s[k]->workspace_bytes(N, h, w));
    cws = std::max(cws, c2s[k]->workspace_bytes(N, oh, ow));
    if (dss[k]) cws = std::max(cws, dss[k]->workspace_bytes(N, h, w));
    t[ix[k]].bytes = (size_t)N * h * w * ch * es;
    t[ix[k]].last_op = dss[k] ? o + 1 : o + 2;  // identity shortcuts are read by conv2
    iy1[k] = add(o, o + 2, (size_t)N * oh * ow * f * es);
    iidn[k] = dss[k] ? add(o, o + 2, (size_t)N * oh * ow * f * es) : -1;
    ix[k + 1] = add(o + 2, o + 3, 0);
    h = oh; w = ow; ch = f;
  }
  t[ix[nb]].bytes = (size_t)N * h * w * ch * es;
  t[ix[nb]].last_op = 26;
  const int i_pooled = add(26, 27, (size_t)N * 512 * es);
  const int i_cws = add(0, 27, cws);
  const int linger = (overlap_hint() >= 3 && N >= 16 && !arena_linger_forced()) ? 0 : arena_linger();  // see overlap_hint
  for (auto& e : t) e.last_op = std::min(27, e.last_op + linger);
  p.total = plan_offsets(t, 256) + 4096;
  p.stem_out = t[i_stem].offset; p.pooled = t[i_pooled].offset; p.cws = t[i_cws].offset;
  for (int k = 0; k <= nb; ++k) p.x[k] = t[ix[k]].offset;
  for (int k = 0; k < nb; ++k) { p.y1[k] = t[iy1[k]].offset; p.idn[k] = iidn[k] >= 0 ? t[iidn[k]].offset : 0; }
  return p;
}

static Plan plan_of(const ConvLayer& stem, const std::vector<ResNet18::Block>& blocks, int dt, int N, int H, int W) {
  std::vector<const ConvLayer*> c1s, c2s, dss;
  for (const ResNet18::Block& b : blocks) { c1s.push_back(b.c1.get()); c2s.push_back(b.c2.get()); dss.push_back(b.ds.get()); }
  NNCV_REQUIRE(c1s.size() == 8, "ResNet-18 has eight BasicBlocks");
  return make_plan(stem, c1s, c2s, dss, dt, N, H, W);
}

size_t ResNet18::workspace_bytes(int N, int H, int W) const { return plan_of(*stem_, blocks_, dt_, N, H, W).total; }

void ResNet18::forward(const void* src, int N, int H, int W, void* logits, void* ws, hipStream_t s, int tap_stage,
                       void* tap) const {
  NNCV_REQUIRE(N > 0 && H >= 32 && W >= 32, "ResNet-18: input must be at least 32x32");
  const Plan p = plan_of(*stem_, blocks_, dt_, N, H, W);
  char* base = static_cast<char*>(ws);
  char* stem_out = base + p.stem_out;
  char* pooled = base + p.pooled;
  char* cws = base + p.cws;
  char* x0 = base + p.x[0];

  // stem: conv7x7 s2 + BN + ReLU (Res18.mlir:118-142), then maxpool 3x3 s2 (:144-151)
  if (!stem_->forward_stem_pool(src, N, H, W, x0, s)) {
    stem_->forward(src, N, H, W, nullptr, stem_out, cws, s);
    launch_maxpool3x3s2_nhwc(stem_out, x0, dt_, N, p.h1, p.w1, 64, s);
  }
  int h = p.h2, w = p.w2, nblk = 0, ch = 64;
  const size_t es = dtype_size(dt_);
  if (tap_stage == 0) NNCV_HIP_CHECK(hipMemcpyAsync(tap, x0, (size_t)N * h * w * 64 * es, hipMemcpyDeviceToDevice, s));
  for (const Block& b : blocks_) {
    // BasicBlock (Res18.mlir:152-203, :255-320): y = relu(bn2(conv2(relu(bn1(conv1(x))))) + shortcut(x))
    char* x = base + p.x[nblk];
    char* y1 = base + p.y1[nblk];
    char* idn = base + p.idn[nblk];
    char* y2 = base + p.x[nblk + 1];
    const int oh = b.c1->out_h(h), ow = b.c1->out_w(w);
    const void* shortcut = x;
    if (b.ds && b.c1->has_shortcut()) {
      b.c1->forward_with_shortcut(x, N, h, w, y1, idn, cws, s);
      shortcut = idn;
    } else {
      b.c1->forward(x, N, h, w, nullptr, y1, cws, s);
      if (b.ds) {
        b.ds->forward(x, N, h, w, nullptr, idn, cws, s);
        shortcut = idn;
      }
    }
    b.c2->forward(y1, N, oh, ow, shortcut, y2, cws, s);
    h = oh; w = ow;
    ch = b.c2->desc().F;
    ++nblk;
    if (nblk % 2 == 0 && tap_stage == nblk / 2)
      NNCV_HIP_CHECK(hipMemcpyAsync(tap, y2, (size_t)N * h * w * ch * es, hipMemcpyDeviceToDevice, s));
  }
  char* body_out = base + p.x[8];
  // head: global average pool (sum, one divide), FC with bias (Res18.mlir:609-628)
  static const bool never_fused = getenv("NNCV_HIP_NO_HEAD_FUSION") != nullptr;
  // see overlap_hint (arena_plan.hpp); at small batches the fused head is a few dozen workgroups and one launch less
  const bool split_head = never_fused || (overlap_hint() >= 3 && N >= 16);
  if (!split_head) {
    launch_avgpool_fc(body_out, fc_w_.get(), fc_b_.as<float>(), static_cast<float*>(logits), dt_, N, h * w, 512, 1000, s);
    return;
  }
  launch_global_avgpool_nhwc(body_out, pooled, dt_, N, h * w, 512, s);
  IgemmArgs a{};
  a.in = pooled; a.wt = fc_w_.get(); a.out = logits; a.shift = fc_b_.as<float>();
  a.N = N; a.H = 1; a.W = 1; a.C = 512; a.F = 1000; a.R = 1; a.S = 1; a.OH = 1; a.OW = 1;
  a.stride_h = a.stride_w = 1; a.ldo = 1000; a.batch = 1;
  launch_igemm(a, dt_, kF32, s);
}

}  // namespace nncv_hip
