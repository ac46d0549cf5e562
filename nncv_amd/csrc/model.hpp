// Host-side objects of the path: one convolution with its prepared weights and fused epilogue,
// and the ResNet-18 graph of tests/Nets/Res18.mlir built from them.
#pragma once
#include <memory>
#include <vector>

#include "runtime.hpp"

namespace nncv_hip {

enum ConvAlgo : int { kAlgoAuto = 0, kAlgoWinograd = 1, kAlgoIgemm = 2 };

// linalg.conv_2d_nchw_fchw + BatchNorm + (residual add) + ReLU as one device operation.
// Weights arrive in the reference's FCHW order; they are re-laid once at creation:
//   igemm    : [F][R][S][C]   (K = (r,s,c) contiguous per filter); 3x3 stride-1 layers also keep
//              a fragment-major copy for the LDS-patch kernel (conv3x3_patch.hip)
//   winograd : U[36][F][C]    (filter transform done here, like the reference folds it at
//                              compile time, OptimizeConv2dUsingWinograd.cpp:106-150)
class ConvLayer {
 public:
  struct Desc {
    int dt = kF32;  // element type of activations and weights
    int C = 0, F = 0, R = 0, S = 0, stride = 1, pad = 0;
    int relu = 0;  // activation applied last (enum Act); 1 = ReLU
    int algo = kAlgoAuto;
    bool stem = false;  // 7x7 s2 p3 over 3 channels read from NCHW (pixel-pair packing)
  };
  // w: device pointer to FCHW weights of type `dt`; bn: device pointers gamma,beta,mean,var of
  // type `dt` (all null -> no scale/shift).
  ConvLayer(const Desc& d, const void* w_dev, const void* gamma, const void* beta, const void* mean, const void* var,
            hipStream_t s);

  const Desc& desc() const { return d_; }
  int algo() const { return algo_; }
  int out_h(int H) const { return (H + 2 * d_.pad - d_.R) / d_.stride + 1; }
  int out_w(int W) const { return (W + 2 * d_.pad - d_.S) / d_.stride + 1; }
  size_t workspace_bytes(int N, int H, int W, bool strided = false) const;
  // in/out/residual: NHWC device tensors of type dt (stem: `in` is NCHW [N,3,H,W]).
  // `ws` must hold workspace_bytes().  `counters`: kSplitKCounterInts zeroed ints to use as the K split's tickets
  // instead of the layer's own (null = the layer's own).
  void forward(const void* in, int N, int H, int W, const void* residual, void* out, void* ws, hipStream_t s,
               int* counters = nullptr) const;
  static constexpr int kSplitKCounterInts = 256;
  // generic-layout form used by the operator-level ABI: strides for in / out (residual shares out's)
  void forward_strided(const void* in, Strides4 in_st, int N, int H, int W, const void* residual, void* out, Strides4 out_st,
                       bool accumulate, void* ws, hipStream_t s) const;
  // Fuses the 1x1 shortcut convolution `ds` of a down-sampling block (same input, same stride, no
  // padding) into this 3x3 pad-1 convolution: one launch then produces both tensors.  Returns
  // false (and changes nothing) when the pair does not qualify.
  // stem only: conv + BN + ReLU + the 3x3 stride-2 max-pool in one launch, NCHW in, pooled NHWC
  // out.  Returns false (nothing launched) when the fused kernel does not cover the case.
  bool forward_stem_pool(const void* in, int N, int H, int W, void* pooled_out, hipStream_t s) const;
  bool fuse_shortcut(const ConvLayer& ds, hipStream_t s);
  bool has_shortcut() const { return aux_F_ > 0; }
  // forward() of this layer into `out` and of the fused shortcut into `shortcut_out`
  void forward_with_shortcut(const void* in, int N, int H, int W, void* out, void* shortcut_out, void* ws, hipStream_t s) const;

 private:
  Desc d_;
  int algo_;
  DeviceBuffer wt_, wfrag_, wfrag32_, U_, scale_, shift_, wt_shift_;
  DeviceBuffer wt_cat_, scale_cat_, shift_cat_;  // this layer's filters followed by the fused shortcut's
  DeviceBuffer aux_wfrag_;  // the fused shortcut's filters alone, fragment-major (stride-2 patch kernel)
  DeviceBuffer splitk_counters_;  // tickets of the patch kernel's K split (fp32); zero between launches
  int aux_F_ = 0;
  int aux_relu_ = 0;
  double aux_flops_per_pixel_ = 0.0;
};

class ResNet18 {
 public:
  // params_dev: flat device blob of `n_elems` elements of type dt in the canonical tensor order.
  ResNet18(const void* params_dev, long long n_elems, int dt, int algo3x3, hipStream_t s);
  int dtype() const { return dt_; }
  size_t workspace_bytes(int N, int H, int W) const;
  // src: NCHW [N,3,H,W] of type dt (device); logits: [N,1000] of type dt (device).
  // tap_stage >= 0 also copies the NHWC activation after that stage to `tap`
  // (0: after the max-pool, 1..4: after layer1..layer4).
  void forward(const void* src, int N, int H, int W, void* logits, void* ws, hipStream_t s, int tap_stage = -1,
               void* tap = nullptr) const;

  struct Block {
    std::unique_ptr<ConvLayer> c1, c2, ds;
  };

 private:
  int dt_;
  std::unique_ptr<ConvLayer> stem_;
  std::vector<Block> blocks_;
  DeviceBuffer fc_w_, fc_b_;  // [1000][512] dt ; [1000] f32
};

static constexpr long long kResNet18Elems = 11699112;

}  // namespace nncv_hip
