// A network as a list of operators over numbered NHWC tensors: what a compiled object for the
// reference's other fixtures (tests/Nets/MobileNetV3.mlir, Yolov5s.mlir) is made of once BatchNorm
// is folded and the elementwise tails are fused into their producers.  The reference has no such
// object at run time -- its compiler bakes the graph into straight-line code -- so the description
// is this library's own; its vocabulary is the fixtures' (conv_2d_nchw_fchw,
// depthwise_conv_2d_nchw_chw, pooling_nchw_max / _sum, concat, the activation generics).
#pragma once
#include <memory>
#include <vector>

#include "../../include/nncv_hip.h"
#include "runtime.hpp"

namespace nncv_hip {

typedef nncv_hip_graph_op GraphOp;

class Graph {
 public:
  // ops: n operators in execution order.  Tensor 0 is the network input (NCHW, in_channels
  // channels); every other tensor is the `out` of exactly one operator and may only be read by
  // later ones.  The `out` of the last operator is the network output.
  // params_dev: flat device blob of n_elems elements of type dt that the operators' offsets index.
  // params_dev == nullptr builds the structure only (shapes, merged launches, concatenation views, the
  // workspace plan): no device is touched and forward() must not be called.
  Graph(const GraphOp* ops, int n, int in_channels, const void* params_dev, long long n_elems, int dt, hipStream_t s);
  int dtype() const { return dt_; }
  int in_channels() const { return c_in_; }
  int num_ops() const { return (int)nodes_.size(); }
  // channels / height / width of the network output for an H x W input
  void output_shape(int H, int W, int* C, int* OH, int* OW) const;
  size_t workspace_bytes(int N, int H, int W) const;
  int num_tensors() const { return n_tensors_; }
  // The workspace plan for an input shape, for inspection: tensor_info[4*t..] = {tensor whose memory t
  // lives in, byte offset of t, bytes of that memory block, channel offset of t inside it}; launch_dst[i]
  // = the tensor operator i's launch writes first, -1 when the operator was merged into another launch
  // or writes no workspace tensor.  Returns the workspace size.  Host arithmetic only.
  size_t describe_plan(int N, int H, int W, long long* tensor_info, int* launch_dst) const;
  // src: NCHW [N,in_channels,H,W] of type dt; out: NCHW fp32 of the output shape (both device)
  void forward(const void* src, int N, int H, int W, float* out, void* ws, hipStream_t s) const;

 private:
  struct Node {
    GraphOp op;
    int C = 0;  // channels of in[0] as stored (the network input is padded to a whole vector)
    DeviceBuffer wt, wfrag, wfrag32, scale, shift;
    // Set on a GAVGPOOL that starts "pool -> 1x1 conv + bias -> 1x1 conv + bias -> SCALE of the pooled
    // tensor" whose three intermediate tensors have no other reader: the four operators run as one
    // squeeze-excitation launch and the next three nodes are skipped.
    bool se_head = false, skip = false;
    // Set on a CONV whose only reader is the ADD that follows it (x + act(conv), a YOLOv5
    // Bottleneck): the convolution adds `add_res` after its activation and writes the ADD's
    // output tensor `add_out`; the ADD node is skipped.
    int add_res = -1, add_out = -1;
    DeviceBuffer wt_pairs;  // see pair_stem_
  };
  struct Dims { int C, H, W; };
  struct Plan {
    int N, H, W;
    std::vector<Dims> dims;      // per tensor
    std::vector<size_t> offset;  // per tensor, in the workspace (tensor 0: its NHWC copy)
    std::vector<size_t> root_bytes;  // per tensor: size of the memory block it lives in
    size_t total;
  };
  const Plan& plan_of(int N, int H, int W) const;
  void launch_io(int i, std::vector<int>* writes, std::vector<int>* reads) const;
  void check_plan(const Plan& p) const;

  int dt_, c_in_, n_tensors_ = 0;
  bool dry_ = false;
  std::vector<Node> nodes_;
  std::vector<int> channels_;  // per tensor, as stored (padded to a whole 16-byte vector)
  std::vector<int> logical_;   // per tensor, as the network defines it
  // Concatenation without copies: a tensor that is an input of one CONCAT, and whose producer and
  // readers can all address rows at a pitch, lives inside the concatenated tensor (`view_of_` =
  // that tensor, `view_c0_` = its channel offset there).  Chains are resolved by root_of().
  std::vector<int> view_of_, view_c0_;
  // Index of the one convolution that reads the network input, when it is an fp16 stride-2
  // convolution over <= 4 channels: for even W the input is then stored as pixel pairs (4 channels
  // per pixel) and that convolution walks pairs (launch_weight_pairs); -1 otherwise.
  int pair_stem_ = -1;
  void root_of(int t, int* root, int* c0) const;
  std::vector<float> detect_anchor_wh_, detect_stride_;  // YOLO_DETECT: host copies of anchors * stride, strides
  std::vector<int> last_use_;  // per tensor: index of the last operator that reads it
  mutable std::vector<Plan> plans_;
};

// The operator list and parameter count of torchvision's MobileNetV3-small as exported in
// tests/Nets/MobileNetV3.mlir (parameters in state_dict order without num_batches_tracked).
std::vector<GraphOp> mobilenetv3_small_ops(long long* n_elems);

}  // namespace nncv_hip
