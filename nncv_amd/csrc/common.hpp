// Shared declarations of the gfx950 hot-path library: element types, error handling, kernel
// argument blocks and the launcher prototypes each .hip file exports to the host layer.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <stdexcept>
#include <string>

namespace nncv_hip {

typedef _Float16 half_t;

enum DType : int { kF32 = 1, kF16 = 2 };  // numbering of nncv::rt::dataType (DataType.hpp:118-124)
enum Layout : int { kNCHW = 0, kNHWC = 1 };

inline size_t dtype_size(int dt) { return dt == kF16 ? 2 : 4; }

struct Error : std::runtime_error {
  using std::runtime_error::runtime_error;
};

[[noreturn]] inline void fail(const std::string& msg) { throw Error(msg); }

#define NNCV_HIP_CHECK(expr)                                                              \
  do {                                                                                    \
    hipError_t _e = (expr);                                                               \
    if (_e != hipSuccess)                                                                 \
      ::nncv_hip::fail(std::string(#expr) + ": " + hipGetErrorString(_e) + " (" __FILE__ ":" + \
                       std::to_string(__LINE__) + ")");                                   \
  } while (0)

#define NNCV_REQUIRE(cond, msg)                     \
  do {                                              \
    if (!(cond)) ::nncv_hip::fail(std::string(msg)); \
  } while (0)

// ---------------------------------------------------------------------------------------------
// Activations fused into the epilogues, written the way the reference's fixtures spell them
// (tests/Nets/Res18.mlir:139-141 ReLU; tests/Nets/MobileNetV3.mlir:259-293 hard-swish,
// :349-379 hard-sigmoid; Yolov5s.mlir SiLU = x * 1/(1+exp(-x))).
// ---------------------------------------------------------------------------------------------
enum Act : int { kActNone = 0, kActRelu = 1, kActHardSwish = 2, kActHardSigmoid = 3, kActSilu = 4, kActSigmoid = 5 };
// flag on the activation code of a convolution epilogue: the residual is added after the activation
// (a YOLOv5 Bottleneck, x + SiLU(conv)) instead of before it (a ResNet BasicBlock, ReLU(conv + x))
constexpr int kActResidualAfter = 0x100;

// The fixtures divide by 6.0 (arith.divf).  Where the result is rounded to fp16 anyway (HALF_OUT),
// multiplying by the correctly rounded 1/6 instead -- at most one ulp of the fp32 intermediate away --
// saves the ten-instruction IEEE division sequence per element (MobileNetV3-small: 2.4 % of a
// batch-32 pass, 5 % at batch 256); fp32 outputs keep the division and stay bit-exact.
constexpr float kSixth = 0.16666667163372039794921875f;

// `arith.cmpf ugt` + select: NaN is kept, everything not greater than zero becomes +0.
// One instruction on gfx950: v_maximum3_f32(x, 0, 0) is the IEEE-754-2019 maximum, which propagates NaN and orders
// -0 below +0, i.e. the same values as the compare + select.
__device__ __forceinline__ float relu_ugt(float x) { return __builtin_elementwise_maximum(x, 0.0f); }

// 1 / (1 + exp(-x)) on the hardware's exp2 and reciprocal units (v_exp_f32, v_rcp_f32: about 1 ulp
// each, so the result is within a few ulp of the correctly rounded one -- far inside the 1e-4 / 1e-2
// parity bars).  The library expf plus an IEEE division is ~40 instructions per element, which made
// the SiLU epilogue of YOLOv5's memory-bound layers cost as much as their memory traffic.
// Limits: x -> -inf gives +0, x -> +inf gives 1, NaN stays NaN.
__device__ __forceinline__ float sigmoid_fast(float x) {
  return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(x * -1.44269504088896340736f));
}

template <bool HALF_OUT = false>
__device__ __forceinline__ float act_apply(float x, int act) {
  switch (act) {
    case kActRelu: return relu_ugt(x);
    case kActHardSwish: {  // (min(relu(x + 3), 6) / 6) * x ; min is `olt` + select; the division may be a multiplication, see kSixth
      float t = relu_ugt(x + 3.0f);
      t = t < 6.0f ? t : 6.0f;
      return (HALF_OUT ? t * kSixth : t / 6.0f) * x;
    }
    case kActHardSigmoid: {  // max(0, min(1, (x + 3) / 6)) ; `olt(1,t) ? 1 : t` then `ogt(0,m) ? 0 : m`
      float t = HALF_OUT ? (x + 3.0f) * kSixth : (x + 3.0f) / 6.0f;
      t = 1.0f < t ? 1.0f : t;
      return 0.0f > t ? 0.0f : t;
    }
    case kActSilu: return x * sigmoid_fast(x);
    case kActSigmoid: return sigmoid_fast(x);
    default: return x;
  }
}

// The same for N values of one lane with ONE dispatch on the activation code.  Epilogues use this
// form: calling act_apply per element inside an unrolled loop leaves a chain of scalar branches
// per element in the code (some 400 taken branches per wave in a 64-value epilogue, which was most
// of the run time of the memory-bound SiLU / hard-swish layers).
template <bool HALF_OUT = false, int N>
__device__ __forceinline__ void act_apply_n(float (&y)[N], int act) {
  switch (act) {
    case kActRelu:
#pragma unroll
      for (int e = 0; e < N; ++e) y[e] = act_apply<HALF_OUT>(y[e], kActRelu);
      break;
    case kActHardSwish:
#pragma unroll
      for (int e = 0; e < N; ++e) y[e] = act_apply<HALF_OUT>(y[e], kActHardSwish);
      break;
    case kActHardSigmoid:
#pragma unroll
      for (int e = 0; e < N; ++e) y[e] = act_apply<HALF_OUT>(y[e], kActHardSigmoid);
      break;
    case kActSilu:
#pragma unroll
      for (int e = 0; e < N; ++e) y[e] = act_apply<HALF_OUT>(y[e], kActSilu);
      break;
    case kActSigmoid:
#pragma unroll
      for (int e = 0; e < N; ++e) y[e] = act_apply<HALF_OUT>(y[e], kActSigmoid);
      break;
    default: break;
  }
}

// ---------------------------------------------------------------------------------------------
// Optional event timing of every launch (profiler.cpp).  `name` must be a string literal or
// otherwise outlive the scope; flops / bytes are the ALGORITHMIC work of the launch.
// ---------------------------------------------------------------------------------------------
bool profiler_enabled();
void profiler_enable(bool on);
std::string profiler_report();  // JSON {tag: {launches, ms, flops, bytes}}; waits for the work, clears
class ProfScope {
 public:
  ProfScope(const char* name, double flops, double bytes, hipStream_t s);
  ~ProfScope();
  ProfScope(const ProfScope&) = delete;
  ProfScope& operator=(const ProfScope&) = delete;

 private:
  hipStream_t s_;
  bool on_;
};

// ---------------------------------------------------------------------------------------------
// Implicit-GEMM convolution / batched GEMM on MFMA.
//   out[b][p][f] = epilogue( sum_k  X[b][p][k] * Wt[b][f][k] )
// p = output pixel (n, oy, ox) of an NHWC activation tensor, k = (r, s, c) with c fastest,
// X gathered on the fly with zero fill outside the image (the reference materialises the halo
// with tensor.pad; here it never exists).  With R = S = 1, stride 1, pad 0 this is a plain
// K-contiguous GEMM, which is how the 36 transformed-domain GEMMs of Winograd and the FC use it.
// ---------------------------------------------------------------------------------------------
struct IgemmArgs {
  const void* in;        // [batch][N][H][W][C]
  const void* wt;        // [batch][F][R*S*C]   (K-contiguous rows)
  void* out;             // [batch][P][ldo], channel f at out[p*ldo + f]
  const float* scale;    // [F] or null (1)
  const float* shift;    // [F] or null (0)
  const void* residual;  // same indexing as out, or null
  int N, H, W, C, F, R, S, OH, OW;
  int stride_h, stride_w, pad_h, pad_w;
  int relu;    // activation code (enum Act), optionally | kActResidualAfter; 0 none, 1 ReLU
  int ldo;     // out/residual row pitch in elements
  int batch;   // grid.z
  long long in_bs, wt_bs, out_bs;  // batch strides in elements
  double alg_flops;  // algorithmic flops of the launch for reporting; 0 = 2*P*F*R*S*C*batch
  int pix_stride;    // elements between horizontally adjacent pixels; 0 = C (the stem reads 32
                     // contiguous elements = 4 packed pixel pairs at a pixel pitch of 8)
  unsigned in_bytes, wt_bytes;  // size of one batch slice of in / wt; 0 = derived from the geometry
  const void* wt_frag;  // the same 3x3 filters in fragment-major order (launch_weight_frag3x3), or null
  const void* wt_frag32;  // fp16 3x3 stride-1 filters in the stream kernel's order (launch_weight_frag32), or null
  // Auxiliary filters fused into the same launch (the 1x1 stride-2 shortcut convolution of a
  // down-sampling block rides on the 3x3 stride-2 one: same input pixels, centre tap only).
  // Filters [aux_f0, F) are auxiliary: their rows of `wt` are zero outside tap `aux_tap`
  // (= r*S + s), only that tap's K range is walked for them, and their results go to `aux_out`
  // (row pitch aux_ldo, channel f - aux_f0) with aux_relu and no residual.  scale/shift cover
  // all F filters.  aux_f0 = 0: none; otherwise a multiple of 128.  Fast kernel only.
  int aux_f0, aux_tap, aux_relu, aux_ldo;
  void* aux_out;
  const void* aux_wt_frag;  // the auxiliary 1x1 filters alone, fragment-major (launch_weight_frag1x1), or null
  // Optional scratch for splitting K over workgroups (conv3x3_patch.hip, small fp32 launches only):
  // splitk_ws holds fp32 partial tiles for the duration of the launch; splitk_counters are
  // splitk_counters_n ints that are zero before the launch and zero again after it.  Null: no split.
  void* splitk_ws;
  size_t splitk_ws_bytes;
  int* splitk_counters;
  int splitk_counters_n;
};
// in_dt: element type of in/wt (kF32 | kF16); out_dt: element type of out/residual.
// Dispatches to the fast kernel (igemm_fast.hip) when C is a multiple of one K step and the
// tensors are below 2 GiB, else to the generic one (igemm.hip).
void launch_igemm(const IgemmArgs& a, int in_dt, int out_dt, hipStream_t s);
// 3x3 pad-1 layers at stride 1 or 2: direct convolution with the haloed input patch resident in LDS
// (conv3x3_patch.hip); same arguments and epilogue as the igemm kernels.
bool conv3x3_patch_applicable(const IgemmArgs& a, int in_dt);
// The tile plan that kernel would use for N x OH x OW output pixels, F filters and `slabs` 128-byte
// channel slabs: out = {WS, TN, TH, TW, NTX, rw_log, LDS cells available, loader coverage}.  Host
// arithmetic only (no device needed); false = no plan.
bool conv3x3_patch_plan(int stride, int N, int OH, int OW, int F, int slabs, int out[8]);
void launch_conv3x3_patch(const IgemmArgs& a, int in_dt, int out_dt, hipStream_t s);
// fp16 3x3 stride-1 pad-1 layers over whole 128-byte channel slabs and whole 32-filter groups: persistent
// workgroups, double-buffered LDS patch, 128 x 32 wave tiles (conv3x3_f16.hip).  launch returns false when no
// tile plan exists for the shape (nothing launched).
bool conv3x3_stream_applicable(const IgemmArgs& a, int in_dt, int out_dt);
bool launch_conv3x3_stream(const IgemmArgs& a, hipStream_t s);
// The stream kernel's launch plan for N images of H x W with C channels and F filters: out = {TH, S, top, aligned, tiles,
// segments per patch row, pixel groups, filter groups, K groups, filter blocks, workgroups per filter block, segment
// capacity of a patch buffer}; host arithmetic only (no device needed); false = no plan.
bool conv3x3_stream_plan(int N, int H, int W, int C, int F, int out[14]);
size_t weight_frag32_bytes(int F, int C);
void launch_weight_frag32(const void* w, int w_dt, void* dst, int F, int C, hipStream_t s);
// Stride-2 image convolutions over pixel pairs (C = 8, fp16, 6x3 and 3x2 windows, at most 64 filters):
// the whole K axis in one step (conv_pairs.hip); same arguments and epilogue as the igemm kernels.
bool conv_pairs_applicable(const IgemmArgs& a, int in_dt, int out_dt);
void launch_conv_pairs(const IgemmArgs& a, hipStream_t s);
bool igemm_fast_applicable(const IgemmArgs& a, int in_dt, int out_dt);
void launch_igemm_fast(const IgemmArgs& a, int in_dt, int out_dt, hipStream_t s);

// fp32 row-major C += A.B  (linalg.matmul)
void launch_gemm_nn_f32(const float* A, const float* B, float* C, int M, int N, int K, hipStream_t s);

// ---------------------------------------------------------------------------------------------
// Winograd F(4x4,3x3)
// ---------------------------------------------------------------------------------------------
struct Strides4 { long long n, c, h, w; };  // element strides of a logical [N][C][H][W] tensor
inline Strides4 strides_of(int layout, int C, int H, int W) {
  if (layout == kNHWC) return {(long long)H * W * C, 1, (long long)W * C, C};
  return {(long long)C * H * W, (long long)H * W, W, 1};
}

// U[36][F][C] = G g G^T from w[F][C][3][3]; U stored as u_dt, optionally scaled by 2^u_shift.
void launch_wino43_filter(const void* w, int w_dt, void* U, int u_dt, int F, int C, hipStream_t s);
// V[36][tiles][C] = B^T d B; input addressed through `st` (any layout), zero halo of `pad`.
void launch_wino43_input(const void* in, int in_dt, Strides4 st, void* V, int v_dt, int N, int C, int H,
                         int W, int pad, hipStream_t s);
// out = epilogue(A^T M A), M[36][tiles][F] of m_dt; out/residual addressed through `st`.
struct WinoOutArgs {
  const void* M; void* out; const void* residual; const float* scale; const float* shift;
  Strides4 st; int N, F, OH, OW; int relu; int accumulate;  // accumulate: out += result (ABI conv form)
};
void launch_wino43_output(const WinoOutArgs& a, int m_dt, int out_dt, hipStream_t s);

// ---------------------------------------------------------------------------------------------
// Pooling, layout and parameter preparation
// ---------------------------------------------------------------------------------------------
void launch_maxpool3x3s2_nhwc(const void* in, void* out, int dt, int N, int H, int W, int C, hipStream_t s);
void launch_global_avgpool_nhwc(const void* in, void* out, int dt, int N, int HW, int C, hipStream_t s);
// head: global average pool + fully connected layer with bias, fp32 logits (C must be 512)
void launch_avgpool_fc(const void* in, const void* w, const float* bias, float* out, int dt, int N, int HW, int C, int F,
                       hipStream_t s);
// the reference driver's image preparation (u8 HWC -> normalised NCHW) and top-1 scan, on the device
void launch_preprocess_u8(const void* src, void* dst, int dst_dt, int N, int H, int W, int channels, hipStream_t s);
void launch_argmax_rows(const float* x, int* idx, int N, int F, hipStream_t s);
// generic strided copy/cast between layouts: dst[n,c,h,w] (+)= (c < Csrc ? src[n,c,h,w] : 0) for c < Cdst
void launch_relayout(const void* src, int src_dt, Strides4 ss, void* dst, int dst_dt, Strides4 ds, int N,
                     int Csrc, int Cdst, int H, int W, bool accumulate, hipStream_t s);
// image [N,C,H,W] with C <= one 16-byte vector -> NHWC [N,H,W,vector], zero padded channels
bool image_to_nhwc_applicable(int dt, int C);
// (Cp: channels per pixel of dst, 0 = one vector; 4 with fp16 = the pixel-pair form)
void launch_image_to_nhwc(const void* src, void* dst, int dt, int N, int C, int H, int W, hipStream_t s, int Cp = 0);
// fp16 filters [F,C<=4,K,K] of a stride-2 convolution re-laid for an image stored as pixel pairs:
// dst [Fp][K][S2][8], S2 = ceil((K + pad%2) / 2); the convolution then runs with S = S2, stride 1 and
// padding (pad + 1) / 2 along x over W/2 pairs of 8 channels
void launch_weight_pairs(const void* w, int w_dt, void* dst, int F, int Fp, int C, int K, int pad, hipStream_t s);
// stem input: NCHW [N,3,H,W] -> zero-haloed pixel-pair image [N][H+6][(W+8)/2][8]
void launch_stem_pack(const void* src, int src_dt, void* dst, int dst_dt, int N, int H, int W, hipStream_t s);
// weights FCRS -> [F][R][S][Cp] (Cp >= C, zero filled), cast to dst_dt
void launch_weight_frsc(const void* w, int w_dt, void* dst, int dst_dt, int F, int C, int R, int S, int Cp,
                        hipStream_t s);
// 3x3 weights FCHW -> fragment-major order of conv3x3_patch.hip, F padded to a multiple of 64
void launch_weight_frag3x3(const void* w, int w_dt, void* dst, int dst_dt, int F, int C, hipStream_t s);
// 1x1 weights [F][C] in the same order with one tap per slab (IgemmArgs::aux_wt_frag)
void launch_weight_frag1x1(const void* w, int w_dt, void* dst, int dst_dt, int F, int C, hipStream_t s);
// stem weights [64,3,7,7] -> [64][7][4][8] over (pixel-pair, channel4); pair sp / pixel p holds
// filter column 2*sp + p - col_shift (zero outside 0..6)
void launch_stem_weight(const void* w, int w_dt, void* dst, int dst_dt, int F, int col_shift, hipStream_t s);
// fused stem: conv7x7 s2 p3 + scale/shift + ReLU + maxpool 3x3 s2 p1, NCHW fp16 in, NHWC out
// (stem_pool.hip); wt in the col_shift = 1 layout above
bool stem_pool_applicable(int dt, int N, int H, int W, int F);
void launch_stem_pool(const void* in, const void* wt, const float* scale, const float* shift, void* out, int N, int H, int W,
                      hipStream_t s);
// BN fold: scale = gamma / sqrt(var + eps), shift = beta - mean*scale (fp32 out)
void launch_bn_fold(const void* gamma, const void* beta, const void* mean, const void* var, int dt, float* scale,
                    float* shift, int C, hipStream_t s, float eps = 1e-5f);

// ---------------------------------------------------------------------------------------------
// Operators of the other network fixtures (MobileNetV3.mlir, Yolov5s.mlir), NHWC, elementwise.hip
// ---------------------------------------------------------------------------------------------
// linalg.depthwise_conv_2d_nchw_chw (+ zero halo of `pad`) + scale/shift + activation.
// wt: [K][K][C] of type dt (launch_weight_dw); K in {3, 5}; C a multiple of the 16-byte vector.
struct DwConvArgs {
  const void* in; const void* wt; void* out; const float* scale; const float* shift;
  int N, H, W, C, K, stride, pad, OH, OW, act;
};
void launch_dwconv(const DwConvArgs& a, int dt, hipStream_t s);
// depthwise weights [C][1][K][K] (or [C][K][K]) -> [K][K][C]
void launch_weight_dw(const void* w, int w_dt, void* dst, int dst_dt, int C, int K, hipStream_t s);
// out[n,p,c] = x[n,p,c] * g[n,c]   (squeeze-excitation gate; MobileNetV3.mlir:380-384)
void launch_scale_channels(const void* x, const void* g, void* out, int dt, int N, int HW, int C, hipStream_t s);
// Whole squeeze-excitation block: out = x * act2(W2 . act1(W1 . mean_hw(x) + b1) + b2), one launch.
// w1 [SQ][C], w2 [C][SQ] of type dt; b1, b2 fp32.
struct SeArgs {
  const void* x; const void* w1; const float* b1; const void* w2; const float* b2; void* out;
  int N, HW, C, SQ, act1, act2;
};
bool se_block_applicable(int dt, int HW, int C, int SQ);
void launch_se_block(const SeArgs& a, int dt, hipStream_t s);
// out = act(a (+ b));  b may be null;  n elements, n a multiple of the 16-byte vector
void launch_eltwise(const void* a, const void* b, void* out, int dt, long long n, int act, hipStream_t s);
// the same over [P][C] tensors with row pitches lda / ldb / ldo (elements): slices of wider tensors
void launch_eltwise_pitched(const void* a, int lda, const void* b, int ldb, void* out, int ldo, int dt, long long P, int C, int act,
                            hipStream_t s);
// copies x [P][C] into channels [c0, c0 + C) of out [P][ldo]   (torch.cat over channels, NHWC)
// (ldi: row pitch of x, 0 = C)
void launch_concat_slice(const void* x, void* out, int dt, long long P, int C, int ldo, int c0, hipStream_t s, int ldi = 0);
// nearest-neighbour 2x up-sampling [N,H,W,C] -> [N,2H,2W,C], written at channel offset c0 of pitch ldo
void launch_upsample2x(const void* x, void* out, int dt, int N, int H, int W, int C, int ldo, int c0, hipStream_t s, int ldi = 0);
// max-pool K x K, any stride / padding (-inf halo), NHWC
// y1 = m(x), y2 = m(y1), y3 = m(y2) with m = max-pool 5x5 stride 1 pad 2, all three kept, in one launch
// (maps of at most 1600 pixels); ld*: elements between pixels of each tensor.
bool maxpool5_chain3_applicable(int dt, int H, int W, int C);
void launch_maxpool5_chain3(const void* in, void* o1, void* o2, void* o3, int dt, int N, int H, int W, int C, int ldi, int ld1, int ld2,
                            int ld3, hipStream_t s);
void launch_maxpool_nhwc(const void* in, void* out, int dt, int N, int H, int W, int C, int K, int stride, int pad,
                         hipStream_t s, int ldi = 0, int ldo = 0);  // pixel pitches of in / out, 0 = C
// YOLOv5 Detect decode of one level: head [N,H,W,ldc] (A*F used channels, anchor-major) ->
// out[n][box0 + (a*H + y)*W + x][0..F) fp32, rows of `boxes_total` boxes per image.
// anchor_wh: A (w, h) pairs already multiplied by the stride.
struct DetectArgs {
  const void* head; float* out; int N, H, W, A, F, ldc; long long box0, boxes_total; float stride; float anchor_wh[8];
  float inv_f, inv_w;  // filled in by the launcher
};
void launch_yolo_detect(const DetectArgs& a, int dt, hipStream_t s);
void launch_cast(const void* src, int src_dt, void* dst, int dst_dt, long long n, hipStream_t s);
void launch_fill_f32(float* dst, float v, long long n, hipStream_t s);

}  // namespace nncv_hip
