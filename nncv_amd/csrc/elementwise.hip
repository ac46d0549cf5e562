// Bandwidth-bound operators of the reference's other network fixtures, NHWC, one 16-byte channel
// group per lane:
//   linalg.depthwise_conv_2d_nchw_chw + BatchNorm + activation   (tests/Nets/MobileNetV3.mlir:284-303)
//   squeeze-excitation gate  x[n,c,h,w] * g[n,c]                 (MobileNetV3.mlir:380-384)
//   add / activation, channel concatenation, nearest 2x up-sampling, K x K max-pool
//                                                                (tests/Nets/Yolov5s.mlir)
// None of them has arithmetic intensity worth MFMA: the bound is HBM (or L2 for the small maps),
// so the only rules are whole-vector coalesced accesses along the channel axis and no
// materialised halo (tensor.pad becomes a predicate).
#include "common.hpp"

namespace nncv_hip {

namespace {

template <typename T>
struct V16;
template <>
struct V16<float> {
  typedef float type __attribute__((ext_vector_type(4)));
  static constexpr int n = 4;
};
template <>
struct V16<half_t> {
  typedef half_t type __attribute__((ext_vector_type(8)));
  static constexpr int n = 8;
};

// arith.maximumf: NaN in either operand wins
__device__ __forceinline__ float max_nan(float m, float v) { return (v > m || v != v) ? v : m; }

inline unsigned grid_for(long long work) {
  const long long g = (work + 255) / 256;
  NNCV_REQUIRE(g >= 1 && g < (1ll << 31), "elementwise: grid out of range");
  return (unsigned)g;
}

}  // namespace

// ---------------------------------------------------------------------------------------------
// Depthwise convolution.  One thread = one output pixel x one channel group; the K*K input
// vectors it needs are shared with its neighbours through L1/L2 (the maps of the MobileNet
// stages are at most a few MB).  fp32 accumulation in (kh, kw) order like the reference's loop
// nest; scale/shift (folded BatchNorm) and the activation are applied before the one rounding.
// ---------------------------------------------------------------------------------------------
template <typename T, int K>
__global__ __launch_bounds__(256) void dwconv_kernel(const DwConvArgs a) {
  constexpr int VN = V16<T>::n;
  typedef typename V16<T>::type V;
  const int CG = a.C / VN;
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long long)a.N * a.OH * a.OW * CG) return;
  const int cg = (int)(idx % CG);
  long long p = idx / CG;
  const int ox = (int)(p % a.OW);
  p /= a.OW;
  const int oy = (int)(p % a.OH);
  const int n = (int)(p / a.OH);
  const T* in = static_cast<const T*>(a.in) + (long long)n * a.H * a.W * a.C + cg * VN;
  const T* wt = static_cast<const T*>(a.wt) + cg * VN;
  float acc[VN];
#pragma unroll
  for (int e = 0; e < VN; ++e) acc[e] = 0.0f;
#pragma unroll
  for (int r = 0; r < K; ++r) {
    const int iy = oy * a.stride - a.pad + r;
    if ((unsigned)iy >= (unsigned)a.H) continue;
#pragma unroll
    for (int s = 0; s < K; ++s) {
      const int ix = ox * a.stride - a.pad + s;
      if ((unsigned)ix >= (unsigned)a.W) continue;
      const V x = *reinterpret_cast<const V*>(in + ((long long)iy * a.W + ix) * a.C);
      const V w = *reinterpret_cast<const V*>(wt + (r * K + s) * a.C);
#pragma unroll
      for (int e = 0; e < VN; ++e) acc[e] += (float)x[e] * (float)w[e];
    }
  }
  V o;
#pragma unroll
  for (int e = 0; e < VN; ++e) {
    float y = acc[e];
    if (a.scale) y *= a.scale[cg * VN + e];
    if (a.shift) y += a.shift[cg * VN + e];
    o[e] = (T)act_apply(y, a.act);
  }
  *reinterpret_cast<V*>(static_cast<T*>(a.out) + (((long long)n * a.OH + oy) * a.OW + ox) * a.C + cg * VN) = o;
}

void launch_dwconv(const DwConvArgs& a, int dt, hipStream_t s) {
  const int vn = dt == kF16 ? 8 : 4;
  NNCV_REQUIRE(a.K == 3 || a.K == 5, "dwconv: kernel size must be 3 or 5");
  NNCV_REQUIRE(a.C % vn == 0, "dwconv: C must be a multiple of the 16-byte vector");
  NNCV_REQUIRE(a.stride >= 1 && a.pad >= 0 && a.N >= 1 && a.H >= 1 && a.W >= 1, "dwconv: bad geometry");
  NNCV_REQUIRE(a.OH == (a.H + 2 * a.pad - a.K) / a.stride + 1 && a.OW == (a.W + 2 * a.pad - a.K) / a.stride + 1 && a.OH >= 1 &&
                   a.OW >= 1,
               "dwconv: output size does not match input/filter/stride/pad");
  const long long work = (long long)a.N * a.OH * a.OW * (a.C / vn);
  const unsigned grid = grid_for(work);
  const double px_in = (double)a.N * a.H * a.W, px_out = (double)a.N * a.OH * a.OW;
  ProfScope prof(a.K == 3 ? "dwconv3x3" : "dwconv5x5", 2.0 * px_out * a.C * a.K * a.K,
                 (double)dtype_size(dt) * a.C * (px_in + px_out + a.K * a.K), s);
#define LAUNCH(T, KK) hipLaunchKernelGGL((dwconv_kernel<T, KK>), dim3(grid), dim3(256), 0, s, a)
  if (dt == kF16) {
    if (a.K == 3) LAUNCH(half_t, 3); else LAUNCH(half_t, 5);
  } else {
    if (a.K == 3) LAUNCH(float, 3); else LAUNCH(float, 5);
  }
#undef LAUNCH
  NNCV_HIP_CHECK(hipGetLastError());
}

template <typename Ts, typename Td>
__global__ void weight_dw_kernel(const Ts* __restrict__ w, Td* __restrict__ dst, int C, int KK) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;  // destination index: tap * C + c
  if (i >= C * KK) return;
  const int c = i % C, tap = i / C;
  dst[i] = (Td)(float)w[c * KK + tap];
}

void launch_weight_dw(const void* w, int w_dt, void* dst, int dst_dt, int C, int K, hipStream_t s) {
  const int n = C * K * K;
  const unsigned grid = grid_for(n);
#define LAUNCH(TS, TD) hipLaunchKernelGGL((weight_dw_kernel<TS, TD>), dim3(grid), dim3(256), 0, s, (const TS*)w, (TD*)dst, C, K * K)
  if (w_dt == kF32 && dst_dt == kF32) LAUNCH(float, float);
  else if (w_dt == kF16 && dst_dt == kF16) LAUNCH(half_t, half_t);
  else if (w_dt == kF32 && dst_dt == kF16) LAUNCH(float, half_t);
  else LAUNCH(half_t, float);
#undef LAUNCH
  NNCV_HIP_CHECK(hipGetLastError());
}

// ---------------------------------------------------------------------------------------------
// out[n,p,:] = x[n,p,:] * g[n,:]
// ---------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void scale_channels_kernel(const T* __restrict__ x, const T* __restrict__ g, T* __restrict__ out,
                                                             long long total, int HWCG, int CG) {
  constexpr int VN = V16<T>::n;
  typedef typename V16<T>::type V;
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const int n = (int)(idx / HWCG);
  const int cg = (int)(idx % CG);
  const V xv = *reinterpret_cast<const V*>(x + idx * VN);
  const V gv = *reinterpret_cast<const V*>(g + ((long long)n * CG + cg) * VN);
  V o;
#pragma unroll
  for (int e = 0; e < VN; ++e) o[e] = (T)((float)gv[e] * (float)xv[e]);
  *reinterpret_cast<V*>(out + idx * VN) = o;
}

void launch_scale_channels(const void* x, const void* g, void* out, int dt, int N, int HW, int C, hipStream_t s) {
  const int vn = dt == kF16 ? 8 : 4;
  NNCV_REQUIRE(C % vn == 0, "scale_channels: C must be a multiple of the 16-byte vector");
  const int CG = C / vn;
  NNCV_REQUIRE((long long)HW * CG < (1ll << 31), "scale_channels: image too large");
  const long long total = (long long)N * HW * CG;
  if (total == 0) return;
  ProfScope prof("scale_channels", (double)total * vn, (double)dtype_size(dt) * (2.0 * total * vn + (double)N * C), s);
  if (dt == kF16)
    hipLaunchKernelGGL((scale_channels_kernel<half_t>), dim3(grid_for(total)), dim3(256), 0, s, (const half_t*)x, (const half_t*)g,
                       (half_t*)out, total, HW * CG, CG);
  else
    hipLaunchKernelGGL((scale_channels_kernel<float>), dim3(grid_for(total)), dim3(256), 0, s, (const float*)x, (const float*)g,
                       (float*)out, total, HW * CG, CG);
  NNCV_HIP_CHECK(hipGetLastError());
}

// ---------------------------------------------------------------------------------------------
// out = act(a + b)
// ---------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void eltwise_kernel(const T* __restrict__ a, const T* __restrict__ b, T* __restrict__ out,
                                                      long long nvec, int act) {
  constexpr int VN = V16<T>::n;
  typedef typename V16<T>::type V;
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= nvec) return;
  const V av = *reinterpret_cast<const V*>(a + idx * VN);
  float y[VN];
#pragma unroll
  for (int e = 0; e < VN; ++e) y[e] = (float)av[e];
  if (b) {
    const V bv = *reinterpret_cast<const V*>(b + idx * VN);
#pragma unroll
    for (int e = 0; e < VN; ++e) y[e] += (float)bv[e];
  }
  V o;
#pragma unroll
  for (int e = 0; e < VN; ++e) o[e] = (T)act_apply(y[e], act);
  *reinterpret_cast<V*>(out + idx * VN) = o;
}

void launch_eltwise(const void* a, const void* b, void* out, int dt, long long n, int act, hipStream_t s) {
  const int vn = dt == kF16 ? 8 : 4;
  NNCV_REQUIRE(n % vn == 0, "eltwise: element count must be a multiple of the 16-byte vector");
  if (n == 0) return;
  ProfScope prof(b ? "eltwise_add" : "eltwise_act", (double)n, (double)dtype_size(dt) * n * (b ? 3 : 2), s);
  if (dt == kF16)
    hipLaunchKernelGGL((eltwise_kernel<half_t>), dim3(grid_for(n / vn)), dim3(256), 0, s, (const half_t*)a, (const half_t*)b,
                       (half_t*)out, n / vn, act);
  else
    hipLaunchKernelGGL((eltwise_kernel<float>), dim3(grid_for(n / vn)), dim3(256), 0, s, (const float*)a, (const float*)b,
                       (float*)out, n / vn, act);
  NNCV_HIP_CHECK(hipGetLastError());
}

// ---------------------------------------------------------------------------------------------
// Channel concatenation (a strided copy into a slice of the wider tensor) and nearest 2x
// up-sampling written straight into such a slice; both move raw 16-byte vectors.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void concat_slice_kernel(const uint4* __restrict__ x, uint4* __restrict__ out, long long total,
                                                           int CG, int ldg, int g0) {
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const long long p = idx / CG;
  const int cg = (int)(idx % CG);
  out[p * ldg + g0 + cg] = x[idx];
}

void launch_concat_slice(const void* x, void* out, int dt, long long P, int C, int ldo, int c0, hipStream_t s) {
  const int vn = dt == kF16 ? 8 : 4;
  NNCV_REQUIRE(C % vn == 0 && ldo % vn == 0 && c0 % vn == 0 && c0 >= 0 && c0 + C <= ldo,
               "concat: channel counts and offset must be multiples of the 16-byte vector");
  const long long total = P * (C / vn);
  if (total == 0) return;
  ProfScope prof("concat_slice", 0.0, 2.0 * dtype_size(dt) * P * C, s);
  hipLaunchKernelGGL(concat_slice_kernel, dim3(grid_for(total)), dim3(256), 0, s, (const uint4*)x, (uint4*)out, total, C / vn,
                     ldo / vn, c0 / vn);
  NNCV_HIP_CHECK(hipGetLastError());
}

__global__ __launch_bounds__(256) void upsample2x_kernel(const uint4* __restrict__ x, uint4* __restrict__ out, long long total,
                                                         int H, int W, int CG, int ldg, int g0) {
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;  // over output vectors
  if (idx >= total) return;
  const int cg = (int)(idx % CG);
  long long p = idx / CG;
  const int ox = (int)(p % (2 * W));
  p /= 2 * W;
  const int oy = (int)(p % (2 * H));
  const long long n = p / (2 * H);
  out[((n * 2 * H + oy) * 2 * W + ox) * ldg + g0 + cg] = x[((n * H + (oy >> 1)) * W + (ox >> 1)) * CG + cg];
}

void launch_upsample2x(const void* x, void* out, int dt, int N, int H, int W, int C, int ldo, int c0, hipStream_t s) {
  const int vn = dt == kF16 ? 8 : 4;
  NNCV_REQUIRE(C % vn == 0 && ldo % vn == 0 && c0 % vn == 0 && c0 >= 0 && c0 + C <= ldo,
               "upsample: channel counts and offset must be multiples of the 16-byte vector");
  const long long total = (long long)N * 4 * H * W * (C / vn);
  if (total == 0) return;
  ProfScope prof("upsample2x", 0.0, 5.0 * dtype_size(dt) * N * H * W * C, s);
  hipLaunchKernelGGL(upsample2x_kernel, dim3(grid_for(total)), dim3(256), 0, s, (const uint4*)x, (uint4*)out, total, H, W, C / vn,
                     ldo / vn, c0 / vn);
  NNCV_HIP_CHECK(hipGetLastError());
}

// ---------------------------------------------------------------------------------------------
// linalg.pooling_nchw_max with any window / stride over a -inf halo (Yolov5s.mlir: 5x5 stride 1
// pad 2 in the SPPF block), NHWC
// ---------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void maxpool_kernel(const T* __restrict__ in, T* __restrict__ out, int N, int H, int W, int C,
                                                      int K, int stride, int pad, int OH, int OW) {
  constexpr int VN = V16<T>::n;
  typedef typename V16<T>::type V;
  const int CG = C / VN;
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long long)N * OH * OW * CG) return;
  const int cg = (int)(idx % CG);
  long long p = idx / CG;
  const int ox = (int)(p % OW);
  p /= OW;
  const int oy = (int)(p % OH);
  const int n = (int)(p / OH);
  float m[VN];
#pragma unroll
  for (int e = 0; e < VN; ++e) m[e] = -INFINITY;
  for (int r = 0; r < K; ++r) {
    const int iy = oy * stride - pad + r;
    if ((unsigned)iy >= (unsigned)H) continue;
    for (int q = 0; q < K; ++q) {
      const int ix = ox * stride - pad + q;
      if ((unsigned)ix >= (unsigned)W) continue;
      const V v = *reinterpret_cast<const V*>(in + (((long long)n * H + iy) * W + ix) * C + cg * VN);
#pragma unroll
      for (int e = 0; e < VN; ++e) m[e] = max_nan(m[e], (float)v[e]);
    }
  }
  V o;
#pragma unroll
  for (int e = 0; e < VN; ++e) o[e] = (T)m[e];
  *reinterpret_cast<V*>(out + (((long long)n * OH + oy) * OW + ox) * C + cg * VN) = o;
}

void launch_maxpool_nhwc(const void* in, void* out, int dt, int N, int H, int W, int C, int K, int stride, int pad,
                         hipStream_t s) {
  const int vn = dt == kF16 ? 8 : 4;
  NNCV_REQUIRE(C % vn == 0, "maxpool: C must be a multiple of the 16-byte vector");
  NNCV_REQUIRE(K >= 1 && stride >= 1 && pad >= 0 && 2 * pad <= K && H + 2 * pad >= K && W + 2 * pad >= K, "maxpool: bad geometry");
  const int OH = (H + 2 * pad - K) / stride + 1, OW = (W + 2 * pad - K) / stride + 1;
  const long long work = (long long)N * OH * OW * (C / vn);
  if (work == 0) return;
  ProfScope prof("maxpool", 0.0, (double)dtype_size(dt) * N * C * ((double)H * W + (double)OH * OW), s);
  if (dt == kF16)
    hipLaunchKernelGGL((maxpool_kernel<half_t>), dim3(grid_for(work)), dim3(256), 0, s, (const half_t*)in, (half_t*)out, N, H, W, C,
                       K, stride, pad, OH, OW);
  else
    hipLaunchKernelGGL((maxpool_kernel<float>), dim3(grid_for(work)), dim3(256), 0, s, (const float*)in, (float*)out, N, H, W, C, K,
                       stride, pad, OH, OW);
  NNCV_HIP_CHECK(hipGetLastError());
}

}  // namespace nncv_hip
