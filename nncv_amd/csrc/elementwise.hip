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
// Depthwise convolution.  One thread = OXT horizontally adjacent output pixels x one channel
// group: per filter row it loads the (OXT-1)*S + K input vectors the strip needs once and each
// filter tap once, instead of K*K of both per output pixel -- the kernel is bound by the number of
// vector-memory instructions, not by HBM (the maps of the MobileNet stages are a few MB and the
// halo reuse between neighbouring threads is served by L1/L2).  fp32 accumulation in (kh, kw)
// order like the reference's loop nest; scale/shift (folded BatchNorm) and the activation are
// applied before the one rounding.
// ---------------------------------------------------------------------------------------------
template <typename T, int K, int S, int OXT>
__global__ __launch_bounds__(128) void dwconv_kernel(const DwConvArgs a, int strips) {
  constexpr int VN = V16<T>::n;
  constexpr int LW = (OXT - 1) * S + K;  // input pixels one strip touches per filter row
  typedef typename V16<T>::type V;
  const int CG = a.C / VN;
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long long)a.N * a.OH * strips * CG) return;
  const int cg = (int)(idx % CG);
  long long p = idx / CG;
  const int sx = (int)(p % strips);
  p /= strips;
  const int oy = (int)(p % a.OH);
  const int n = (int)(p / a.OH);
  const int ox0 = sx * OXT;
  const T* in = static_cast<const T*>(a.in) + (long long)n * a.H * a.W * a.C + cg * VN;
  const T* wt = static_cast<const T*>(a.wt) + cg * VN;
  const int ix0 = ox0 * S - a.pad;
  float acc[OXT][VN];
#pragma unroll
  for (int j = 0; j < OXT; ++j)
#pragma unroll
    for (int e = 0; e < VN; ++e) acc[j][e] = 0.0f;
  // Every load is unconditional from a clamped address and zeroed afterwards when it lies in the
  // halo: no control flow in the tap loops, so the loads of all rows can be in flight together.
#pragma unroll
  for (int r = 0; r < K; ++r) {
    const int iy = oy * S - a.pad + r;
    const bool rok = (unsigned)iy < (unsigned)a.H;
    const T* row = in + (long long)min(max(iy, 0), a.H - 1) * a.W * a.C;
    V x[LW];
#pragma unroll
    for (int q = 0; q < LW; ++q) {
      const int ix = ix0 + q;
      const bool ok = rok && (unsigned)ix < (unsigned)a.W;
      x[q] = *reinterpret_cast<const V*>(row + (long long)min(max(ix, 0), a.W - 1) * a.C);
      if (!ok) {
#pragma unroll
        for (int e = 0; e < VN; ++e) x[q][e] = (T)0.0f;
      }
    }
#pragma unroll
    for (int s = 0; s < K; ++s) {
      const V w = *reinterpret_cast<const V*>(wt + (r * K + s) * a.C);
#pragma unroll
      for (int j = 0; j < OXT; ++j)
#pragma unroll
        for (int e = 0; e < VN; ++e) acc[j][e] += (float)x[j * S + s][e] * (float)w[e];
    }
  }
  float sc[VN], sh[VN];
#pragma unroll
  for (int e = 0; e < VN; ++e) {
    sc[e] = a.scale ? a.scale[cg * VN + e] : 1.0f;
    sh[e] = a.shift ? a.shift[cg * VN + e] : 0.0f;
  }
  T* out = static_cast<T*>(a.out) + (((long long)n * a.OH + oy) * a.OW) * a.C + cg * VN;
#pragma unroll
  for (int j = 0; j < OXT; ++j) {
    if (ox0 + j >= a.OW) break;
    V o;
    float y[VN];
#pragma unroll
    for (int e = 0; e < VN; ++e) y[e] = acc[j][e] * sc[e] + sh[e];
    act_apply_n<sizeof(T) == 2>(y, a.act);
#pragma unroll
    for (int e = 0; e < VN; ++e) o[e] = (T)y[e];
    *reinterpret_cast<V*>(out + (long long)(ox0 + j) * a.C) = o;
  }
}

template <typename T, int K, int S, int OXT>
static void launch_dwconv_oxt(const DwConvArgs& a, hipStream_t s) {
  const int strips = (a.OW + OXT - 1) / OXT;
  const long long work = (long long)a.N * a.OH * strips * (a.C / V16<T>::n);
  const long long grid = (work + 127) / 128;
  NNCV_REQUIRE(grid >= 1 && grid < (1ll << 31), "dwconv: grid out of range");
  hipLaunchKernelGGL((dwconv_kernel<T, K, S, OXT>), dim3((unsigned)grid), dim3(128), 0, s, a, strips);
}

// A lane-FMA is all the arithmetic there is (a wave retires one per 4 cycles), so the launch is as
// long as the FMA chain of one thread unless there are many waves per CU to interleave.  Strips
// of 4 or 2 outputs per thread save vector loads, but only pay once the grid is large enough to
// fill the machine with them (256 CUs x 8 waves).
template <typename T, int K, int S>
static void launch_dwconv_cfg(const DwConvArgs& a, hipStream_t s) {
  const long long vecs = (long long)a.N * a.OH * (a.C / V16<T>::n);
  auto waves = [&](int oxt) { return vecs * ((a.OW + oxt - 1) / oxt) / 64; };
  if (waves(4) >= 2048 && !(K == 5 && S == 2)) launch_dwconv_oxt<T, K, S, 4>(a, s);
  else if (waves(2) >= 2048) launch_dwconv_oxt<T, K, S, 2>(a, s);
  else launch_dwconv_oxt<T, K, S, 1>(a, s);
}

void launch_dwconv(const DwConvArgs& a, int dt, hipStream_t s) {
  const int vn = dt == kF16 ? 8 : 4;
  NNCV_REQUIRE(a.K == 3 || a.K == 5, "dwconv: kernel size must be 3 or 5");
  NNCV_REQUIRE(a.stride == 1 || a.stride == 2, "dwconv: stride must be 1 or 2");
  NNCV_REQUIRE(a.C % vn == 0, "dwconv: C must be a multiple of the 16-byte vector");
  NNCV_REQUIRE(a.pad >= 0 && a.N >= 1 && a.H >= 1 && a.W >= 1, "dwconv: bad geometry");
  NNCV_REQUIRE(a.OH == (a.H + 2 * a.pad - a.K) / a.stride + 1 && a.OW == (a.W + 2 * a.pad - a.K) / a.stride + 1 && a.OH >= 1 &&
                   a.OW >= 1,
               "dwconv: output size does not match input/filter/stride/pad");
  const double px_in = (double)a.N * a.H * a.W, px_out = (double)a.N * a.OH * a.OW;
  ProfScope prof(a.K == 3 ? "dwconv3x3" : "dwconv5x5", 2.0 * px_out * a.C * a.K * a.K,
                 (double)dtype_size(dt) * a.C * (px_in + px_out + a.K * a.K), s);
  const int sel = (dt == kF16 ? 0 : 4) + (a.K == 3 ? 0 : 2) + (a.stride == 1 ? 0 : 1);
  switch (sel) {
    case 0: launch_dwconv_cfg<half_t, 3, 1>(a, s); break;
    case 1: launch_dwconv_cfg<half_t, 3, 2>(a, s); break;
    case 2: launch_dwconv_cfg<half_t, 5, 1>(a, s); break;
    case 3: launch_dwconv_cfg<half_t, 5, 2>(a, s); break;
    case 4: launch_dwconv_cfg<float, 3, 1>(a, s); break;
    case 5: launch_dwconv_cfg<float, 3, 2>(a, s); break;
    case 6: launch_dwconv_cfg<float, 5, 1>(a, s); break;
    default: launch_dwconv_cfg<float, 5, 2>(a, s); break;
  }
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
// Squeeze-excitation block in one launch (MobileNetV3.mlir:322-384): global average pool, 1x1
// convolution + bias + act1 (C -> SQ), 1x1 convolution + bias + act2 (SQ -> C), and the gate
// multiplied back onto the input.  One workgroup per image: its activation (at most a few
// hundred KB in these networks) is read twice, the second time out of L2, and nothing but the
// gated result is written.  The pooled vector, the squeezed vector and the gate stay in fp32 in
// LDS -- they are never rounded to the storage type.  1024 threads and batched loads, because
// with one workgroup per image the launch is as long as its longest chain of dependent loads.
// ---------------------------------------------------------------------------------------------
constexpr int kSeMaxC = 1024, kSeMaxSq = 256, kSeThreads = 1024;

template <typename T>
__global__ __launch_bounds__(kSeThreads) void se_block_kernel(const SeArgs a) {
  constexpr int VN = V16<T>::n;
  constexpr int NT = kSeThreads, NW = NT / 64;
  typedef typename V16<T>::type V;
  __shared__ float part[NT * VN];
  __shared__ float mean[kSeMaxC];
  __shared__ float hid[kSeMaxSq];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n = blockIdx.x;
  const int CG = a.C / VN;
  const T* __restrict__ x = static_cast<const T*>(a.x) + (long long)n * a.HW * a.C;

  // 1. pool: thread = (pixel phase pp, channel group cg), eight loads in flight
  const int ppb = NT / CG;  // CG <= 256
  const int pp = tid / CG, cg = tid - pp * CG;
  if (pp < ppb) {
    float acc[VN];
#pragma unroll
    for (int e = 0; e < VN; ++e) acc[e] = 0.0f;
    constexpr int U = 8;
    for (int p = pp; p < a.HW; p += U * ppb) {
      V v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) v[u] = *reinterpret_cast<const V*>(x + (long long)min(p + u * ppb, a.HW - 1) * a.C + cg * VN);
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (p + u * ppb < a.HW) {
#pragma unroll
          for (int e = 0; e < VN; ++e) acc[e] += (float)v[u][e];
        }
    }
#pragma unroll
    for (int e = 0; e < VN; ++e) part[tid * VN + e] = acc[e];
  }
  __syncthreads();
  // the ppb partial rows (C floats each, row q at part[q * C]) are folded in two steps so that a
  // narrow tensor (C = 16: 512 rows) is not one thread's chain of 512 dependent LDS reads
  const int GA = min(ppb, max(1, NT / a.C));
  {
    const int g = tid / a.C, c = tid - g * a.C;
    if (g < GA) {
      float s = 0.0f;
#pragma unroll 8
      for (int q = g; q < ppb; q += GA) s += part[q * a.C + c];
      part[g * a.C + c] = s;  // row g is read by this thread only
    }
  }
  __syncthreads();
  for (int c = tid; c < a.C; c += NT) {
    float s = 0.0f;
#pragma unroll 8
    for (int q = 0; q < GA; ++q) s += part[q * a.C + c];
    mean[c] = s / (float)a.HW;
  }
  __syncthreads();

  // 2. squeeze: a wave takes four outputs at a time, lanes along C
  const T* __restrict__ w1 = static_cast<const T*>(a.w1);
  constexpr int JB = 4;
  for (int j0 = wave; j0 < a.SQ; j0 += NW * JB) {
    float s[JB];
#pragma unroll
    for (int b = 0; b < JB; ++b) s[b] = 0.0f;
    for (int v = lane; v < CG; v += 64) {
      V w[JB];
#pragma unroll
      for (int b = 0; b < JB; ++b) w[b] = *reinterpret_cast<const V*>(w1 + (long long)min(j0 + b * NW, a.SQ - 1) * a.C + v * VN);
#pragma unroll
      for (int b = 0; b < JB; ++b)
#pragma unroll
        for (int e = 0; e < VN; ++e) s[b] += mean[v * VN + e] * (float)w[b][e];
    }
#pragma unroll
    for (int b = 0; b < JB; ++b) {
#pragma unroll
      for (int o = 32; o >= 1; o >>= 1) s[b] += __shfl_xor(s[b], o);
      const int j = j0 + b * NW;
      if (lane == 0 && j < a.SQ) hid[j] = act_apply(s[b] + a.b1[j], a.act1);
    }
  }
  __syncthreads();

  // 3. excite: one thread per channel, six filter vectors in flight; the gate overwrites the means
  const T* __restrict__ w2 = static_cast<const T*>(a.w2);
  const int SG = a.SQ / VN;
  for (int c = tid; c < a.C; c += NT) {
    float s = 0.0f;
    constexpr int U = 6;
    for (int v0 = 0; v0 < SG; v0 += U) {
      V w[U];
#pragma unroll
      for (int u = 0; u < U; ++u) w[u] = *reinterpret_cast<const V*>(w2 + (long long)c * a.SQ + min(v0 + u, SG - 1) * VN);
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (v0 + u < SG) {
#pragma unroll
          for (int e = 0; e < VN; ++e) s += hid[(v0 + u) * VN + e] * (float)w[u][e];
        }
    }
    mean[c] = act_apply(s + a.b2[c], a.act2);
  }
  __syncthreads();

  // 4. gate the image, four vectors in flight per thread
  T* __restrict__ out = static_cast<T*>(a.out) + (long long)n * a.HW * a.C;
  const int total = a.HW * CG;
  constexpr int UG = 4;
  for (int i0 = tid; i0 < total; i0 += UG * NT) {
    V xv[UG];
#pragma unroll
    for (int u = 0; u < UG; ++u) xv[u] = *reinterpret_cast<const V*>(x + (long long)min(i0 + u * NT, total - 1) * VN);
#pragma unroll
    for (int u = 0; u < UG; ++u) {
      const int i = i0 + u * NT;
      if (i < total) {
        const int g = i % CG;
        V o;
#pragma unroll
        for (int e = 0; e < VN; ++e) o[e] = (T)(mean[g * VN + e] * (float)xv[u][e]);
        *reinterpret_cast<V*>(out + (long long)i * VN) = o;
      }
    }
  }
}

bool se_block_applicable(int dt, int HW, int C, int SQ) {
  const int vn = dt == kF16 ? 8 : 4;
  return C % vn == 0 && SQ % vn == 0 && C / vn <= 256 && C <= kSeMaxC && SQ <= kSeMaxSq && HW >= 1 &&
         (long long)HW * C < (1ll << 31);
}

void launch_se_block(const SeArgs& a, int dt, hipStream_t s) {
  NNCV_REQUIRE(se_block_applicable(dt, a.HW, a.C, a.SQ), "se_block: shape not covered");
  NNCV_REQUIRE(a.N >= 1 && a.b1 && a.b2, "se_block: bad arguments");
  const double es = (double)dtype_size(dt);
  ProfScope prof("se_block", 4.0 * a.N * a.C * a.SQ + 2.0 * a.N * a.HW * a.C, es * (2.0 * a.N * a.HW * a.C + 2.0 * a.C * a.SQ), s);
  if (dt == kF16)
    hipLaunchKernelGGL((se_block_kernel<half_t>), dim3(a.N), dim3(kSeThreads), 0, s, a);
  else
    hipLaunchKernelGGL((se_block_kernel<float>), dim3(a.N), dim3(kSeThreads), 0, s, a);
  NNCV_HIP_CHECK(hipGetLastError());
}

// ---------------------------------------------------------------------------------------------
// out = act(a + b) over [P][C] tensors whose rows may sit inside wider ones (row pitches lda, ldb,
// ldo in elements): a tensor that is one input of a channel concatenation lives in its slice of the
// concatenated tensor.
// ---------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void eltwise_kernel(const T* __restrict__ a, const T* __restrict__ b, T* __restrict__ out,
                                                      long long nvec, int CG, int lda, int ldb, int ldo, int act) {
  constexpr int VN = V16<T>::n;
  typedef typename V16<T>::type V;
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= nvec) return;
  const long long p = idx / CG;
  const int c = (int)(idx - p * CG) * VN;
  const V av = *reinterpret_cast<const V*>(a + p * lda + c);
  float y[VN];
#pragma unroll
  for (int e = 0; e < VN; ++e) y[e] = (float)av[e];
  if (b) {
    const V bv = *reinterpret_cast<const V*>(b + p * ldb + c);
#pragma unroll
    for (int e = 0; e < VN; ++e) y[e] += (float)bv[e];
  }
  V o;
  act_apply_n<sizeof(T) == 2>(y, act);
#pragma unroll
  for (int e = 0; e < VN; ++e) o[e] = (T)y[e];
  *reinterpret_cast<V*>(out + p * ldo + c) = o;
}

void launch_eltwise_pitched(const void* a, int lda, const void* b, int ldb, void* out, int ldo, int dt, long long P, int C, int act,
                            hipStream_t s) {
  const int vn = dt == kF16 ? 8 : 4;
  NNCV_REQUIRE(C % vn == 0 && lda % vn == 0 && ldb % vn == 0 && ldo % vn == 0 && lda >= C && ldo >= C && (!b || ldb >= C),
               "eltwise: channel count and pitches must be multiples of the 16-byte vector");
  const long long n = P * C;
  if (n == 0) return;
  ProfScope prof(b ? "eltwise_add" : "eltwise_act", (double)n, (double)dtype_size(dt) * n * (b ? 3 : 2), s);
  if (dt == kF16)
    hipLaunchKernelGGL((eltwise_kernel<half_t>), dim3(grid_for(n / vn)), dim3(256), 0, s, (const half_t*)a, (const half_t*)b,
                       (half_t*)out, n / vn, C / vn, lda, ldb, ldo, act);
  else
    hipLaunchKernelGGL((eltwise_kernel<float>), dim3(grid_for(n / vn)), dim3(256), 0, s, (const float*)a, (const float*)b,
                       (float*)out, n / vn, C / vn, lda, ldb, ldo, act);
  NNCV_HIP_CHECK(hipGetLastError());
}

void launch_eltwise(const void* a, const void* b, void* out, int dt, long long n, int act, hipStream_t s) {
  const int vn = dt == kF16 ? 8 : 4;
  NNCV_REQUIRE(n % vn == 0, "eltwise: element count must be a multiple of the 16-byte vector");
  launch_eltwise_pitched(a, vn, b, vn, out, vn, dt, n / vn, vn, act, s);  // a dense tensor is [n / vn][vn]
}

// ---------------------------------------------------------------------------------------------
// Channel concatenation (a strided copy into a slice of the wider tensor) and nearest 2x
// up-sampling written straight into such a slice; both move raw 16-byte vectors.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void concat_slice_kernel(const uint4* __restrict__ x, uint4* __restrict__ out, long long total,
                                                           int CG, int ldig, int ldg, int g0) {
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const long long p = idx / CG;
  const int cg = (int)(idx % CG);
  out[p * ldg + g0 + cg] = x[p * ldig + cg];
}

void launch_concat_slice(const void* x, void* out, int dt, long long P, int C, int ldo, int c0, hipStream_t s, int ldi) {
  const int vn = dt == kF16 ? 8 : 4;
  if (ldi == 0) ldi = C;
  NNCV_REQUIRE(C % vn == 0 && ldo % vn == 0 && c0 % vn == 0 && c0 >= 0 && c0 + C <= ldo && ldi % vn == 0 && ldi >= C,
               "concat: channel counts and offset must be multiples of the 16-byte vector");
  const long long total = P * (C / vn);
  if (total == 0) return;
  ProfScope prof("concat_slice", 0.0, 2.0 * dtype_size(dt) * P * C, s);
  hipLaunchKernelGGL(concat_slice_kernel, dim3(grid_for(total)), dim3(256), 0, s, (const uint4*)x, (uint4*)out, total, C / vn,
                     ldi / vn, ldo / vn, c0 / vn);
  NNCV_HIP_CHECK(hipGetLastError());
}

__global__ __launch_bounds__(256) void upsample2x_kernel(const uint4* __restrict__ x, uint4* __restrict__ out, long long total,
                                                         int H, int W, int CG, int ldig, int ldg, int g0) {
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;  // over output vectors
  if (idx >= total) return;
  const int cg = (int)(idx % CG);
  long long p = idx / CG;
  const int ox = (int)(p % (2 * W));
  p /= 2 * W;
  const int oy = (int)(p % (2 * H));
  const long long n = p / (2 * H);
  out[((n * 2 * H + oy) * 2 * W + ox) * ldg + g0 + cg] = x[((n * H + (oy >> 1)) * W + (ox >> 1)) * ldig + cg];
}

void launch_upsample2x(const void* x, void* out, int dt, int N, int H, int W, int C, int ldo, int c0, hipStream_t s, int ldi) {
  const int vn = dt == kF16 ? 8 : 4;
  if (ldi == 0) ldi = C;
  NNCV_REQUIRE(C % vn == 0 && ldo % vn == 0 && c0 % vn == 0 && c0 >= 0 && c0 + C <= ldo && ldi % vn == 0 && ldi >= C,
               "upsample: channel counts and offset must be multiples of the 16-byte vector");
  const long long total = (long long)N * 4 * H * W * (C / vn);
  if (total == 0) return;
  ProfScope prof("upsample2x", 0.0, 5.0 * dtype_size(dt) * N * H * W * C, s);
  hipLaunchKernelGGL(upsample2x_kernel, dim3(grid_for(total)), dim3(256), 0, s, (const uint4*)x, (uint4*)out, total, H, W, C / vn,
                     ldi / vn, ldo / vn, c0 / vn);
  NNCV_HIP_CHECK(hipGetLastError());
}

// ---------------------------------------------------------------------------------------------
// linalg.pooling_nchw_max with any window / stride over a -inf halo (Yolov5s.mlir: 5x5 stride 1
// pad 2 in the SPPF block), NHWC
// ---------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void maxpool_kernel(const T* __restrict__ in, T* __restrict__ out, int N, int H, int W, int C,
                                                      int K, int stride, int pad, int OH, int OW, int ldi, int ldo) {
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
      const V v = *reinterpret_cast<const V*>(in + (((long long)n * H + iy) * W + ix) * ldi + cg * VN);
#pragma unroll
      for (int e = 0; e < VN; ++e) m[e] = max_nan(m[e], (float)v[e]);
    }
  }
  V o;
#pragma unroll
  for (int e = 0; e < VN; ++e) o[e] = (T)m[e];
  *reinterpret_cast<V*>(out + (((long long)n * OH + oy) * OW + ox) * ldo + cg * VN) = o;
}

void launch_maxpool_nhwc(const void* in, void* out, int dt, int N, int H, int W, int C, int K, int stride, int pad,
                         hipStream_t s, int ldi, int ldo) {
  const int vn = dt == kF16 ? 8 : 4;
  if (ldi == 0) ldi = C;
  if (ldo == 0) ldo = C;
  NNCV_REQUIRE(C % vn == 0 && ldi % vn == 0 && ldo % vn == 0 && ldi >= C && ldo >= C,
               "maxpool: C and the pitches must be multiples of the 16-byte vector");
  NNCV_REQUIRE(K >= 1 && stride >= 1 && pad >= 0 && 2 * pad <= K && H + 2 * pad >= K && W + 2 * pad >= K, "maxpool: bad geometry");
  const int OH = (H + 2 * pad - K) / stride + 1, OW = (W + 2 * pad - K) / stride + 1;
  const long long work = (long long)N * OH * OW * (C / vn);
  if (work == 0) return;
  ProfScope prof("maxpool", 0.0, (double)dtype_size(dt) * N * C * ((double)H * W + (double)OH * OW), s);
  if (dt == kF16)
    hipLaunchKernelGGL((maxpool_kernel<half_t>), dim3(grid_for(work)), dim3(256), 0, s, (const half_t*)in, (half_t*)out, N, H, W, C,
                       K, stride, pad, OH, OW, ldi, ldo);
  else
    hipLaunchKernelGGL((maxpool_kernel<float>), dim3(grid_for(work)), dim3(256), 0, s, (const float*)in, (float*)out, N, H, W, C, K,
                       stride, pad, OH, OW, ldi, ldo);
  NNCV_HIP_CHECK(hipGetLastError());
}

// ---------------------------------------------------------------------------------------------
// Three 5x5 stride-1 pad-2 max-pools in a row, each result kept (YOLOv5's SPPF block,
// Yolov5s.mlir: y1 = m(x), y2 = m(y1), y3 = m(y2), all four concatenated): one launch instead of
// three.  A workgroup owns one image x one 16-byte channel vector: the H*W map sits in LDS, each
// stage takes five row maxima and then five of those down the column (the -inf halo is a skipped
// tap) and writes its result both to memory and to the other LDS map.  The maps are 20x20 for a 640x640 input, so the three
// stand-alone launches were nothing but latency (16 us each for 3 MB).
// ---------------------------------------------------------------------------------------------
constexpr int kPoolChainMaxHW = 1600;

template <typename T>
__global__ __launch_bounds__(256) void maxpool5_chain3_kernel(const T* __restrict__ in, T* __restrict__ o1, T* __restrict__ o2,
                                                              T* __restrict__ o3, int H, int W, int CG, int ldi, int ld1, int ld2,
                                                              int ld3) {
  constexpr int VN = V16<T>::n;
  typedef typename V16<T>::type V;
  extern __shared__ __align__(16) unsigned char pool_smem[];
  const int HW = H * W, tid = threadIdx.x;
  V* bufs = reinterpret_cast<V*>(pool_smem);  // two maps that take turns + the row maxima of the current stage
  V* rowmax = bufs + 2 * HW;
  const int n = blockIdx.x / CG, cg = blockIdx.x - n * CG;
  const float inv_w = 1.0f / (float)W;
  in += (long long)n * HW * ldi + cg * VN;
  for (int p = tid; p < HW; p += 256) bufs[p] = *reinterpret_cast<const V*>(in + (long long)p * ldi);
  __syncthreads();
#pragma unroll
  for (int stage = 0; stage < 3; ++stage) {
    const V* src = bufs + (stage & 1) * HW;
    V* dst = bufs + ((stage + 1) & 1) * HW;
    const int ldo = stage == 0 ? ld1 : stage == 1 ? ld2 : ld3;
    T* out = (stage == 0 ? o1 : stage == 1 ? o2 : o3) + ((long long)n * HW * ldo + cg * VN);
    // the 5x5 maximum as five columns of row maxima (the maximum does not depend on the order, NaN included)
    for (int p = tid; p < HW; p += 256) {
      int y = (int)((float)p * inv_w), x = p - y * W;  // exact for p < 2^24 after the correction
      if (x >= W) { ++y; x -= W; }
      if (x < 0) { --y; x += W; }
      float m[VN];
#pragma unroll
      for (int e = 0; e < VN; ++e) m[e] = -INFINITY;
#pragma unroll
      for (int q = -2; q <= 2; ++q) {
        const V v = src[(unsigned)(x + q) < (unsigned)W ? p + q : p];  // outside the map: the centre again, which changes nothing
#pragma unroll
        for (int e = 0; e < VN; ++e) m[e] = max_nan(m[e], (float)v[e]);
      }
      V o;
#pragma unroll
      for (int e = 0; e < VN; ++e) o[e] = (T)m[e];
      rowmax[p] = o;
    }
    __syncthreads();
    for (int p = tid; p < HW; p += 256) {
      float m[VN];
#pragma unroll
      for (int e = 0; e < VN; ++e) m[e] = -INFINITY;
#pragma unroll
      for (int r = -2; r <= 2; ++r) {
        const V v = rowmax[(unsigned)(p + r * W) < (unsigned)HW ? p + r * W : p];
#pragma unroll
        for (int e = 0; e < VN; ++e) m[e] = max_nan(m[e], (float)v[e]);
      }
      V o;
#pragma unroll
      for (int e = 0; e < VN; ++e) o[e] = (T)m[e];
      dst[p] = o;
      *reinterpret_cast<V*>(out + (long long)p * ldo) = o;
    }
    __syncthreads();
  }
}

bool maxpool5_chain3_applicable(int dt, int H, int W, int C) {
  static const bool off = getenv("NNCV_HIP_NO_POOL_CHAIN") != nullptr;
  const int vn = dt == kF16 ? 8 : 4;
  return !off && H >= 1 && W >= 1 && H * W <= kPoolChainMaxHW && C % vn == 0;
}

void launch_maxpool5_chain3(const void* in, void* o1, void* o2, void* o3, int dt, int N, int H, int W, int C, int ldi, int ld1, int ld2,
                            int ld3, hipStream_t s) {
  const int vn = dt == kF16 ? 8 : 4;
  NNCV_REQUIRE(maxpool5_chain3_applicable(dt, H, W, C) && ldi % vn == 0 && ld1 % vn == 0 && ld2 % vn == 0 && ld3 % vn == 0 &&
                   ldi >= C && ld1 >= C && ld2 >= C && ld3 >= C && (long long)N * (C / vn) < (1ll << 31),
               "maxpool chain: shape not covered");
  ProfScope prof("maxpool5_chain3", 0.0, (double)dtype_size(dt) * N * C * 4.0 * H * W, s);
  const dim3 grid((unsigned)((long long)N * (C / vn)));
  static const bool once = [] {
    NNCV_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(maxpool5_chain3_kernel<half_t>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, 3 * kPoolChainMaxHW * 16));
    NNCV_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(maxpool5_chain3_kernel<float>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, 3 * kPoolChainMaxHW * 16));
    return true;
  }();
  (void)once;
  const size_t smem = (size_t)3 * H * W * 16;
  if (dt == kF16)
    hipLaunchKernelGGL((maxpool5_chain3_kernel<half_t>), grid, dim3(256), smem, s, (const half_t*)in, (half_t*)o1, (half_t*)o2, (half_t*)o3,
                       H, W, C / vn, ldi, ld1, ld2, ld3);
  else
    hipLaunchKernelGGL((maxpool5_chain3_kernel<float>), grid, dim3(256), smem, s, (const float*)in, (float*)o1, (float*)o2, (float*)o3, H, W,
                       C / vn, ldi, ld1, ld2, ld3);
  NNCV_HIP_CHECK(hipGetLastError());
}

// ---------------------------------------------------------------------------------------------
// YOLOv5 Detect decode, one level (Yolov5s.mlir:1348-1448): expand [N,A*F,H,W] to [N,A,H,W,F],
// sigmoid, xy = (2 s + (x, y) - 0.5) * stride, wh = (2 s)^2 * anchor (powf(., 2) is the square),
// everything else the sigmoid itself; boxes ordered (anchor, y, x).  One thread per output value,
// F fastest, so both the NHWC read (F consecutive channels of one anchor) and the fp32 write are
// contiguous runs of F elements.
// ---------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void yolo_detect_kernel(const DetectArgs a) {
  // blockIdx.y = (image, anchor); blockIdx.x walks the H*W*F values of that anchor, F fastest
  const int n = blockIdx.y / a.A, an = blockIdx.y - n * a.A;
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  const int HWF = a.H * a.W * a.F;
  if (i >= HWF) return;
  // i / F and pix / W by float reciprocal + correction (exact below 2^24, which the launcher checks):
  // the integer-divide expansion was half of this kernel's instructions
  int pix = (int)((float)i * a.inv_f), k = i - pix * a.F;
  if (k >= a.F) { ++pix; k -= a.F; }
  if (k < 0) { --pix; k += a.F; }
  const T* head = static_cast<const T*>(a.head);
  const float v = (float)head[((long long)n * a.H * a.W + pix) * a.ldc + an * a.F + k];
  const float sg = sigmoid_fast(v);
  float o = sg;
  if (k < 4) {
    int y = (int)((float)pix * a.inv_w), x = pix - y * a.W;
    if (x >= a.W) { ++y; x -= a.W; }
    if (x < 0) { --y; x += a.W; }
    if (k < 2) {
      const float g = (float)(k == 0 ? x : y) - 0.5f;
      o = (sg * 2.0f + g) * a.stride;
    } else {
      const float t = sg * 2.0f;
      o = (t * t) * a.anchor_wh[an * 2 + (k - 2)];
    }
  }
  a.out[((long long)n * a.boxes_total + a.box0 + (long long)an * a.H * a.W) * a.F + i] = o;
}

// The same with four consecutive values per thread and one 16-byte store (the launcher uses it when
// H*W*F is a multiple of 4 and the level's first output value is 16-byte aligned): a quarter of the
// index arithmetic and store instructions per value.
template <typename T>
__global__ __launch_bounds__(256) void yolo_detect4_kernel(const DetectArgs a) {
  const int n = blockIdx.y / a.A, an = blockIdx.y - n * a.A;
  const int i = (blockIdx.x * blockDim.x + threadIdx.x) * 4;
  const int HWF = a.H * a.W * a.F;
  if (i >= HWF) return;
  int pix = (int)((float)i * a.inv_f), k = i - pix * a.F;
  if (k >= a.F) { ++pix; k -= a.F; }
  if (k < 0) { --pix; k += a.F; }
  const T* head = static_cast<const T*>(a.head) + (long long)n * a.H * a.W * a.ldc + an * a.F;
  float v[4];
  int kk[4], pp[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    kk[e] = k;
    pp[e] = pix;
    v[e] = (float)head[(long long)pix * a.ldc + k];
    if (++k == a.F) { k = 0; ++pix; }
  }
  float o[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const float sg = sigmoid_fast(v[e]);
    o[e] = sg;
    if (kk[e] < 4) {
      int y = (int)((float)pp[e] * a.inv_w), x = pp[e] - y * a.W;
      if (x >= a.W) { ++y; x -= a.W; }
      if (x < 0) { --y; x += a.W; }
      if (kk[e] < 2) {
        const float g = (float)(kk[e] == 0 ? x : y) - 0.5f;
        o[e] = (sg * 2.0f + g) * a.stride;
      } else {
        const float t = sg * 2.0f;
        o[e] = (t * t) * a.anchor_wh[an * 2 + (kk[e] - 2)];
      }
    }
  }
  typedef float f4 __attribute__((ext_vector_type(4)));
  *reinterpret_cast<f4*>(a.out + ((long long)n * a.boxes_total + a.box0 + (long long)an * a.H * a.W) * a.F + i) = f4{o[0], o[1], o[2], o[3]};
}

void launch_yolo_detect(const DetectArgs& a, int dt, hipStream_t s) {
  NNCV_REQUIRE(a.A >= 1 && a.A <= 4 && a.F >= 5 && a.A * a.F <= a.ldc && a.N >= 1 && a.H >= 1 && a.W >= 1, "yolo_detect: bad shape");
  NNCV_REQUIRE((long long)a.H * a.W * a.F < (1ll << 24) && (long long)a.N * a.A <= 65535, "yolo_detect: level too large");
  DetectArgs b = a;
  b.inv_f = 1.0f / (float)a.F;
  b.inv_w = 1.0f / (float)a.W;
  const long long work = (long long)a.N * a.A * a.H * a.W * a.F;
  ProfScope prof("yolo_detect", 0.0, (double)work * (dtype_size(dt) + 4.0), s);
  // four values per thread when every (image, anchor) block of the output starts on a 16-byte boundary
  const long long hwf = (long long)a.H * a.W * a.F;
  const bool vec4 = hwf % 4 == 0 && (a.boxes_total * a.F) % 4 == 0 && (a.box0 * a.F) % 4 == 0 &&
                    reinterpret_cast<uintptr_t>(a.out) % 16 == 0;
  if (vec4) {
    dim3 grid4((unsigned)((hwf / 4 + 255) / 256), (unsigned)(a.N * a.A));
    if (dt == kF16)
      hipLaunchKernelGGL((yolo_detect4_kernel<half_t>), grid4, dim3(256), 0, s, b);
    else
      hipLaunchKernelGGL((yolo_detect4_kernel<float>), grid4, dim3(256), 0, s, b);
    NNCV_HIP_CHECK(hipGetLastError());
    return;
  }
  dim3 grid((unsigned)(((long long)a.H * a.W * a.F + 255) / 256), (unsigned)(a.N * a.A));
  if (dt == kF16)
    hipLaunchKernelGGL((yolo_detect_kernel<half_t>), grid, dim3(256), 0, s, b);
  else
    hipLaunchKernelGGL((yolo_detect_kernel<float>), grid, dim3(256), 0, s, b);
  NNCV_HIP_CHECK(hipGetLastError());
}

}  // namespace nncv_hip
