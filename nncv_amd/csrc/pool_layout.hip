// Bandwidth-bound helpers of the ResNet-18 path: pooling, layout packing and one-time parameter
// preparation.  Activations are NHWC inside the library (channels contiguous), so every kernel
// here maps lanes to the channel axis and moves 16 bytes per lane where the shape allows.
#include <type_traits>

#include "common.hpp"

namespace nncv_hip {

template <typename T>
struct Vec16;  // 16-byte vector of T
template <>
struct Vec16<float> {
  typedef float type __attribute__((ext_vector_type(4)));
  static constexpr int n = 4;
};
template <>
struct Vec16<half_t> {
  typedef half_t type __attribute__((ext_vector_type(8)));
  static constexpr int n = 8;
};

// arith.maximumf (tests/Nets/Pool2DMax.mlir:24): NaN in either operand wins.
__device__ __forceinline__ float max_nan(float m, float v) { return (v > m || v != v) ? v : m; }

// ---------------------------------------------------------------------------------------------
// linalg.pooling_nchw_max 3x3 stride 2 over a -inf halo of 1 (tests/Nets/Res18.mlir:144-151),
// NHWC.  One thread = one output pixel x one 16-byte channel group; the halo is a predicate.
// ---------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void maxpool3x3s2_kernel(const T* __restrict__ in, T* __restrict__ out, int N, int H,
                                                           int W, int C, int OH, int OW) {
  constexpr int VN = Vec16<T>::n;
  typedef typename Vec16<T>::type V;
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
#pragma unroll
  for (int r = 0; r < 3; ++r) {
    const int iy = oy * 2 - 1 + r;
    if ((unsigned)iy >= (unsigned)H) continue;
#pragma unroll
    for (int s = 0; s < 3; ++s) {
      const int ix = ox * 2 - 1 + s;
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

// The same pooling for whole images at a time: one workgroup per output row, one thread per pair of neighbouring output
// pixels and 16-byte channel group (the two windows share a column: 15 loads for two results instead of 18), 32-bit
// index arithmetic throughout (the generic kernel above spends more time dividing 64-bit indices than loading).
// fp16 keeps the halves packed: the running maximum is
// v_pk_max_f16, which returns the other operand when one is a NaN, so NaNs are tracked next to it as the unsigned maximum
// of the magnitudes (a NaN is a magnitude above infinity's 0x7c00) and put back at the end -- arith.maximumf
// (tests/Nets/Pool2DMax.mlir:24) propagates them.
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned short ushort8_t __attribute__((ext_vector_type(8)));
typedef half_t half8_t __attribute__((ext_vector_type(8)));

template <typename T>
__global__ __launch_bounds__(256) void maxpool3x3s2_rows_kernel(const T* __restrict__ in, T* __restrict__ out, int H, int W, int C,
                                                                int OH, int OW, unsigned in_bytes, unsigned inv_cg, unsigned n_rows) {
  constexpr int VN = Vec16<T>::n;
  const int CG = C / VN, pairs = (OW + 1) >> 1;
  // Hardware deals workgroups to the 8 XCDs round-robin; neighbouring output rows share an input row, so each XCD takes a
  // contiguous band of rows and its L2 serves the shared row (otherwise every shared row is fetched by two L2s).
  const unsigned per_xcd = (n_rows + 7u) >> 3;
  const unsigned row = (blockIdx.x & 7u) * per_xcd + (blockIdx.x >> 3);  // n * OH + oy
  if (row >= n_rows) return;
  const unsigned n = row / (unsigned)OH, oy = row - n * (unsigned)OH;
  const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(in), 0, (int)in_bytes, 0x00020000);
  const unsigned pix_b = (unsigned)C * sizeof(T);
  for (unsigned e = threadIdx.x; e < (unsigned)(pairs * CG); e += 256) {
    const unsigned px = __umulhi(e, inv_cg), cg = e - px * (unsigned)CG;  // e / CG, e % CG
    const int ox0 = 2 * (int)px, ix0 = 2 * ox0 - 1;
    // Coordinates outside the image are clamped to its border instead of being answered with -inf: a window that hangs
    // over the border by its one halo row or column then reads a pixel it holds anyway, and a maximum does not mind
    // seeing a value twice.  (The second output pixel of a last, odd pair reads clamped columns and is not stored.)
    u32x4 v[3][5];
    unsigned coff[5];
#pragma unroll
    for (int c = 0; c < 5; ++c) coff[c] = (unsigned)min(max(ix0 + c, 0), W - 1) * pix_b + cg * 16u;
#pragma unroll
    for (int r = 0; r < 3; ++r) {
      const int iy = min(max(2 * (int)oy - 1 + r, 0), H - 1);
      const unsigned roff = (n * (unsigned)H + (unsigned)iy) * (unsigned)W * pix_b;
#pragma unroll
      for (int c = 0; c < 5; ++c) v[r][c] = __builtin_amdgcn_raw_buffer_load_b128(rs, roff + coff[c], 0, 0);
    }
    T* o = out + ((size_t)row * OW + ox0) * C + cg * VN;
    if constexpr (sizeof(T) == 2) {
      // Packed halves, one instruction per dword and operation, written out: the compiler's own rendering of the vector
      // maximum canonicalises every operand first and splits the 16-bit masks into byte moves (600 instructions per
      // thread, which made the kernel issue-bound).
      const u32x4 ninf4 = {0xfc00fc00u, 0xfc00fc00u, 0xfc00fc00u, 0xfc00fc00u};  // -inf in both halves
      u32x4 m0 = ninf4, m1 = ninf4, a0 = {0u, 0u, 0u, 0u}, a1 = a0;
      auto fmax2 = [](unsigned x, unsigned y) {
        unsigned d;
        asm("v_pk_max_f16 %0, %1, %2" : "=v"(d) : "v"(x), "v"(y));
        return d;
      };
      auto umax2 = [](unsigned x, unsigned y) {
        unsigned d;
        asm("v_pk_max_u16 %0, %1, %2" : "=v"(d) : "v"(x), "v"(y));
        return d;
      };
#pragma unroll
      for (int r = 0; r < 3; ++r)
#pragma unroll
        for (int c = 0; c < 5; ++c)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const unsigned x = v[r][c][q], mag = x & 0x7fff7fffu;
            if (c <= 2) {
              m0[q] = fmax2(m0[q], x);
              a0[q] = umax2(a0[q], mag);
            }
            if (c >= 2) {
              m1[q] = fmax2(m1[q], x);
              a1[q] = umax2(a1[q], mag);
            }
          }
      // a magnitude above infinity's 0x7c00 among the nine: the result is a NaN
      auto with_nans = [&](u32x4 m, u32x4 a) {
        u32x4 o4;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const unsigned lo = (a[q] & 0xffffu) > 0x7c00u ? 0xffffu : 0u, hi = (a[q] >> 16) > 0x7c00u ? 0xffff0000u : 0u;
          const unsigned mk = lo | hi;
          o4[q] = (m[q] & ~mk) | (mk & 0x7e007e00u);
        }
        return o4;
      };
      *reinterpret_cast<u32x4*>(o) = with_nans(m0, a0);
      if (ox0 + 1 < OW) *reinterpret_cast<u32x4*>(o + C) = with_nans(m1, a1);
    } else {
      float m0[4], m1[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) m0[q] = m1[q] = -INFINITY;
#pragma unroll
      for (int r = 0; r < 3; ++r) {
#pragma unroll
        for (int c = 0; c < 5; ++c) {
          typedef float f4v __attribute__((ext_vector_type(4)));
          const f4v vf = __builtin_bit_cast(f4v, v[r][c]);  // the whole vector: a bit cast of one element reads element 0
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            if (c <= 2) m0[q] = max_nan(m0[q], vf[q]);
            if (c >= 2) m1[q] = max_nan(m1[q], vf[q]);
          }
        }
      }
      typedef float f4 __attribute__((ext_vector_type(4)));
      *reinterpret_cast<f4*>(o) = f4{m0[0], m0[1], m0[2], m0[3]};
      if (ox0 + 1 < OW) *reinterpret_cast<f4*>(o + C) = f4{m1[0], m1[1], m1[2], m1[3]};
    }
  }
}

void launch_maxpool3x3s2_nhwc(const void* in, void* out, int dt, int N, int H, int W, int C, hipStream_t s) {
  const int OH = (H + 2 - 3) / 2 + 1, OW = (W + 2 - 3) / 2 + 1;
  const int vn = dt == kF16 ? 8 : 4;
  NNCV_REQUIRE(C % vn == 0, "maxpool: C must be a multiple of the 16-byte vector");
  const long long work = (long long)N * OH * OW * (C / vn);
  const long long grid = (work + 255) / 256;
  NNCV_REQUIRE(grid < (1ll << 31), "maxpool: grid too large");
  ProfScope prof("maxpool3x3s2", 0.0, (double)dtype_size(dt) * N * C * ((double)H * W + (double)OH * OW), s);
  const long long in_bytes = (long long)N * H * W * C * (long long)dtype_size(dt);
  static const bool generic = getenv("NNCV_HIP_MAXPOOL_GENERIC") != nullptr;
  // the row form addresses the input with 32-bit byte offsets and wants rows that give a workgroup something to do
  if (!generic && in_bytes < (1ll << 31) && (long long)N * OH < (1ll << 31) && C / vn >= 2 && ((OW + 1) / 2) * (C / vn) >= 64) {
    const unsigned inv_cg = C / vn == 1 ? 0u : (unsigned)(0xffffffffull / (unsigned)(C / vn) + 1);
    const unsigned grid_rows = ((unsigned)(N * OH) + 7u) / 8u * 8u;
    if (dt == kF16)
      hipLaunchKernelGGL((maxpool3x3s2_rows_kernel<half_t>), dim3(grid_rows), dim3(256), 0, s, (const half_t*)in, (half_t*)out, H, W, C, OH, OW,
                         (unsigned)in_bytes, inv_cg, (unsigned)(N * OH));
    else
      hipLaunchKernelGGL((maxpool3x3s2_rows_kernel<float>), dim3(grid_rows), dim3(256), 0, s, (const float*)in, (float*)out, H, W, C, OH, OW,
                         (unsigned)in_bytes, inv_cg, (unsigned)(N * OH));
    NNCV_HIP_CHECK(hipGetLastError());
    return;
  }
  if (dt == kF16)
    hipLaunchKernelGGL((maxpool3x3s2_kernel<half_t>), dim3((unsigned)grid), dim3(256), 0, s, (const half_t*)in, (half_t*)out, N, H, W, C, OH, OW);
  else
    hipLaunchKernelGGL((maxpool3x3s2_kernel<float>), dim3((unsigned)grid), dim3(256), 0, s, (const float*)in, (float*)out, N, H, W, C, OH, OW);
  NNCV_HIP_CHECK(hipGetLastError());
}

// ---------------------------------------------------------------------------------------------
// linalg.pooling_nchw_sum over the whole image followed by one divf by H*W
// (tests/Nets/Res18.mlir:609-614).  NHWC [N][HW][C] -> [N][C].
// A workgroup handles one image x 64 channels: each of its 4 waves sums a quarter of the pixels
// with lanes along the channels (one contiguous 128/256-byte segment per wave per pixel), then
// the four partial sums meet in LDS.  fp32 accumulation; sum first, one divide.
// ---------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void global_avgpool_kernel(const T* __restrict__ in, T* __restrict__ out, int HW, int C) {
  __shared__ float part[4][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c = blockIdx.x * 64 + lane, n = blockIdx.y;
  float s = 0.0f;
  if (c < C)
    for (int p = wave; p < HW; p += 4) s += (float)in[((long long)n * HW + p) * C + c];
  part[wave][lane] = s;
  __syncthreads();
  if (wave == 0 && c < C) {
    const float tot = ((part[0][lane] + part[1][lane]) + part[2][lane]) + part[3][lane];
    out[(long long)n * C + c] = (T)(tot / (float)HW);
  }
}

// Whole-vector form for C % (16 bytes) == 0: a workgroup owns one image x up to 32 channel
// groups; its threads split into pixel phases x channel groups, keep four 16-byte loads in
// flight each, and meet in LDS.  Same arithmetic (fp32 sums, one divide).
template <typename T>
__global__ __launch_bounds__(256) void global_avgpool_vec_kernel(const T* __restrict__ in, T* __restrict__ out, int HW, int C,
                                                                 int cgb) {
  constexpr int VN = Vec16<T>::n;
  typedef typename Vec16<T>::type V;
  __shared__ float part[256 * VN];
  const int tid = threadIdx.x, n = blockIdx.y;
  const int CG = C / VN;
  const int g0 = blockIdx.x * cgb;
  const int ng = min(cgb, CG - g0);  // channel groups of this workgroup
  const int ppb = 256 / ng;
  const int pp = tid / ng, cg = g0 + (tid - pp * ng);
  const T* x = in + (long long)n * HW * C + cg * VN;
  float acc[VN];
#pragma unroll
  for (int e = 0; e < VN; ++e) acc[e] = 0.0f;
  if (pp < ppb) {
    int p = pp;
    for (; p + 3 * ppb < HW; p += 4 * ppb) {
      V v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) v[u] = *reinterpret_cast<const V*>(x + (long long)(p + u * ppb) * C);
#pragma unroll
      for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int e = 0; e < VN; ++e) acc[e] += (float)v[u][e];
    }
    for (; p < HW; p += ppb) {
      const V v = *reinterpret_cast<const V*>(x + (long long)p * C);
#pragma unroll
      for (int e = 0; e < VN; ++e) acc[e] += (float)v[e];
    }
#pragma unroll
    for (int e = 0; e < VN; ++e) part[tid * VN + e] = acc[e];
  }
  __syncthreads();
  if (tid < ng * VN) {
    const int g = tid / VN, e = tid % VN;
    float s = 0.0f;
    for (int q = 0; q < ppb; ++q) s += part[(q * ng + g) * VN + e];
    out[(long long)n * C + (g0 + g) * VN + e] = (T)(s / (float)HW);
  }
}

void launch_global_avgpool_nhwc(const void* in, void* out, int dt, int N, int HW, int C, hipStream_t s) {
  ProfScope prof("global_avgpool", 0.0, (double)dtype_size(dt) * N * C * (HW + 1.0), s);
  const int vn = dt == kF16 ? 8 : 4;
  if (C % vn == 0) {
    const int CG = C / vn;
    // fewer channel groups per workgroup when that is what it takes to give every CU one
    int cgb = 32;
    while (cgb > 2 && (long long)((CG + cgb - 1) / cgb) * N < 256) cgb >>= 1;
    dim3 grid((CG + cgb - 1) / cgb, N);
    if (dt == kF16)
      hipLaunchKernelGGL((global_avgpool_vec_kernel<half_t>), grid, dim3(256), 0, s, (const half_t*)in, (half_t*)out, HW, C, cgb);
    else
      hipLaunchKernelGGL((global_avgpool_vec_kernel<float>), grid, dim3(256), 0, s, (const float*)in, (float*)out, HW, C, cgb);
    NNCV_HIP_CHECK(hipGetLastError());
    return;
  }
  dim3 grid((C + 63) / 64, N);
  if (dt == kF16)
    hipLaunchKernelGGL((global_avgpool_kernel<half_t>), grid, dim3(256), 0, s, (const half_t*)in, (half_t*)out, HW, C);
  else
    hipLaunchKernelGGL((global_avgpool_kernel<float>), grid, dim3(256), 0, s, (const float*)in, (float*)out, HW, C);
  NNCV_HIP_CHECK(hipGetLastError());
}

// ---------------------------------------------------------------------------------------------
// Network head in one launch: global average pool (sum over the image, one divide,
// tests/Nets/Res18.mlir:609-614) and the 512 -> F fully connected layer with bias (:615-628).
// A workgroup = one image x a slice of the F outputs.  Phase 1: a wave sums every fourth pixel of the
// image, a lane eight channels of it (16-byte loads: one kilobyte per instruction), fp32, in pixel
// order; the four waves' sums meet in LDS and are added in wave order, one divide; the pooled vector
// is never rounded to the storage type.  Phase 2: a wave takes eight outputs per trip, its 64 lanes
// each hold 8 of the 512 means and read 8 consecutive weights of each filter (a filter row is one
// contiguous kilobyte); the eight dot products are added over the lanes together (see below).
// Slices recompute the pooling instead of synchronising across workgroups.
// ---------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void avgpool_fc_kernel(const T* __restrict__ in, const T* __restrict__ w,
                                                         const float* __restrict__ bias, float* __restrict__ out, int N, int HW,
                                                         int F, int f_per_block) {
  // images per workgroup.  More would read the filters less often (once per IG images); measured at batch 32 with slices
  // of 64 outputs: 6.2 us with one, 6.7 with two, 9.0 with four (longer chains per workgroup, fewer workgroups).
  constexpr int IG = 1;
  typedef float floatx4 __attribute__((ext_vector_type(4)));
  typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
  __shared__ __align__(16) float part[IG][4][512];  // per image and wave: the sums over the wave's pixels
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n0 = blockIdx.y * IG;
  {
    // A wave takes every fourth pixel, a lane eight channels of it: one kilobyte (fp32: two) per load instruction.  (Two
    // channels per lane, 4-byte loads, kept the vector-memory path busy for a quarter of the instructions' worth of
    // data: 5.4 of the launch's 7.8 us at batch 32.)  Through buffer descriptors of exactly one image each (none for an
    // image past N): what lies past the end reads as zeros, and a sum that started at +0 is the same with +0 added.
    typedef T V8 __attribute__((ext_vector_type(8)));
    constexpr int PB = 16 / IG;  // pixels per wave and trip
    const unsigned pix_bytes = 512u * (unsigned)sizeof(T), img_bytes = (unsigned)HW * pix_bytes;
    const unsigned loff = (unsigned)lane * 8u * (unsigned)sizeof(T);
    __amdgpu_buffer_rsrc_t rs[IG];
    float ps[IG][8];
#pragma unroll
    for (int g = 0; g < IG; ++g) {
      const bool have = n0 + g < N;
      rs[g] = __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(in + (long long)(have ? n0 + g : 0) * HW * 512), 0, have ? img_bytes : 0u, 0x00020000);
#pragma unroll
      for (int e = 0; e < 8; ++e) ps[g][e] = 0.0f;
    }
    for (int p = wave; p < HW; p += 4 * PB) {  // the additions of a wave stay in pixel order
      V8 v[IG][PB];
#pragma unroll
      for (int g = 0; g < IG; ++g)
#pragma unroll
        for (int u = 0; u < PB; ++u) {
          const unsigned off = (unsigned)(p + 4 * u) * pix_bytes + loff;
          if constexpr (sizeof(T) == 2) {
            v[g][u] = __builtin_bit_cast(V8, __builtin_amdgcn_raw_buffer_load_b128(rs[g], off, 0, 0));
          } else {
            typedef unsigned u32x8 __attribute__((ext_vector_type(8)));
            const u32x4 lo = __builtin_amdgcn_raw_buffer_load_b128(rs[g], off, 0, 0), hi = __builtin_amdgcn_raw_buffer_load_b128(rs[g], off + 16u, 0, 0);
            v[g][u] = __builtin_bit_cast(V8, u32x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]});
          }
        }
#pragma unroll
      for (int g = 0; g < IG; ++g)
#pragma unroll
        for (int u = 0; u < PB; ++u)
#pragma unroll
          for (int e = 0; e < 8; ++e) ps[g][e] += (float)v[g][u][e];
    }
#pragma unroll
    for (int g = 0; g < IG; ++g) {
      *reinterpret_cast<floatx4*>(&part[g][wave][lane * 8]) = floatx4{ps[g][0], ps[g][1], ps[g][2], ps[g][3]};
      *reinterpret_cast<floatx4*>(&part[g][wave][lane * 8 + 4]) = floatx4{ps[g][4], ps[g][5], ps[g][6], ps[g][7]};
    }
  }
  __syncthreads();
  float m[IG][8];  // the means of this lane's eight channels: the four waves' sums in wave order, one divide
#pragma unroll
  for (int g = 0; g < IG; ++g)
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      floatx4 a = *reinterpret_cast<const floatx4*>(&part[g][0][lane * 8 + 4 * h]);
#pragma unroll
      for (int k = 1; k < 4; ++k) a += *reinterpret_cast<const floatx4*>(&part[g][k][lane * 8 + 4 * h]);
#pragma unroll
      for (int e = 0; e < 4; ++e) m[g][4 * h + e] = a[e] / (float)HW;
    }
  const int f_begin = blockIdx.x * f_per_block;
  const int f_end = f_begin + f_per_block < F ? f_begin + f_per_block : F;
  typedef T V8 __attribute__((ext_vector_type(8)));
  for (int f0 = f_begin + wave; f0 < f_end; f0 += 32) {  // eight filters of this wave per trip: eight loads in flight
    V8 wv[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int f = f0 + 4 * u < f_end ? f0 + 4 * u : f0;
      wv[u] = *reinterpret_cast<const V8*>(w + (long long)f * 512 + lane * 8);
    }
    // The V = 8 * IG dot products of a trip are added over the 64 lanes together: at distance 32 a lane keeps the lower or
    // the upper half of the values (by its bit 5), hands the other half to its partner and adds what it receives, and so
    // on at 16, 8 ...; V - 1 lane exchanges and a few more for the bits that are left, instead of six per value, and
    // the same additions (own + partner's, the same pairs at the same distances: bit-identical to a tree per value).
    // A lane ends with the sum of value (g, u) = (vi >> 3, vi & 7), vi read off its upper bits.
    constexpr int V = 8 * IG;
    int vi = 0, dd = 32;
#pragma unroll
    for (int n = V; n > 1; n >>= 1, dd >>= 1) vi += (lane & dd) ? n / 2 : 0;
    const int gl = vi >> 3, fl = f0 + 4 * (vi & 7);
    const bool writer = (lane & (2 * dd - 1)) == 0 && fl < f_end && n0 + gl < N;
    const float bl = (bias && fl < f_end) ? bias[fl] : 0.0f;  // with the weights: fetched where it is added it is a trip to memory per output
    float x[V];
#pragma unroll
    for (int g = 0; g < IG; ++g)
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        float acc = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; ++e) acc += m[g][e] * (float)wv[u][e];
        x[g * 8 + u] = acc;
      }
    // (compile-time recursion: as a loop over halving n the compiler kept x[] indexed at run time)
    auto fold = [&](auto self, auto n_c, auto d_c) -> void {
      constexpr int n = decltype(n_c)::value, d = decltype(d_c)::value;
      if constexpr (n > 1) {
        const bool hi = (lane & d) != 0;
#pragma unroll
        for (int v = 0; v < n / 2; ++v) {
          const float keep = hi ? x[v + n / 2] : x[v];
          const float send = hi ? x[v] : x[v + n / 2];
          x[v] = keep + __shfl_xor(send, d);
        }
        self(self, std::integral_constant<int, n / 2>(), std::integral_constant<int, d / 2>());
      } else if constexpr (d >= 1) {
        x[0] += __shfl_xor(x[0], d);
        self(self, n_c, std::integral_constant<int, d / 2>());
      }
    };
    fold(fold, std::integral_constant<int, V>(), std::integral_constant<int, 32>());
    if (writer) out[(long long)(n0 + gl) * F + fl] = x[0] + bl;
  }
}

// in: NHWC [N][HW][512] of dt; w: [F][512] of dt; bias: [F] fp32 or null; out: [N][F] fp32.
void launch_avgpool_fc(const void* in, const void* w, const float* bias, float* out, int dt, int N, int HW, int C, int F,
                       hipStream_t s) {
  NNCV_REQUIRE(C == 512, "avgpool_fc: the head is built for 512 channels");
  NNCV_REQUIRE(N > 0 && N <= 65535 && HW > 0 && F > 0 && (long long)HW * 512 * (long long)dtype_size(dt) < (1ll << 31), "avgpool_fc: bad shape");
  // Slices of 64 outputs (two trips of eight filters per wave) once the images alone fill the CUs twice over, 32 (one
  // trip: the kernel is a chain of memory latencies) below that.  Batch 32: 6.5 us with 32, 6.2 with 64, 7.5 with 128.
  const int fpb = N >= 16 ? 64 : 32;
  dim3 grid((F + fpb - 1) / fpb, N);
  const double es = (double)dtype_size(dt);
  ProfScope prof("avgpool_fc", 2.0 * N * F * 512.0, es * ((double)N * HW * 512 + (double)F * 512) + 4.0 * N * F, s);
  if (dt == kF16)
    hipLaunchKernelGGL((avgpool_fc_kernel<half_t>), grid, dim3(256), 0, s, (const half_t*)in, (const half_t*)w, bias, out, N, HW, F, fpb);
  else
    hipLaunchKernelGGL((avgpool_fc_kernel<float>), grid, dim3(256), 0, s, (const float*)in, (const float*)w, bias, out, N, HW, F, fpb);
  NNCV_HIP_CHECK(hipGetLastError());
}

// ---------------------------------------------------------------------------------------------
// The driver's pre- and post-processing on the device (examples/Res18/main.cpp:38-77, :103-111).
//   preprocess: 8-bit HWC image (3 or 4 interleaved channels, the first three used) ->
//     NCHW, x = ((u8 / 255.f) - mean[c]) / std[c] with the driver's constants and its fp32
//     operation order (two IEEE divisions), stored as fp32 or rounded once to fp16.
//   argmax: the driver's scan `max = -100; idx = 0; if (v > max) {max = v; idx = i;}` per row:
//     the FIRST index of the largest value above -100 (NaNs never win, index 0 if nothing does).
// ---------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void preprocess_u8_kernel(const unsigned char* __restrict__ src, T* __restrict__ dst, int N,
                                                            int HW, int channels) {
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;  // one pixel each
  if (idx >= (long long)N * HW) return;
  const int n = (int)(idx / HW), p = (int)(idx - (long long)n * HW);
  const unsigned char* px = src + idx * channels;
  const float mean[3] = {0.485f, 0.456f, 0.406f}, sd[3] = {0.229f, 0.224f, 0.225f};
#pragma unroll
  for (int c = 0; c < 3; ++c) {
    const float v = (float)px[c] / 255.f;
    dst[((long long)n * 3 + c) * HW + p] = (T)((v - mean[c]) / sd[c]);
  }
}

void launch_preprocess_u8(const void* src, void* dst, int dst_dt, int N, int H, int W, int channels, hipStream_t s) {
  NNCV_REQUIRE(channels == 3 || channels == 4, "preprocess: 3 or 4 interleaved channels");
  const long long work = (long long)N * H * W;
  const long long grid = (work + 255) / 256;
  NNCV_REQUIRE(work > 0 && grid < (1ll << 31), "preprocess: bad size");
  ProfScope prof("preprocess_u8", 0.0, (double)work * (channels + 3.0 * dtype_size(dst_dt)), s);
  if (dst_dt == kF16)
    hipLaunchKernelGGL((preprocess_u8_kernel<half_t>), dim3((unsigned)grid), dim3(256), 0, s, (const unsigned char*)src, (half_t*)dst, N, H * W, channels);
  else
    hipLaunchKernelGGL((preprocess_u8_kernel<float>), dim3((unsigned)grid), dim3(256), 0, s, (const unsigned char*)src, (float*)dst, N, H * W, channels);
  NNCV_HIP_CHECK(hipGetLastError());
}

__global__ __launch_bounds__(256) void argmax_rows_kernel(const float* __restrict__ x, int* __restrict__ idx_out, int F) {
  __shared__ float smax[4];
  __shared__ int sidx[4];
  const float* row = x + (long long)blockIdx.x * F;
  float best = -100.f;
  int bi = 0x7fffffff;  // "nothing above -100 yet"
  for (int i = threadIdx.x; i < F; i += 256) {
    const float v = row[i];
    if (v > best) { best = v; bi = i; }  // strided scan: equal values keep the earlier index
  }
  // wave, then workgroup: larger value wins, equal values -> smaller index
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) {
    const float ov = __shfl_xor(best, d);
    const int oi = __shfl_xor(bi, d);
    if (ov > best || (ov == best && oi < bi)) { best = ov; bi = oi; }
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) { smax[wave] = best; sidx[wave] = bi; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 4; ++w)
      if (smax[w] > best || (smax[w] == best && sidx[w] < bi)) { best = smax[w]; bi = sidx[w]; }
    idx_out[blockIdx.x] = bi == 0x7fffffff ? 0 : bi;
  }
}

void launch_argmax_rows(const float* x, int* idx, int N, int F, hipStream_t s) {
  NNCV_REQUIRE(N > 0 && F > 0, "argmax: empty");
  ProfScope prof("argmax_rows", 0.0, 4.0 * N * (F + 1.0), s);
  hipLaunchKernelGGL(argmax_rows_kernel, dim3(N), dim3(256), 0, s, x, idx, F);
  NNCV_HIP_CHECK(hipGetLastError());
}

// ---------------------------------------------------------------------------------------------
// generic strided relayout / cast, dst (+)= src (operator-level ABI only; not on the ResNet-18 path)
// ---------------------------------------------------------------------------------------------
template <typename Ts, typename Td>
__global__ void relayout_kernel(const Ts* __restrict__ src, Strides4 ss, Td* __restrict__ dst, Strides4 ds, int N, int Cs,
                                int Cd, int H, int W, int dst_c_fastest, int accumulate) {
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long long)N * Cd * H * W) return;
  int n, c, h, w;
  long long r = idx;
  if (dst_c_fastest) {
    c = (int)(r % Cd); r /= Cd; w = (int)(r % W); r /= W; h = (int)(r % H); n = (int)(r / H);
  } else {
    w = (int)(r % W); r /= W; h = (int)(r % H); r /= H; c = (int)(r % Cd); n = (int)(r / Cd);
  }
  const float v = c < Cs ? (float)src[n * ss.n + c * ss.c + h * ss.h + w * ss.w] : 0.0f;
  Td* d = dst + (n * ds.n + c * ds.c + h * ds.h + w * ds.w);
  *d = accumulate ? (Td)((float)*d + v) : (Td)v;
}

void launch_relayout(const void* src, int src_dt, Strides4 ss, void* dst, int dst_dt, Strides4 ds, int N, int Cs, int Cd,
                     int H, int W, bool accumulate, hipStream_t s) {
  const long long work = (long long)N * Cd * H * W;
  if (work == 0) return;
  const long long grid = (work + 255) / 256;
  NNCV_REQUIRE(grid < (1ll << 31), "relayout: grid too large");
  const int cf = ds.c == 1;
#define LAUNCH(TS, TD) \
  hipLaunchKernelGGL((relayout_kernel<TS, TD>), dim3((unsigned)grid), dim3(256), 0, s, (const TS*)src, ss, (TD*)dst, ds, N, Cs, Cd, H, W, cf, accumulate ? 1 : 0)
  if (src_dt == kF32 && dst_dt == kF32) LAUNCH(float, float);
  else if (src_dt == kF32 && dst_dt == kF16) LAUNCH(float, half_t);
  else if (src_dt == kF16 && dst_dt == kF16) LAUNCH(half_t, half_t);
  else if (src_dt == kF16 && dst_dt == kF32) LAUNCH(half_t, float);
#undef LAUNCH
  NNCV_HIP_CHECK(hipGetLastError());
}

// ---------------------------------------------------------------------------------------------
// Network input of the graph executor: NCHW with a few channels (an image: 3) -> NHWC padded to
// one 16-byte vector per pixel.  One thread per pixel: the C plane reads are coalesced across the
// wave (consecutive pixels), the write is one whole vector per lane.
// ---------------------------------------------------------------------------------------------
template <typename T, int CP>
__global__ __launch_bounds__(256) void image_to_nhwc_kernel(const T* __restrict__ src, T* __restrict__ dst, int C, long long HW,
                                                            long long total) {
  typedef T V __attribute__((ext_vector_type(CP)));
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const long long n = idx / HW, p = idx - n * HW;
  V v;
#pragma unroll
  for (int c = 0; c < CP; ++c) v[c] = c < C ? src[(n * C + c) * HW + p] : (T)0.0f;
  *reinterpret_cast<V*>(dst + idx * CP) = v;
}

bool image_to_nhwc_applicable(int dt, int C) { return C >= 1 && C <= (dt == kF16 ? 8 : 4); }

// Cp: channels per pixel in dst; one 16-byte vector (8 halves / 4 floats), or for fp16 half a
// vector (4), which makes two horizontally adjacent pixels one vector (the pixel-pair form).
void launch_image_to_nhwc(const void* src, void* dst, int dt, int N, int C, int H, int W, hipStream_t s, int Cp) {
  const int vn = dt == kF16 ? 8 : 4;
  if (Cp == 0) Cp = vn;
  NNCV_REQUIRE(image_to_nhwc_applicable(dt, C) && C <= Cp && (Cp == vn || (dt == kF16 && Cp == 4)),
               "image_to_nhwc: channel count not covered");
  const long long HW = (long long)H * W, total = HW * N;
  if (total == 0) return;
  const long long grid = (total + 255) / 256;
  NNCV_REQUIRE(grid < (1ll << 31), "image_to_nhwc: grid too large");
  ProfScope prof("image_to_nhwc", 0.0, (double)dtype_size(dt) * total * (C + Cp), s);
  if (dt == kF16 && Cp == 8)
    hipLaunchKernelGGL((image_to_nhwc_kernel<half_t, 8>), dim3((unsigned)grid), dim3(256), 0, s, (const half_t*)src, (half_t*)dst, C, HW, total);
  else if (dt == kF16)
    hipLaunchKernelGGL((image_to_nhwc_kernel<half_t, 4>), dim3((unsigned)grid), dim3(256), 0, s, (const half_t*)src, (half_t*)dst, C, HW, total);
  else
    hipLaunchKernelGGL((image_to_nhwc_kernel<float, 4>), dim3((unsigned)grid), dim3(256), 0, s, (const float*)src, (float*)dst, C, HW, total);
  NNCV_HIP_CHECK(hipGetLastError());
}

// Filters of a stride-2 convolution over an image stored as pixel pairs ([N][H][W/2][2 pixels x 4
// channels], fp16): with ix = 2*ox - pad + s, the pair holding column ix is ox - pad2 + s2, so the
// horizontal walk becomes stride 1 over S2 pairs and the K axis shrinks from K*K*8 (3 channels
// padded to a whole vector) to K*S2*8.
//   pad even: pad2 = pad/2,     S2 = ceil(K/2),     element (s2, p) is filter column 2*s2 + p
//   pad odd : pad2 = (pad+1)/2, S2 = ceil((K+1)/2), element (s2, p) is filter column 2*s2 + p - 1
// (zero outside 0..K-1 and for channels >= C).  dst: [Fp][K][S2][8], rows >= F zero.
template <typename Ts>
__global__ void weight_pairs_kernel(const Ts* __restrict__ w, half_t* __restrict__ dst, int F, int C, int K, int S2, int shift,
                                    int total) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const int e = i & 7, c = e & 3, pp = e >> 2;
  int r = i >> 3;
  const int s2 = r % S2; r /= S2;
  const int kr = r % K;
  const int f = r / K;
  const int sc = 2 * s2 + pp - shift;
  float v = 0.0f;
  if (f < F && c < C && sc >= 0 && sc < K) v = (float)w[((f * C + c) * K + kr) * K + sc];
  dst[i] = (half_t)v;
}

void launch_weight_pairs(const void* w, int w_dt, void* dst, int F, int Fp, int C, int K, int pad, hipStream_t s) {
  NNCV_REQUIRE(C >= 1 && C <= 4 && K >= 1 && Fp >= F, "weight_pairs: shape not covered");
  const int shift = pad & 1, S2 = (K + shift + 1) / 2;
  const int total = Fp * K * S2 * 8;
  const unsigned grid = (unsigned)((total + 255) / 256);
  if (w_dt == kF16)
    hipLaunchKernelGGL((weight_pairs_kernel<half_t>), dim3(grid), dim3(256), 0, s, (const half_t*)w, (half_t*)dst, F, C, K, S2, shift, total);
  else
    hipLaunchKernelGGL((weight_pairs_kernel<float>), dim3(grid), dim3(256), 0, s, (const float*)w, (half_t*)dst, F, C, K, S2, shift, total);
  NNCV_HIP_CHECK(hipGetLastError());
}

// ---------------------------------------------------------------------------------------------
// Stem input packing.  The 7x7 stride-2 pad-3 convolution over 3 channels
// (tests/Nets/Res18.mlir:118-124) is run by the implicit-GEMM kernel as a 7x4 stride-(2,1)
// convolution over "pixel pairs": the NCHW image becomes [N][H+6][Wp][8] where element
// (y', xp, 4*p + c) = in[c][y'-3][2*xp + p - 3] (zero outside the image and for c = 3), so that
// one 16-byte chunk holds two horizontally adjacent pixels and a stride-2 walk in x becomes a
// stride-1 walk over pairs.  Wp = (W + 9) / 2.
// ---------------------------------------------------------------------------------------------
template <typename Ts, typename Td>
__global__ __launch_bounds__(256) void stem_pack_kernel(const Ts* __restrict__ src, Td* __restrict__ dst, int N, int H, int W,
                                                        int HP, int WP) {
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long long)N * HP * WP) return;
  const int xp = (int)(idx % WP);
  const int yp = (int)((idx / WP) % HP);
  const int n = (int)(idx / ((long long)WP * HP));
  const int iy = yp - 3;
  Td v[8];
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    const int ix = 2 * xp + p - 3;
    const bool ok = (unsigned)iy < (unsigned)H && (unsigned)ix < (unsigned)W;
#pragma unroll
    for (int c = 0; c < 3; ++c) v[4 * p + c] = ok ? (Td)(float)src[(((long long)n * 3 + c) * H + iy) * W + ix] : (Td)0.0f;
    v[4 * p + 3] = (Td)0.0f;
  }
  Td* d = dst + idx * 8;
#pragma unroll
  for (int e = 0; e < 8; ++e) d[e] = v[e];
}

void launch_stem_pack(const void* src, int src_dt, void* dst, int dst_dt, int N, int H, int W, hipStream_t s) {
  const int HP = H + 6, WP = (W + 9) / 2;
  const long long work = (long long)N * HP * WP;
  const long long grid = (work + 255) / 256;
  NNCV_REQUIRE(grid < (1ll << 31), "stem_pack: grid too large");
  ProfScope prof("stem_pack", 0.0, (double)dtype_size(src_dt) * N * 3 * H * W + (double)dtype_size(dst_dt) * work * 8, s);
#define LAUNCH(TS, TD) \
  hipLaunchKernelGGL((stem_pack_kernel<TS, TD>), dim3((unsigned)grid), dim3(256), 0, s, (const TS*)src, (TD*)dst, N, H, W, HP, WP)
  if (src_dt == kF32 && dst_dt == kF32) LAUNCH(float, float);
  else if (src_dt == kF16 && dst_dt == kF16) LAUNCH(half_t, half_t);
  else if (src_dt == kF32 && dst_dt == kF16) LAUNCH(float, half_t);
  else fail("stem_pack: unsupported dtype combination");
#undef LAUNCH
  NNCV_HIP_CHECK(hipGetLastError());
}

// ---------------------------------------------------------------------------------------------
// one-time parameter preparation
// ---------------------------------------------------------------------------------------------
template <typename Ts, typename Td>
__global__ void weight_frsc_kernel(const Ts* __restrict__ w, Td* __restrict__ dst, int F, int C, int R, int S, int Cp) {
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long long)F * R * S * Cp) return;
  const int c = (int)(idx % Cp);
  long long r = idx / Cp;
  const int s = (int)(r % S); r /= S;
  const int rr = (int)(r % R);
  const int f = (int)(r / R);
  dst[idx] = c < C ? (Td)(float)w[(((long long)f * C + c) * R + rr) * S + s] : (Td)0.0f;
}

void launch_weight_frsc(const void* w, int w_dt, void* dst, int dst_dt, int F, int C, int R, int S, int Cp, hipStream_t s) {
  const long long work = (long long)F * R * S * Cp;
  const unsigned grid = (unsigned)((work + 255) / 256);
#define LAUNCH(TS, TD) hipLaunchKernelGGL((weight_frsc_kernel<TS, TD>), dim3(grid), dim3(256), 0, s, (const TS*)w, (TD*)dst, F, C, R, S, Cp)
  if (w_dt == kF32 && dst_dt == kF32) LAUNCH(float, float);
  else if (w_dt == kF16 && dst_dt == kF16) LAUNCH(half_t, half_t);
  else if (w_dt == kF32 && dst_dt == kF16) LAUNCH(float, half_t);
  else fail("weight_frsc: unsupported dtype combination");
#undef LAUNCH
  NNCV_HIP_CHECK(hipGetLastError());
}

// Fragment-major 3x3 weights for conv3x3_patch.hip: a wave's MFMA weight operand for
// (64-filter block fb, 128-byte channel slab sl, tap, K sub-step kk, filter half i) is one
// contiguous kilobyte, lane L holding filter fb*64 + i*32 + L%32, channels
// sl*SLAB + (L/32 + 2*kk)*CE .. +CE-1 (CE = elements per 16 bytes, SLAB = 8*CE):
//   offset(fb, sl, tap, kk, i, L) = (((((fb*nslab + sl)*9 + tap)*4 + kk)*2 + i)*64 + L) * 16 bytes.
// Filters beyond F are zero.  TAPS = 1 is the same order for 1x1 filters (the shortcut convolution
// that rides on a stride-2 3x3 one).
template <typename Ts, typename Td, int TAPS>
__global__ void weight_frag3x3_kernel(const Ts* __restrict__ w, Td* __restrict__ dst, int F, int C, int Fp) {
  constexpr int CE = 16 / (int)sizeof(Td);
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;  // one 16-byte chunk each
  const int nslab = C / (8 * CE);
  const long long total = (long long)(Fp / 64) * nslab * TAPS * 4 * 2 * 64;
  if (idx >= total) return;
  const int L = (int)(idx & 63);
  long long r = idx >> 6;
  const int i = (int)(r & 1); r >>= 1;
  const int kk = (int)(r & 3); r >>= 2;
  const int tap = (int)(r % TAPS); r /= TAPS;
  const int sl = (int)(r % nslab);
  const int fb = (int)(r / nslab);
  const int f = fb * 64 + i * 32 + (L & 31);
  const int c0 = sl * 8 * CE + ((L >> 5) + 2 * kk) * CE;
  Td* d = dst + idx * CE;
#pragma unroll
  for (int e = 0; e < CE; ++e) d[e] = f < F ? (Td)(float)w[((long long)f * C + c0 + e) * TAPS + tap] : (Td)0.0f;
}

template <int TAPS>
static void launch_weight_frag(const void* w, int w_dt, void* dst, int dst_dt, int F, int C, hipStream_t s) {
  const int ce = dst_dt == kF16 ? 8 : 4;
  NNCV_REQUIRE(C % (8 * ce) == 0, "weight_frag: C must be a multiple of the 128-byte slab");
  const int Fp = (F + 63) / 64 * 64;
  const long long total = (long long)(Fp / 64) * (C / (8 * ce)) * TAPS * 4 * 2 * 64;
  const unsigned grid = (unsigned)((total + 255) / 256);
#define LAUNCH(TS, TD) hipLaunchKernelGGL((weight_frag3x3_kernel<TS, TD, TAPS>), dim3(grid), dim3(256), 0, s, (const TS*)w, (TD*)dst, F, C, Fp)
  if (w_dt == kF32 && dst_dt == kF32) LAUNCH(float, float);
  else if (w_dt == kF16 && dst_dt == kF16) LAUNCH(half_t, half_t);
  else fail("weight_frag: unsupported dtype combination");
#undef LAUNCH
  NNCV_HIP_CHECK(hipGetLastError());
}

void launch_weight_frag3x3(const void* w, int w_dt, void* dst, int dst_dt, int F, int C, hipStream_t s) {
  launch_weight_frag<9>(w, w_dt, dst, dst_dt, F, C, s);
}
void launch_weight_frag1x1(const void* w, int w_dt, void* dst, int dst_dt, int F, int C, hipStream_t s) {
  launch_weight_frag<1>(w, w_dt, dst, dst_dt, F, C, s);
}

template <typename Ts, typename Td>
__global__ void stem_weight_kernel(const Ts* __restrict__ w, Td* __restrict__ dst, int F, int col_shift) {
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;  // over [F][7][4][8]
  if (idx >= F * 7 * 4 * 8) return;
  const int e = idx & 7, sp = (idx >> 3) & 3, r = (idx >> 5) % 7, f = idx / 224;
  const int p = e >> 2, c = e & 3, s = 2 * sp + p - col_shift;
  dst[idx] = (c < 3 && s >= 0 && s < 7) ? (Td)(float)w[((f * 3 + c) * 7 + r) * 7 + s] : (Td)0.0f;
}

void launch_stem_weight(const void* w, int w_dt, void* dst, int dst_dt, int F, int col_shift, hipStream_t s) {
  const unsigned grid = (unsigned)((F * 224 + 255) / 256);
#define LAUNCH(TS, TD) \
  hipLaunchKernelGGL((stem_weight_kernel<TS, TD>), dim3(grid), dim3(256), 0, s, (const TS*)w, (TD*)dst, F, col_shift)
  if (w_dt == kF32 && dst_dt == kF32) LAUNCH(float, float);
  else if (w_dt == kF16 && dst_dt == kF16) LAUNCH(half_t, half_t);
  else if (w_dt == kF32 && dst_dt == kF16) LAUNCH(float, half_t);
  else fail("stem_weight: unsupported dtype combination");
#undef LAUNCH
  NNCV_HIP_CHECK(hipGetLastError());
}

// BN (tests/Nets/Res18.mlir:127-136) folded to y = x*scale + shift:
//   r = 1/sqrt(var + (float)1e-5) ; scale = gamma * r ; shift = beta - mean * scale
// evaluated in fp64 and rounded once, so the fold adds less than one fp32 ulp to each factor.
template <typename T>
__global__ void bn_fold_kernel(const T* g, const T* b, const T* m, const T* v, float* scale, float* shift, int C, float eps_f) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const double eps = (double)eps_f;  // the reference truncates its f64 epsilon to f32 first
  const double r = 1.0 / sqrt((double)(float)v[c] + eps);
  const double sc = (double)(float)g[c] * r;
  scale[c] = (float)sc;
  shift[c] = (float)((double)(float)b[c] - (double)(float)m[c] * sc);
}

void launch_bn_fold(const void* g, const void* b, const void* m, const void* v, int dt, float* scale, float* shift, int C,
                    hipStream_t s, float eps) {
  const unsigned grid = (unsigned)((C + 255) / 256);
  if (dt == kF16)
    hipLaunchKernelGGL((bn_fold_kernel<half_t>), dim3(grid), dim3(256), 0, s, (const half_t*)g, (const half_t*)b, (const half_t*)m, (const half_t*)v, scale, shift, C, eps);
  else
    hipLaunchKernelGGL((bn_fold_kernel<float>), dim3(grid), dim3(256), 0, s, (const float*)g, (const float*)b, (const float*)m, (const float*)v, scale, shift, C, eps);
  NNCV_HIP_CHECK(hipGetLastError());
}

template <typename Ts, typename Td>
__global__ void cast_kernel(const Ts* __restrict__ src, Td* __restrict__ dst, long long n) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) dst[i] = (Td)(float)src[i];
}

void launch_cast(const void* src, int src_dt, void* dst, int dst_dt, long long n, hipStream_t s) {
  if (n == 0) return;
  const unsigned grid = (unsigned)((n + 255) / 256);
#define LAUNCH(TS, TD) hipLaunchKernelGGL((cast_kernel<TS, TD>), dim3(grid), dim3(256), 0, s, (const TS*)src, (TD*)dst, n)
  if (src_dt == kF32 && dst_dt == kF32) LAUNCH(float, float);
  else if (src_dt == kF16 && dst_dt == kF16) LAUNCH(half_t, half_t);
  else if (src_dt == kF32 && dst_dt == kF16) LAUNCH(float, half_t);
  else LAUNCH(half_t, float);
#undef LAUNCH
  NNCV_HIP_CHECK(hipGetLastError());
}

__global__ void fill_f32_kernel(float* dst, float v, long long n) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) dst[i] = v;
}
void launch_fill_f32(float* dst, float v, long long n, hipStream_t s) {
  if (n == 0) return;
  hipLaunchKernelGGL(fill_f32_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, dst, v, n);
  NNCV_HIP_CHECK(hipGetLastError());
}

}  // namespace nncv_hip
