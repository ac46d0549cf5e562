// Winograd F(4x4,3x3) transforms for gfx950.
//
// Counterparts in the reference (which implements F(6x6,3x3) as IR rewrites and never enables it
// in a CPU pipeline): filter fold  OptimizeConv2dUsingWinograd.cpp:41-83, input transform
// TileAndDecoWinogradPass.cpp:149-232 (V = B^T d B, ragged tiles zero padded :208-211), output
// transform :357-413 (Y = A^T M A) and the final extract_slice
// OptimizeConv2dUsingWinograd.cpp:272-278.  The F(4,3) matrices are the textbook Lavin & Gray
// set (interpolation points 0, +-1, +-2, inf).
//
// Data layout in HBM, t = 6*i + j over the 36 transformed positions:
//   U[t][F][C]      filters, K(=C)-contiguous rows  -> "weights" operand of the batched GEMM
//   V[t][tiles][C]  inputs,  K(=C)-contiguous rows  -> "pixels" operand
//   M[t][tiles][F]  products
// tiles = N * ceil(OH/4) * ceil(OW/4), tile = (n*TH + ty)*TW + tx.
//
// These kernels are pure data movement plus a few adds per element: they are HBM-bandwidth
// bound.  Work is split so that the lanes of a wave run along the channel axis, which is the
// contiguous axis of V, M and of NHWC activations, so every access of a wave is one contiguous
// segment (2 elements per lane).  All transform arithmetic is fp32 regardless of storage type.
#include "common.hpp"

namespace nncv_hip {

template <typename T>
struct Pair;
template <>
struct Pair<float> {
  typedef float type __attribute__((ext_vector_type(2)));
};
template <>
struct Pair<half_t> {
  typedef half_t type __attribute__((ext_vector_type(2)));
};


// rows of B^T applied to a 6-vector
__device__ __forceinline__ void bt6(const float d[6], float o[6]) {
  o[0] = 4.0f * d[0] - 5.0f * d[2] + d[4];
  o[1] = -4.0f * d[1] - 4.0f * d[2] + d[3] + d[4];
  o[2] = 4.0f * d[1] - 4.0f * d[2] - d[3] + d[4];
  o[3] = -2.0f * d[1] - d[2] + 2.0f * d[3] + d[4];
  o[4] = 2.0f * d[1] - d[2] - 2.0f * d[3] + d[4];
  o[5] = 4.0f * d[1] - 5.0f * d[3] + d[5];
}
// rows of A^T applied to a 6-vector
__device__ __forceinline__ void at6(const float m[6], float o[4]) {
  o[0] = m[0] + m[1] + m[2] + m[3] + m[4];
  o[1] = m[1] - m[2] + 2.0f * m[3] - 2.0f * m[4];
  o[2] = m[1] + m[2] + 4.0f * m[3] + 4.0f * m[4];
  o[3] = m[1] - m[2] + 8.0f * m[3] - 8.0f * m[4] + m[5];
}

// ---------------------------------------------------------------------------------------------
// filter: one thread per (f, c); evaluated in fp64, runs once per model load.
// ---------------------------------------------------------------------------------------------
template <typename Tw, typename Tu>
__global__ void wino43_filter_kernel(const Tw* __restrict__ w, Tu* __restrict__ U, int F, int C) {
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= F * C) return;
  const int f = idx / C, c = idx - f * C;
  const double G[6][3] = {{1.0 / 4, 0, 0},           {-1.0 / 6, -1.0 / 6, -1.0 / 6}, {-1.0 / 6, 1.0 / 6, -1.0 / 6},
                          {1.0 / 24, 1.0 / 12, 1.0 / 6}, {1.0 / 24, -1.0 / 12, 1.0 / 6}, {0, 0, 1}};
  double g[3][3], t[6][3];
  for (int p = 0; p < 3; ++p)
    for (int q = 0; q < 3; ++q) g[p][q] = (double)(float)w[(long long)idx * 9 + p * 3 + q];
  for (int i = 0; i < 6; ++i)
    for (int q = 0; q < 3; ++q) t[i][q] = G[i][0] * g[0][q] + G[i][1] * g[1][q] + G[i][2] * g[2][q];
  for (int i = 0; i < 6; ++i)
    for (int j = 0; j < 6; ++j) {
      const double u = t[i][0] * G[j][0] + t[i][1] * G[j][1] + t[i][2] * G[j][2];
      U[((long long)(i * 6 + j) * F + f) * C + c] = (Tu)(float)u;
    }
}

// ---------------------------------------------------------------------------------------------
// input: one thread per (tile, channel pair).
// ---------------------------------------------------------------------------------------------
template <typename Tin, typename Tv, bool kContigC>
__global__ __launch_bounds__(256) void wino43_input_kernel(const Tin* __restrict__ in, Strides4 st, Tv* __restrict__ V,
                                                           int N, int C, int H, int W, int pad, int TH, int TW) {
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const int C2 = C >> 1;
  const long long tiles = (long long)N * TH * TW;
  if (idx >= tiles * C2) return;
  const int c = (int)(idx % C2) * 2;
  const long long tile = idx / C2;
  const int tx = (int)(tile % TW);
  const int ty = (int)((tile / TW) % TH);
  const int n = (int)(tile / ((long long)TW * TH));
  const int y0 = ty * 4 - pad, x0 = tx * 4 - pad;
  const Tin* base = in + (long long)n * st.n + (long long)c * st.c;

  float t0[6][6], t1[6][6];  // B^T d, per channel
#pragma unroll
  for (int x = 0; x < 6; ++x) {
    float d0[6], d1[6];
    const int ix = x0 + x;
#pragma unroll
    for (int y = 0; y < 6; ++y) {
      const int iy = y0 + y;
      float a = 0.0f, b = 0.0f;
      if ((unsigned)iy < (unsigned)H && (unsigned)ix < (unsigned)W) {
        const Tin* p = base + (long long)iy * st.h + (long long)ix * st.w;
        if (kContigC) {
          const typename Pair<Tin>::type v = *reinterpret_cast<const typename Pair<Tin>::type*>(p);
          a = (float)v[0];
          b = (float)v[1];
        } else {
          a = (float)p[0];
          b = (float)p[st.c];
        }
      }
      d0[y] = a;
      d1[y] = b;
    }
    float o0[6], o1[6];
    bt6(d0, o0);
    bt6(d1, o1);
#pragma unroll
    for (int i = 0; i < 6; ++i) {
      t0[i][x] = o0[i];
      t1[i][x] = o1[i];
    }
  }
#pragma unroll
  for (int i = 0; i < 6; ++i) {
    float o0[6], o1[6];
    bt6(t0[i], o0);
    bt6(t1[i], o1);
#pragma unroll
    for (int j = 0; j < 6; ++j) {
      typename Pair<Tv>::type v;
      v[0] = (Tv)o0[j];
      v[1] = (Tv)o1[j];
      *reinterpret_cast<typename Pair<Tv>::type*>(V + ((long long)(i * 6 + j) * tiles + tile) * C + c) = v;
    }
  }
}

// ---------------------------------------------------------------------------------------------
// output: one thread per (tile, channel pair); fused BN scale/shift, residual add and ReLU.
// ---------------------------------------------------------------------------------------------
template <typename Tm, typename Tout, bool kContigC>
__global__ __launch_bounds__(256) void wino43_output_kernel(const WinoOutArgs a, int TH, int TW) {
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const int F2 = a.F >> 1;
  const long long tiles = (long long)a.N * TH * TW;
  if (idx >= tiles * F2) return;
  const int f = (int)(idx % F2) * 2;
  const long long tile = idx / F2;
  const int tx = (int)(tile % TW);
  const int ty = (int)((tile / TW) % TH);
  const int n = (int)(tile / ((long long)TW * TH));
  const Tm* M = static_cast<const Tm*>(a.M);

  float t0[4][6], t1[4][6];  // A^T m, per channel
#pragma unroll
  for (int j = 0; j < 6; ++j) {
    float m0[6], m1[6];
#pragma unroll
    for (int i = 0; i < 6; ++i) {
      const typename Pair<Tm>::type v =
          *reinterpret_cast<const typename Pair<Tm>::type*>(M + ((long long)(i * 6 + j) * tiles + tile) * a.F + f);
      m0[i] = (float)v[0];
      m1[i] = (float)v[1];
    }
    float o0[4], o1[4];
    at6(m0, o0);
    at6(m1, o1);
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      t0[r][j] = o0[r];
      t1[r][j] = o1[r];
    }
  }
  const float sc0 = a.scale ? a.scale[f] : 1.0f, sc1 = a.scale ? a.scale[f + 1] : 1.0f;
  const float sh0 = a.shift ? a.shift[f] : 0.0f, sh1 = a.shift ? a.shift[f + 1] : 0.0f;
  Tout* out = static_cast<Tout*>(a.out);
  const Tout* res = static_cast<const Tout*>(a.residual);
  const long long base = (long long)n * a.st.n + (long long)f * a.st.c;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    float y0[4], y1[4];
    at6(t0[r], y0);
    at6(t1[r], y1);
    const int oy = ty * 4 + r;
    if (oy >= a.OH) continue;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int ox = tx * 4 + q;
      if (ox >= a.OW) continue;
      const long long o = base + (long long)oy * a.st.h + (long long)ox * a.st.w;
      float v0 = y0[q] * sc0 + sh0, v1 = y1[q] * sc1 + sh1;
      if (kContigC) {
        typedef typename Pair<Tout>::type P2;
        if (res) {
          const P2 rv = *reinterpret_cast<const P2*>(res + o);
          v0 += (float)rv[0];
          v1 += (float)rv[1];
        }
        if (a.accumulate) {
          const P2 ov = *reinterpret_cast<const P2*>(out + o);
          v0 += (float)ov[0];
          v1 += (float)ov[1];
        }
        if (a.relu) {
          v0 = relu_ugt(v0);
          v1 = relu_ugt(v1);
        }
        P2 w;
        w[0] = (Tout)v0;
        w[1] = (Tout)v1;
        *reinterpret_cast<P2*>(out + o) = w;
      } else {
        if (res) {
          v0 += (float)res[o];
          v1 += (float)res[o + a.st.c];
        }
        if (a.accumulate) {
          v0 += (float)out[o];
          v1 += (float)out[o + a.st.c];
        }
        if (a.relu) {
          v0 = relu_ugt(v0);
          v1 = relu_ugt(v1);
        }
        out[o] = (Tout)v0;
        out[o + a.st.c] = (Tout)v1;
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------
// LDS-staged forms for dense NHWC tensors whose channel count is a multiple of 64: the 2-D
// transform is done as two 1-D passes with the intermediate in LDS (fp32), so that a thread never
// holds more than one 6-vector per channel, and every global access is 16 bytes per lane with 8
// (fp16) or 16 (fp32) consecutive lanes covering the 64 channels of one pixel / one V or M row.
// A workgroup owns kTiles tiles x 64 channels.
//   input : pass 1  thread = (tile, column x, 16-byte channel group): 6 loads down the column,
//                   B^T along y, 6 vectors to LDS[tile][i][x][c];
//           pass 2  thread = (tile, row i, channel group): 6 vectors from LDS, B^T along x,
//                   6 stores to V[6i+j][tile][c].
//   output: pass 1  thread = (tile, column j, channel group): 6 loads M[6i+j][tile][f], A^T along
//                   i, 4 vectors to LDS[tile][r][j][f];
//           pass 2  thread = (tile, row r, channel group): 6 vectors from LDS, A^T along j, then
//                   scale/shift, residual, ReLU and one rounding, up to 4 pixel stores.
// ---------------------------------------------------------------------------------------------
template <typename T>
struct WinoLds {
  static constexpr int VW = 16 / (int)sizeof(T);  // channels per thread
  static constexpr int CG = 64 / VW;              // channel groups per 64 channels
  static constexpr int kTiles = 240 / (6 * CG);   // fp16: 5, fp32: 2
  // floats per row of 64 channels in LDS: four more than it holds.  The lanes of a wave are (channel group, u) pairs and u
  // moves by one row: at a pitch of 64 floats all six u would meet in the same banks, at 68 the 16-byte accesses of any
  // 16 neighbouring lanes fall into 16 different bank groups.
  static constexpr int kRow = 68;
  typedef T Vec __attribute__((ext_vector_type(VW)));
};
typedef float wf4 __attribute__((ext_vector_type(4)));

template <typename T>
__global__ __launch_bounds__(256) void wino43_input_lds_kernel(const T* __restrict__ in, T* __restrict__ V, int N, int C, int H,
                                                               int W, int pad, int TH, int TW) {
  typedef WinoLds<T> L;
  constexpr int VW = L::VW, CG = L::CG, KT = L::kTiles;
  typedef typename L::Vec Vec;
  __shared__ __align__(16) float mid[KT][6][6][L::kRow];
  const int tid = threadIdx.x;
  const long long tiles = (long long)N * TH * TW;
  // Workgroups go to the 8 XCDs round-robin; tile rows share two input rows with the row below, so each XCD takes a
  // contiguous range of tile blocks and its L2 serves the shared rows (measured: 1.64x the input bytes fetched otherwise).
  const unsigned per_xcd = (gridDim.x + 7u) >> 3;
  const unsigned blk = (blockIdx.x & 7u) * per_xcd + (blockIdx.x >> 3);
  const long long tile0 = (long long)blk * KT;
  const int c0 = blockIdx.y * 64;
  const int cg = tid % CG, u = (tid / CG) % 6, tl = tid / (6 * CG);
  const long long tile = tile0 + tl;
  const bool live = tl < KT && tile < tiles;
  if (live) {  // pass 1: u = column x
    const int tx = (int)(tile % TW), ty = (int)((tile / TW) % TH), n = (int)(tile / ((long long)TW * TH));
    const int ix = tx * 4 - pad + u, y0 = ty * 4 - pad;
    Vec d[6];
#pragma unroll
    for (int y = 0; y < 6; ++y) {
      const int iy = y0 + y;
      const bool ok = (unsigned)iy < (unsigned)H && (unsigned)ix < (unsigned)W;
      // out-of-image taps read pixel 0 (a valid address) and are zeroed: no divergent branch
      const long long off = ok ? (((long long)n * H + iy) * W + ix) * C + c0 + cg * VW : 0;
      Vec v = *reinterpret_cast<const Vec*>(in + off);
      if (!ok)
        for (int e = 0; e < VW; ++e) v[e] = (T)0.0f;
      d[y] = v;
    }
    float t[6][VW];
#pragma unroll
    for (int e = 0; e < VW; ++e) {
      float col[6], o[6];
#pragma unroll
      for (int y = 0; y < 6; ++y) col[y] = (float)d[y][e];
      bt6(col, o);
#pragma unroll
      for (int i = 0; i < 6; ++i) t[i][e] = o[i];
    }
#pragma unroll
    for (int i = 0; i < 6; ++i)
#pragma unroll
      for (int e0 = 0; e0 < VW; e0 += 4)
        *reinterpret_cast<wf4*>(&mid[tl][i][u][cg * VW + e0]) = wf4{t[i][e0], t[i][e0 + 1], t[i][e0 + 2], t[i][e0 + 3]};
  }
  __syncthreads();
  if (live) {  // pass 2: u = row i
    // all VW channels of the lane at once: every store is 16 bytes, eight neighbouring lanes fill one 128-byte line
    // (four channels at a time, the fp16 lanes wrote every line of V in two half-filled passes)
    float o[6][VW];
#pragma unroll
    for (int e0 = 0; e0 < VW; e0 += 4) {
      wf4 rx[6];
#pragma unroll
      for (int x = 0; x < 6; ++x) rx[x] = *reinterpret_cast<const wf4*>(&mid[tl][u][x][cg * VW + e0]);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float row[6], r[6];
#pragma unroll
        for (int x = 0; x < 6; ++x) row[x] = rx[x][e];
        bt6(row, r);
#pragma unroll
        for (int j = 0; j < 6; ++j) o[j][e0 + e] = r[j];
      }
    }
#pragma unroll
    for (int j = 0; j < 6; ++j) {
      Vec w;
#pragma unroll
      for (int e = 0; e < VW; ++e) w[e] = (T)o[j][e];
      *reinterpret_cast<Vec*>(V + ((long long)(u * 6 + j) * tiles + tile) * C + c0 + cg * VW) = w;
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void wino43_output_lds_kernel(const WinoOutArgs a, int TH, int TW) {
  typedef WinoLds<T> L;
  constexpr int VW = L::VW, CG = L::CG, KT = L::kTiles;
  typedef typename L::Vec Vec;
  __shared__ __align__(16) float mid[KT][4][6][L::kRow];
  const int tid = threadIdx.x;
  const long long tiles = (long long)a.N * TH * TW;
  const long long tile0 = (long long)blockIdx.x * KT;
  const int f0 = blockIdx.y * 64;
  const int cg = tid % CG, u = (tid / CG) % 6, tl = tid / (6 * CG);
  const long long tile = tile0 + tl;
  const bool live = tl < KT && tile < tiles;
  const T* M = static_cast<const T*>(a.M);
  if (live) {  // pass 1: u = column j
    Vec m[6];
#pragma unroll
    for (int i = 0; i < 6; ++i) m[i] = *reinterpret_cast<const Vec*>(M + ((long long)(i * 6 + u) * tiles + tile) * a.F + f0 + cg * VW);
    float t[4][VW];
#pragma unroll
    for (int e = 0; e < VW; ++e) {
      float col[6], o[4];
#pragma unroll
      for (int i = 0; i < 6; ++i) col[i] = (float)m[i][e];
      at6(col, o);
#pragma unroll
      for (int r = 0; r < 4; ++r) t[r][e] = o[r];
    }
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
      for (int e0 = 0; e0 < VW; e0 += 4)
        *reinterpret_cast<wf4*>(&mid[tl][r][u][cg * VW + e0]) = wf4{t[r][e0], t[r][e0 + 1], t[r][e0 + 2], t[r][e0 + 3]};
  }
  __syncthreads();
  if (live && u < 4) {  // pass 2: u = row r
    const int tx = (int)(tile % TW), ty = (int)((tile / TW) % TH), n = (int)(tile / ((long long)TW * TH));
    const int oy = ty * 4 + u;
    if (oy < a.OH) {
      T* out = static_cast<T*>(a.out);
      const T* res = static_cast<const T*>(a.residual);
      const int f = f0 + cg * VW;
      float y[4][VW];
#pragma unroll
      for (int e0 = 0; e0 < VW; e0 += 4) {
        wf4 rj[6];
#pragma unroll
        for (int j = 0; j < 6; ++j) rj[j] = *reinterpret_cast<const wf4*>(&mid[tl][u][j][cg * VW + e0]);
#pragma unroll
        for (int e1 = 0; e1 < 4; ++e1) {
          const int e = e0 + e1;
          float row[6], o[4];
#pragma unroll
          for (int j = 0; j < 6; ++j) row[j] = rj[j][e1];
          at6(row, o);
          const float sc = a.scale ? a.scale[f + e] : 1.0f, sh = a.shift ? a.shift[f + e] : 0.0f;
#pragma unroll
          for (int q = 0; q < 4; ++q) y[q][e] = o[q] * sc + sh;
        }
      }
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int ox = tx * 4 + q;
        if (ox >= a.OW) continue;
        const long long o = (((long long)n * a.OH + oy) * a.OW + ox) * a.F + f;
        if (res) {
          const Vec rv = *reinterpret_cast<const Vec*>(res + o);
#pragma unroll
          for (int e = 0; e < VW; ++e) y[q][e] += (float)rv[e];
        }
        if (a.accumulate) {
          const Vec ov = *reinterpret_cast<const Vec*>(out + o);
#pragma unroll
          for (int e = 0; e < VW; ++e) y[q][e] += (float)ov[e];
        }
        Vec w;
#pragma unroll
        for (int e = 0; e < VW; ++e) w[e] = (T)(a.relu ? relu_ugt(y[q][e]) : y[q][e]);
        *reinterpret_cast<Vec*>(out + o) = w;
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------
// launchers
// ---------------------------------------------------------------------------------------------
void launch_wino43_filter(const void* w, int w_dt, void* U, int u_dt, int F, int C, hipStream_t s) {
  const int n = F * C, blk = 256, grid = (n + blk - 1) / blk;
  if (w_dt == kF32 && u_dt == kF32)
    hipLaunchKernelGGL((wino43_filter_kernel<float, float>), dim3(grid), dim3(blk), 0, s, (const float*)w, (float*)U, F, C);
  else if (w_dt == kF16 && u_dt == kF16)
    hipLaunchKernelGGL((wino43_filter_kernel<half_t, half_t>), dim3(grid), dim3(blk), 0, s, (const half_t*)w, (half_t*)U, F, C);
  else if (w_dt == kF32 && u_dt == kF16)
    hipLaunchKernelGGL((wino43_filter_kernel<float, half_t>), dim3(grid), dim3(blk), 0, s, (const float*)w, (half_t*)U, F, C);
  else
    fail("wino43_filter: unsupported dtype combination");
  NNCV_HIP_CHECK(hipGetLastError());
}

void launch_wino43_input(const void* in, int in_dt, Strides4 st, void* V, int v_dt, int N, int C, int H, int W, int pad,
                         hipStream_t s) {
  NNCV_REQUIRE(C % 2 == 0, "wino43_input: C must be even");
  const int OH = H + 2 * pad - 2, OW = W + 2 * pad - 2;
  NNCV_REQUIRE(OH >= 1 && OW >= 1, "wino43_input: empty output");
  const int TH = (OH + 3) / 4, TW = (OW + 3) / 4;
  const long long work = (long long)N * TH * TW * (C / 2);
  const int blk = 256;
  const long long grid = (work + blk - 1) / blk;
  NNCV_REQUIRE(grid < (1ll << 31), "wino43_input: grid too large");
  const bool contig = st.c == 1;
  const double es = dtype_size(in_dt), vs = dtype_size(v_dt);
  ProfScope prof(contig ? "wino43_input<nhwc>" : "wino43_input<strided>", 0.0,
                 es * N * C * H * W + vs * 36.0 * N * TH * TW * C, s);
  // dense NHWC with whole 64-channel groups: the LDS-staged kernel
  if (contig && in_dt == v_dt && C % 64 == 0 && st.w == C && st.h == (long long)W * C && st.n == (long long)H * W * C &&
      getenv("NNCV_HIP_WINO_SIMPLE") == nullptr) {
    const long long tiles = (long long)N * TH * TW;
    if (in_dt == kF16) {
      dim3 g((unsigned)(((tiles + WinoLds<half_t>::kTiles - 1) / WinoLds<half_t>::kTiles + 7) / 8 * 8), C / 64);
      hipLaunchKernelGGL((wino43_input_lds_kernel<half_t>), g, dim3(256), 0, s, (const half_t*)in, (half_t*)V, N, C, H, W, pad, TH, TW);
    } else {
      dim3 g((unsigned)(((tiles + WinoLds<float>::kTiles - 1) / WinoLds<float>::kTiles + 7) / 8 * 8), C / 64);
      hipLaunchKernelGGL((wino43_input_lds_kernel<float>), g, dim3(256), 0, s, (const float*)in, (float*)V, N, C, H, W, pad, TH, TW);
    }
    NNCV_HIP_CHECK(hipGetLastError());
    return;
  }
#define LAUNCH(TI, TV, CC)                                                                               \
  hipLaunchKernelGGL((wino43_input_kernel<TI, TV, CC>), dim3((unsigned)grid), dim3(blk), 0, s, (const TI*)in, st, \
                     (TV*)V, N, C, H, W, pad, TH, TW)
  if (in_dt == kF32 && v_dt == kF32) { if (contig) LAUNCH(float, float, true); else LAUNCH(float, float, false); }
  else if (in_dt == kF16 && v_dt == kF16) { if (contig) LAUNCH(half_t, half_t, true); else LAUNCH(half_t, half_t, false); }
  else fail("wino43_input: unsupported dtype combination");
#undef LAUNCH
  NNCV_HIP_CHECK(hipGetLastError());
}

void launch_wino43_output(const WinoOutArgs& a, int m_dt, int out_dt, hipStream_t s) {
  NNCV_REQUIRE(a.F % 2 == 0, "wino43_output: F must be even");
  const int TH = (a.OH + 3) / 4, TW = (a.OW + 3) / 4;
  const long long work = (long long)a.N * TH * TW * (a.F / 2);
  const int blk = 256;
  const long long grid = (work + blk - 1) / blk;
  NNCV_REQUIRE(grid < (1ll << 31), "wino43_output: grid too large");
  const bool contig = a.st.c == 1;
  const double ms = dtype_size(m_dt), os = dtype_size(out_dt);
  ProfScope prof(contig ? "wino43_output<nhwc>" : "wino43_output<strided>", 0.0,
                 ms * 36.0 * a.N * TH * TW * a.F + os * (double)a.N * a.F * a.OH * a.OW * (a.residual ? 2 : 1), s);
  if (contig && m_dt == out_dt && a.F % 64 == 0 && a.st.w == a.F && a.st.h == (long long)a.OW * a.F &&
      a.st.n == (long long)a.OH * a.OW * a.F && getenv("NNCV_HIP_WINO_SIMPLE") == nullptr) {
    const long long tiles = (long long)a.N * TH * TW;
    if (m_dt == kF16) {
      dim3 g((unsigned)((tiles + WinoLds<half_t>::kTiles - 1) / WinoLds<half_t>::kTiles), a.F / 64);
      hipLaunchKernelGGL((wino43_output_lds_kernel<half_t>), g, dim3(256), 0, s, a, TH, TW);
    } else {
      dim3 g((unsigned)((tiles + WinoLds<float>::kTiles - 1) / WinoLds<float>::kTiles), a.F / 64);
      hipLaunchKernelGGL((wino43_output_lds_kernel<float>), g, dim3(256), 0, s, a, TH, TW);
    }
    NNCV_HIP_CHECK(hipGetLastError());
    return;
  }
#define LAUNCH(TM, TO, CC) \
  hipLaunchKernelGGL((wino43_output_kernel<TM, TO, CC>), dim3((unsigned)grid), dim3(blk), 0, s, a, TH, TW)
  if (m_dt == kF32 && out_dt == kF32) { if (contig) LAUNCH(float, float, true); else LAUNCH(float, float, false); }
  else if (m_dt == kF16 && out_dt == kF16) { if (contig) LAUNCH(half_t, half_t, true); else LAUNCH(half_t, half_t, false); }
  else if (m_dt == kF32 && out_dt == kF16) { if (contig) LAUNCH(float, half_t, true); else LAUNCH(float, half_t, false); }
  else fail("wino43_output: unsupported dtype combination");
#undef LAUNCH
  NNCV_HIP_CHECK(hipGetLastError());
}

}  // namespace nncv_hip
