// Image convolution over pixel pairs: the stride-2 first layer of a network whose input has at most
// four channels, once the graph executor has packed the image as [N][H][W/2][2 pixels x 4 channels]
// (fp16).  The horizontal walk is then stride 1 over S pairs, every filter tap is one 16-byte chunk
// and the whole K axis is R*S chunks, 18 for YOLOv5s' 6x6 window, 6 for MobileNetV3's 3x3.
// Replaces the compiler's tiling of linalg.conv_2d_nchw_fchw for those layers
// (src/nncv/compiler/Conversion/CodeGen/LlvmCpu/ModernTile.cpp:124-286; the layers are
// tests/Nets/Yolov5s.mlir's and tests/Nets/MobileNetV3.mlir's first convolutions).
//
// K is so short that a pipelined K walk through LDS only adds barriers.  A wave owns 64 pixels x 32
// or 64 filters and needs no staging at all: lane (pixel l%32, chunk half l/32) of MFMA step kk reads
// chunk 2*kk + l/32 of its pixel straight from global memory (half a wave reads 32 consecutive
// pairs = 512 contiguous bytes), ALL steps requested back to back (one latency), the filters sit in
// registers.  The epilogue (scale/shift, activation, one rounding) runs on the accumulators; the
// halves pass through a small LDS tile only to leave as whole pixel rows, 16 bytes per lane.  With
// 5-10 KB of LDS per wave tile the kernel runs at the occupancy its registers allow.  HBM bound:
// the packed image is read once (window overlap is served by the caches), the result written once.
#include "mfma_tile.hpp"

namespace nncv_hip {

using namespace mt;

namespace {
constexpr unsigned kOOBc = 0x7fff0000u;  // byte offset beyond any buffer this kernel accepts
}

template <int R, int S, int NI>
__global__ __launch_bounds__(256) void conv_pairs_kernel(const IgemmArgs a) {
  constexpr int NCH = R * S, KST = NCH / 2;
  constexpr int TP = 64 * NI + 16;  // bytes per pixel row of the output tile: 32*NI halves + pad
  static_assert(NCH % 2 == 0, "an MFMA step takes two chunks");
  __shared__ __align__(16) unsigned char smem[4 * 64 * TP];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lrow = lane & 31, lchunk = lane >> 5;
  const int P = a.N * a.OH * a.OW;
  const int f0 = blockIdx.y * (32 * NI);
  const int p0 = blockIdx.x * 256 + wave * 64;
  const __amdgpu_buffer_rsrc_t rs_in = make_rsrc(a.in, a.in_bytes);
  const __amdgpu_buffer_rsrc_t rs_wt = make_rsrc(a.wt, a.wt_bytes);

  // ---- this lane's two pixels and its chunk of every step, requested back to back ----
  int base[2], iy0[2], ix0[2];
  const int ohow = a.OH * a.OW;
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int p = p0 + j * 32 + lrow;
    const int n = p / ohow, rem = p - n * ohow;
    const int oy = rem / a.OW, ox = rem - oy * a.OW;
    iy0[j] = p < P ? oy * a.stride_h - a.pad_h : -(1 << 28);  // pixels past the end: never inside the image
    ix0[j] = ox * a.stride_w - a.pad_w;
    base[j] = (n * a.H + iy0[j]) * a.W + ix0[j];  // in pairs; only used when the tap is in bounds
  }
  u32x4 b[KST][2];
#pragma unroll
  for (int kk = 0; kk < KST; ++kk) {
    const int c = 2 * kk + lchunk, r = c / S, s = c - r * S;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const bool ok = ((unsigned)(iy0[j] + r) < (unsigned)a.H) & ((unsigned)(ix0[j] + s) < (unsigned)a.W);
      b[kk][j] = __builtin_amdgcn_raw_buffer_load_b128(rs_in, ok ? (unsigned)(base[j] + r * a.W + s) * 16u : kOOBc, 0, 0);
    }
  }
  // ---- the filters: row f is R*S chunks; lane (filter l%32, chunk half l/32) of step kk holds
  //      chunk 2*kk + l/32.  Rows past the tensor read as zero. ----
  u32x4 w[KST][NI];
#pragma unroll
  for (int kk = 0; kk < KST; ++kk)
#pragma unroll
    for (int i = 0; i < NI; ++i)
      w[kk][i] = __builtin_amdgcn_raw_buffer_load_b128(rs_wt, (unsigned)(((f0 + i * 32 + lrow) * NCH + 2 * kk + lchunk) * 16), 0, 0);
  // scale/shift of this lane's accumulator channels f0 + 32 i + 8 q + 4 (l/32) .. + 3
  floatx4 sc[NI][4], sh[NI][4];
#pragma unroll
  for (int i = 0; i < NI; ++i)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int f = f0 + i * 32 + 8 * q + 4 * lchunk;
      const bool fin = f < a.F;
      sc[i][q] = (a.scale && fin) ? *reinterpret_cast<const floatx4*>(a.scale + f) : floatx4{1.f, 1.f, 1.f, 1.f};
      sh[i][q] = (a.shift && fin) ? *reinterpret_cast<const floatx4*>(a.shift + f) : floatx4{0.f, 0.f, 0.f, 0.f};
    }

  floatx16 acc[NI][2];
#pragma unroll
  for (int i = 0; i < NI; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;
#pragma unroll
  for (int kk = 0; kk < KST; ++kk)
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) Mma<half_t>::run(w[kk][i], b[kk][j], acc[i][j]);

  // ---- epilogue on the accumulators, halves to this wave's tile [pixel][channel] ----
  unsigned char* tile = smem + wave * (64 * TP);
  const int act = a.relu & 0xff;
#pragma unroll
  for (int i = 0; i < NI; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        float y[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) y[e] = acc[i][j][4 * q + e] * sc[i][q][e] + sh[i][q][e];
        act_apply_n<true>(y, act);
        half4 h;
#pragma unroll
        for (int e = 0; e < 4; ++e) h[e] = (half_t)y[e];
        *reinterpret_cast<half4*>(tile + (j * 32 + lrow) * TP + (i * 32 + 8 * q + 4 * lchunk) * 2) = h;
      }
  __syncthreads();
  // ---- whole pixel rows out: 4*NI lanes cover the 32*NI channels of one pixel ----
  constexpr int LPR = 4 * NI, RPI = 64 / LPR;
  const int fc = (lane % LPR) * 8;
  half_t* out = static_cast<half_t*>(a.out);
#pragma unroll
  for (int it = 0; it < 64 / RPI; ++it) {
    const int row = it * RPI + lane / LPR;
    const u32x4 v = *reinterpret_cast<const u32x4*>(tile + row * TP + fc * 2);
    if (p0 + row < P && f0 + fc < a.F) *reinterpret_cast<u32x4*>(out + (long long)(p0 + row) * a.ldo + f0 + fc) = v;
  }
}

bool conv_pairs_applicable(const IgemmArgs& a, int in_dt, int out_dt) {
  static const bool off = getenv("NNCV_HIP_NO_CONV_PAIRS") != nullptr;
  const bool window = (a.R == 6 && a.S == 3) || (a.R == 3 && a.S == 2);
  const long long P = (long long)a.N * a.OH * a.OW;
  return !off && in_dt == kF16 && out_dt == kF16 && window && a.C == 8 && (a.pix_stride == 0 || a.pix_stride == 8) && a.batch == 1 &&
         a.aux_f0 == 0 && a.residual == nullptr && (a.relu & ~0xff) == 0 && a.F % 8 == 0 && a.F <= 64 && a.ldo % 8 == 0 && a.ldo >= a.F && P * a.ldo < (1ll << 31) &&
         (long long)a.N * a.H * a.W * 16 < (long long)kOOBc && a.in_bytes > 0 && a.in_bytes < kOOBc && a.wt_bytes > 0;
}

template <int R, int S, int NI>
static void launch_pairs_cfg(const IgemmArgs& a, const char* tag, hipStream_t s) {
  auto kern = conv_pairs_kernel<R, S, NI>;
  const long long P = (long long)a.N * a.OH * a.OW;
  const double flops = a.alg_flops > 0 ? a.alg_flops : 2.0 * P * a.F * R * S * 8.0;
  const double bytes = 2.0 * ((double)a.N * a.H * a.W * 8 + (double)a.F * R * S * 8 + (double)P * a.F * (a.residual ? 2 : 1));
  ProfScope prof(tag, flops, bytes, s);
  dim3 grid((unsigned)((P + 255) / 256), (unsigned)((a.F + 32 * NI - 1) / (32 * NI)));
  hipLaunchKernelGGL(kern, grid, dim3(256), 0, s, a);
}

void launch_conv_pairs(const IgemmArgs& a, hipStream_t s) {
  if (a.R == 6) {
    if (a.F > 32) launch_pairs_cfg<6, 3, 2>(a, "conv_pairs<f16,6x3,64>", s);
    else launch_pairs_cfg<6, 3, 1>(a, "conv_pairs<f16,6x3,32>", s);
  } else {
    if (a.F > 32) launch_pairs_cfg<3, 2, 2>(a, "conv_pairs<f16,3x2,64>", s);
    else launch_pairs_cfg<3, 2, 1>(a, "conv_pairs<f16,3x2,32>", s);
  }
  NNCV_HIP_CHECK(hipGetLastError());
}

}  // namespace nncv_hip
