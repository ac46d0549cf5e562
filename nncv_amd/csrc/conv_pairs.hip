// Convolutions whose whole K axis is a handful of 16-byte chunks (fp16), in two forms:
//  * the stride-2 first layer of a network whose input has at most four channels, once the graph
//    executor has packed the image as [N][H][W/2][2 pixels x 4 channels]: the horizontal walk is
//    stride 1 over S pairs, every filter tap is one chunk and K is R*S chunks, 18 for YOLOv5s'
//    6x6 window, 6 for MobileNetV3's 3x3 (tests/Nets/Yolov5s.mlir, tests/Nets/MobileNetV3.mlir);
//  * 1x1 convolutions over at most 144 channels in multiples of 8 (MobileNetV3's expansion and
//    projection layers, 16..144 channels: none of them a multiple of the 64-byte K step of the
//    pipelined kernel), with the residual add of an inverted-residual block.
// Replaces the compiler's tiling of linalg.conv_2d_nchw_fchw for those layers
// (src/nncv/compiler/Conversion/CodeGen/LlvmCpu/ModernTile.cpp:124-286).
//
// K is so short that a pipelined K walk through LDS only adds barriers.  A wave owns 64 pixels x 32
// or 64 filters and needs no staging at all: lane (pixel l%32, chunk half l/32) of MFMA step kk reads
// chunk 2*kk + l/32 of its pixel straight from global memory, ALL steps requested back to back (one
// latency), the filters sit in registers.  The epilogue (scale/shift, residual, activation, one
// rounding) runs on the accumulators; the halves pass through a small LDS tile only to leave as
// whole pixel rows, 16 bytes per lane.  With 5-10 KB of LDS per wave tile the kernel runs at the
// occupancy its registers allow.  HBM bound: input read once (window overlap and the re-reads of
// further filter blocks are served by the caches), result written once.
#include "mfma_tile.hpp"

namespace nncv_hip {

using namespace mt;

namespace {
constexpr unsigned kOOBc = 0x7fff0000u;  // byte offset beyond any buffer this kernel accepts
}

// PW = false: R x S window over pixel pairs (C = 8), KST = R*S/2.
// PW = true : 1x1 window over C = 8*nch channels, nch <= 2*KST chunks (chunks past nch read as zero).
// WV waves per workgroup, 64 pixels each (1 for small launches: more, smaller workgroups).
// RES: the launch has a residual input (instances without one carry no registers or code for it).
template <bool PW, int R, int S, int KST, int NI, int WV, bool RES>
__global__ __launch_bounds__(64 * WV) void conv_pairs_kernel(const IgemmArgs a) {
  constexpr int TP = 64 * NI + 16;  // bytes per pixel row of the output tile: 32*NI halves + pad
  static_assert(PW || R * S == 2 * KST, "an MFMA step takes two chunks");
  __shared__ __align__(16) unsigned char smem[WV * 64 * TP];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lrow = lane & 31, lchunk = lane >> 5;
  const int P = a.N * a.OH * a.OW;
  const int f0 = blockIdx.y * (32 * NI);
  const int p0 = blockIdx.x * (64 * WV) + wave * 64;
  const int nch = PW ? a.C / 8 : R * S;  // chunks per pixel = chunks per filter row
  const __amdgpu_buffer_rsrc_t rs_in = make_rsrc(a.in, a.in_bytes);
  const __amdgpu_buffer_rsrc_t rs_wt = make_rsrc(a.wt, a.wt_bytes);

  // ---- this lane's two pixels and its chunk of every step, requested back to back ----
  u32x4 b[KST][2];
  if constexpr (PW) {
    const int pix = a.pix_stride ? a.pix_stride : a.C;
#pragma unroll
    for (int kk = 0; kk < KST; ++kk) {
      const int c = 2 * kk + lchunk;
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int p = p0 + j * 32 + lrow;
        const bool ok = (p < P) & (c < nch);
        b[kk][j] = __builtin_amdgcn_raw_buffer_load_b128(rs_in, ok ? (unsigned)(p * pix + c * 8) * 2u : kOOBc, 0, 0);
      }
    }
  } else {
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
#pragma unroll
    for (int kk = 0; kk < KST; ++kk) {
      const int c = 2 * kk + lchunk, r = c / S, s = c - r * S;
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const bool ok = ((unsigned)(iy0[j] + r) < (unsigned)a.H) & ((unsigned)(ix0[j] + s) < (unsigned)a.W);
        b[kk][j] = __builtin_amdgcn_raw_buffer_load_b128(rs_in, ok ? (unsigned)(base[j] + r * a.W + s) * 16u : kOOBc, 0, 0);
      }
    }
  }
  // ---- the filters: row f is nch chunks; lane (filter l%32, chunk half l/32) of step kk holds
  //      chunk 2*kk + l/32.  Rows past the tensor read as zero. ----
  u32x4 w[KST][NI];
#pragma unroll
  for (int kk = 0; kk < KST; ++kk)
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int c = 2 * kk + lchunk;
      w[kk][i] = __builtin_amdgcn_raw_buffer_load_b128(rs_wt, c < nch ? (unsigned)(((f0 + i * 32 + lrow) * nch + c) * 16) : kOOBc, 0, 0);
    }
  // scale/shift of this lane's accumulator channels f0 + 32 i + 8 q + 4 (l/32) .. + 3, and the
  // residual values at the same places (element offsets; rows past the end read element 0)
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
  const half_t* res = static_cast<const half_t*>(a.residual);
  half4 rv[NI][2][4];
  if constexpr (RES) {
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int p = p0 + j * 32 + lrow, f = f0 + i * 32 + 8 * q + 4 * lchunk;
          const long long off = (p < P && f < a.F) ? (long long)p * a.ldo + f : 0;
          rv[i][j][q] = *reinterpret_cast<const half4*>(res + off);
        }
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
  const bool res_after = a.relu & kActResidualAfter;  // y = act(conv) + residual instead of act(conv + residual)
#pragma unroll
  for (int i = 0; i < NI; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        float y[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) y[e] = acc[i][j][4 * q + e] * sc[i][q][e] + sh[i][q][e];
        if (RES && !res_after) {
#pragma unroll
          for (int e = 0; e < 4; ++e) y[e] += (float)rv[i][j][q][e];
        }
        act_apply_n<true>(y, act);
        if (RES && res_after) {
#pragma unroll
          for (int e = 0; e < 4; ++e) y[e] += (float)rv[i][j][q][e];
        }
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
  static const bool off_pw = getenv("NNCV_HIP_NO_CONV_SHORTK") != nullptr;
  const int pix = a.pix_stride ? a.pix_stride : a.C;
  const long long P = (long long)a.N * a.OH * a.OW;
  const bool common = in_dt == kF16 && out_dt == kF16 && a.batch == 1 && a.aux_f0 == 0 && a.F % 8 == 0 && a.ldo % 8 == 0 && a.ldo >= a.F &&
                      P * a.ldo < (1ll << 31) && a.in_bytes > 0 && a.in_bytes < kOOBc && a.wt_bytes > 0 && a.wt_bytes < kOOBc &&
                      (a.relu & ~(0xff | kActResidualAfter)) == 0;
  if (!common) return false;
  const bool window = (a.R == 6 && a.S == 3) || (a.R == 3 && a.S == 2);
  if (window)
    return !off && a.C == 8 && pix == 8 && a.F <= 64 && a.residual == nullptr && (a.relu & ~0xff) == 0 &&
           (long long)a.N * a.H * a.W * 16 < (long long)kOOBc;
  // 1x1, stride 1, no padding: the output pixel is the input pixel.  Channel counts that the pipelined
  // kernel takes as well (multiples of 32) come here only for small launches, where its barriers per K
  // step are all latency (MobileNetV3's 96-channel layers at 14x14 and 7x7: 0.449 -> 0.444 ms per
  // batch of 32); on YOLOv5s' large 1x1 layers it is the faster one (1.27 against 1.32 ms).
  return !off_pw && a.R == 1 && a.S == 1 && a.stride_h == 1 && a.stride_w == 1 && a.pad_h == 0 && a.pad_w == 0 && a.OH == a.H &&
         a.OW == a.W && a.C % 8 == 0 && (a.C % 32 != 0 || P <= 8192) && a.C <= 144 && pix % 8 == 0 && P * pix * 2 < (long long)kOOBc;
}

template <bool PW, int R, int S, int KST, int NI>
static void launch_pairs_cfg(const IgemmArgs& a, const char* tag, hipStream_t s) {
  const long long P = (long long)a.N * a.OH * a.OW;
  const double flops = a.alg_flops > 0 ? a.alg_flops : 2.0 * P * a.F * a.R * a.S * a.C;
  const double bytes = 2.0 * ((double)a.N * a.H * a.W * a.C + (double)a.F * a.R * a.S * a.C + (double)P * a.F * (a.residual ? 2 : 1));
  ProfScope prof(tag, flops, bytes, s);
  const unsigned gy = (unsigned)((a.F + 32 * NI - 1) / (32 * NI));
  // fewer four-wave workgroups than CUs: one wave per workgroup instead
  const bool small = (P + 255) / 256 * gy < 256;
  const dim3 grid(small ? (unsigned)((P + 63) / 64) : (unsigned)((P + 255) / 256), gy), block(small ? 64 : 256);
  if constexpr (PW) {
    if (a.residual && small) hipLaunchKernelGGL((conv_pairs_kernel<PW, R, S, KST, NI, 1, true>), grid, block, 0, s, a);
    else if (a.residual) hipLaunchKernelGGL((conv_pairs_kernel<PW, R, S, KST, NI, 4, true>), grid, block, 0, s, a);
    else if (small) hipLaunchKernelGGL((conv_pairs_kernel<PW, R, S, KST, NI, 1, false>), grid, block, 0, s, a);
    else hipLaunchKernelGGL((conv_pairs_kernel<PW, R, S, KST, NI, 4, false>), grid, block, 0, s, a);
  } else {  // the image layers have no residual input (conv_pairs_applicable)
    if (small) hipLaunchKernelGGL((conv_pairs_kernel<PW, R, S, KST, NI, 1, false>), grid, block, 0, s, a);
    else hipLaunchKernelGGL((conv_pairs_kernel<PW, R, S, KST, NI, 4, false>), grid, block, 0, s, a);
  }
}

void launch_conv_pairs(const IgemmArgs& a, hipStream_t s) {
  if (a.R == 6) {
    if (a.F > 32) launch_pairs_cfg<false, 6, 3, 9, 2>(a, "conv_pairs<f16,6x3,64>", s);
    else launch_pairs_cfg<false, 6, 3, 9, 1>(a, "conv_pairs<f16,6x3,32>", s);
  } else if (a.R == 3) {
    if (a.F > 32) launch_pairs_cfg<false, 3, 2, 3, 2>(a, "conv_pairs<f16,3x2,64>", s);
    else launch_pairs_cfg<false, 3, 2, 3, 1>(a, "conv_pairs<f16,3x2,32>", s);
  } else {
    // K steps in registers: 1 (16 channels), 3 (..48), 6 (..96), 9 (..144); 64 filters per wave tile
    // while the registers allow it
    const int kst = (a.C / 8 + 1) / 2;
    if (kst <= 1) {
      if (a.F > 32) launch_pairs_cfg<true, 1, 1, 1, 2>(a, "conv1x1_shortk<f16,16,64>", s);
      else launch_pairs_cfg<true, 1, 1, 1, 1>(a, "conv1x1_shortk<f16,16,32>", s);
    } else if (kst <= 3) {
      if (a.F > 32) launch_pairs_cfg<true, 1, 1, 3, 2>(a, "conv1x1_shortk<f16,48,64>", s);
      else launch_pairs_cfg<true, 1, 1, 3, 1>(a, "conv1x1_shortk<f16,48,32>", s);
    } else if (kst <= 6) {
      launch_pairs_cfg<true, 1, 1, 6, 1>(a, "conv1x1_shortk<f16,96,32>", s);
    } else {
      launch_pairs_cfg<true, 1, 1, 9, 1>(a, "conv1x1_shortk<f16,144,32>", s);
    }
  }
  NNCV_HIP_CHECK(hipGetLastError());
}

}  // namespace nncv_hip
