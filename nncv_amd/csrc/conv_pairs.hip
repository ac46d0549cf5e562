// Image convolution over pixel pairs: the stride-2 first layer of a network whose input has at most
// four channels, once the graph executor has packed the image as [N][H][W/2][2 pixels x 4 channels]
// (fp16).  The horizontal walk is then stride 1 over S pairs, every filter tap is one 16-byte chunk
// and the whole K axis is R*S chunks, 18 for YOLOv5s' 6x6 window, 6 for MobileNetV3's 3x3.
// Replaces the compiler's tiling of linalg.conv_2d_nchw_fchw for those layers
// (src/nncv/compiler/Conversion/CodeGen/LlvmCpu/ModernTile.cpp:124-286; the layers are
// tests/Nets/Yolov5s.mlir's and tests/Nets/MobileNetV3.mlir's first convolutions).
//
// K is so short that a pipelined K walk only adds barriers: a workgroup (4 waves, 256 pixels, one
// pixel per thread) requests ALL chunks of its pixels at once (one latency, consecutive lanes read
// consecutive pairs), parks them in LDS as [pixel][chunk] rows (an odd number of 16-byte cells per
// row: conflict-free 16-byte reads), holds its 32 or 64 filters in registers, issues R*S/2 MFMA
// steps per wave and leaves through the coalescing epilogue shared with the other convolution
// kernels (scale/shift, residual, activation, whole rows stored).  HBM bound: the packed image is
// read once (window overlap is served by the caches) and the result written once.
#include "mfma_tile.hpp"

namespace nncv_hip {

using namespace mt;

namespace {
constexpr unsigned kOOBc = 0x7fff0000u;  // byte offset beyond any buffer this kernel accepts
}

template <int R, int S, int NI>
__global__ __launch_bounds__(256) void conv_pairs_kernel(const IgemmArgs a) {
  constexpr int NCH = R * S, KST = NCH / 2, PITCH = (NCH + 1) * 16;
  static_assert(NCH % 2 == 0, "an MFMA step takes two chunks");
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lrow = lane & 31, lchunk = lane >> 5;
  const int P = a.N * a.OH * a.OW;
  const int f0 = blockIdx.y * (32 * NI);
  const __amdgpu_buffer_rsrc_t rs_in = make_rsrc(a.in, a.in_bytes);
  const __amdgpu_buffer_rsrc_t rs_wt = make_rsrc(a.wt, a.wt_bytes);

  // ---- this thread's pixel: all of its taps requested back to back ----
  const int p = blockIdx.x * 256 + tid;
  const int ohow = a.OH * a.OW;
  const int n = p / ohow, rem = p - n * ohow;
  const int oy = rem / a.OW, ox = rem - oy * a.OW;
  const int iy0 = oy * a.stride_h - a.pad_h, ix0 = ox * a.stride_w - a.pad_w;
  const int base = (n * a.H + iy0) * a.W + ix0;  // in pairs; may be negative, only used when in bounds
  u32x4 v[NCH];
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int s = 0; s < S; ++s) {
      const bool ok = (p < P) & ((unsigned)(iy0 + r) < (unsigned)a.H) & ((unsigned)(ix0 + s) < (unsigned)a.W);
      v[r * S + s] = __builtin_amdgcn_raw_buffer_load_b128(rs_in, ok ? (unsigned)(base + r * a.W + s) * 16u : kOOBc, 0, 0);
    }
  // ---- the filters: row f is R*S chunks; lane (filter lrow, chunk half lchunk) of step kk holds
  //      chunk 2*kk + lchunk.  Rows past the tensor read as zero. ----
  u32x4 w[KST][NI];
#pragma unroll
  for (int kk = 0; kk < KST; ++kk)
#pragma unroll
    for (int i = 0; i < NI; ++i)
      w[kk][i] = __builtin_amdgcn_raw_buffer_load_b128(rs_wt, (unsigned)(((f0 + i * 32 + lrow) * NCH + 2 * kk + lchunk) * 16), 0, 0);
  EpiScale<half_t> ess;
  ess.load(lane, f0, a.F, a.scale, a.shift);

#pragma unroll
  for (int c = 0; c < NCH; ++c) *reinterpret_cast<u32x4*>(smem + tid * PITCH + c * 16) = v[c];
  __syncthreads();

  floatx16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;
  const unsigned char* mine = smem + (wave * 64 + lrow) * PITCH + lchunk * 16;
#pragma unroll
  for (int kk = 0; kk < KST; ++kk) {
    u32x4 b[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) b[j] = *reinterpret_cast<const u32x4*>(mine + j * 32 * PITCH + kk * 32);
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) Mma<half_t>::run(w[kk][i], b[j], acc[i][j]);
  }
  __syncthreads();  // every wave is done with the pixel rows: LDS becomes the output tiles

  int rowoff[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int pj = blockIdx.x * 256 + wave * 64 + j * 32 + lrow;
    rowoff[j] = pj < P ? pj * a.ldo : -1;
  }
  tile_reduce_store<half_t, 1, NI, true>(acc, smem + wave * kTileBytes, 0, lane, rowoff, f0, a.F, ess,
                                         static_cast<const half_t*>(a.residual), static_cast<half_t*>(a.out), a.relu);
}

template <int R, int S>
static constexpr int pairs_smem() {
  return 256 * (R * S + 1) * 16 > 4 * kTileBytes ? 256 * (R * S + 1) * 16 : 4 * kTileBytes;
}

bool conv_pairs_applicable(const IgemmArgs& a, int in_dt, int out_dt) {
  static const bool off = getenv("NNCV_HIP_NO_CONV_PAIRS") != nullptr;
  const bool window = (a.R == 6 && a.S == 3) || (a.R == 3 && a.S == 2);
  const long long P = (long long)a.N * a.OH * a.OW;
  return !off && in_dt == kF16 && out_dt == kF16 && window && a.C == 8 && (a.pix_stride == 0 || a.pix_stride == 8) && a.batch == 1 &&
         a.aux_f0 == 0 && a.F % 8 == 0 && a.F <= 64 && a.ldo % 8 == 0 && a.ldo >= a.F && P * a.ldo < (1ll << 31) &&
         (long long)a.N * a.H * a.W * 16 < (long long)kOOBc && a.in_bytes > 0 && a.in_bytes < kOOBc && a.wt_bytes > 0;
}

template <int R, int S, int NI>
static void launch_pairs_cfg(const IgemmArgs& a, const char* tag, hipStream_t s) {
  auto kern = conv_pairs_kernel<R, S, NI>;
  constexpr int smem = pairs_smem<R, S>();
  static const bool once = [&] {
    NNCV_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, smem));
    return true;
  }();
  (void)once;
  const long long P = (long long)a.N * a.OH * a.OW;
  const double flops = a.alg_flops > 0 ? a.alg_flops : 2.0 * P * a.F * R * S * 8.0;
  const double bytes = 2.0 * ((double)a.N * a.H * a.W * 8 + (double)a.F * R * S * 8 + (double)P * a.F * (a.residual ? 2 : 1));
  ProfScope prof(tag, flops, bytes, s);
  dim3 grid((unsigned)((P + 255) / 256), (unsigned)((a.F + 32 * NI - 1) / (32 * NI)));
  hipLaunchKernelGGL(kern, grid, dim3(256), smem, s, a);
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
