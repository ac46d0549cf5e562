// 3x3 stride-1 pad-1 convolution with the haloed input patch resident in LDS (gfx950).
//
// The implicit-GEMM kernels gather every input pixel once per filter tap, i.e. nine times, from
// L2.  Here a workgroup owns an output tile of TN images x TH rows x the full width W (at most
// 64*WS pixel "slots") and 64 filters, and per 128-byte channel slab (64 halves / 32 floats):
//   * loads the (TH+2) x (W+2) haloed input patch ONCE into LDS (zero halo straight from the
//     buffer-load range check; the reference materialises it with tensor.pad,
//     tests/Nets/Res18.mlir:152-155),
//   * walks the nine taps; a tap is a constant byte offset into the patch, so the MFMA pixel
//     operand of tap (r,s) is read from the same LDS data at  slot_base + (r*(W+2)+s)*pitch,
//   * streams the tap's 64x128-byte weight slice through a double-buffered LDS tile.
// Input traffic from L2 drops from 9x to (TH+2)/TH x, LDS writes per MFMA by ~5x.
//
// Wave layout WS x WK: WS waves each own 64 slots x 64 filters (2x2 accumulators of
// v_mfma_f32_32x32x16_f16; fp32: 4x v_mfma_f32_32x32x2_f32 per chunk pair), and WK "K groups"
// split the four 32-byte K sub-steps of every tap between them (their partial sums meet in LDS
// at the end).  Splitting K inside the workgroup rather than shrinking the pixel tile keeps one
// 16-byte LDS read per MFMA while giving every SIMD two resident waves whose LDS latencies and
// MFMAs overlap, and lets small feature maps (14x14, 7x7) still fill 256 CUs:
//   56x56, 28x28 -> WS=4, WK=2 ; 14x14 -> WS=2, WK=4 ; 7x7 -> WS=1, WK=4.
// Weights are the MFMA "A" rows so a lane ends up with 4 consecutive channels of one pixel; the
// epilogue (scale/shift, residual, ReLU) goes through LDS for whole-row stores (mfma_tile.hpp).
// LDS pixel pitch is 128 + 16 bytes: consecutive pixels land 36 banks apart.
#include "mfma_tile.hpp"

namespace nncv_hip {

using namespace mt;

namespace {
constexpr int kPitch = 144;            // LDS bytes per pixel / per filter row: 128 payload + 16 pad
constexpr int kWBytes = 64 * kPitch;   // one weight buffer: 64 filters x 128 B
constexpr unsigned kOOBp = 0x7fff0000u;
constexpr int kXcdsP = 8;

template <int WS> struct PatchCap;  // patch capacity in pixels for 64*WS slots
template <> struct PatchCap<4> { static constexpr int pix = 384; };
template <> struct PatchCap<2> { static constexpr int pix = 256; };
template <> struct PatchCap<1> { static constexpr int pix = 128; };
}  // namespace

struct PatchArgs {
  const void* in;        // NHWC [N][H][W][C]
  const void* wt;        // [F][3][3][C]
  void* out;             // NHWC [N][H][W][F]
  const float* scale;    // [F] or null
  const float* shift;    // [F] or null
  const void* residual;  // like out, or null
  int N, H, W, C, F, relu;
  int TN, TH;            // tile: TN images x TH rows x W columns
  int tiles_y;           // ceil(H / TH)
  int tiles;             // ceil(N / TN) * tiles_y
  unsigned in_bytes, wt_bytes;
  float inv_php, inv_pw, inv_thw, inv_w;  // 1/(PH*PW), 1/PW, 1/(TH*W), 1/W
};

template <int WS, int WK>
struct PatchCfg {
  static constexpr int NW = WS * WK, NT = 64 * NW;
  static constexpr int cap = PatchCap<WS>::pix;
  static constexpr int PCH = (cap * 8 + NT - 1) / NT;  // 16-byte patch chunks per thread
  static constexpr int patch_bytes = PCH * (NT / 8) * kPitch;
  static constexpr int WCH = (512 + NT - 1) / NT;      // 16-byte weight chunks per thread
  static constexpr int main_bytes = patch_bytes + 3 * kWBytes;  // patch + weight ring
  static constexpr int red_bytes = WK > 1 ? WS * 64 * 64 * 4 : 0;
  static constexpr int epi_bytes = WS * kEpiWaveBytes;
  static constexpr int smem = main_bytes > red_bytes ? (main_bytes > epi_bytes ? main_bytes : epi_bytes)
                                                     : (red_bytes > epi_bytes ? red_bytes : epi_bytes);
};

template <typename T, typename OutT, int WS, int WK>
__global__ __launch_bounds__(64 * WS * WK) void conv3x3_patch_kernel(const PatchArgs a) {
  typedef PatchCfg<WS, WK> Cfg;
  constexpr int NT = Cfg::NT, PCH = Cfg::PCH, WCH = Cfg::WCH;
  constexpr int ES = sizeof(T);
  constexpr int SLAB = 128 / ES;  // channels per slab
  constexpr int KPG = 4 / WK;     // 32-byte K sub-steps per K group and tap
  static_assert(WK == 1 || WK == 2 || WK == 4, "K groups split the four sub-steps of a tap");
  extern __shared__ __align__(16) unsigned char smem[];
  unsigned char* patch = smem;
  unsigned char* wbuf = smem + Cfg::patch_bytes;  // ring of 3 buffers

  const int per_xcd = (a.tiles + kXcdsP - 1) / kXcdsP;
  const int tile = (blockIdx.x % kXcdsP) * per_xcd + blockIdx.x / kXcdsP;
  if (tile >= a.tiles) return;
  const int f0blk = blockIdx.y * 64;
  const int n0 = (tile / a.tiles_y) * a.TN, y0 = (tile % a.tiles_y) * a.TH;
  const int PH = a.TH + 2, PW = a.W + 2;
  const int ppix = a.TN * PH * PW;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int ws = wave % WS, wk = wave / WS;
  const int lrow = lane & 31, lchunk = lane >> 5;
  const __amdgpu_buffer_rsrc_t rs_in = make_rsrc(a.in, a.in_bytes);
  const __amdgpu_buffer_rsrc_t rs_wt = make_rsrc(a.wt, a.wt_bytes);

  // epilogue scale/shift of this lane's output channels: requested now, used at the very end
  EpiScale<OutT> ess;
  ess.load(lane, f0blk, a.F, a.scale, a.shift);

  // ---- weight loader: chunk q = tid + NT*i -> filter row q/8, piece q%8 (512 chunks per tap) ----
  unsigned wvoff[WCH];
#pragma unroll
  for (int i = 0; i < WCH; ++i) {
    const int f = f0blk + (tid >> 3) + (NT / 8) * i;
    wvoff[i] = f < a.F ? (unsigned)((f * 9 * a.C) * ES + (tid & 7) * 16) : kOOBp;
  }
  unsigned char* const wdst = wbuf + (tid >> 3) * kPitch + (tid & 7) * 16;
  // Weights of tap-iteration `it` live at byte offset ((it%9)*C + (it/9)*SLAB)*ES of a filter row.
  // Three register sets keep the loads of iterations it+1 .. it+3 in flight (an iteration is only
  // 4-16 MFMAs long, far less than an L2 round trip).
  const int nslab = a.C / SLAB;
  const int niter = nslab * 9;
  auto wload = [&](u32x4(&r)[WCH], int it) {
    const int sl = it / 9, tp = it - sl * 9;  // scalar
    const unsigned ko = (unsigned)((tp * a.C + sl * SLAB) * ES);
#pragma unroll
    for (int i = 0; i < WCH; ++i)
      r[i] = __builtin_amdgcn_raw_buffer_load_b128(rs_wt, it < niter ? wvoff[i] + ko : kOOBp, 0, 0);
  };
  u32x4 wregs[3][WCH];
  wload(wregs[0], 0);
  wload(wregs[1], 1);
  wload(wregs[2], 2);

  // ---- patch loader: chunk q = tid + NT*i -> pixel q/8, 16-byte piece q%8 ----
  unsigned pvoff[PCH];
#pragma unroll
  for (int i = 0; i < PCH; ++i) {
    const int pixel = (tid >> 3) + (NT / 8) * i;
    unsigned off = kOOBp;
    if (pixel < ppix) {
      int rem, px;
      const int nl = fast_div(pixel, PH * PW, a.inv_php, &rem);
      const int py = fast_div(rem, PW, a.inv_pw, &px);
      const int n = n0 + nl, iy = y0 + py - 1, ix = px - 1;
      if (n < a.N && (unsigned)iy < (unsigned)a.H && (unsigned)ix < (unsigned)a.W)
        off = (unsigned)((((n * a.H + iy) * a.W + ix) * a.C) * ES + (tid & 7) * 16);
    }
    pvoff[i] = off;
  }
  unsigned char* const pdst = patch + (tid >> 3) * kPitch + (tid & 7) * 16;
  u32x4 pregs[PCH];
#pragma unroll
  for (int i = 0; i < PCH; ++i) pregs[i] = __builtin_amdgcn_raw_buffer_load_b128(rs_in, pvoff[i], 0, 0);

  // ---- this lane's two pixel slots ----
  const int nslots = a.TN * a.TH * a.W;
  int sbase[2];  // byte offset of the slot's tap-(0,0) pixel in the patch
  int obase[2];  // element offset of the slot's output pixel row, or -1
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int sl = ws * 64 + j * 32 + lrow;
    int nl = 0, ty = 0, tx = 0;
    bool ok = sl < nslots;
    if (ok) {
      int rem;
      nl = fast_div(sl, a.TH * a.W, a.inv_thw, &rem);
      ty = fast_div(rem, a.W, a.inv_w, &tx);
      ok = (n0 + nl) < a.N && (y0 + ty) < a.H;
    }
    sbase[j] = ((nl * PH + ty) * PW + tx) * kPitch + (lchunk + 2 * wk * KPG) * 16;
    obase[j] = ok ? (((n0 + nl) * a.H + y0 + ty) * a.W + tx) * a.F : -1;
  }
  const unsigned char* const wsrc = wbuf + lrow * kPitch + (lchunk + 2 * wk * KPG) * 16;

  floatx16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  static_assert(WCH * NT == 512, "every thread stores all of its weight chunks");
  auto wstore = [&](const u32x4(&r)[WCH], int buf) {
#pragma unroll
    for (int i = 0; i < WCH; ++i) *reinterpret_cast<u32x4*>(wdst + buf * kWBytes + i * (NT / 8) * kPitch) = r[i];
  };
  auto ldw = [&](u32x4(&f)[2], int slot, int kk) {
#pragma unroll
    for (int i = 0; i < 2; ++i) f[i] = *reinterpret_cast<const u32x4*>(wsrc + slot * kWBytes + i * 32 * kPitch + kk * 32);
  };
  auto ldp = [&](u32x4(&f)[2], int tapoff, int kk) {
#pragma unroll
    for (int j = 0; j < 2; ++j) f[j] = *reinterpret_cast<const u32x4*>(patch + sbase[j] + tapoff + kk * 32);
  };

  // Pipeline.  Weights of iteration `it` (= one tap of one slab) sit in LDS ring slot it%3 and in
  // register set it%3 on their way there; at iteration `it` the weights of it+2 are stored and
  // those of it+5 requested, so three iterations of loads are always in flight, and because the
  // weights of it+1 were stored one iteration earlier, the first MFMA operands of iteration it+1
  // are read from LDS BEFORE the barrier that ends iteration it: no wave waits on LDS latency
  // right after a barrier.
  wstore(wregs[0], 0);
  wload(wregs[0], 3);
  wstore(wregs[1], 1);
  wload(wregs[1], 4);
#pragma unroll
  for (int i = 0; i < PCH; ++i) *reinterpret_cast<u32x4*>(pdst + i * (NT / 8) * kPitch) = pregs[i];
  __syncthreads();

  u32x4 fw[2], fp[2];
  ldw(fw, 0, 0);
  ldp(fp, 0, 0);
  // One trip = one filter row = three taps, so ring slots and register sets rotate statically.
  int tr = 0, slab = 0;
  for (int it0 = 0; it0 < niter; it0 += 3) {
    // next slab's patch is requested at the first tap of this slab and lands after its last tap
    if (tr == 0 && slab + 1 < nslab) {
      const unsigned so = (unsigned)((slab + 1) * 128);
#pragma unroll
      for (int i = 0; i < PCH; ++i) pregs[i] = __builtin_amdgcn_raw_buffer_load_b128(rs_in, pvoff[i] + so, 0, 0);
    }
    const int ntr = tr == 2 ? 0 : tr + 1;
#pragma unroll
    for (int ts = 0; ts < 3; ++ts) {
      const int it = it0 + ts;
      wstore(wregs[(ts + 2) % 3], (ts + 2) % 3);  // weights of it+2
      wload(wregs[(ts + 2) % 3], it + 5);
      const bool new_patch = ts == 2 && tr == 2 && slab + 1 < nslab;  // the patch changes after this tap
      const int tapoff = (tr * PW + ts) * kPitch;
      const int ntapoff = ts == 2 ? (ntr * PW) * kPitch : tapoff + kPitch;
#pragma unroll
      for (int kk = 0; kk < KPG; ++kk) {
        u32x4 nw[2], np[2];
        if (kk + 1 < KPG) {
          ldw(nw, ts, kk + 1);
          ldp(np, tapoff, kk + 1);
        } else {
          ldw(nw, (ts + 1) % 3, 0);
          if (!new_patch) ldp(np, ntapoff, 0);
        }
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j) Mma<T>::run(fw[i], fp[j], acc[i][j]);
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          fw[i] = nw[i];
          fp[i] = np[i];
        }
      }
      if (new_patch) {
        __syncthreads();  // every wave is done with the old patch
#pragma unroll
        for (int i = 0; i < PCH; ++i) *reinterpret_cast<u32x4*>(pdst + i * (NT / 8) * kPitch) = pregs[i];
      }
      __syncthreads();
      if (new_patch) ldp(fp, 0, 0);
    }
    tr = ntr;
    if (tr == 0) ++slab;
  }
  __syncthreads();

  // ---- K groups meet in LDS, one group per round (the last barrier freed all of LDS) ----
  if (WK > 1) {
    float* red = reinterpret_cast<float*>(smem) + (size_t)ws * 64 * 64 + lane;
#pragma unroll 1
    for (int g = 1; g < WK; ++g) {
      if (wk == g) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) red[((i * 2 + j) * 16 + v) * 64] = acc[i][j][v];
      }
      __syncthreads();
      if (wk == 0) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] += red[((i * 2 + j) * 16 + v) * 64];
      }
      __syncthreads();
    }
  }

  epilogue_64x64<OutT>(acc, smem + ws * kEpiWaveBytes, wk == 0, lane, obase, f0blk, a.F, ess,
                       static_cast<const OutT*>(a.residual), static_cast<OutT*>(a.out), a.relu);
}

// Tile choice for 64*ws slots: TN images x TH rows x W columns with a patch of at most `cap` pixels.
static bool plan_tile(int N, int H, int W, int slots, int cap, int* TN, int* TH) {
  if (W > slots || 3 * (W + 2) > cap) return false;
  int thmax = 0;
  for (int th = 1; th <= H; ++th)
    if (th * W <= slots && (th + 2) * (W + 2) <= cap) thmax = th;
  if (thmax == 0) return false;
  if (thmax < H) {
    const int nt = (H + thmax - 1) / thmax;
    *TH = (H + nt - 1) / nt;  // balanced rows per tile
    *TN = 1;
    return true;
  }
  int tn = 1;
  while (tn + 1 <= N && (tn + 1) * H * W <= slots && (tn + 1) * (H + 2) * (W + 2) <= cap) ++tn;
  *TN = tn;
  *TH = H;
  return true;
}

// Picks the wave arrangement: the largest pixel tile that still gives (about) every CU a workgroup.
static bool plan_patch(int N, int H, int W, int F, int* WS, int* TN, int* TH) {
  static const int force = [] {
    const char* e = getenv("NNCV_HIP_PATCH_WS");
    return e ? atoi(e) : 0;
  }();
  const int fb = (F + 63) / 64;
  long long best_blocks = 0;
  for (int ws : {4, 2, 1}) {
    if (force && ws != force) continue;
    const int cap = ws == 4 ? PatchCap<4>::pix : ws == 2 ? PatchCap<2>::pix : PatchCap<1>::pix;
    int tn, th;
    if (!plan_tile(N, H, W, 64 * ws, cap, &tn, &th)) continue;
    const long long blocks = (long long)((N + tn - 1) / tn) * ((H + th - 1) / th) * fb;
    // the first (largest) arrangement that fills the chip wins; failing that, the one with the
    // most workgroups
    if (blocks > best_blocks) {
      best_blocks = blocks; *WS = ws; *TN = tn; *TH = th;
    }
    if (blocks >= 224) break;
  }
  return best_blocks != 0;
}

bool conv3x3_patch_applicable(const IgemmArgs& a, int in_dt) {
  static const bool off = getenv("NNCV_HIP_NO_PATCH") != nullptr;
  const int slab = in_dt == kF16 ? 64 : 32;
  int ws, tn, th;
  return !off && a.R == 3 && a.S == 3 && a.stride_h == 1 && a.stride_w == 1 && a.pad_h == 1 && a.pad_w == 1 && a.batch == 1 &&
         a.pix_stride == 0 && a.C % slab == 0 && a.F % 8 == 0 && a.ldo == a.F &&
         (long long)a.N * a.H * a.W * a.F < (1ll << 31) && a.in_bytes < kOOBp && a.wt_bytes < kOOBp &&
         plan_patch(a.N, a.H, a.W, a.F, &ws, &tn, &th);
}

template <typename T, typename OutT, int WS, int WK>
static void launch_patch_cfg(const PatchArgs& a, double flops, double bytes, const char* tag, hipStream_t s) {
  typedef PatchCfg<WS, WK> Cfg;
  auto kern = conv3x3_patch_kernel<T, OutT, WS, WK>;
  static const bool attr = [&] {
    NNCV_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, Cfg::smem));
    return true;
  }();
  (void)attr;
  ProfScope prof(tag, flops, bytes, s);
  dim3 grid((a.tiles + kXcdsP - 1) / kXcdsP * kXcdsP, (a.F + 63) / 64);
  hipLaunchKernelGGL(kern, grid, dim3(Cfg::NT), Cfg::smem, s, a);
}

void launch_conv3x3_patch(const IgemmArgs& g, int in_dt, int out_dt, hipStream_t s) {
  PatchArgs a{};
  a.in = g.in; a.wt = g.wt; a.out = g.out; a.scale = g.scale; a.shift = g.shift; a.residual = g.residual;
  a.N = g.N; a.H = g.H; a.W = g.W; a.C = g.C; a.F = g.F; a.relu = g.relu;
  int ws = 0;
  NNCV_REQUIRE(plan_patch(a.N, a.H, a.W, a.F, &ws, &a.TN, &a.TH), "conv3x3_patch: no tile fits");
  a.tiles_y = (a.H + a.TH - 1) / a.TH;
  a.tiles = ((a.N + a.TN - 1) / a.TN) * a.tiles_y;
  a.in_bytes = g.in_bytes; a.wt_bytes = g.wt_bytes;
  a.inv_php = 1.0f / ((a.TH + 2) * (a.W + 2)); a.inv_pw = 1.0f / (a.W + 2);
  a.inv_thw = 1.0f / (a.TH * a.W); a.inv_w = 1.0f / a.W;
  const double P = (double)a.N * a.H * a.W;
  const double flops = 2.0 * P * a.F * 9.0 * a.C;
  const double es = dtype_size(in_dt), os = dtype_size(out_dt);
  const double bytes = es * (P * a.C + 9.0 * a.C * a.F) + os * P * a.F * (a.residual ? 2 : 1);
  const bool h = in_dt == kF16 && out_dt == kF16, f = in_dt == kF32 && out_dt == kF32;
  NNCV_REQUIRE(h || f, "conv3x3_patch: unsupported dtype combination");
  if (h) {
    if (ws == 4) launch_patch_cfg<half_t, half_t, 4, 2>(a, flops, bytes, "conv3x3_patch<f16,4,2>", s);
    else if (ws == 2) launch_patch_cfg<half_t, half_t, 2, 4>(a, flops, bytes, "conv3x3_patch<f16,2,4>", s);
    else launch_patch_cfg<half_t, half_t, 1, 4>(a, flops, bytes, "conv3x3_patch<f16,1,4>", s);
  } else {
    if (ws == 4) launch_patch_cfg<float, float, 4, 2>(a, flops, bytes, "conv3x3_patch<f32,4,2>", s);
    else if (ws == 2) launch_patch_cfg<float, float, 2, 4>(a, flops, bytes, "conv3x3_patch<f32,2,4>", s);
    else launch_patch_cfg<float, float, 1, 4>(a, flops, bytes, "conv3x3_patch<f32,1,4>", s);
  }
  NNCV_HIP_CHECK(hipGetLastError());
}

}  // namespace nncv_hip
