// Fast path of the implicit-GEMM convolution / batched K-contiguous GEMM (same contract as the
// generic kernel in igemm.hip) for the shapes ResNet-18 actually has: the channel count is a
// multiple of one K step (32 halves / 16 floats), so every K step lies inside one filter tap
// (r, s) and all K bookkeeping is wave-uniform scalar work.
//
// What differs from the generic kernel, and why:
//  * Gathers are raw buffer loads. A lane whose pixel falls in the halo (or past the end of the
//    tensor) gets an offset beyond the buffer's size and the hardware returns zeros: no branches,
//    no exec-mask juggling in the main loop.
//  * The K walk is a scalar (kr, ks, kc) triple advanced once per step; the prologue decodes
//    pixel indices with float-reciprocal division (an integer divide is ~40 VALU instructions).
//  * Waves are arranged WP x WF x WK: WP*WF waves tile the workgroup's (64*WP) x (64*WF) output
//    block with 64x64 sub-tiles (2x2 MFMA 32x32 accumulators: one 16-byte LDS read per MFMA), and
//    WK "K groups" each take every WK-th K step of the same output block; their partial sums meet
//    in LDS at the end.  Small-P layers (14x14, 7x7 maps at batch 32) use WK = 4 so that 64x64
//    output blocks still give every SIMD of the chip a 64x64 accumulator tile to work on.
//  * A stage is KS K-steps; global loads run two stages ahead of the MFMAs (two register sets,
//    two LDS buffers, one barrier per stage).
//  * K groups meet in an fp32 LDS tile and the epilogue reads it back so that residual reads and
//    result stores are whole 128-byte rows (mfma_tile.hpp).
//  * Workgroups are renumbered so that each XCD (8 of them, round-robin over the linear workgroup
//    id) gets a contiguous range of pixel tiles: neighbouring tiles share input rows, and each
//    XCD has its own L2.
#include "mfma_tile.hpp"

namespace nncv_hip {

using namespace mt;

namespace {
constexpr int kRow = 80;                 // LDS row pitch in bytes: 64 payload + 16 pad
constexpr unsigned kOOB = 0x7fffff00u;   // byte offset beyond any buffer this kernel accepts
constexpr int kXcds = 8;
}  // namespace

template <typename T, typename OutT, int WP, int WF, int WK, int KS, int NI>
__global__ __launch_bounds__(64 * WP * WF * WK) void igemm_fast_kernel(const IgemmArgs a, const int tiles_x,
                                                                       const float inv_ohow, const float inv_ow) {
  constexpr int NT = 64 * WP * WF * WK;
  static_assert(NT == 256, "loader mapping assumes 256 threads");
  constexpr int ES = sizeof(T);
  constexpr int CE = 16 / ES;       // elements per 16-byte chunk
  constexpr int BKE = 4 * CE;       // elements per K step
  constexpr int BP = 64 * WP, BF = 64 * WF, ROWS = BP + BF;
  // NI = 1: a workgroup owns 32 filters instead of 64 (twice the workgroups for small problems).
  // The LDS stage keeps its 64 weight rows; the upper 32 are loaded as zeros and never multiplied.
  static_assert(NI == 2 || WF == 1, "half filter blocks only with one filter wave");
  constexpr int BFE = NI == 2 ? BF : 32;  // filters per workgroup
  constexpr int R64 = ROWS / 64;    // 64-row groups per K step
  constexpr int LPT = KS * R64;     // 16-byte loads per thread per stage
  constexpr int STAGE = KS * ROWS * kRow;
  static_assert(KS % WK == 0, "every K group needs the same number of steps per stage");

  extern __shared__ __align__(16) unsigned char smem[];  // max(2 * STAGE, output tiles) bytes

  // ---- which output block (XCD-aware renumbering along x) ----
  const int per_xcd = (tiles_x + kXcds - 1) / kXcds;
  const int bx = (blockIdx.x % kXcds) * per_xcd + blockIdx.x / kXcds;
  if (bx >= tiles_x) return;  // uniform for the whole workgroup
  const int by = blockIdx.y, bz = blockIdx.z;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wpos = wave % (WP * WF), wk = wave / (WP * WF);
  const int wp = wpos % WP, wf = wpos / WP;
  const int P = a.N * a.OH * a.OW;
  const int nk_row = (a.R * a.S * a.C) / BKE;  // K steps of a whole filter row (exact: C % BKE == 0)
  // auxiliary filter blocks walk one tap only
  const bool aux = a.aux_f0 > 0 && by * BFE >= a.aux_f0;
  const int spt = a.C / BKE;  // K steps per tap
  const int k_begin = aux ? a.aux_tap * spt : 0;
  const int nk = aux ? k_begin + spt : nk_row;  // end of the K walk
  const int pix = a.pix_stride ? a.pix_stride : a.C;

  const __amdgpu_buffer_rsrc_t rs_in = make_rsrc(static_cast<const T*>(a.in) + (long long)bz * a.in_bs, a.in_bytes);
  const __amdgpu_buffer_rsrc_t rs_wt = make_rsrc(static_cast<const T*>(a.wt) + (long long)bz * a.wt_bs, a.wt_bytes);

  // ---- per-thread loader state: rows (tid>>2) + 64*g, chunk tid&3 ----
  const int ck = tid & 3, r0 = tid >> 2;
  int pbase[WP], piy[WP], pix0[WP];
#pragma unroll
  for (int g = 0; g < WP; ++g) {
    const int gp = bx * BP + r0 + 64 * g;
    if (gp < P) {
      int rem, ox;
      const int n = fast_div(gp, a.OH * a.OW, inv_ohow, &rem);
      const int oy = fast_div(rem, a.OW, inv_ow, &ox);
      piy[g] = oy * a.stride_h - a.pad_h;
      pix0[g] = ox * a.stride_w - a.pad_w;
      pbase[g] = (((n * a.H + piy[g]) * a.W + pix0[g]) * pix + ck * CE) * ES;
    } else {
      piy[g] = pix0[g] = -(1 << 28);
      pbase[g] = 0;
    }
  }
  int wbase[WF];
#pragma unroll
  for (int g = 0; g < WF; ++g) {
    const int f = by * BFE + r0 + 64 * g;
    wbase[g] = (f < a.F && r0 + 64 * g < BFE) ? (f * (nk_row * BKE) + ck * CE) * ES : -1;
  }

  // epilogue scale/shift of this lane's output channels: requested now, used at the very end
  EpiScale<OutT> ess;
  ess.load(lane, by * BFE + wf * 64, a.F, a.scale, a.shift);

  // scalar K walk
  int kstep = k_begin, kr = aux ? a.aux_tap / a.S : 0, ks = aux ? a.aux_tap % a.S : 0, kc = 0;

  u32x4 regs[2][LPT];
  auto issue = [&](u32x4(&r)[LPT]) {
#pragma unroll
    for (int st = 0; st < KS; ++st) {
      const bool kval = kstep < nk;
      const int koff = ((kr * a.W + ks) * pix + kc) * ES;
#pragma unroll
      for (int g = 0; g < WP; ++g) {
        const bool ok = kval && (unsigned)(piy[g] + kr) < (unsigned)a.H && (unsigned)(pix0[g] + ks) < (unsigned)a.W;
        r[st * R64 + g] = __builtin_amdgcn_raw_buffer_load_b128(rs_in, ok ? (unsigned)(pbase[g] + koff) : kOOB, 0, 0);
      }
      const int wko = kstep * (BKE * ES);
#pragma unroll
      for (int g = 0; g < WF; ++g) {
        const bool ok = kval && wbase[g] >= 0;
        r[st * R64 + WP + g] = __builtin_amdgcn_raw_buffer_load_b128(rs_wt, ok ? (unsigned)(wbase[g] + wko) : kOOB, 0, 0);
      }
      ++kstep;
      kc += BKE;
      if (kc == a.C) {
        kc = 0;
        if (++ks == a.S) {
          ks = 0;
          ++kr;
        }
      }
    }
  };
  auto store = [&](const u32x4(&r)[LPT], int buf) {
    unsigned char* base = smem + buf * STAGE + r0 * kRow + ck * 16;
#pragma unroll
    for (int st = 0; st < KS; ++st)
#pragma unroll
      for (int g = 0; g < R64; ++g)
        *reinterpret_cast<u32x4*>(base + (st * ROWS + 64 * g) * kRow) = r[st * R64 + g];
  };

  floatx16 acc[2][2];  // [f sub-tile][pixel sub-tile]
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  const int lrow = lane & 31, lchunk = lane >> 5;
  auto compute = [&](int buf) {
    const unsigned char* sP = smem + buf * STAGE + (wp * 64 + lrow) * kRow + lchunk * 16;
    const unsigned char* sW = smem + buf * STAGE + (BP + wf * 64 + lrow) * kRow + lchunk * 16;
#pragma unroll
    for (int st = wk; st < KS; st += WK) {
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        u32x4 fw[2], fp[2];
#pragma unroll
        for (int i = 0; i < NI; ++i) fw[i] = *reinterpret_cast<const u32x4*>(sW + (st * ROWS + i * 32) * kRow + kk * 32);
#pragma unroll
        for (int j = 0; j < 2; ++j) fp[j] = *reinterpret_cast<const u32x4*>(sP + (st * ROWS + j * 32) * kRow + kk * 32);
#pragma unroll
        for (int i = 0; i < NI; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j) Mma<T>::run(fw[i], fp[j], acc[i][j]);
      }
    }
  };

  const int nst = (nk - k_begin + KS - 1) / KS;
  issue(regs[0]);
  if (nst > 1) issue(regs[1]);
  store(regs[0], 0);
  __syncthreads();
  int s = 0;
  // Steady state, two stages per trip.  Both issues are unconditional so that the wait before each
  // LDS store only covers the loads of the stage being stored (issued a whole stage earlier) and
  // leaves the newest stage's loads in flight.
  for (; s + 3 < nst; s += 2) {
    issue(regs[0]);        // stage s+2
    compute(0);            // stage s
    store(regs[1], 1);     // stage s+1
    __syncthreads();
    issue(regs[1]);        // stage s+3
    compute(1);            // stage s+1
    store(regs[0], 0);     // stage s+2
    __syncthreads();
  }
  // Tail: stage s sits in buffer 0, stage s+1 (if any) is in flight in regs[1], stage s+2 (if any)
  // has not been requested yet.
  if (s + 2 < nst) issue(regs[0]);
  compute(0);
  if (s + 1 < nst) {
    store(regs[1], 1);
    __syncthreads();
    compute(1);
    if (s + 2 < nst) {
      store(regs[0], 0);
      __syncthreads();
      compute(0);
    }
  }
  __syncthreads();

  // ---- K groups meet in an LDS tile, then whole-row stores (all stage buffers are free after the
  // last barrier) ----
  int rowoff[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int gp = bx * BP + wp * 64 + j * 32 + lrow;
    rowoff[j] = gp < P ? gp * (aux ? a.aux_ldo : a.ldo) : -1;
  }
  OutT* out = aux ? static_cast<OutT*>(a.aux_out) : static_cast<OutT*>(a.out) + (long long)bz * a.out_bs;
  const OutT* res = (a.residual && !aux) ? static_cast<const OutT*>(a.residual) + (long long)bz * a.out_bs : nullptr;
  const int fo = aux ? a.aux_f0 : 0;                     // first filter of this output tensor
  const int fend = (aux || a.aux_f0 == 0) ? a.F : a.aux_f0;  // one past its last filter
  tile_reduce_store<OutT, WK, NI>(acc, smem + wpos * WK * kTileBytes, wk, lane, rowoff, by * BFE + wf * 64 - fo, fend - fo, ess, res, out,
                              aux ? a.aux_relu : a.relu);
}

namespace {

template <typename T> constexpr const char* tn();
template <> constexpr const char* tn<half_t>() { return "f16"; }
template <> constexpr const char* tn<float>() { return "f32"; }

template <typename T, typename OutT, int WP, int WF, int WK, int KS, int NI = 2>
void launch_fast_cfg(const IgemmArgs& a, hipStream_t s) {
  constexpr int BP = 64 * WP, BF = 64 * WF, BFE = NI == 2 ? BF : 32;
  constexpr int stage2 = 2 * KS * (BP + BF) * kRow;
  constexpr int epi = WP * WF * WK * kTileBytes;  // one output-tile copy per K group
  constexpr int smem = stage2 > epi ? stage2 : epi;
  static const std::string tag = std::string("igemm_fast<") + tn<T>() + "," + tn<OutT>() + "," + std::to_string(WP) + "," +
                                 std::to_string(WF) + "," + std::to_string(WK) + "," + std::to_string(KS) + (NI == 1 ? ",half>" : ">");
  auto kern = igemm_fast_kernel<T, OutT, WP, WF, WK, KS, NI>;
  static const bool attr_set = [&] {
    NNCV_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, smem));
    return true;
  }();
  (void)attr_set;
  const int P = a.N * a.OH * a.OW;
  const double K = (double)a.R * a.S * a.C;
  const double flops = a.alg_flops > 0 ? a.alg_flops : 2.0 * P * a.F * K * a.batch;
  const double bytes = sizeof(T) * ((double)a.in_bytes / sizeof(T) + (double)a.F * K) * a.batch +
                       sizeof(OutT) * (double)P * a.F * a.batch * (a.residual ? 2 : 1);
  ProfScope prof(tag.c_str(), flops, bytes, s);
  const int tiles_x = (P + BP - 1) / BP;
  dim3 grid((tiles_x + kXcds - 1) / kXcds * kXcds, (a.F + BFE - 1) / BFE, a.batch);
  hipLaunchKernelGGL(kern, grid, dim3(64 * WP * WF * WK), smem, s, a, tiles_x, 1.0f / (float)(a.OH * a.OW), 1.0f / (float)a.OW);
}

template <typename T, typename OutT>
void launch_fast_typed(const IgemmArgs& a, hipStream_t s) {
  const long long P = (long long)a.N * a.OH * a.OW;
  auto blocks = [&](int bp, int bf) { return ((P + bp - 1) / bp) * ((a.F + bf - 1) / bf) * a.batch; };
  static const int force = [] {
    const char* e = getenv("NNCV_HIP_IGEMM_FAST_TILE");
    return e ? atoi(e) : 0;
  }();
  int pick = force;
  if (!pick) {
    // 256 CUs: prefer the largest output block that still leaves no CU idle; when even 128x64
    // blocks cannot do that, fall to 64x64 blocks whose four waves split K.
    if (a.F % 128 == 0 && blocks(128, 128) >= 256) pick = 1;
    else if (a.F <= 64 && blocks(256, 64) >= 256) pick = 2;
    else if (blocks(128, 64) >= 256) pick = 3;
    else if (blocks(64, 64) >= 128 || a.F % 32 != 0) pick = 4;
    else pick = 5;  // fewer than 128 workgroups of 64x64: halve the filter blocks
  }
  switch (pick) {
    case 1: launch_fast_cfg<T, OutT, 2, 2, 1, 1>(a, s); break;
    case 2: launch_fast_cfg<T, OutT, 4, 1, 1, 1>(a, s); break;
    case 3: launch_fast_cfg<T, OutT, 2, 1, 2, 2>(a, s); break;
    case 5: launch_fast_cfg<T, OutT, 1, 1, 4, 4, 1>(a, s); break;
    default: launch_fast_cfg<T, OutT, 1, 1, 4, 4>(a, s); break;
  }
}

}  // namespace

bool igemm_fast_applicable(const IgemmArgs& a, int in_dt, int out_dt) {
  const int bke = in_dt == kF16 ? 32 : 16;
  const int fvec = out_dt == kF16 ? 8 : 4;  // channels per 16-byte store of the epilogue
  static const bool off = getenv("NNCV_HIP_IGEMM_GENERIC") != nullptr;
  const long long P = (long long)a.N * a.OH * a.OW;
  return !off && a.C % bke == 0 && a.F % fvec == 0 && a.ldo % fvec == 0 && a.in_bytes > 0 && a.in_bytes < kOOB &&
         a.wt_bytes > 0 && a.wt_bytes < kOOB && P < (1 << 24) && P * a.ldo < (1ll << 31) &&
         (a.aux_f0 == 0 || (a.aux_f0 % 128 == 0 && a.batch == 1 && a.aux_out && a.aux_ldo % fvec == 0 &&
                            P * a.aux_ldo < (1ll << 31) && a.aux_tap >= 0 && a.aux_tap < a.R * a.S));
}

void launch_igemm_fast(const IgemmArgs& a, int in_dt, int out_dt, hipStream_t s) {
  if (in_dt == kF16 && out_dt == kF16) launch_fast_typed<half_t, half_t>(a, s);
  else if (in_dt == kF16 && out_dt == kF32) launch_fast_typed<half_t, float>(a, s);
  else if (in_dt == kF32 && out_dt == kF32) launch_fast_typed<float, float>(a, s);
  else fail("igemm: unsupported dtype combination");
}

}  // namespace nncv_hip
