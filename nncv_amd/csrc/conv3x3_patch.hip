// 3x3 pad-1 convolution, stride 1 or 2, with the haloed input patch resident in LDS (gfx950).
// The text below describes stride 1; what stride 2 changes (a 2TH+1 x 2TW+1 patch with its even and
// odd columns kept apart, the 1x1 shortcut convolution of a down-sampling block as extra filter
// blocks) is said where the code does it, and so is the split of K over workgroups that small
// fp32 launches use (tile_reduce_store_splitk).
//
// The implicit-GEMM kernels gather every input pixel once per filter tap, i.e. nine times, from
// L2, and need a workgroup barrier per K step.  Here a workgroup owns an output tile of TN images
// x TH rows x TW columns (at most 64*WS pixel "slots"; TW is the full width unless a row is wider
// than the 64 pixels the loader walks, in which case rows are cut into column tiles) and 64
// filters, and per 128-byte channel slab (64 halves / 32 floats):
//   * loads the (TH+2) x (TW+2) haloed input patch ONCE into LDS (zero halo straight from the
//     buffer-load range check; the reference materialises it with tensor.pad,
//     tests/Nets/Res18.mlir:152-155),
//   * walks the nine taps; a tap is a constant byte offset into the patch, so the MFMA pixel
//     operand of tap (r,s) is read from the same LDS data at  slot_base + (r*(TW+2)+s)*pitch,
//   * takes the MFMA weight operand straight from global memory into registers: the filters are
//     stored fragment-major at model load (launch_weight_frag3x3), so each operand load of a wave
//     is one contiguous kilobyte at a scalar offset, three taps of loads are always in flight,
//     and the main loop has no barrier at all (only the slab change has).
//
// Wave layout WS x WK: WS waves each own 64 slots x 64 filters (2x2 accumulators of
// v_mfma_f32_32x32x16_f16; fp32: 4x v_mfma_f32_32x32x2_f32 per chunk pair), and WK "K groups"
// split the four 32-byte K sub-steps of every tap between them; their partial sums meet in an
// fp32 LDS tile from which the epilogue (scale/shift, residual, ReLU) stores whole rows
// (mfma_tile.hpp).  Splitting K inside the workgroup rather than shrinking the pixel tile keeps
// one 16-byte LDS read per MFMA, gives every SIMD two resident waves, and lets small feature maps
// still fill 256 CUs.  All instances are 4 waves (one per SIMD; two workgroups share a CU):
//   56x56, 28x28 -> WS=4, WK=1 ; 14x14 -> WS=2, WK=2 ; 7x7 -> WS=1, WK=4.
// LDS pixel pitch is 128 + 16 bytes: consecutive pixels land 36 banks apart.
#include <type_traits>

#include "mfma_tile.hpp"

namespace nncv_hip {

using namespace mt;

namespace {
constexpr int kPitch = 144;            // LDS bytes per patch pixel: 128 payload + 16 pad
constexpr unsigned kOOBp = 0x7fff0000u;
constexpr int kXcdsP = 8;

template <int WS> struct PatchCap;     // patch capacity in pixels for 64*WS slots
template <> struct PatchCap<4> { static constexpr int pix = 384; };
template <> struct PatchCap<2> { static constexpr int pix = 256; };
template <> struct PatchCap<1> { static constexpr int pix = 192; };
}  // namespace

struct PatchArgs {
  const void* in;        // NHWC [N][H][W][C]
  const void* wf;        // fragment-major weights (launch_weight_frag3x3)
  void* out;             // NHWC [N][H][W][F]
  const float* scale;    // [F] or null
  const float* shift;    // [F] or null
  const void* residual;  // like out, or null
  int N, H, W, C, F, relu;
  int TN, TH;            // tile: TN images x TH output rows x TW output columns
  int tiles_y;           // tiles per group of TN images: ceil(OH / TH) row bands x NTX column tiles
  int tiles;             // ceil(N / TN) * tiles_y
  int ldo, pix;          // elements between pixels of out (and residual) / of in: F and C unless they are slices of wider tensors
  int txw;               // TW | NTX << 16.  NTX = 1 (TW = the full output width) unless a row is too wide for the loader
  int rw_log;            // patch loader: 2^rw_log >= patch columns per loader row
  int rowx;              // stride 1: spare bytes behind the cells of a patch row (see the row pitch in the kernel)
  int OH, OW;            // output size (stride 2; stride 1: H, W)
  int xcd_by_filter;     // XCD <- filter block instead of XCD <- tile range
  unsigned in_bytes, wf_bytes;
  float inv_ph, inv_thw, inv_w;  // 1/(patch rows per image), 1/(TH*TW), 1/TW
  // Stride 2 only: filter blocks >= aux_fb0 (in units of the workgroup's 32*NI filters) belong to a
  // 1x1 stride-2 convolution over the same input (the shortcut of a down-sampling block), with its
  // own output tensor [N][OH][OW][aux_F], scale/shift and ReLU flag.  aux_F = 0: none.
  const void* aux_wf;    // fragment-major, one tap per slab (launch_weight_frag1x1)
  void* aux_out;
  const float* aux_scale;
  const float* aux_shift;
  int aux_F, aux_relu, aux_fb0;
  int aux_inline;  // the workgroup of filter block b also computes block b of the auxiliary filters (aux_F == F): no extra blocks
  unsigned aux_wf_bytes;
  // K split over workgroups (the SK instances): grid.z = ksplit workgroups share an output tile, each
  // walks `spk` channel slabs; their fp32 partial tiles meet in `partial` and the last one to
  // arrive (ticket from `counters`) sums them in slab order and runs the epilogue.
  float* partial;  // [tiles * filter blocks][ksplit][64][64]
  int* counters;   // [tiles * filter blocks], zero between launches
  int ksplit, spk;
};

// tile_reduce_store (mfma_tile.hpp) for one of `ksplit` workgroups that hold partial sums of the same
// output tile.  Every workgroup reduces its K groups through LDS as usual, writes the fp32 result to
// its slot of `partial`, and takes a ticket; the workgroup that draws the last ticket adds the ksplit
// tiles in index order (so the sum does not depend on which one was last), applies the epilogue and
// stores.  It also returns the counter to zero for the next launch.  No workgroup ever waits.
constexpr int kMaxSplit = 16;  // workgroups per output tile at most

template <typename OutT, int NG, int NI>
__device__ __forceinline__ void tile_reduce_store_splitk(const floatx16 (&acc)[2][2], unsigned char* tile, int g, int lane, int tid,
                                                         const int (&rowoff)[2], int f0, int F, const EpiScale<OutT>& ss,
                                                         const OutT* res, OutT* out, int relu, float* partial, int* counter, int z,
                                                         int ksplit) {
  const int lrow = lane & 31, lchunk = lane >> 5;
  constexpr int FPL = EpiScale<OutT>::FPL, LPR = EpiScale<OutT>::LPR;
  constexpr int RPI = 64 / LPR, NIT = 64 / NG / RPI;
  static_assert(NIT >= 1, "too many K groups for this output type");
  typedef OutT VO __attribute__((ext_vector_type(FPL)));
  const int fc = (lane % LPR) * FPL;
  const bool lane_on = fc < 32 * NI;
  const bool fok = f0 + fc < F && lane_on;
  int o[NIT];
  VO rv[NIT];
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    const int row = g * (64 / NG) + it * RPI + lane / LPR;
    const int o0 = __shfl(rowoff[0], row & 31), o1 = __shfl(rowoff[1], row & 31);
    o[it] = (row & 32) ? o1 : o0;
    if (!fok) o[it] = -1;
  }
  if (res) {
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
      const long long off = o[it] >= 0 ? (long long)o[it] + f0 + fc : 0;
      rv[it] = *reinterpret_cast<const VO*>(res + off);
    }
  }
  unsigned char* mine = tile + g * kTileBytes;
#pragma unroll
  for (int j = 0; j < 2; ++j)
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        floatx4* p = reinterpret_cast<floatx4*>(mine + (j * 32 + lrow) * kTilePitch + (i * 32 + 8 * q + 4 * lchunk) * 4);
        *p = floatx4{acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
      }
  __syncthreads();
  floatx4 v[NIT][FPL / 4];
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    const int row = g * (64 / NG) + it * RPI + lane / LPR;
#pragma unroll
    for (int q = 0; q < FPL / 4; ++q) {
      floatx4 sum = *reinterpret_cast<const floatx4*>(tile + row * kTilePitch + fc * 4 + q * 16);
#pragma unroll
      for (int k = 1; k < NG; ++k) sum += *reinterpret_cast<const floatx4*>(tile + k * kTileBytes + row * kTilePitch + fc * 4 + q * 16);
      v[it][q] = sum;
    }
  }
  // This workgroup's partial tile -> global memory, then the ticket.  The tile is written and later
  // read with device-scope relaxed atomics (8 bytes each): those are performed where all XCDs see
  // them, so no cache write-back / invalidate fence is needed (a device-scope fence writes the whole
  // L2 back and costs tens of microseconds here); waiting for the stores to be acknowledged orders
  // them before the ticket.
  typedef unsigned long long u64;
  typedef u64 u64x2 __attribute__((ext_vector_type(2)));
  if (lane_on) {
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
      const int row = g * (64 / NG) + it * RPI + lane / LPR;
#pragma unroll
      for (int q = 0; q < FPL / 4; ++q) {
        u64* p = reinterpret_cast<u64*>(partial + ((size_t)z * 64 + row) * 64 + fc + 4 * q);
        const u64x2 bits = __builtin_bit_cast(u64x2, v[it][q]);
        __hip_atomic_store(p, bits[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(p + 1, bits[1], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __builtin_amdgcn_s_waitcnt(0);  // every store of this wave has been acknowledged
  __syncthreads();                // ... and of every wave (all are done reading the LDS tiles, too)
  int* flag = reinterpret_cast<int*>(tile);
  if (tid == 0) *flag = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __syncthreads();
  if (*flag != ksplit - 1) return;  // uniform for the workgroup
  if (tid == 0) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
  // all kMaxSplit loads of a row segment are requested before the first addition (a chain of
  // dependent round trips to memory would cost more than the split saves); slots past ksplit read
  // tile 0 and are not added
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    const int row = g * (64 / NG) + it * RPI + lane / LPR;
#pragma unroll
    for (int q = 0; q < FPL / 4; ++q) {
      u64x2 bits[kMaxSplit];
#pragma unroll
      for (int zz = 0; zz < kMaxSplit; ++zz) {
        u64* p = reinterpret_cast<u64*>(partial + ((size_t)(zz < ksplit ? zz : 0) * 64 + row) * 64 + (lane_on ? fc : 0) + 4 * q);
        bits[zz][0] = __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        bits[zz][1] = __hip_atomic_load(p + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      floatx4 sum = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int zz = 0; zz < kMaxSplit; ++zz)
        if (zz < ksplit) sum += __builtin_bit_cast(floatx4, bits[zz]);
      v[it][q] = sum;
    }
  }
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    float y[FPL];
#pragma unroll
    for (int q = 0; q < FPL / 4; ++q)
#pragma unroll
      for (int e = 0; e < 4; ++e) y[4 * q + e] = v[it][q][e] * ss.sc[4 * q + e] + ss.sh[4 * q + e];
    if (res) {
#pragma unroll
      for (int e = 0; e < FPL; ++e) y[e] += (float)rv[it][e];
    }
    if (relu == kActRelu) {
#pragma unroll
      for (int e = 0; e < FPL; ++e) y[e] = relu_ugt(y[e]);
    }
    VO ov;
#pragma unroll
    for (int e = 0; e < FPL; ++e) ov[e] = (OutT)y[e];
    if (o[it] >= 0) *reinterpret_cast<VO*>(out + (long long)o[it] + f0 + fc) = ov;
  }
}

template <int WS, int WK, int ST = 1>
struct PatchCfg {
  static constexpr int NW = WS * WK, NT = 64 * NW;
  // padded patch pixels the loader can walk.  A stride-2 tile reads four input pixels per output
  // pixel: its patch is about four times the size for the same number of slots.
  static constexpr int cover = ST == 2 ? (WS == 2 ? 576 : 288) : WS == 4 ? 384 : WS == 2 ? 256 : 192;
  static constexpr int passes = cover / (NT / 8);  // loader passes per thread: NT/8 pixels each
  static constexpr int nset = WK == 4 ? 9 : 3;  // weight register sets = taps in flight; divides 9
  static constexpr int cap = ST == 2 ? (WS == 2 ? 522 : 288) : PatchCap<WS>::pix;
  // instances whose tap loop keeps no patch prefetch registers alive: single-slab layers only
  static constexpr bool reload = ST == 2 ? WS == 1 : WS != 4;
  static constexpr int patch_bytes = cap * kPitch;
  static constexpr int load_bytes = patch_bytes + NT * 16;  // + one dump slot per thread
  static constexpr int tile_bytes = WS * WK * kTileBytes;  // one copy per K group
  static constexpr int smem = load_bytes > tile_bytes ? load_bytes : tile_bytes;
};

// The auxiliary 1x1 stride-2 filter blocks of a stride-2 launch.  Their pixels are the centre taps
// of the tile's slots, so the "patch" is just those 64*WS pixels, one LDS cell per slot, and the
// walk is one tap per slab.  A ninth of the work of a 3x3 block: these workgroups have the highest
// block indices and fill the tail of the launch.
template <typename T, typename OutT, int WS, int WK, int NI>
__device__ __forceinline__ void patch_aux_1x1(const PatchArgs& a, unsigned char* smem, int n0, int y0, int x0, int fb, int tid) {
  constexpr int NT = 64 * WS * WK, ES = sizeof(T), KPG = 4 / WK;
  constexpr int AP = 64 * WS / (NT / 8);  // loader passes: NT/8 pixels each
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ws = wave % WS, wk = wave / WS;
  const int lrow = lane & 31, lchunk = lane >> 5;
  const __amdgpu_buffer_rsrc_t rs_in = make_rsrc(a.in, a.in_bytes);
  const __amdgpu_buffer_rsrc_t rs_wf = make_rsrc(a.aux_wf, a.aux_wf_bytes);
  const int nslab = a.C * ES / 128;
  const int TW = a.txw & 0xffff;
  const int nslots = a.TN * a.TH * TW;
  auto decode = [&](int sl, int* n, int* oy, int* ox) {
    int nl = 0, rem = sl, tx;
    if (a.TN > 1) nl = fast_div(sl, a.TH * TW, a.inv_thw, &rem);
    const int ty = fast_div(rem, TW, a.inv_w, &tx);
    *n = n0 + nl;
    *oy = y0 + ty;
    *ox = x0 + tx;
    return (sl < nslots) & (*n < a.N) & (*oy < a.OH) & (*ox < a.OW);
  };
  const int p8 = tid >> 3, pc = (tid & 7) * 16;
  const unsigned ces = (unsigned)(a.pix * ES);
  unsigned aoff[AP];
#pragma unroll
  for (int i = 0; i < AP; ++i) {
    int n, oy, ox;
    const bool ok = decode(i * (NT / 8) + p8, &n, &oy, &ox);
    aoff[i] = ok ? __umul24((unsigned)((n * a.H + 2 * oy) * a.W + 2 * ox), ces) + pc : kOOBp;
  }
  u32x4 aregs[AP];
  auto aload = [&](int slab) {
#pragma unroll
    for (int i = 0; i < AP; ++i) aregs[i] = __builtin_amdgcn_raw_buffer_load_b128(rs_in, aoff[i] + slab * 128, 0, 0);
  };
  auto astore = [&]() {
#pragma unroll
    for (int i = 0; i < AP; ++i) *reinterpret_cast<u32x4*>(smem + (i * (NT / 8) + p8) * kPitch + pc) = aregs[i];
  };
  aload(0);
  const int wbase = NI == 2 ? (fb * nslab * 8 + wk * KPG * 2) * 1024 : ((fb >> 1) * nslab * 8 + wk * KPG * 2 + (fb & 1)) * 1024;
  const unsigned wlane = lane * 16;
  EpiScale<OutT> ess;
  ess.load(lane, fb * (32 * NI), a.aux_F, a.aux_scale, a.aux_shift);
  int cell[2], obase[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int sl = ws * 64 + j * 32 + lrow;
    int n, oy, ox;
    const bool ok = decode(sl, &n, &oy, &ox);
    cell[j] = sl * kPitch + (lchunk + 2 * wk * KPG) * 16;
    obase[j] = ok ? ((n * a.OH + oy) * a.OW + ox) * a.aux_F : -1;
  }
  floatx16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;
  astore();
  __syncthreads();
  for (int slab = 0; slab < nslab; ++slab) {
    const bool more = slab + 1 < nslab;
    if (more) aload(slab + 1);
    u32x4 w[KPG][NI];
#pragma unroll
    for (int k = 0; k < KPG; ++k)
#pragma unroll
      for (int i = 0; i < NI; ++i)
        w[k][i] = __builtin_amdgcn_raw_buffer_load_b128(rs_wf, wlane, wbase + slab * 8192 + (k * 2 + i) * 1024, 0);
#pragma unroll
    for (int k = 0; k < KPG; ++k) {
      u32x4 p[2];
#pragma unroll
      for (int j = 0; j < 2; ++j) p[j] = *reinterpret_cast<const u32x4*>(smem + cell[j] + k * 32);
#pragma unroll
      for (int i = 0; i < NI; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) Mma<T>::run(w[k][i], p[j], acc[i][j]);
    }
    if (more) {
      __syncthreads();  // every wave is done with this slab's pixels
      astore();
      __syncthreads();
    }
  }
  __syncthreads();  // LDS becomes the output tiles
  tile_reduce_store<OutT, WK, NI, false>(acc, smem + ws * WK * kTileBytes, wk, lane, obase, fb * (32 * NI), a.aux_F, ess,
                                         static_cast<const OutT*>(nullptr), static_cast<OutT*>(a.aux_out), a.aux_relu);
}

// ACT: the epilogue knows every fused activation (and the residual-after-activation form); without
// it only ReLU / none, which keeps the register-tight ResNet instances as they were.
template <typename T, typename OutT, int WS, int WK, int NI, int ST, bool SK, bool ACT>
__global__ __launch_bounds__(64 * WS * WK) __attribute__((amdgpu_waves_per_eu(2, 2))) void conv3x3_patch_kernel(
    // the values the patch addressing needs first, as plain leading arguments: those are preloaded
    // into SGPRs at wave launch, the struct behind them is fetched by a scalar load as usual
    const void* in_p, int tiles_p, int tiles_y_p, int tn_p, int th_p, int n_p, int h_p, int w_p, int c_p, int rw_log_p,
    int xcd_by_filter_p, unsigned in_bytes_p, int txw_p, const PatchArgs a_rest) {
  PatchArgs a = a_rest;
  a.txw = txw_p;
  a.in = in_p; a.tiles = tiles_p; a.tiles_y = tiles_y_p; a.TN = tn_p; a.TH = th_p; a.N = n_p; a.H = h_p; a.W = w_p; a.C = c_p;
  a.rw_log = rw_log_p; a.xcd_by_filter = xcd_by_filter_p; a.in_bytes = in_bytes_p;
  typedef PatchCfg<WS, WK, ST> Cfg;
  static_assert(ST == 1 || ST == 2, "stride 1 or 2");
  constexpr int NT = Cfg::NT, kPasses = Cfg::passes, NSET = Cfg::nset;
  constexpr int kDepth = WK == 1 ? 3 : 4;  // pixel-operand ring: LDS reads run kDepth-1 steps ahead of their MFMAs
  constexpr int ES = sizeof(T);
  constexpr int KPG = 4 / WK;     // 32-byte K sub-steps per K group and tap
  constexpr int NF = NI * KPG;    // weight fragments (kilobytes) per wave and tap
  static_assert(NI == 1 || NI == 2, "a wave owns one or two 32-filter halves");
  static_assert(WK == 1 || WK == 2 || WK == 4, "K groups split the four sub-steps of a tap");
  extern __shared__ __align__(16) unsigned char smem[];
  unsigned char* patch = smem;

  // Workgroups are dealt to the 8 XCDs (each with its own L2) round-robin by linear id.  Normally an
  // XCD takes a contiguous range of pixel tiles (neighbouring tiles share halo rows); when the
  // filters outgrow one L2 it takes one 64-filter block instead, so that its weights stay resident.
  int tile, fblk;
  if (a.xcd_by_filter) {
    const int lin = blockIdx.y * gridDim.x + blockIdx.x, per = gridDim.y / kXcdsP;
    const int k = lin / kXcdsP;
    fblk = lin % kXcdsP + kXcdsP * (k % per);
    tile = k / per;
  } else {
    const int per_xcd = (a.tiles + kXcdsP - 1) / kXcdsP;
    tile = (blockIdx.x % kXcdsP) * per_xcd + blockIdx.x / kXcdsP;
    fblk = blockIdx.y;
  }
  if (tile >= a.tiles) return;
  const int f0blk = fblk * (32 * NI);
  // tile -> image group, row band, column tile (one column tile unless the rows are too wide)
  const int TW = a.txw & 0xffff, ntx = a.txw >> 16;
  const int n0 = (tile / a.tiles_y) * a.TN;
  int band = tile % a.tiles_y, x0 = 0;
  if (ntx > 1) {
    x0 = (band % ntx) * TW;
    band /= ntx;
  }
  const int y0 = band * a.TH;
  if constexpr (ST == 2) {
    if (fblk >= a.aux_fb0) {  // uniform for the workgroup
      if (SK && blockIdx.z != 0) return;  // the auxiliary blocks do not split K
      patch_aux_1x1<T, OutT, WS, WK, NI>(a, smem, n0, y0, x0, fblk - a.aux_fb0, threadIdx.x);
      return;
    }
  }
  // Stride 2: output row ty / column tx of the tile reads patch rows 2ty..2ty+2 and columns
  // 2tx..2tx+2.  The patch keeps the even and the odd columns of a row apart (PWh pixels each), so
  // that the slots of consecutive output pixels stay consecutive in LDS for every tap.
  const int OH = ST == 1 ? a.H : a.OH, OW = ST == 1 ? a.W : a.OW;
  const int PH = ST == 1 ? a.TH + 2 : 2 * a.TH + 1, PW = ST == 1 ? TW + 2 : 2 * TW + 1;
  const int PWh = TW + 1;
  // Stride 1: consecutive slots wrap from the end of one tile row to the start of the next, and a 16-byte LDS read of a
  // wave is free of bank conflicts when the 16-byte units of the slots continue the sequence of a row (9 units per
  // slot) across the wrap.  A patch row is TW + 2 cells, two more than the tile row: with 14 spare units behind it the
  // row pitch is 9 * TW units mod 16.  (7x7 tiles: 40 % of the LDS cycles of a launch were conflict cycles without it.)
  const int RP = PW * kPitch + (ST == 1 ? a.rowx : 0);  // bytes from one patch row to the next (stride 1)

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform, kept in an SGPR
  const int ws = wave % WS, wk = wave / WS;
  const int lrow = lane & 31, lchunk = lane >> 5;
  const __amdgpu_buffer_rsrc_t rs_in = make_rsrc(a.in, a.in_bytes);
  const __amdgpu_buffer_rsrc_t rs_wf = make_rsrc(a.wf, a.wf_bytes);
  // The widest tile keeps no patch prefetch registers alive in the tap loop: the host only picks it
  // for single-slab layers, and its loop never reloads the patch.
  constexpr bool kReload = Cfg::reload;
  const int nslab_all = a.C * ES / 128;
  const int slab0 = SK ? (int)blockIdx.z * a.spk : 0;  // this workgroup's first slab and how many it walks
  const int nslab = SK ? min(a.spk, nslab_all - slab0) : nslab_all;
  const int niter = nslab * 9;  // one iteration = one tap of one slab

  // ---- patch loader: 8 threads per pixel, NT/8 pixels per pass; the patch is walked as rows of
  //      2^rw_log pixels (>= W+2), so row and column of a pass are shifts and masks ----
  const int p8 = tid >> 3, pc = (tid & 7) * 16;
  const int prows = a.TN * PH;
  const int rwm = (1 << a.rw_log) - 1;
  const unsigned ces = (unsigned)(a.pix * ES);
  unsigned pvoff[kPasses];
  if (a.TN == 1) {  // one image per tile: patch row r is image row y0 - 1 + r
    const int rowbase = (n0 * a.H + ST * y0 - 1) * a.W + ST * x0 - 1;
#pragma unroll
    for (int i = 0; i < kPasses; ++i) {
      const int q = i * (NT / 8) + p8;
      const int r = q >> a.rw_log, px = q & rwm;
      const bool ok = (r < prows) & ((unsigned)(ST * y0 - 1 + r) < (unsigned)a.H) & ((unsigned)(ST * x0 + px - 1) < (unsigned)a.W);
      const unsigned off = __umul24((unsigned)(rowbase + (int)__umul24(r, a.W) + px), ces) + pc;
      pvoff[i] = ok ? off : kOOBp;
    }
  } else {
#pragma unroll
    for (int i = 0; i < kPasses; ++i) {
      const int q = i * (NT / 8) + p8;
      const int r = q >> a.rw_log, px = q & rwm;
      int py;
      const int n = n0 + fast_div(r, PH, a.inv_ph, &py);
      const int iy = ST * y0 + py - 1;
      const bool ok = (r < prows) & (n < a.N) & ((unsigned)iy < (unsigned)a.H) & ((unsigned)(ST * x0 + px - 1) < (unsigned)a.W);
      const unsigned off = __umul24((unsigned)((n * a.H + iy) * a.W + ST * x0 + px - 1), ces) + pc;
      pvoff[i] = ok ? off : kOOBp;
    }
  }
  u32x4 pregs[kPasses];
  auto pload = [&](int slab) {
#pragma unroll
    for (int i = 0; i < kPasses; ++i) pregs[i] = __builtin_amdgcn_raw_buffer_load_b128(rs_in, pvoff[i] + (slab0 + slab) * 128, 0, 0);
  };
  // Lanes whose pass lies outside the patch store to a private dump slot behind it: no divergence.
  const int dump = Cfg::patch_bytes + tid * 16;
  auto pstore = [&]() {
#pragma unroll
    for (int i = 0; i < kPasses; ++i) {
      const int q = i * (NT / 8) + p8;
      const int r = q >> a.rw_log, px = q & rwm;
      const int dst = (ST == 1 ? (int)__umul24(r, RP) + (int)__umul24(px, kPitch)
                               : (int)__umul24(__umul24(2 * r + (px & 1), PWh) + (px >> 1), kPitch)) + pc;
      *reinterpret_cast<u32x4*>(patch + (((px < PW) & (r < prows)) ? dst : dump)) = pregs[i];
    }
  };
  pload(0);  // first in the queue: the patch gates the tap loop, the weights below only its first taps
  __builtin_amdgcn_sched_barrier(0);

  // ---- weights: iteration `it`, sub-step k of this K group, filter half i of 64-filter block fb is
  //      the kilobyte at (fb*niter*8 + it*8 + k*2 + i)*1024; NSET register sets hold iterations
  //      it .. it+NSET-1.  An NI = 1 workgroup owns one half of a 64-filter block. ----
  const int niter_all = nslab_all * 9;
  const int wbase = (NI == 2 ? (fblk * niter_all * 8 + wk * KPG * 2) * 1024 : ((fblk >> 1) * niter_all * 8 + wk * KPG * 2 + (fblk & 1)) * 1024) +
                    slab0 * 9 * 8192;
  const unsigned wlane = lane * 16;
  auto wfrag = [](int k, int i) { return (k * 2 + i) * 1024; };  // byte offset of fragment (k, i) inside an iteration
  auto wload = [&](u32x4(&r)[NF], int it) {
    const int so = it < niter ? wbase + it * 8192 : 0;  // past the end: re-read block 0 (never used)
#pragma unroll
    for (int k = 0; k < KPG; ++k)
#pragma unroll
      for (int i = 0; i < NI; ++i) r[k * NI + i] = __builtin_amdgcn_raw_buffer_load_b128(rs_wf, wlane, so + wfrag(k, i), 0);
  };
  u32x4 wregs[NSET][NF];
#pragma unroll
  for (int q = 0; q < NSET; ++q) wload(wregs[q], q);

  // epilogue scale/shift of this lane's output channels: requested now, used at the very end --
  // except in the instances whose tap loop has no 16 registers to spare for them (they would be
  // spilled to scratch memory around the loop: a wait for every load in flight at the loop's door
  // and 13 KB of extra HBM writes per workgroup), which request them behind the loop instead
  constexpr bool kLateScale = sizeof(T) == 2 && (WS == 4 || (ST == 2 && WS == 1 && NI == 2));
  EpiScale<OutT> ess;
  if constexpr (!kLateScale) ess.load(lane, f0blk, a.F, a.scale, a.shift);

  // ---- this lane's two pixel slots ----
  const int nslots = a.TN * a.TH * TW;
  int sbase[2];  // byte offset of the slot's tap-(0,0) pixel in the patch
  int obase[2];  // element offset of the slot's output pixel row, or -1
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int sl0 = ws * 64 + j * 32 + lrow;
    // a slot beyond the tile reads with the slot 16, 32 ... before it (the same LDS banks as if it had a pixel: fifteen
    // lanes on one cell were a bank conflict per read on 7x7 tiles); its results are never stored
    int sl = sl0;
    if (sl0 >= nslots) {
      const int back = (((sl0 - nslots) >> 4) + 1) << 4;
      sl = sl0 >= back ? sl0 - back : 0;
    }
    int nl = 0, rem = sl, tx;
    if (a.TN > 1) nl = fast_div(sl, a.TH * TW, a.inv_thw, &rem);
    const int ty = fast_div(rem, TW, a.inv_w, &tx);
    const bool ok = (sl < nslots) & ((n0 + nl) < a.N) & ((y0 + ty) < OH) & ((x0 + tx) < OW);
    // slots whose pixel lies outside the image read pixel 0 of the patch
    const int celloff = ST == 1 ? (int)__umul24(__umul24(nl, PH) + ty, RP) + (int)__umul24(tx, kPitch)
                                : (int)__umul24(__umul24(__umul24(nl, PH) + 2 * ty, 2 * PWh) + tx, kPitch);
    sbase[j] = (ok ? celloff : 0) + (lchunk + 2 * wk * KPG) * 16;
    obase[j] = (ok && sl0 < nslots) ? (((n0 + nl) * OH + y0 + ty) * OW + x0 + tx) * a.ldo : -1;
  }

  // [filter half][pixel half]; with NI = 1 only acc[0] is used.  The first step of the first slab starts the sums from a
  // zero C operand: clearing the registers instead cost 64 moves between the patch barrier and the first MFMA.
  // (fp16 instances; the fp32 ones, four chained MFMAs per product, are at their register limit and keep the moves.)
  constexpr bool kZeroC = sizeof(T) == 2;
  floatx16 acc[2][2];
#pragma unroll
  for (int i = kZeroC ? 1 : 0; i < 2; ++i)  // fp16, NI = 1: acc[1] is never written by an MFMA and never read for a result
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  // ---- tap loop.  One trip = one slab = 9 taps x KPG K sub-steps ("steps"), fully unrolled, so
  // that tap offsets, weight register sets (NSET divides 9) and the ring slot of the pixel
  // operands are all static.  Per step: four MFMAs; the pixel operands come from LDS kDepth-1
  // steps ahead, a weight register is refilled (NSET taps ahead) right after its last use.
  // Scheduling fences pin that software pipeline: left alone, the scheduler sinks both kinds of
  // load to just before their consumers and the loop runs at memory latency.
  constexpr int kSteps = 9 * KPG;
  int rowbase[3][2];  // slot base + filter row r
#pragma unroll
  for (int r = 0; r < 3; ++r)
#pragma unroll
    for (int j = 0; j < 2; ++j) rowbase[r][j] = sbase[j] + r * (ST == 1 ? RP : 2 * PWh * kPitch);
  const int odd_col = PWh * kPitch;  // stride 2: from an even column to the odd one right of it
  u32x4 ring[kDepth][2];
  auto ldp = [&](auto step_c) {
    constexpr int st = decltype(step_c)::value;
    constexpr int t = st / KPG, k = st % KPG;
#pragma unroll
    for (int j = 0; j < 2; ++j)
      if constexpr (ST == 1)
        ring[st % kDepth][j] = *reinterpret_cast<const u32x4*>(patch + rowbase[t / 3][j] + (t % 3) * kPitch + k * 32);
      else  // filter columns 0, 1, 2 = even column, the odd one after it, the next even one
        ring[st % kDepth][j] = *reinterpret_cast<const u32x4*>(patch + rowbase[t / 3][j] + (t % 3 == 1 ? odd_col : 0) + (t % 3 == 2 ? kPitch : 0) + k * 32);
  };
  auto ldp1 = [&](auto step_c, int j) {
    constexpr int st = decltype(step_c)::value;
    constexpr int t = st / KPG, k = st % KPG;
    if constexpr (ST == 1)
      ring[st % kDepth][j] = *reinterpret_cast<const u32x4*>(patch + rowbase[t / 3][j] + (t % 3) * kPitch + k * 32);
    else
      ring[st % kDepth][j] = *reinterpret_cast<const u32x4*>(patch + rowbase[t / 3][j] + (t % 3 == 1 ? odd_col : 0) + (t % 3 == 2 ? kPitch : 0) + k * 32);
  };
  // the fp16 instances spread a step's other instructions between its MFMAs (see the tap loop)
  constexpr bool kSpread = sizeof(T) == 2;
  auto prime = [&](auto self, auto d_c) -> void {  // the first kDepth-1 steps of a fresh patch
    constexpr int d = decltype(d_c)::value;
    if constexpr (d < kDepth - 1) {
      ldp(d_c);
      __builtin_amdgcn_sched_barrier(0);  // in step order: left alone the compiler issued the first step's reads last
      self(self, std::integral_constant<int, d + 1>());
    }
  };

  pstore();
  __syncthreads();
  prime(prime, std::integral_constant<int, 0>());

  for (int slab = 0; slab < nslab; ++slab) {
    const bool more = kReload && slab + 1 < nslab;
    if (kReload && more) pload(slab + 1);  // lands after the last tap of this slab
    auto steps = [&](auto self, auto step_c) -> void {
      constexpr int st = decltype(step_c)::value;
      if constexpr (st < kSteps) {
        constexpr int t = st / KPG, k = st % KPG, set = t % NSET;
        const int it_next = slab * 9 + t + NSET;
        const int wso = it_next < niter ? wbase + it_next * 8192 : 0;  // past the end: re-read block 0 (never used)
        if constexpr (kSpread) {
          // every MFMA is followed by its share of the step's other instructions (an LDS read of the step kDepth - 1
          // ahead, a weight refill), so that they issue under it instead of behind the four: 7x7x512 at batch 32
          // 13.3 -> 12.9 us (one wave per SIMD), the stride-2 launches 10.0 -> 9.4, 56x56x64 14.4 -> 14.05
#pragma unroll
          for (int i = 0; i < NI; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
              if (kZeroC && st == 0 && slab == 0) Mma<T>::start(wregs[set][k * NI + i], ring[st % kDepth][j], acc[i][j]);
              else Mma<T>::run(wregs[set][k * NI + i], ring[st % kDepth][j], acc[i][j]);
              __builtin_amdgcn_sched_barrier(0);
              if constexpr (st + kDepth - 1 < kSteps) {
                if (i == 0) ldp1(std::integral_constant<int, st + kDepth - 1>(), j);
              }
              if (j == 1) wregs[set][k * NI + i] = __builtin_amdgcn_raw_buffer_load_b128(rs_wf, wlane, wso + wfrag(k, i), 0);
              __builtin_amdgcn_sched_barrier(0);
            }
        } else {
          if constexpr (st + kDepth - 1 < kSteps) ldp(std::integral_constant<int, st + kDepth - 1>());
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int i = 0; i < NI; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
              if (kZeroC && st == 0 && slab == 0) Mma<T>::start(wregs[set][k * NI + i], ring[st % kDepth][j], acc[i][j]);
              else Mma<T>::run(wregs[set][k * NI + i], ring[st % kDepth][j], acc[i][j]);
            }
#pragma unroll
          for (int i = 0; i < NI; ++i)
            wregs[set][k * NI + i] = __builtin_amdgcn_raw_buffer_load_b128(rs_wf, wlane, wso + wfrag(k, i), 0);
          __builtin_amdgcn_sched_barrier(0);
        }
        self(self, std::integral_constant<int, st + 1>());
      }
    };
    steps(steps, std::integral_constant<int, 0>());
    if (kReload && more) {
      __syncthreads();  // every wave is done with the old patch
      pstore();
      __syncthreads();
      prime(prime, std::integral_constant<int, 0>());
    }
  }
  // ---- inline form of the auxiliary 1x1 stride-2 filters: this workgroup's own block of them, computed after its
  //      3x3 block.  Its operands (the centre pixels of the slots, every slab at once, and all its weight
  //      fragments) are requested here and arrive under the epilogue of the 3x3 block. ----
  constexpr int AP = 64 * WS / (NT / 8);       // loader passes over the slots: NT/8 pixels each
  constexpr int kAuxSlabs = WS == 1 ? 4 : 1;   // slabs the inline form holds in registers
  u32x4 aregs[kAuxSlabs][AP];
  u32x4 awreg[kAuxSlabs][NF];
  EpiScale<OutT> aess;
  if constexpr (ST == 2) {
    if (a.aux_inline) {
      const __amdgpu_buffer_rsrc_t rs_awf = make_rsrc(a.aux_wf, a.aux_wf_bytes);
#pragma unroll
      for (int i = 0; i < AP; ++i) {
        const int sl = i * (NT / 8) + p8;
        int nl = 0, rem = sl, tx;
        if (a.TN > 1) nl = fast_div(sl, a.TH * TW, a.inv_thw, &rem);
        const int ty = fast_div(rem, TW, a.inv_w, &tx);
        const bool ok = (sl < nslots) & ((n0 + nl) < a.N) & ((y0 + ty) < OH) & ((x0 + tx) < OW);
        const unsigned off = __umul24((unsigned)(((n0 + nl) * a.H + 2 * (y0 + ty)) * a.W + 2 * (x0 + tx)), ces) + pc;
#pragma unroll
        for (int sb = 0; sb < kAuxSlabs; ++sb)
          aregs[sb][i] = __builtin_amdgcn_raw_buffer_load_b128(rs_in, ok && sb < nslab_all ? off + sb * 128 : kOOBp, 0, 0);
      }
      const int awbase = NI == 2 ? (fblk * nslab_all * 8 + wk * KPG * 2) * 1024 : ((fblk >> 1) * nslab_all * 8 + wk * KPG * 2 + (fblk & 1)) * 1024;
#pragma unroll
      for (int sb = 0; sb < kAuxSlabs; ++sb)
#pragma unroll
        for (int k = 0; k < KPG; ++k)
#pragma unroll
          for (int i = 0; i < NI; ++i)
            awreg[sb][k * NI + i] = __builtin_amdgcn_raw_buffer_load_b128(rs_awf, wlane, sb < nslab_all ? awbase + sb * 8192 + wfrag(k, i) : 0, 0);
      aess.load(lane, f0blk, a.aux_F, a.aux_scale, a.aux_shift);
    }
  }
  if constexpr (kLateScale) ess.load(lane, f0blk, a.F, a.scale, a.shift);
  __syncthreads();  // every wave is done with the patch: LDS becomes the output tiles

  if constexpr (SK) {
    const int wg = tile * gridDim.y + fblk;
    tile_reduce_store_splitk<OutT, WK, NI>(acc, smem + ws * WK * kTileBytes, wk, lane, tid, obase, f0blk, a.F, ess,
                                           static_cast<const OutT*>(a.residual), static_cast<OutT*>(a.out), a.relu,
                                           a.partial + (size_t)wg * a.ksplit * 4096, a.counters + wg, blockIdx.z, a.ksplit);
  } else {
    tile_reduce_store<OutT, WK, NI, ACT>(acc, smem + ws * WK * kTileBytes, wk, lane, obase, f0blk, a.F, ess,
                                         static_cast<const OutT*>(a.residual), static_cast<OutT*>(a.out), a.relu);
  }
  if constexpr (ST == 2 && !SK) {
    if (a.aux_inline) {
      __syncthreads();  // the output tiles have been read: LDS becomes the slots' centre pixels, [slot][slab][64 ch] + 16 pad
      const int apitch = nslab_all * 128 + 16;
#pragma unroll
      for (int i = 0; i < AP; ++i)
#pragma unroll
        for (int sb = 0; sb < kAuxSlabs; ++sb)
          if (sb < nslab_all) *reinterpret_cast<u32x4*>(smem + (i * (NT / 8) + p8) * apitch + sb * 128 + pc) = aregs[sb][i];
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;
      __syncthreads();
#pragma unroll
      for (int sb = 0; sb < kAuxSlabs; ++sb)
        if (sb < nslab_all) {  // uniform
#pragma unroll
          for (int k = 0; k < KPG; ++k) {
            u32x4 p[2];
#pragma unroll
            for (int j = 0; j < 2; ++j)
              p[j] = *reinterpret_cast<const u32x4*>(smem + (ws * 64 + j * 32 + lrow) * apitch + sb * 128 + (lchunk + 2 * wk * KPG) * 16 + k * 32);
#pragma unroll
            for (int i = 0; i < NI; ++i)
#pragma unroll
              for (int j = 0; j < 2; ++j) Mma<T>::run(awreg[sb][k * NI + i], p[j], acc[i][j]);
          }
        }
      __syncthreads();  // every wave is done with the pixels: LDS becomes the output tiles again
      tile_reduce_store<OutT, WK, NI, false>(acc, smem + ws * WK * kTileBytes, wk, lane, obase, f0blk, a.aux_F, aess,
                                             static_cast<const OutT*>(nullptr), static_cast<OutT*>(a.aux_out), a.aux_relu);
    }
  }
}

// Tile choice for 64*ws slots: TN images x TH output rows x TW output columns, patch of at most
// `cap` cells, which the loader walks as rows of 2^rw_log <= 64 pixels, `cover` padded pixels at
// most.  H, W: output size (= input size at stride 1).  Rows whose patch is wider than the loader
// takes are cut into NTX column tiles of equal width.
struct TilePlan { int TN, TH, TW, NTX, rw_log; };
constexpr int kRowSpare = 14 * 16;  // (9 * TW - 9 * (TW + 2)) mod 16 units of 16 bytes
static bool plan_tile_ntx(int st, int N, int H, int W_full, int ntx, int slots, int cap, int cover, TilePlan* t) {
  const int W = (W_full + ntx - 1) / ntx;
  const int PW = st == 1 ? W + 2 : 2 * W + 1;       // patch columns the loader walks
  const int cells = st == 1 ? W + 2 : 2 * (W + 1);  // LDS cells per patch row
  auto prow = [&](int th) { return st == 1 ? th + 2 : 2 * th + 1; };
  int lg = 0;
  while ((1 << lg) < PW) ++lg;
  if ((1 << lg) > 64 || W > slots) return false;
  const int max_rows = cover >> lg;  // patch rows the loader can cover
  // stride 1: every patch row carries kRowSpare spare bytes (the kernel's conflict-free row pitch)
  auto fits = [&](int tn, int th) {
    return tn * th * W <= slots && tn * prow(th) * (cells * kPitch + (st == 1 ? kRowSpare : 0)) <= cap * kPitch && tn * prow(th) <= max_rows;
  };
  int thmax = 0;
  for (int th = 1; th <= H; ++th)
    if (fits(1, th)) thmax = th;
  if (thmax == 0) return false;
  t->rw_log = lg; t->TW = W; t->NTX = ntx; t->TN = 1;
  if (thmax < H) {
    const int nt = (H + thmax - 1) / thmax;
    t->TH = (H + nt - 1) / nt;  // balanced rows per tile
    return true;
  }
  t->TH = H;
  if (ntx == 1)
    while (t->TN + 1 <= N && fits(t->TN + 1, H)) ++t->TN;
  return true;
}

static bool plan_tile(int st, int N, int H, int W, int slots, int cap, int cover, TilePlan* t) {
  const int max_tw = std::min(slots, st == 1 ? 62 : 31);
  const int ntx0 = (W + max_tw - 1) / max_tw;
  // The loader walks the patch as rows of a power of two, so the widest cut is not always the one
  // that fills the slots best (40 columns: a 42-wide patch is walked as 64 and leaves room for two
  // output rows, 80 of 128 slots; two column tiles of 20 take six rows, 120 slots).  Try a few cuts
  // and keep the one with the fewest tiles; ties go to the wider tile (less halo).
  long long best_tiles = 0;
  for (int ntx = ntx0; ntx <= ntx0 + 6 && ntx <= W; ++ntx) {
    TilePlan c;
    if (!plan_tile_ntx(st, N, H, W, ntx, slots, cap, cover, &c)) continue;
    const long long tiles = (long long)((N + c.TN - 1) / c.TN) * ((H + c.TH - 1) / c.TH) * ntx;
    if (best_tiles == 0 || tiles < best_tiles) {
      best_tiles = tiles;
      *t = c;
    }
  }
  return best_tiles > 0;
}

// Picks the wave arrangement: the largest pixel tile that still gives (about) every CU a workgroup.
static bool plan_patch(int st, int N, int H, int W, int F, int slabs, int* WS, TilePlan* plan) {
  static const int force = [] {
    const char* e = getenv("NNCV_HIP_PATCH_WS");
    return e ? atoi(e) : 0;
  }();
  const int fb = (F + 63) / 64;
  // Score = fraction of the MFMA slots that carry real pixels x fraction of the 256 CUs that get
  // a workgroup.  A narrower tile has to beat a wider one by a quarter: its workgroups re-read the
  // weights more often, split K across waves and pay the fixed prologue / epilogue per fewer
  // MFMAs (measured on 56x56x64 at batch 32: 15.8 / 17.1 / 20.7 us for 256 / 128 / 64 slots, and the
  // same order on 28x28x128, 14x14x256, 80x80x64 and 40x40x128; 64 slots win where the wider tiles
  // leave CUs idle, 7x7x512 and small batches).
  double best = 0.0;
  for (int ws : {4, 2, 1}) {
    if (force && ws != force) continue;
    int cap, cover;
    if (st == 1) {
      if (ws == 4 && slabs != 1) continue;  // the WS=4 instance handles one slab
      cap = ws == 4 ? PatchCfg<4, 1>::cap : ws == 2 ? PatchCfg<2, 2>::cap : PatchCfg<1, 4>::cap;
      cover = ws == 4 ? PatchCfg<4, 1>::cover : ws == 2 ? PatchCfg<2, 2>::cover : PatchCfg<1, 4>::cover;
    } else {
      if (ws == 4 || (ws == 2 && slabs != 1)) continue;  // stride 2: the WS=2 instance handles one slab
      cap = ws == 2 ? PatchCfg<2, 2, 2>::cap : PatchCfg<1, 4, 2>::cap;
      cover = ws == 2 ? PatchCfg<2, 2, 2>::cover : PatchCfg<1, 4, 2>::cover;
    }
    TilePlan t;
    if (!plan_tile(st, N, H, W, 64 * ws, cap, cover, &t)) continue;
    const long long tiles = (long long)((N + t.TN - 1) / t.TN) * ((H + t.TH - 1) / t.TH) * t.NTX;
    const double used = (double)N * H * W / ((double)tiles * 64 * ws);
    // "every CU busy" saturates at 7/8 of them: past that a narrower tile only adds halo re-reads
    const double fill = tiles * fb >= 224 ? 1.0 : (double)(tiles * fb) / 224.0;
    const double score = used * fill;
    if (score > best * 1.25) {
      best = score; *WS = ws; *plan = t;
    }
  }
  return best > 0.0;
}

bool conv3x3_patch_plan(int stride, int N, int OH, int OW, int F, int slabs, int out[8]) {
  int ws = 0;
  TilePlan t{};
  if ((stride != 1 && stride != 2) || N < 1 || OH < 1 || OW < 1 || F < 1 || slabs < 1 || !plan_patch(stride, N, OH, OW, F, slabs, &ws, &t))
    return false;
  out[0] = ws; out[1] = t.TN; out[2] = t.TH; out[3] = t.TW; out[4] = t.NTX; out[5] = t.rw_log;
  if (stride == 1) {
    out[6] = ws == 4 ? PatchCfg<4, 1>::cap : ws == 2 ? PatchCfg<2, 2>::cap : PatchCfg<1, 4>::cap;
    out[7] = ws == 4 ? PatchCfg<4, 1>::cover : ws == 2 ? PatchCfg<2, 2>::cover : PatchCfg<1, 4>::cover;
  } else {
    out[6] = ws == 2 ? PatchCfg<2, 2, 2>::cap : PatchCfg<1, 4, 2>::cap;
    out[7] = ws == 2 ? PatchCfg<2, 2, 2>::cover : PatchCfg<1, 4, 2>::cover;
  }
  return true;
}

bool conv3x3_patch_applicable(const IgemmArgs& a, int in_dt) {
  static const bool off = getenv("NNCV_HIP_NO_PATCH") != nullptr;
  const int slab = in_dt == kF16 ? 64 : 32;
  int ws;
  TilePlan tp;
  static const bool off2 = getenv("NNCV_HIP_NO_PATCH_S2") != nullptr;
  const int st = a.stride_h;
  // auxiliary filters: the centre tap of a stride-2 launch, given fragment-major
  const int fmain = a.aux_f0 ? a.aux_f0 : a.F, faux = a.F - fmain;
  const bool aux_ok = a.aux_f0 == 0 || (st == 2 && a.aux_tap == 4 && a.aux_wt_frag && a.aux_out && a.aux_relu <= kActRelu && a.aux_f0 % 64 == 0 &&
                                        faux % 8 == 0 && a.aux_ldo == faux);
  // other activations than ReLU (and the residual added after them): fp16 instances only
  static const bool off_act = getenv("NNCV_HIP_NO_PATCH_ACT") != nullptr;
  const bool act_ok = a.relu <= kActRelu || (in_dt == kF16 && !off_act && a.aux_f0 == 0 && (a.relu & 0xff) <= kActSigmoid &&
                                             (a.relu & ~(0xff | kActResidualAfter)) == 0);
  const int pix = a.pix_stride ? a.pix_stride : a.C;
  // Stride 2 pays while the launch is small: its workgroups load four input pixels per output pixel
  // in front of the same K walk, which the implicit-GEMM kernel overtakes once it has enough
  // 128x128 tiles for several rounds per CU (measured at 15 GFLOP per launch: 29-34 us there, 35-38
  // here; at 3.7 GFLOP: 13-17 us there, 10-11 here).
  const double s2_flops = 2.0 * a.N * a.OH * a.OW * (double)fmain * 9.0 * a.C;
  if (st == 2 && s2_flops > 8e9) return false;
  return !off && aux_ok && act_ok && a.wt_frag && a.R == 3 && a.S == 3 && (st == 1 || (st == 2 && !off2)) && a.stride_w == st &&
         a.pad_h == 1 && a.pad_w == 1 && a.OH == (a.H - 1) / st + 1 && a.OW == (a.W - 1) / st + 1 &&
         a.batch == 1 && pix % (slab / 8) == 0 && a.C % slab == 0 && fmain % 8 == 0 && a.ldo >= fmain && a.ldo % (slab / 8) == 0 &&
         (long long)a.N * a.OH * a.OW * std::max(a.ldo, faux) < (1ll << 31) && (long long)a.N * a.H * a.W < (1 << 24) && a.in_bytes < kOOBp &&
         (long long)pix * (long long)dtype_size(in_dt) < (1 << 24) &&
         (long long)((std::max(fmain, faux) + 63) / 64) * 64 * 9 * a.C * (long long)dtype_size(in_dt) < (1ll << 31) &&
         plan_patch(st, a.N, a.OH, a.OW, fmain, a.C / slab, &ws, &tp);
}

template <typename T, typename OutT, int WS, int WK, int NI, int ST = 1, bool SK = false, bool ACT = false>
static void launch_patch_cfg(const PatchArgs& a, double flops, double bytes, const char* tag, hipStream_t s) {
  typedef PatchCfg<WS, WK, ST> Cfg;
  auto kern = conv3x3_patch_kernel<T, OutT, WS, WK, NI, ST, SK, ACT>;
  static const bool attr = [&] {
    NNCV_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, Cfg::smem));
    return true;
  }();
  (void)attr;
  ProfScope prof(tag, flops, bytes, s);
  PatchArgs b = a;
  b.aux_fb0 = (a.F + 32 * NI - 1) / (32 * NI);
  // inline form of the auxiliary filters: same count as the 3x3 filters, rows of the same length, every slab held at once
  // ... and only where the 3x3 blocks alone fill the CUs: on a small launch the separate blocks are extra parallelism
  b.aux_inline = ST == 2 && !SK && a.aux_inline && a.aux_F == a.F && a.ldo == a.aux_F && a.C * (int)sizeof(T) / 128 <= (WS == 1 ? 4 : 1) &&
                 (long long)a.tiles * b.aux_fb0 >= 200;
  const int fblocks = b.aux_fb0 + (b.aux_inline ? 0 : (a.aux_F + 32 * NI - 1) / (32 * NI));
  if (b.xcd_by_filter && fblocks % kXcdsP != 0) b.xcd_by_filter = 0;
  dim3 grid((a.tiles + kXcdsP - 1) / kXcdsP * kXcdsP, fblocks, SK ? a.ksplit : 1);
  hipLaunchKernelGGL(kern, grid, dim3(Cfg::NT), Cfg::smem, s, b.in, b.tiles, b.tiles_y, b.TN, b.TH, b.N, b.H, b.W, b.C, b.rw_log,
                     b.xcd_by_filter, b.in_bytes, b.txw, b);
}

void launch_conv3x3_patch(const IgemmArgs& g, int in_dt, int out_dt, hipStream_t s) {
  PatchArgs a{};
  a.in = g.in; a.wf = g.wt_frag; a.out = g.out; a.scale = g.scale; a.shift = g.shift; a.residual = g.residual;
  a.N = g.N; a.H = g.H; a.W = g.W; a.C = g.C; a.F = g.aux_f0 ? g.aux_f0 : g.F; a.relu = g.relu;
  a.ldo = g.ldo; a.pix = g.pix_stride ? g.pix_stride : g.C;
  if (g.aux_f0) {
    a.aux_F = g.F - g.aux_f0; a.aux_wf = g.aux_wt_frag; a.aux_out = g.aux_out; a.aux_relu = g.aux_relu;
    a.aux_scale = g.scale ? g.scale + g.aux_f0 : nullptr; a.aux_shift = g.shift ? g.shift + g.aux_f0 : nullptr;
    a.aux_wf_bytes = (unsigned)((size_t)((a.aux_F + 63) / 64) * 64 * g.C * dtype_size(in_dt));
  }
  static const bool no_inline = getenv("NNCV_HIP_NO_AUX_INLINE") != nullptr;
  a.aux_inline = a.aux_F > 0 && !no_inline;
  int ws = 0;
  const int st = g.stride_h;
  a.OH = g.OH; a.OW = g.OW;
  TilePlan tp;
  NNCV_REQUIRE(plan_patch(st, a.N, a.OH, a.OW, a.F, a.C * (int)dtype_size(in_dt) / 128, &ws, &tp), "conv3x3_patch: no tile fits");
  a.TN = tp.TN; a.TH = tp.TH; a.rw_log = tp.rw_log;
  a.rowx = st == 1 ? kRowSpare : 0;
  a.txw = tp.TW | (tp.NTX << 16);
  a.tiles_y = ((a.OH + a.TH - 1) / a.TH) * tp.NTX;
  a.tiles = ((a.N + a.TN - 1) / a.TN) * a.tiles_y;
  a.in_bytes = g.in_bytes;
  a.wf_bytes = (unsigned)((size_t)((a.F + 63) / 64) * 64 * 9 * a.C * dtype_size(in_dt));
  a.xcd_by_filter = ((a.F + 63) / 64) % kXcdsP == 0 && a.wf_bytes > (2u << 20);
  a.inv_ph = 1.0f / (st == 1 ? a.TH + 2 : 2 * a.TH + 1);
  a.inv_thw = 1.0f / (a.TH * tp.TW);
  a.inv_w = 1.0f / tp.TW;
  const double P = (double)a.N * a.OH * a.OW;
  const double flops = 2.0 * P * a.C * (9.0 * a.F + a.aux_F);
  const double es = dtype_size(in_dt), os = dtype_size(out_dt);
  const double bytes = es * ((double)a.N * a.H * a.W * a.C + a.C * (9.0 * a.F + a.aux_F)) + os * P * (a.F * (a.residual ? 2 : 1) + a.aux_F);
  const bool h = in_dt == kF16 && out_dt == kF16, f = in_dt == kF32 && out_dt == kF32;
  NNCV_REQUIRE(h || f, "conv3x3_patch: unsupported dtype combination");
  // Few workgroups (small batch on the deep layers: each streams its filter block's weights through
  // one CU's 64 B/clk vector-memory path): split the 64-filter blocks in two and use twice the CUs.
  // (measured on 7x7x512 -> 512: at 128 whole blocks, batch 16, halves take 10.1 us against 12.1; at 256, batch 32, 15.7 against 13.9)
  const bool halves = ws == 1 && (long long)a.tiles * ((a.F + 63) / 64 + (a.aux_F + 63) / 64) <= 128 && a.F % 64 == 0;
  if (halves) a.xcd_by_filter = (a.F / 32) % kXcdsP == 0 && a.wf_bytes > (2u << 20);
  // fp32, still few workgroups, several slabs: split K over up to 256 / workgroups workgroups.  An
  // fp32 wave needs 64 cycles of the matrix pipe per 32x32x2 product, so a deep layer at batch 1
  // (16 workgroups = 64 of the chip's 1024 SIMDs) is bound by those few waves' matrix time, and
  // spreading K over more SIMDs pays for the reduction through memory (about 5 us).  In fp16 the
  // same launches are four times shorter and the reduction costs more than it saves (measured:
  // layer4 at batch 1 6.5 -> 10 us), so the split is fp32 only.
  static const int sk_env = [] {
    const char* e = getenv("NNCV_HIP_SPLITK");
    return e ? atoi(e) : -1;
  }();
  a.ksplit = 1;
  if (halves && in_dt == kF32 && sk_env != 0 && g.splitk_ws && g.splitk_counters) {
    const int nslab = a.C * (int)dtype_size(in_dt) / 128;
    const long long wgs = (long long)a.tiles * (a.F / 32 + (a.aux_F + 31) / 32);
    const int want = (int)std::min<long long>(std::min(nslab, kMaxSplit), sk_env > 0 ? sk_env : 256 / wgs);
    // Only walks of eight slabs and more are split: the reduction through memory costs about as much as four slabs of
    // taps (one fp32 layer [1,64,56,56] -> 64, two slabs: 8.3 us whole against 12.4 split in two; the fp32 network at
    // [1,3,256,256]: 0.282 ms splitting from two slabs, 0.265 from four, 0.263 from eight, 0.289 from sixteen, 0.360 never).
    static const int min_slabs = [] {
      const char* e = getenv("NNCV_HIP_SPLITK_MINSLAB");
      return e ? atoi(e) : 8;
    }();
    if (want >= 2 && nslab >= min_slabs && wgs <= g.splitk_counters_n) {
      a.spk = (nslab + want - 1) / want;
      a.ksplit = (nslab + a.spk - 1) / a.spk;
      if ((size_t)wgs * a.ksplit * 4096 * sizeof(float) > g.splitk_ws_bytes) a.ksplit = 1;
    }
    a.partial = static_cast<float*>(g.splitk_ws);
    a.counters = g.splitk_counters;
  }
  const bool act = a.relu > kActRelu;
  if (act) {
    NNCV_REQUIRE(h, "conv3x3_patch: activations other than ReLU are fp16 only");
    if (st == 2) {
      if (ws == 2) launch_patch_cfg<half_t, half_t, 2, 2, 2, 2, false, true>(a, flops, bytes, "conv3x3s2_patch<f16,2,2,act>", s);
      else if (halves) launch_patch_cfg<half_t, half_t, 1, 4, 1, 2, false, true>(a, flops, bytes, "conv3x3s2_patch<f16,1,4,half,act>", s);
      else launch_patch_cfg<half_t, half_t, 1, 4, 2, 2, false, true>(a, flops, bytes, "conv3x3s2_patch<f16,1,4,act>", s);
    } else {
      if (ws == 4) launch_patch_cfg<half_t, half_t, 4, 1, 2, 1, false, true>(a, flops, bytes, "conv3x3_patch<f16,4,1,act>", s);
      else if (ws == 2) launch_patch_cfg<half_t, half_t, 2, 2, 2, 1, false, true>(a, flops, bytes, "conv3x3_patch<f16,2,2,act>", s);
      else if (halves) launch_patch_cfg<half_t, half_t, 1, 4, 1, 1, false, true>(a, flops, bytes, "conv3x3_patch<f16,1,4,half,act>", s);
      else launch_patch_cfg<half_t, half_t, 1, 4, 2, 1, false, true>(a, flops, bytes, "conv3x3_patch<f16,1,4,act>", s);
    }
  } else if (st == 2) {
    if (h) {
      if (ws == 2) launch_patch_cfg<half_t, half_t, 2, 2, 2, 2>(a, flops, bytes, "conv3x3s2_patch<f16,2,2>", s);
      else if (halves) launch_patch_cfg<half_t, half_t, 1, 4, 1, 2>(a, flops, bytes, "conv3x3s2_patch<f16,1,4,half>", s);
      else launch_patch_cfg<half_t, half_t, 1, 4, 2, 2>(a, flops, bytes, "conv3x3s2_patch<f16,1,4>", s);
    } else {
      if (ws == 2) launch_patch_cfg<float, float, 2, 2, 2, 2>(a, flops, bytes, "conv3x3s2_patch<f32,2,2>", s);
      else if (a.ksplit > 1) launch_patch_cfg<float, float, 1, 4, 1, 2, true>(a, flops, bytes, "conv3x3s2_patch<f32,1,4,half,splitk>", s);
      else if (halves) launch_patch_cfg<float, float, 1, 4, 1, 2>(a, flops, bytes, "conv3x3s2_patch<f32,1,4,half>", s);
      else launch_patch_cfg<float, float, 1, 4, 2, 2>(a, flops, bytes, "conv3x3s2_patch<f32,1,4>", s);
    }
  } else if (h) {
    if (ws == 4) launch_patch_cfg<half_t, half_t, 4, 1, 2>(a, flops, bytes, "conv3x3_patch<f16,4,1>", s);
    else if (ws == 2) launch_patch_cfg<half_t, half_t, 2, 2, 2>(a, flops, bytes, "conv3x3_patch<f16,2,2>", s);
    else if (halves) launch_patch_cfg<half_t, half_t, 1, 4, 1>(a, flops, bytes, "conv3x3_patch<f16,1,4,half>", s);
    else launch_patch_cfg<half_t, half_t, 1, 4, 2>(a, flops, bytes, "conv3x3_patch<f16,1,4>", s);
  } else {
    if (ws == 4) launch_patch_cfg<float, float, 4, 1, 2>(a, flops, bytes, "conv3x3_patch<f32,4,1>", s);
    else if (ws == 2) launch_patch_cfg<float, float, 2, 2, 2>(a, flops, bytes, "conv3x3_patch<f32,2,2>", s);
    else if (a.ksplit > 1) launch_patch_cfg<float, float, 1, 4, 1, 1, true>(a, flops, bytes, "conv3x3_patch<f32,1,4,half,splitk>", s);
    else if (halves) launch_patch_cfg<float, float, 1, 4, 1>(a, flops, bytes, "conv3x3_patch<f32,1,4,half>", s);
    else launch_patch_cfg<float, float, 1, 4, 2>(a, flops, bytes, "conv3x3_patch<f32,1,4>", s);
  }
  NNCV_HIP_CHECK(hipGetLastError());
}

}  // namespace nncv_hip
