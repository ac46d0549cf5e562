// ResNet stem in one launch (gfx950, fp16): conv 7x7 stride 2 pad 3 over 3 channels + BN + ReLU
// (tests/Nets/Res18.mlir:118-142) followed by max-pool 3x3 stride 2 over a -inf halo of 1
// (tests/Nets/Res18.mlir:144-151), NCHW image in, NHWC pooled activation out.
//
// The 112x112x64 convolution output (51 MB at batch 32, four times the pooled tensor) never
// reaches memory.  A workgroup owns a 7x8 tile of pooled pixels, i.e. a 15x17 tile of convolution
// pixels (255 of the 256 MFMA pixel slots of four 64x64 wave tiles) and a 35x40 tile of the image:
//   1. the image tile is packed into LDS as rows of pixel PAIRS, [row][pair][2 px][c0 c1 c2 0]
//      (one 16-byte write per pair),
//      so that one filter row (8 px x 4 ch = 32 halves) is 64 contiguous bytes starting at the
//      pair of the output pixel (stride 2 = one pair per output pixel): every MFMA operand is one
//      aligned 16-byte LDS read at a constant offset, with no im2col anywhere;
//   2. K = 7 filter rows x 32 halves; the 64x224 filter matrix sits in registers for the whole
//      life of the (persistent) workgroup, so the tap loop is 14 x (2 LDS reads + 4 MFMAs);
//   3. scale/shift + ReLU in fp32, one rounding to fp16, tile to LDS ([slot][64 ch]); pixels
//      outside the convolution output become +0, a neutral pooling halo after ReLU (every window
//      holds at least one real, non-negative pixel);
//   4. each thread takes one pooled pixel x 16 channels: nine 32-byte LDS reads, a packed
//      UNSIGNED 16-bit max per tap (on non-negative halves the bit patterns sort like the values
//      and NaNs sort above +inf, so this is arith.maximumf with its NaN propagation), one 32-byte
//      store: four threads write a pixel's 128 contiguous bytes.
// Workgroups are persistent (tiles strided by the grid) and request the next tile's image
// pixels before the MFMAs of the current one.
#include "mfma_tile.hpp"

namespace nncv_hip {

using namespace mt;

namespace {
constexpr int kPTH = 7, kPTW = 8;      // pooled tile
constexpr int kCTW = 17;               // convolution tile: 15 rows x 17 columns = 255 slots
constexpr int kITH = 35, kPairs = 20;  // image tile: 35 rows x 20 pixel pairs
constexpr int kInPitch = kPairs * 16 + 16;
constexpr int kInBytes = kITH * kInPitch;
constexpr int kConvPitch = 144;        // 64 halves + 16 pad
constexpr int kConvBytes = 256 * kConvPitch;
constexpr int kTabBytes = 2 * 64 * 4;  // scale, shift
constexpr unsigned kOOBs = 0x7fff0000u;

typedef unsigned short ushort2v __attribute__((ext_vector_type(2)));
typedef half_t half2v __attribute__((ext_vector_type(2)));
}  // namespace

struct StemPoolArgs {
  const half_t* in;    // [N][3][H][W]
  const half_t* wt;    // [64][7][4 pairs][2 px][4 ch], pair sp / px p holds filter column 2*sp + p - 1
  const float* scale;  // [64]
  const float* shift;  // [64]
  half_t* out;         // [N][PH][PW][64]
  int N, H, W, OH, OW, PH, PW;
  int tiles_x, tiles_y, ntiles;
  unsigned in_bytes;
};

__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void stem_pool_kernel(const StemPoolArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  unsigned char* in_t = smem;
  unsigned char* conv_t = smem + kInBytes;
  float* tab = reinterpret_cast<float*>(smem + kInBytes + kConvBytes);

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lrow = lane & 31, lchunk = lane >> 5;
  const __amdgpu_buffer_rsrc_t rs_in = make_rsrc(a.in, a.in_bytes);

  // ---- loader: element e = i*256 + tid of the [35][20] pixel pairs of an image tile.  A thread
  //      fetches the pair's three channel dwords (two adjacent pixels of one channel each; lanes
  //      walk the pairs of a row, so every channel plane is read in contiguous runs) and deposits
  //      the packed pair [c0 c1 c2 0 | c0 c1 c2 0] as ONE 16-byte LDS write: consecutive lanes hit
  //      consecutive 16-byte bank groups, where per-channel 2-byte deposits collided ----
  constexpr int kElems = (kITH * kPairs + 255) / 256;  // pairs per thread and tile
  int l_off[kElems];
#pragma unroll
  for (int i = 0; i < kElems; ++i) {
    const int e = i * 256 + tid;
    const int row = e / kPairs, pr = e - row * kPairs;
    l_off[i] = e < kITH * kPairs ? row * kInPitch + pr * 16 : -1;
  }
  unsigned pix[kElems][3];
  auto tile_origin = [&](int t, int& n, int& py0, int& px0) {
    n = t / (a.tiles_x * a.tiles_y);
    const int r = t - n * (a.tiles_x * a.tiles_y);
    const int ty = r / a.tiles_x;
    py0 = ty * kPTH;
    px0 = (r - ty * a.tiles_x) * kPTW;
  };
  auto request = [&](int t) {
    int n, py0, px0;
    tile_origin(t, n, py0, px0);
    const int iy0 = 4 * py0 - 5, ix0 = 4 * px0 - 6;  // conv row 2*py0-1 -> image row 2*(2*py0-1)-3; column one further left (pairs)
    const int base = (n * 3 * a.H + iy0) * a.W + ix0;
#pragma unroll
    for (int i = 0; i < kElems; ++i) {
      const int row = l_off[i] / kInPitch, col = ((l_off[i] - row * kInPitch) >> 4) * 2;
      const bool ok = (l_off[i] >= 0) & ((unsigned)(iy0 + row) < (unsigned)a.H) & ((unsigned)(ix0 + col) < (unsigned)a.W);
#pragma unroll
      for (int c = 0; c < 3; ++c) {
        const int g_rel = (c * a.H + row) * a.W + col;
        pix[i][c] = __builtin_amdgcn_raw_buffer_load_b32(rs_in, ok ? (unsigned)(base + g_rel) * 2u : kOOBs, 0, 0);
      }
    }
  };
  auto deposit = [&]() {
#pragma unroll
    for (int i = 0; i < kElems; ++i)
      if (l_off[i] >= 0) {
        u32x4 v;
        v[0] = (pix[i][0] & 0xffffu) | (pix[i][1] << 16);
        v[1] = pix[i][2] & 0xffffu;
        v[2] = (pix[i][0] >> 16) | (pix[i][1] & 0xffff0000u);
        v[3] = pix[i][2] >> 16;
        *reinterpret_cast<u32x4*>(in_t + l_off[i]) = v;
      }
  };

  int t = blockIdx.x;
  if (t >= a.ntiles) return;
  request(t);

  // ---- once per workgroup: zero the image tile (the fourth channel and the row padding stay
  //      zero for good), the scale/shift table, the filters ----
  for (int i = tid; i < kInBytes / 16; i += 256) reinterpret_cast<u32x4*>(in_t)[i] = u32x4{0u, 0u, 0u, 0u};
  if (tid < 64) {
    tab[tid] = a.scale ? a.scale[tid] : 1.0f;
    tab[64 + tid] = a.shift ? a.shift[tid] : 0.0f;
  }
  // The 64 x 224 filter matrix (28 KB) ends up in the registers of EVERY wave.  It comes from memory once per workgroup,
  // through the (still unused) convolution tile in LDS, instead of once per wave: a quarter of the vector-memory traffic
  // of the prologue (58 MB over the 512 workgroups of a launch otherwise).  Filter rows are 464 bytes apart there
  // (448 + 16: the 32 lanes of a fragment read distinct banks).
  constexpr int kWPitch = 448 + 16;
  static_assert(64 * kWPitch <= kConvBytes, "the filters fit the convolution tile");
  {
    u32x4 stage[7];
#pragma unroll
    for (int k = 0; k < 7; ++k) stage[k] = reinterpret_cast<const u32x4*>(a.wt)[tid + 256 * k];  // 1792 chunks of 16 bytes
#pragma unroll
    for (int k = 0; k < 7; ++k) {
      const int c = tid + 256 * k, f = c / 28, w = c - f * 28;
      *reinterpret_cast<u32x4*>(conv_t + f * kWPitch + w * 16) = stage[k];
    }
  }
  __syncthreads();
  u32x4 wreg[7][2][2];  // [filter row][K half][filter half]
#pragma unroll
  for (int r = 0; r < 7; ++r)
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int i = 0; i < 2; ++i)
        wreg[r][h][i] = *reinterpret_cast<const u32x4*>(conv_t + (i * 32 + lrow) * kWPitch + (r * 32 + h * 16 + lchunk * 8) * 2);

  // ---- this lane's two convolution pixels (slots) ----
  int cy[2], cx[2], abase[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int s = wave * 64 + j * 32 + lrow;
    cy[j] = s / kCTW;
    cx[j] = s - cy[j] * kCTW;
    if (s >= 255) cy[j] = cx[j] = 0;  // the spare slot recomputes pixel 0; it is stored as the halo value
    abase[j] = 2 * cy[j] * kInPitch + cx[j] * 16 + lchunk * 16;
  }
  // pooling role: pooled pixel tid/4 of the tile, channels 16*(tid%4)..
  const int pp = tid >> 2, pg = tid & 3;
  const int ppy = pp >> 3, ppx = pp & 7;

  __syncthreads();  // zero fill done before the first deposit

  for (; t < a.ntiles; t += gridDim.x) {
    int n, py0, px0;
    tile_origin(t, n, py0, px0);
    deposit();
    __syncthreads();  // image tile complete; every wave is done pooling the previous tile
    if (t + (int)gridDim.x < a.ntiles) request(t + gridDim.x);
    __builtin_amdgcn_sched_barrier(0);

    floatx16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;
    u32x4 fp[2][2];
#pragma unroll
    for (int j = 0; j < 2; ++j) fp[0][j] = *reinterpret_cast<const u32x4*>(in_t + abase[j]);
#pragma unroll
    for (int st = 0; st < 14; ++st) {
      const int r = st >> 1, h = st & 1;
      if (st + 1 < 14) {
        const int rn = (st + 1) >> 1, hn = (st + 1) & 1;
#pragma unroll
        for (int j = 0; j < 2; ++j) fp[(st + 1) & 1][j] = *reinterpret_cast<const u32x4*>(in_t + abase[j] + rn * kInPitch + hn * 32);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) Mma<half_t>::run(wreg[r][h][i], fp[st & 1][j], acc[i][j]);
      __builtin_amdgcn_sched_barrier(0);
    }

    // ---- scale/shift, ReLU, one rounding, tile to LDS; pixels outside the convolution output
    //      (and the spare slot) become the pooling halo ----
    const int cy0 = 2 * py0 - 1, cx0 = 2 * px0 - 1;
    bool live[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int s = wave * 64 + j * 32 + lrow;
      live[j] = (s < 255) & ((unsigned)(cy0 + cy[j]) < (unsigned)a.OH) & ((unsigned)(cx0 + cx[j]) < (unsigned)a.OW);
    }
    // scale / shift of a channel group are fetched once and used for both of the lane's pixels (the
    // stores to the convolution tile in between keep the compiler from merging the reads itself;
    // with the pixel loop outside, this stage took 38 % of the kernel, now 30 %)
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int c = i * 32 + 8 * q + 4 * lchunk;
        const floatx4 sc = *reinterpret_cast<const floatx4*>(tab + c);
        const floatx4 sh = *reinterpret_cast<const floatx4*>(tab + 64 + c);
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int s = wave * 64 + j * 32 + lrow;
          half4 o;
#pragma unroll
          for (int e = 0; e < 4; ++e) o[e] = (half_t)relu_ugt(acc[i][j][4 * q + e] * sc[e] + sh[e]);
          typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
          u32x2 bits = __builtin_bit_cast(u32x2, o);
          if (!live[j]) bits = u32x2{0u, 0u};
          *reinterpret_cast<u32x2*>(conv_t + s * kConvPitch + c * 2) = bits;
        }
      }
    __syncthreads();

    // ---- 3x3 stride-2 max over the convolution tile ----
    if (pp < kPTH * kPTW && py0 + ppy < a.PH && px0 + ppx < a.PW) {
      // After ReLU every value is +0, positive, +inf or NaN: as unsigned 16-bit patterns they sort
      // like the numbers, with every NaN (either sign) above +inf.  One packed unsigned max per
      // tap is therefore the NaN-propagating maximum of arith.maximumf, and +0 is a neutral halo.
      ushort2v m[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) m[e] = ushort2v{0, 0};
#pragma unroll
      for (int dy = 0; dy < 3; ++dy)
#pragma unroll
        for (int dx = 0; dx < 3; ++dx) {
          const unsigned char* src = conv_t + ((2 * ppy + dy) * kCTW + 2 * ppx + dx) * kConvPitch + pg * 32;
          const u32x4 v0 = *reinterpret_cast<const u32x4*>(src), v1 = *reinterpret_cast<const u32x4*>(src + 16);
#pragma unroll
          for (int e = 0; e < 8; ++e) m[e] = __builtin_elementwise_max(m[e], __builtin_bit_cast(ushort2v, e < 4 ? v0[e] : v1[e - 4]));
        }
      u32x4 o0, o1;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const unsigned w = __builtin_bit_cast(unsigned, m[e]);
        if (e < 4) o0[e] = w; else o1[e - 4] = w;
      }
      half_t* dst = a.out + (((long long)n * a.PH + py0 + ppy) * a.PW + px0 + ppx) * 64 + pg * 16;
      *reinterpret_cast<u32x4*>(dst) = o0;
      *reinterpret_cast<u32x4*>(dst + 8) = o1;
    }
  }
}

bool stem_pool_applicable(int dt, int N, int H, int W, int F) {
  static const bool off = getenv("NNCV_HIP_NO_STEM_FUSION") != nullptr;
  return !off && dt == kF16 && F == 64 && W % 2 == 0 && H >= 7 && W >= 8 && (long long)N * 3 * H * W * 2 < (long long)kOOBs;
}

// wt: launch_stem_weight_shifted layout; out: [N][PH][PW][64] with PH, PW the pooled size.
void launch_stem_pool(const void* in, const void* wt, const float* scale, const float* shift, void* out, int N, int H, int W,
                      hipStream_t s) {
  StemPoolArgs a{};
  a.in = static_cast<const half_t*>(in); a.wt = static_cast<const half_t*>(wt); a.scale = scale; a.shift = shift;
  a.out = static_cast<half_t*>(out);
  a.N = N; a.H = H; a.W = W;
  a.OH = (H + 6 - 7) / 2 + 1; a.OW = (W + 6 - 7) / 2 + 1;
  a.PH = (a.OH + 2 - 3) / 2 + 1; a.PW = (a.OW + 2 - 3) / 2 + 1;
  a.tiles_y = (a.PH + kPTH - 1) / kPTH; a.tiles_x = (a.PW + kPTW - 1) / kPTW;
  const long long nt = (long long)N * a.tiles_x * a.tiles_y;
  NNCV_REQUIRE(nt < (1ll << 30), "stem: too many tiles");
  a.ntiles = (int)nt;
  a.in_bytes = (unsigned)((size_t)N * 3 * H * W * 2);
  constexpr int smem = kInBytes + kConvBytes + kTabBytes;
  static const bool attr = [] {
    NNCV_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(stem_pool_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, smem));
    return true;
  }();
  (void)attr;
  const double flops = 2.0 * N * a.OH * a.OW * 64.0 * 147.0;
  const double bytes = 2.0 * ((double)N * 3 * H * W + (double)N * a.PH * a.PW * 64 + 64.0 * 224);
  ProfScope prof("stem_conv7x7_bn_relu_maxpool<f16>", flops, bytes, s);
  const int grid = a.ntiles < 512 ? a.ntiles : 512;  // two persistent workgroups per CU
  hipLaunchKernelGGL(stem_pool_kernel, dim3(grid), dim3(256), smem, s, a);
  NNCV_HIP_CHECK(hipGetLastError());
}

}  // namespace nncv_hip
