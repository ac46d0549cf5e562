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
//      aligned 16-byte LDS read at a constant offset, with no im2col anywhere (the eighth pixel of a row is the
//      image pixel left of the window under a zero weight: a non-finite pixel there turns into NaN);
//   2. K = 7 filter rows x 32 halves; the 64x224 filter matrix sits in registers for the whole
//      life of the (persistent) workgroup, so the tap loop is 14 x (2 LDS reads + 4 MFMAs);
//   3. scale/shift + ReLU in fp32, one rounding to fp16, tile to LDS ([pixel][64 ch], 16-byte writes: the MFMA rows
//      hold the filters permuted so that a lane ends with 16 consecutive channels); pixels
//      outside the convolution output become +0, a neutral pooling halo after ReLU (every window
//      holds at least one real, non-negative pixel);
//   4. each thread takes eight channels of two pooled pixels: nine 16-byte LDS reads each, a packed
//      UNSIGNED 16-bit max per tap (on non-negative halves the bit patterns sort like the values
//      and NaNs sort above +inf, so this is arith.maximumf with its NaN propagation), one 16-byte
//      store per pixel: eight threads write a pixel's 128 contiguous bytes.
// Workgroups are persistent (tiles strided by the grid).  The image pixels of a tile are requested a whole
// tile ahead, and the pooling of a tile runs in pieces between the MFMAs of the next one: a tile costs two
// barriers.  LDS is the busiest unit of this kernel, so every access pattern is laid out free of bank
// conflicts (they doubled its busy cycles): see the slot order, the pooling roles and the cell pitch below.
#include <type_traits>

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
typedef unsigned short ushort8v __attribute__((ext_vector_type(8)));
}  // namespace

struct StemPoolArgs {
  const half_t* in;    // [N][3][H][W]
  const half_t* wt;    // [64][7][4 pairs][2 px][4 ch], pair sp / px p holds filter column 2*sp + p - 1
  const float* scale;  // [64]
  const float* shift;  // [64]
  half_t* out;         // [N][PH][PW][64]
  int N, H, W, OH, OW, PH, PW;
  int tiles_x, tiles_y, ntiles;
  unsigned in_bytes, out_bytes;
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
  const __amdgpu_buffer_rsrc_t rs_out = make_rsrc(a.out, a.out_bytes);
  const __amdgpu_buffer_rsrc_t rs_wt = make_rsrc(a.wt, 64u * 448u);
  const __amdgpu_buffer_rsrc_t rs_sc = make_rsrc(a.scale ? (const void*)a.scale : (const void*)a.in, a.scale ? 256u : 0u);
  const __amdgpu_buffer_rsrc_t rs_sh = make_rsrc(a.shift ? (const void*)a.shift : (const void*)a.in, a.shift ? 256u : 0u);

  // ---- loader: element e = i*256 + tid of the [35][20] pixel pairs of an image tile.  A thread
  //      fetches the pair's three channel dwords (two adjacent pixels of one channel each; lanes
  //      walk the pairs of a row, so every channel plane is read in contiguous runs) and deposits
  //      the packed pair [c0 c1 c2 0 | c0 c1 c2 0] as ONE 16-byte LDS write: consecutive lanes hit
  //      consecutive 16-byte bank groups, where per-channel 2-byte deposits collided.  What depends on
  //      the thread alone (LDS address, row and column inside the tile, byte offset inside a channel
  //      plane) is worked out once; a tile adds wave-uniform terms, the plane's start travels as the
  //      load's scalar offset ----
  constexpr int kElems = (kITH * kPairs + 255) / 256;  // pairs per thread and tile
  int l_off[kElems], l_row[kElems], l_col[kElems], l_rel[kElems];
#pragma unroll
  for (int i = 0; i < kElems; ++i) {
    const int e = i * 256 + tid;
    const int row = e / kPairs, pr = e - row * kPairs;
    const bool in_tile = e < kITH * kPairs;
    l_off[i] = in_tile ? row * kInPitch + pr * 16 : -1;
    l_row[i] = in_tile ? row : (1 << 20);  // far outside any image: never ok
    l_col[i] = 2 * pr;
    l_rel[i] = (row * a.W + 2 * pr) * 2;
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
    const int tile_rel = (iy0 * a.W + ix0) * 2;      // may be negative; the sum with an in-range element is not
    const unsigned plane = (unsigned)(a.H * a.W) * 2u;
#pragma unroll
    for (int i = 0; i < kElems; ++i) {
      const bool ok = ((unsigned)(iy0 + l_row[i]) < (unsigned)a.H) & ((unsigned)(ix0 + l_col[i]) < (unsigned)a.W);
      const unsigned off = ok ? (unsigned)(tile_rel + l_rel[i]) : kOOBs;
#pragma unroll
      for (int c = 0; c < 3; ++c) pix[i][c] = __builtin_amdgcn_raw_buffer_load_b32(rs_in, off, (unsigned)(n * 3 + c) * plane, 0);
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

  // ---- once per workgroup: the filters, the scale/shift table, zeros in the image tile (the fourth channel and the
  //      row padding stay zero for good).  Every load of the prologue -- filters, scale and shift, the first image
  //      tile -- is requested before anything waits: one trip to memory instead of three in a row ----
  constexpr int kWPitch = 448 + 16;
  static_assert(64 * kWPitch <= kConvBytes, "the filters fit the convolution tile");
  u32x4 stage[7];
#pragma unroll
  for (int k = 0; k < 7; ++k) stage[k] = __builtin_amdgcn_raw_buffer_load_b128(rs_wt, (unsigned)(tid + 256 * k) * 16u, 0, 0);  // 1792 chunks of 16 bytes
  // a missing vector is a buffer of no bytes: the load returns zeros, the select below fills in 1 / 0
  const unsigned tab_raw = __builtin_amdgcn_raw_buffer_load_b32(wave == 0 ? rs_sc : rs_sh, (unsigned)(tid & 63) * 4u, 0, 0);
  request(t);
  __builtin_amdgcn_sched_barrier(0);
  for (int i = tid; i < kInBytes / 16; i += 256) reinterpret_cast<u32x4*>(in_t)[i] = u32x4{0u, 0u, 0u, 0u};
  if (tid < 128) {
    const bool have = wave == 0 ? a.scale != nullptr : a.shift != nullptr;
    tab[tid] = have ? __builtin_bit_cast(float, tab_raw) : (wave == 0 ? 1.0f : 0.0f);
  }
  // The 64 x 224 filter matrix (28 KB) ends up in the registers of EVERY wave.  It comes from memory once per workgroup,
  // through the (still unused) convolution tile in LDS, instead of once per wave: a quarter of the vector-memory traffic
  // of the prologue (58 MB over the 512 workgroups of a launch otherwise).  Filter rows are 464 bytes apart there
  // (448 + 16: the 32 lanes of a fragment read distinct banks).
  {
#pragma unroll
    for (int k = 0; k < 7; ++k) {
      // filter 16h + 4q + e of a half goes to row 8q + 4h + e of its MFMA: the accumulator registers of a lane are
      // then 16 consecutive channels, which go to the convolution tile as 16-byte writes
      const int c = tid + 256 * k, f = c / 28, w = c - f * 28;
      const int row = (f & 32) + 8 * ((f >> 2) & 3) + 4 * ((f >> 4) & 1) + (f & 3);
      *reinterpret_cast<u32x4*>(conv_t + row * kWPitch + w * 16) = stage[k];
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
  // Slots 0 .. 239 are columns 0 .. 15 of the tile's 15 rows, slots 240 .. 254 the seventeenth column: 16 neighbouring
  // lanes then read 16 neighbouring pixel pairs of one image row (no LDS bank conflicts; with 17 slots to a row nearly
  // every group of 16 lanes wrapped to the next row and hit a bank twice).  The spare slot 255 recomputes pixel 0
  // into a cell of its own that no pooling window reads.
  int cy[2], cx[2], abase[2], ccell[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int s = wave * 64 + j * 32 + lrow;
    cy[j] = s < 240 ? s >> 4 : s - 240;
    cx[j] = s < 240 ? s & 15 : 16;
    if (s >= 255) cy[j] = cx[j] = 0;
    ccell[j] = s >= 255 ? 255 * kConvPitch : (cy[j] * kCTW + cx[j]) * kConvPitch;
    abase[j] = 2 * cy[j] * kInPitch + cx[j] * 16 + lchunk * 16;
  }
  // pooling role: 16 bytes (eight channels) of two pooled pixels, (ppy, ppx) and (ppy + 4, ppx).  A 16-byte LDS read of
  // a wave runs at full rate when (measured on this chip) the 16-byte units of lanes 0-15 differ mod 16 AND lane l + 16
  // reads the unit of lane l mod 16 (same for lanes 32-63).  Lanes 0-15 are the eight chunks of the pooled pixels ppx
  // and ppx + 4 of a row (windows 8 cells = 72 units apart); lanes 16-31 take the pixels one row down and one to
  // the left (mod 8), whose windows start 32 or 48 cells further on.  With four lanes to a pixel and neighbouring pixels
  // on neighbouring lanes these reads took 2.8 times the cycles.  Row 7 does not exist: its threads read a row-5
  // window with the same bank pattern and store nowhere.
  const int pchunk = lane & 7, ppar = (lane >> 4) & 1;
  const int ppx = ((((lane >> 5) & 1) + 2 * (wave & 1) - ppar + 4 * ((lane >> 3) & 1)) & 7);
  const int ppy[2] = {2 * (wave >> 1) + ppar, 2 * (wave >> 1) + ppar + 4};
  const bool prole[2] = {true, ppy[1] < kPTH};
  int pool_base[2];
  pool_base[0] = ((2 * ppy[0]) * kCTW + 2 * ppx) * kConvPitch + pchunk * 16;
  pool_base[1] = prole[1] ? ((2 * ppy[1]) * kCTW + 2 * ppx) * kConvPitch + pchunk * 16
                          : ((2 * 5) * kCTW + 2 * ((ppx + 2) & 7)) * kConvPitch + pchunk * 16;

  __syncthreads();  // the filters are in registers, the zero fill is done
  deposit();
  if (t + (int)gridDim.x < a.ntiles) request(t + gridDim.x);
  __syncthreads();  // the first image tile is complete

  // ---- 3x3 stride-2 max over the convolution tile, in pieces that go between the MFMAs of the NEXT tile.
  //      After ReLU every value is +0, positive, +inf or NaN: as unsigned 16-bit patterns they sort
  //      like the numbers, with every NaN (either sign) above +inf.  One packed unsigned max per
  //      tap is therefore the NaN-propagating maximum of arith.maximumf, and +0 is a neutral halo. ----
  ushort8v m0, m1;   // pooled pixel 0 and 1 of this thread
  u32x4 pv0, pv1;
  unsigned pool_dst[2] = {kOOBs, kOOBs};  // byte offsets of this thread's 16 output bytes for the tile being pooled, or out of range
  auto pool_target = [&](int n, int py0, int px0) {
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const bool ok = prole[k] & (py0 + ppy[k] < a.PH) & (px0 + ppx < a.PW);
      pool_dst[k] = ok ? (unsigned)((((n * a.PH + py0 + ppy[k]) * a.PW + px0 + ppx) * 64 + pchunk * 8) * 2) : kOOBs;
    }
  };
  auto pool_read = [&](auto d_c) {
    constexpr int d = decltype(d_c)::value;
    constexpr int off = ((d / 3) * kCTW + d % 3) * kConvPitch;
    pv0 = *reinterpret_cast<const u32x4*>(conv_t + pool_base[0] + off);
    pv1 = *reinterpret_cast<const u32x4*>(conv_t + pool_base[1] + off);
  };
  auto pool_max = [&](auto d_c) {
    constexpr int d = decltype(d_c)::value;
    if constexpr (d == 0) {
      m0 = __builtin_bit_cast(ushort8v, pv0);
      m1 = __builtin_bit_cast(ushort8v, pv1);
    } else {
      m0 = __builtin_elementwise_max(m0, __builtin_bit_cast(ushort8v, pv0));
      m1 = __builtin_elementwise_max(m1, __builtin_bit_cast(ushort8v, pv1));
    }
  };
  auto pool_store = [&]() {
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, m0), rs_out, pool_dst[0], 0, 0);
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, m1), rs_out, pool_dst[1], 0, 0);
  };
  // piece k of the pooling, k = 0 .. 55 (one per MFMA of a tile): tap d is read behind MFMA 4d and folded in behind
  // MFMA 4d + 4, just before the next tap's read (four MFMAs cover the LDS latency, and the wait leaves the step's
  // operand reads in flight); the two stores follow the last tap
  auto pool_piece = [&](auto k_c) {
    constexpr int k = decltype(k_c)::value;
    if constexpr (k % 4 == 0 && k >= 4 && k <= 36) pool_max(std::integral_constant<int, k / 4 - 1>());
    if constexpr (k % 4 == 0 && k < 36) pool_read(std::integral_constant<int, k / 4>());
    if constexpr (k == 38) pool_store();
  };

  for (;;) {
    int n, py0, px0;
    tile_origin(t, n, py0, px0);
    const int tnext = t + (int)gridDim.x;

    // ---- the tile's 56 MFMAs per wave (operands one step ahead; the first step starts the sums from a zero C operand),
    //      each followed by a piece of the previous tile's pooling ----
    floatx16 acc[2][2];
    u32x4 fp[2][2];
#pragma unroll
    for (int j = 0; j < 2; ++j) fp[0][j] = *reinterpret_cast<const u32x4*>(in_t + abase[j]);
    auto steps = [&](auto self, auto st_c) -> void {
      constexpr int st = decltype(st_c)::value;
      if constexpr (st < 14) {
        constexpr int r = st >> 1, h = st & 1;
        if constexpr (st + 1 < 14) {
          constexpr int rn = (st + 1) >> 1, hn = (st + 1) & 1;
#pragma unroll
          for (int j = 0; j < 2; ++j) fp[(st + 1) & 1][j] = *reinterpret_cast<const u32x4*>(in_t + abase[j] + rn * kInPitch + hn * 32);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            if constexpr (st == 0) {
              const floatx16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
              acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8, wreg[r][h][i]), __builtin_bit_cast(half8, fp[st & 1][j]), zero, 0, 0, 0);
            } else {
              Mma<half_t>::run(wreg[r][h][i], fp[st & 1][j], acc[i][j]);
            }
            __builtin_amdgcn_sched_barrier(0);
            if (i == 0 && j == 0) pool_piece(std::integral_constant<int, 4 * st>());
            if (i == 0 && j == 1) pool_piece(std::integral_constant<int, 4 * st + 1>());
            if (i == 1 && j == 0) pool_piece(std::integral_constant<int, 4 * st + 2>());
            if (i == 1 && j == 1) pool_piece(std::integral_constant<int, 4 * st + 3>());
            __builtin_amdgcn_sched_barrier(0);
          }
        self(self, std::integral_constant<int, st + 1>());
      }
    };
    steps(steps, std::integral_constant<int, 0>());
    __syncthreads();  // every wave is done reading the image tile and pooling the previous convolution tile

    // the next image tile (requested a whole tile ago) goes to LDS and the one after it is requested before the
    // epilogue, so that its loads travel under it
    if (tnext < a.ntiles) {
      deposit();
      if (tnext + (int)gridDim.x < a.ntiles) request(tnext + gridDim.x);
    }
    __builtin_amdgcn_sched_barrier(0);

    // ---- scale/shift, ReLU, one rounding, tile to LDS; pixels outside the convolution output become the
    //      pooling halo (only tiles on the image's edges have any: the others skip the test) ----
    const int cy0 = 2 * py0 - 1, cx0 = 2 * px0 - 1;
    const bool interior = (cy0 >= 0) & (cx0 >= 0) & (cy0 + 14 < a.OH) & (cx0 + kCTW - 1 < a.OW);
    bool live[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) live[j] = interior | (((unsigned)(cy0 + cy[j]) < (unsigned)a.OH) & ((unsigned)(cx0 + cx[j]) < (unsigned)a.OW));
    // A lane holds 16 consecutive channels of each half of the filters for its two pixels.  Scale / shift of four
    // channels are fetched once for both pixels and one group ahead of their use: left to the compiler (no registers
    // to spare during the taps) every group waited for its own reads, eight LDS round trips in a row that made this
    // stage longer than the tile's MFMAs.  Eight channels make one 16-byte write to the pixel's cell.
    floatx4 scb[2], shb[2];
    scb[0] = *reinterpret_cast<const floatx4*>(tab + 16 * lchunk);
    shb[0] = *reinterpret_cast<const floatx4*>(tab + 64 + 16 * lchunk);
    half8 o8[2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int g = i * 4 + q;
        if (g + 1 < 8) {
          const int cn = ((g + 1) / 4) * 32 + 16 * lchunk + 4 * ((g + 1) % 4);
          scb[(g + 1) & 1] = *reinterpret_cast<const floatx4*>(tab + cn);
          shb[(g + 1) & 1] = *reinterpret_cast<const floatx4*>(tab + 64 + cn);
        }
        __builtin_amdgcn_sched_barrier(0);
        const floatx4 sc = scb[g & 1], sh = shb[g & 1];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
#pragma unroll
          for (int e = 0; e < 4; ++e) o8[j][4 * (q & 1) + e] = (half_t)relu_ugt(acc[i][j][4 * q + e] * sc[e] + sh[e]);
          if (q & 1) {
            u32x4 bits = __builtin_bit_cast(u32x4, o8[j]);
            if (!interior) {  // wave-uniform
              if (!live[j]) bits = u32x4{0u, 0u, 0u, 0u};
            }
            *reinterpret_cast<u32x4*>(conv_t + ccell[j] + (i * 32 + 16 * lchunk + 8 * (q >> 1)) * 2) = bits;
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    pool_target(n, py0, px0);
    if (tnext >= a.ntiles) break;
    t = tnext;
    __syncthreads();  // convolution tile and next image tile complete
  }

  // ---- the last tile's pooling has no MFMAs to go under ----
  __syncthreads();
  {
    u32x4 tv[9][2];  // the accumulators are dead: all nine taps are requested before the first maximum
#pragma unroll
    for (int d = 0; d < 9; ++d) {
      const int off = ((d / 3) * kCTW + d % 3) * kConvPitch;
      tv[d][0] = *reinterpret_cast<const u32x4*>(conv_t + pool_base[0] + off);
      tv[d][1] = *reinterpret_cast<const u32x4*>(conv_t + pool_base[1] + off);
    }
    m0 = __builtin_bit_cast(ushort8v, tv[0][0]);
    m1 = __builtin_bit_cast(ushort8v, tv[0][1]);
#pragma unroll
    for (int d = 1; d < 9; ++d) {
      m0 = __builtin_elementwise_max(m0, __builtin_bit_cast(ushort8v, tv[d][0]));
      m1 = __builtin_elementwise_max(m1, __builtin_bit_cast(ushort8v, tv[d][1]));
    }
  }
  pool_store();
}

bool stem_pool_applicable(int dt, int N, int H, int W, int F) {
  static const bool off = getenv("NNCV_HIP_NO_STEM_FUSION") != nullptr;
  return !off && dt == kF16 && F == 64 && W % 2 == 0 && H >= 7 && W >= 8 && (long long)N * 3 * H * W * 2 < (long long)kOOBs &&
         (long long)N * ((H + 3) / 4) * ((W + 3) / 4) * 128 < (long long)kOOBs;  // image and pooled tensor within a buffer descriptor's range check
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
  a.out_bytes = (unsigned)((size_t)N * a.PH * a.PW * 64 * 2);
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
