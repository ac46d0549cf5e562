// Implicit-GEMM convolution / batched K-contiguous GEMM on gfx950 MFMA.
//
// Replaces what nncv's ModernTile + ModernVec passes emit for linalg.conv_2d_nchw_fchw
// (src/nncv/compiler/Conversion/CodeGen/LlvmCpu/ModernTile.cpp:124-286) and, through the
// R=S=1 form, linalg.batch_matmul of the Winograd rewrite
// (src/nncv/compiler/Conversion/ConvOptimize/OptimizeConv2dUsingWinograd.cpp:227-248) and the FC
// matmul (tests/Nets/Res18.mlir:621-628).
//
// Design (CDNA4, 64-wide waves):
//  * 256 threads = 4 waves per workgroup; a workgroup owns BP output pixels x BF output channels,
//    each wave a (BP/WP) x (BF/WF) sub-tile made of 32x32 MFMA accumulators.
//  * K = (r, s, c) is walked in steps of four 16-byte chunks per row.  A chunk is 8 halves or
//    4 floats that are contiguous in c, so one 16-byte global load fills it; pixels outside the
//    image contribute zero chunks (no padded copy of the activation exists).
//  * Both operands go global -> registers -> LDS (rows of 4 chunks + 1 chunk of padding = 80 B,
//    which makes every 16-byte LDS read of a wave conflict free) with two LDS buffers so the
//    global loads of step k+1 overlap the MFMAs of step k; one barrier per step.
//  * Operand roles are swapped in the MFMA (weights are the "A" rows, pixels the "B" columns)
//    so that each lane ends up with 4 consecutive output channels of one pixel: the epilogue
//    (BN scale/shift, residual add, ReLU) is applied in registers and stored as one 8/16-byte
//    vector per lane straight into the NHWC result.
//  * fp16: v_mfma_f32_32x32x16_f16 (lane = row l%32, k = 8*(l/32)..+7);
//    fp32: four v_mfma_f32_32x32x2_f32 per chunk pair (lane = row l%32, k = l/32), the K order
//    inside a chunk pair is permuted identically for both operands, which a dot product allows.
#include "common.hpp"

namespace nncv_hip {

typedef half_t half8 __attribute__((ext_vector_type(8)));
typedef half_t half4 __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

template <typename T>
struct Mma;
template <>
struct Mma<half_t> {
  static __device__ __forceinline__ void run(const uint4& a, const uint4& b, floatx16& c) {
    c = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8, a), __builtin_bit_cast(half8, b), c,
                                               0, 0, 0);
  }
};
template <>
struct Mma<float> {
  static __device__ __forceinline__ void run(const uint4& a, const uint4& b, floatx16& c) {
    const floatx4 fa = __builtin_bit_cast(floatx4, a), fb = __builtin_bit_cast(floatx4, b);
#pragma unroll
    for (int j = 0; j < 4; ++j) c = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[j], fb[j], c, 0, 0, 0);
  }
};

template <typename OutT>
struct Vec4;
template <>
struct Vec4<float> {
  typedef floatx4 type;
};
template <>
struct Vec4<half_t> {
  typedef half4 type;
};

constexpr int kThreads = 256;
constexpr int kChunksPerStep = 4;                   // 16-byte chunks per row per K step
constexpr int kRowBytes = (kChunksPerStep + 1) * 16;  // LDS row pitch: 64 B payload + 16 B pad

template <typename T, typename OutT, int BP, int BF, int WP, int WF>
__global__ __launch_bounds__(kThreads) void igemm_kernel(const IgemmArgs a) {
  constexpr int CE = 16 / sizeof(T);            // elements per chunk
  constexpr int BKE = kChunksPerStep * CE;      // elements per K step
  constexpr int PCH = BP / 64, FCH = BF / 64;   // rows of each operand a thread loads per step
  constexpr int TP = BP / WP / 32, TF = BF / WF / 32;
  static_assert(WP * WF == 4 && PCH >= 1 && FCH >= 1 && TP >= 1 && TF >= 1, "tile shape");

  __shared__ __align__(16) unsigned char smem[2][(BP + BF) * kRowBytes];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wp = wave % WP, wf = wave / WP;
  const int P = a.N * a.OH * a.OW;
  const int Ktot = a.R * a.S * a.C;
  const int pix = a.pix_stride ? a.pix_stride : a.C;  // element pitch between adjacent pixels
  const int bz = blockIdx.z;
  const T* in = static_cast<const T*>(a.in) + (long long)bz * a.in_bs;
  const T* wt = static_cast<const T*>(a.wt) + (long long)bz * a.wt_bs;

  // ---- loader state ----
  const int ck = tid & 3, r0 = tid >> 2;
  const T* pbase[PCH];
  int iy0[PCH], ix0[PCH];
#pragma unroll
  for (int i = 0; i < PCH; ++i) {
    const int gp = blockIdx.x * BP + r0 + 64 * i;
    if (gp < P) {
      const int n = gp / (a.OH * a.OW), rem = gp - n * (a.OH * a.OW);
      const int oy = rem / a.OW, ox = rem - oy * a.OW;
      iy0[i] = oy * a.stride_h - a.pad_h;
      ix0[i] = ox * a.stride_w - a.pad_w;
      pbase[i] = in + ((long long)n * a.H * a.W + (long long)iy0[i] * a.W + ix0[i]) * pix;
    } else {
      iy0[i] = ix0[i] = -(1 << 28);  // never inside the image
      pbase[i] = in;
    }
  }
  const T* wrow[FCH];
  bool wvalid[FCH];
#pragma unroll
  for (int i = 0; i < FCH; ++i) {
    const int f = blockIdx.y * BF + r0 + 64 * i;
    wvalid[i] = f < a.F;
    wrow[i] = wt + (long long)(wvalid[i] ? f : 0) * Ktot;
  }
  int kidx = ck * CE;
  int kc = kidx % a.C, ks = (kidx / a.C) % a.S, kr = kidx / (a.C * a.S);

  uint4 regP[PCH], regW[FCH];
  auto load_step = [&]() {
    const bool kval = kidx < Ktot;
    const long long koff = ((long long)kr * a.W + ks) * pix + kc;
#pragma unroll
    for (int i = 0; i < PCH; ++i) {
      const bool ok = kval && (unsigned)(iy0[i] + kr) < (unsigned)a.H && (unsigned)(ix0[i] + ks) < (unsigned)a.W;
      regP[i] = ok ? *reinterpret_cast<const uint4*>(pbase[i] + koff) : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < FCH; ++i)
      regW[i] = (kval && wvalid[i]) ? *reinterpret_cast<const uint4*>(wrow[i] + kidx) : make_uint4(0, 0, 0, 0);
    kidx += BKE;
    kc += BKE;
    while (kc >= a.C) {
      kc -= a.C;
      if (++ks == a.S) { ks = 0; ++kr; }
    }
  };
  auto store_step = [&](int buf) {
    unsigned char* sP = smem[buf];
    unsigned char* sW = smem[buf] + BP * kRowBytes;
#pragma unroll
    for (int i = 0; i < PCH; ++i) *reinterpret_cast<uint4*>(sP + (r0 + 64 * i) * kRowBytes + ck * 16) = regP[i];
#pragma unroll
    for (int i = 0; i < FCH; ++i) *reinterpret_cast<uint4*>(sW + (r0 + 64 * i) * kRowBytes + ck * 16) = regW[i];
  };

  floatx16 acc[TF][TP];
#pragma unroll
  for (int i = 0; i < TF; ++i)
#pragma unroll
    for (int j = 0; j < TP; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  const int nk = (Ktot + BKE - 1) / BKE;
  load_step();
  store_step(0);
  __syncthreads();
  const int lrow = lane & 31, lchunk = lane >> 5;
  for (int kt = 0; kt < nk; ++kt) {
    const bool more = kt + 1 < nk;
    if (more) load_step();
    const unsigned char* sP = smem[kt & 1] + (wp * (BP / WP) + lrow) * kRowBytes + lchunk * 16;
    const unsigned char* sW = smem[kt & 1] + BP * kRowBytes + (wf * (BF / WF) + lrow) * kRowBytes + lchunk * 16;
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      uint4 fw[TF], fp[TP];
#pragma unroll
      for (int i = 0; i < TF; ++i) fw[i] = *reinterpret_cast<const uint4*>(sW + i * 32 * kRowBytes + kk * 32);
#pragma unroll
      for (int j = 0; j < TP; ++j) fp[j] = *reinterpret_cast<const uint4*>(sP + j * 32 * kRowBytes + kk * 32);
#pragma unroll
      for (int i = 0; i < TF; ++i)
#pragma unroll
        for (int j = 0; j < TP; ++j) Mma<T>::run(fw[i], fp[j], acc[i][j]);
    }
    if (more) store_step((kt + 1) & 1);
    __syncthreads();
  }

  // ---- epilogue: lane holds pixel (lane%32) x channels 8g + 4*(lane/32) + {0..3}, g = 0..3 ----
  OutT* out = static_cast<OutT*>(a.out) + (long long)bz * a.out_bs;
  const OutT* res = a.residual ? static_cast<const OutT*>(a.residual) + (long long)bz * a.out_bs : nullptr;
  typedef typename Vec4<OutT>::type V4;
#pragma unroll
  for (int j = 0; j < TP; ++j) {
    const int gp = blockIdx.x * BP + wp * (BP / WP) + j * 32 + lrow;
    if (gp >= P) continue;
#pragma unroll
    for (int i = 0; i < TF; ++i) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int f0 = blockIdx.y * BF + wf * (BF / WF) + i * 32 + 8 * g + 4 * lchunk;
        if (f0 >= a.F) continue;
        floatx4 y = {acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
        if (a.scale) y *= *reinterpret_cast<const floatx4*>(a.scale + f0);
        if (a.shift) y += *reinterpret_cast<const floatx4*>(a.shift + f0);
        const long long o = (long long)gp * a.ldo + f0;
        const bool res_after = a.relu & kActResidualAfter;
        float r4[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        if (res) {
          const V4 rv = *reinterpret_cast<const V4*>(res + o);
#pragma unroll
          for (int e = 0; e < 4; ++e) r4[e] = (float)rv[e];
        }
        if (res && !res_after) {
#pragma unroll
          for (int e = 0; e < 4; ++e) y[e] += r4[e];
        }
        if (a.relu == kActRelu) {
#pragma unroll
          for (int e = 0; e < 4; ++e) y[e] = relu_ugt(y[e]);
        } else if (a.relu) {
          float t[4] = {y[0], y[1], y[2], y[3]};
          act_apply_n<sizeof(OutT) == 2>(t, a.relu & 0xff);
          y = floatx4{t[0], t[1], t[2], t[3]};
        }
        if (res && res_after) {
#pragma unroll
          for (int e = 0; e < 4; ++e) y[e] += r4[e];
        }
        V4 ov;
#pragma unroll
        for (int e = 0; e < 4; ++e) ov[e] = (OutT)y[e];
        *reinterpret_cast<V4*>(out + o) = ov;
      }
    }
  }
}

template <typename T> constexpr const char* tname();
template <> constexpr const char* tname<half_t>() { return "f16"; }
template <> constexpr const char* tname<float>() { return "f32"; }

template <typename T, typename OutT, int BP, int BF, int WP, int WF>
static void launch_cfg(const IgemmArgs& a, hipStream_t s) {
  const int P = a.N * a.OH * a.OW;
  static const std::string tag = std::string("igemm<") + tname<T>() + "," + tname<OutT>() + "," + std::to_string(BP) +
                                 "," + std::to_string(BF) + "," + std::to_string(WP) + "," + std::to_string(WF) + ">";
  const double K = (double)a.R * a.S * a.C;
  const double flops = a.alg_flops > 0 ? a.alg_flops : 2.0 * P * a.F * K * a.batch;
  const double bytes = sizeof(T) * ((double)a.N * a.H * a.W * a.C + (double)a.F * K) * a.batch +
                       sizeof(OutT) * (double)P * a.F * a.batch * (a.residual ? 2 : 1);
  ProfScope prof(tag.c_str(), flops, bytes, s);
  dim3 grid((P + BP - 1) / BP, (a.F + BF - 1) / BF, a.batch);
  hipLaunchKernelGGL((igemm_kernel<T, OutT, BP, BF, WP, WF>), grid, dim3(kThreads), 0, s, a);
}

template <typename T, typename OutT>
static void launch_typed(const IgemmArgs& a, hipStream_t s) {
  const long long P = (long long)a.N * a.OH * a.OW;
  auto blocks = [&](int bp, int bf) { return ((P + bp - 1) / bp) * ((a.F + bf - 1) / bf) * a.batch; };
  static const int force = [] {
    const char* e = getenv("NNCV_HIP_IGEMM_TILE");
    return e ? atoi(e) : 0;
  }();
  int pick = force;
  if (!pick) {
    // largest tile that still gives every CU (256 of them) about two workgroups
    if (a.F > 64 && blocks(128, 128) >= 512) pick = 1;
    else if (a.F <= 64 && blocks(256, 64) >= 512) pick = 2;
    else if (blocks(128, 64) >= 384) pick = 3;
    else pick = 4;
  }
  switch (pick) {
    case 1: launch_cfg<T, OutT, 128, 128, 2, 2>(a, s); break;
    case 2: launch_cfg<T, OutT, 256, 64, 4, 1>(a, s); break;
    case 3: launch_cfg<T, OutT, 128, 64, 2, 2>(a, s); break;
    default: launch_cfg<T, OutT, 64, 64, 2, 2>(a, s); break;
  }
}

void launch_igemm(const IgemmArgs& a_in, int in_dt, int out_dt, hipStream_t s) {
  IgemmArgs a = a_in;
  const int ce = in_dt == kF16 ? 8 : 4;
  const int pix = a.pix_stride ? a.pix_stride : a.C;
  const unsigned long long in_b = (unsigned long long)a.N * a.H * a.W * pix * dtype_size(in_dt);
  const unsigned long long wt_b = (unsigned long long)a.F * a.R * a.S * a.C * dtype_size(in_dt);
  if (!a.in_bytes) a.in_bytes = in_b < 0xffffffffull ? (unsigned)in_b : 0xffffffffu;
  if (!a.wt_bytes) a.wt_bytes = wt_b < 0xffffffffull ? (unsigned)wt_b : 0xffffffffu;
  NNCV_REQUIRE(a.C % ce == 0, "igemm: C must be a multiple of the 16-byte chunk");
  NNCV_REQUIRE(a.F % 4 == 0 && a.ldo % 4 == 0, "igemm: F and ldo must be multiples of 4");
  NNCV_REQUIRE(a.batch >= 1 && a.batch <= 65535, "igemm: batch out of range");
  NNCV_REQUIRE((long long)a.N * a.OH * a.OW < (1ll << 31), "igemm: too many output pixels");
  // fewer output rows/columns than the geometry allows is legal (the packed stem image is wider
  // than needed); more would read outside the image, which the kernel turns into zeros anyway
  NNCV_REQUIRE(a.OH >= 1 && a.OW >= 1 && a.OH <= (a.H + 2 * a.pad_h - a.R) / a.stride_h + 1 &&
                   a.OW <= (a.W + 2 * a.pad_w - a.S) / a.stride_w + 1,
               "igemm: output size does not match input/filter/stride/pad");
  if (conv_pairs_applicable(a, in_dt, out_dt)) {
    launch_conv_pairs(a, s);
    return;
  }
  if (conv3x3_stream_applicable(a, in_dt, out_dt) && launch_conv3x3_stream(a, s)) return;
  if (in_dt == out_dt && conv3x3_patch_applicable(a, in_dt)) {
    launch_conv3x3_patch(a, in_dt, out_dt, s);
    return;
  }
  if (igemm_fast_applicable(a, in_dt, out_dt)) {
    launch_igemm_fast(a, in_dt, out_dt, s);
    NNCV_HIP_CHECK(hipGetLastError());
    return;
  }
  NNCV_REQUIRE(a.aux_f0 == 0, "igemm: auxiliary filters need the fast kernel");
  if (in_dt == kF16 && out_dt == kF16) launch_typed<half_t, half_t>(a, s);
  else if (in_dt == kF16 && out_dt == kF32) launch_typed<half_t, float>(a, s);
  else if (in_dt == kF32 && out_dt == kF32) launch_typed<float, float>(a, s);
  else fail("igemm: unsupported dtype combination");
  NNCV_HIP_CHECK(hipGetLastError());
}

}  // namespace nncv_hip
