// Pieces shared by the MFMA convolution kernels (igemm_fast.hip, conv3x3_patch.hip):
// operand types, the MFMA wrappers, exact small-integer division without the ~40-instruction
// integer divide, and the coalescing epilogue of a 64x64 wave tile.
#pragma once
#include "common.hpp"

namespace nncv_hip {
namespace mt {

typedef half_t half8 __attribute__((ext_vector_type(8)));
typedef half_t half4 __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

template <typename T>
struct Mma;
template <>
struct Mma<half_t> {  // lane = row l%32, k = 8*(l/32) .. +7
  static __device__ __forceinline__ void run(const u32x4& a, const u32x4& b, floatx16& c) {
    c = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8, a), __builtin_bit_cast(half8, b), c, 0, 0, 0);
  }
  // the first product of a sum: a zero C operand instead of sixteen cleared registers
  static __device__ __forceinline__ void start(const u32x4& a, const u32x4& b, floatx16& c) {
    const floatx16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    c = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8, a), __builtin_bit_cast(half8, b), zero, 0, 0, 0);
  }
};
template <>
struct Mma<float> {  // lane = row l%32, k = l/32; the 4 floats of a chunk feed 4 MFMAs
  static __device__ __forceinline__ void run(const u32x4& a, const u32x4& b, floatx16& c) {
    const floatx4 fa = __builtin_bit_cast(floatx4, a), fb = __builtin_bit_cast(floatx4, b);
#pragma unroll
    for (int j = 0; j < 4; ++j) c = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[j], fb[j], c, 0, 0, 0);
  }
  static __device__ __forceinline__ void start(const u32x4& a, const u32x4& b, floatx16& c) { run(a, b, c); }  // fp32 sums are cleared by their owner
};

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes, 0x00020000);
}

using ::nncv_hip::relu_ugt;

// x / d for 0 <= x < 2^24 and 1 <= d, given inv = 1.0f / d computed on the host: one float
// multiply and a +-1 correction instead of the integer-divide expansion (which costs more VALU
// time in a kernel prologue than a whole K step of MFMAs).
__device__ __forceinline__ int fast_div(int x, int d, float inv, int* rem) {
  int q = (int)((float)x * inv);
  int r = x - q * d;
  if (r >= d) { ++q; r -= d; }
  if (r < 0) { --q; r += d; }
  *rem = r;
  return q;
}

// ---------------------------------------------------------------------------------------------
// Reduction + epilogue of one 64 (pixel slots) x 64 (channels) output tile that NG waves ("K
// groups") hold partial sums of, acc[i][j] = channels 32i.. x slots 32j.. in the MFMA layout
// (lane: slot l%32, channels 8q + 4*(l/32) + e).
//   1. Every group writes its accumulators into its own fp32 LDS copy of the tile [slot][channel]
//      (NG copies, kTileBytes apart), all at once, then one barrier.
//   2. Each group then takes 64/NG of the tile's rows, sums them over the copies and writes them out with 8 (fp16) / 16
//      (fp32) consecutive lanes covering the 64 channels of one pixel, so residual reads and
//      stores are whole 128/256-byte rows.  BN scale/shift, residual add and ReLU are applied in
//      fp32 on the way out: one rounding.  The scale/shift values a lane needs there are loaded
//      by EpiScale at kernel start, long before they are used.
// Every wave of the workgroup must call tile_reduce_store (it contains one barrier), after a
// barrier that freed the LDS region; `tile` is the first of the NG copies.
// ---------------------------------------------------------------------------------------------
constexpr int kTilePitch = 68 * 4;                     // bytes per slot row: 64 floats + 16 pad
constexpr int kTileBytes = 64 * kTilePitch;

template <typename OutT>
struct EpiScale {
  static constexpr int FPL = 16 / (int)sizeof(OutT);  // channels per lane on the way out
  static constexpr int LPR = 64 / FPL;                // lanes per pixel row
  float sc[FPL], sh[FPL];
  // F must be a multiple of FPL; lanes past F read the last valid group (their rows are not stored).
  __device__ __forceinline__ void load(int lane, int f0, int F, const float* scale, const float* shift) {
    int f = f0 + (lane % LPR) * FPL;
    f = f < F ? f : F - FPL;
#pragma unroll
    for (int e = 0; e < FPL; ++e) {
      sc[e] = 1.f;
      sh[e] = 0.f;
    }
    if (scale) {
#pragma unroll
      for (int q = 0; q < FPL / 4; ++q) {
        const floatx4 a = *reinterpret_cast<const floatx4*>(scale + f + 4 * q);
#pragma unroll
        for (int e = 0; e < 4; ++e) sc[4 * q + e] = a[e];
      }
    }
    if (shift) {
#pragma unroll
      for (int q = 0; q < FPL / 4; ++q) {
        const floatx4 b = *reinterpret_cast<const floatx4*>(shift + f + 4 * q);
#pragma unroll
        for (int e = 0; e < 4; ++e) sh[4 * q + e] = b[e];
      }
    }
  }
};

// NI = 1: the wave tile is 64 slots x 32 channels (acc[0] only); the LDS tile keeps its 64-channel
// rows and the lanes of the upper 32 channels simply store nothing.
// ACT = false compiles only the ReLU form of the activation (the register-tight patch kernel).
template <typename OutT, int NG, int NI = 2, bool ACT = true>
__device__ __forceinline__ void tile_reduce_store(const floatx16 (&acc)[2][2], unsigned char* tile, int g, int lane,
                                                  const int (&rowoff)[2], int f0, int F, const EpiScale<OutT>& ss,
                                                  const OutT* res, OutT* out, int relu) {
  const int lrow = lane & 31, lchunk = lane >> 5;
  constexpr int FPL = EpiScale<OutT>::FPL, LPR = EpiScale<OutT>::LPR;
  constexpr int RPI = 64 / LPR;          // pixel rows per store instruction
  constexpr int NIT = 64 / NG / RPI;     // store instructions per wave
  static_assert(NIT >= 1, "too many K groups for this output type");
  typedef OutT VO __attribute__((ext_vector_type(FPL)));
  const int fc = (lane % LPR) * FPL;
  const bool fok = f0 + fc < F && fc < 32 * NI;
  // Output offsets of the rows this lane stores, fetched from the lanes that own those slots, and
  // the residual rows requested before the reduction so that their latency hides behind it.
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
      // rows that are not stored read element 0 of the tensor: a valid address, no branch
      const long long off = o[it] >= 0 ? (long long)o[it] + f0 + fc : 0;
      rv[it] = *reinterpret_cast<const VO*>(res + off);
    }
  }
  // every K group writes its partial sums into its own copy of the tile, at the same time; one
  // barrier; the rows are summed over the NG copies on the way out
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
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    float y[FPL];
#pragma unroll
    for (int q = 0; q < FPL / 4; ++q)
#pragma unroll
      for (int e = 0; e < 4; ++e) y[4 * q + e] = v[it][q][e] * ss.sc[4 * q + e] + ss.sh[4 * q + e];
    const bool res_after = ACT && (relu & kActResidualAfter);  // y = act(conv) + residual instead of act(conv + residual)
    if (res && !res_after) {
#pragma unroll
      for (int e = 0; e < FPL; ++e) y[e] += (float)rv[it][e];
    }
    if (relu == kActRelu) {
#pragma unroll
      for (int e = 0; e < FPL; ++e) y[e] = relu_ugt(y[e]);
    } else if (ACT && relu) {
      act_apply_n<sizeof(OutT) == 2>(y, relu & 0xff);
    }
    if (res && res_after) {
#pragma unroll
      for (int e = 0; e < FPL; ++e) y[e] += (float)rv[it][e];
    }
    VO ov;
#pragma unroll
    for (int e = 0; e < FPL; ++e) ov[e] = (OutT)y[e];
    if (o[it] >= 0) *reinterpret_cast<VO*>(out + (long long)o[it] + f0 + fc) = ov;
  }
}

}  // namespace mt
}  // namespace nncv_hip
