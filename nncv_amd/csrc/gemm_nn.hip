// fp32 row-major C += A.B on gfx950 MFMA — the linalg.matmul of
// tests/MatMulOptimization/MatMulDeafult.mlir:6-9, which the reference lowers with 16/8/k8 tiles
// and 8x8x8 vector contracts (ModernTile.cpp:289-296, PrepareModernVec.cpp:43-48) and for which
// its unfinished CUDA kernel intended a 128x128x8 shared-memory tiling
// (src/libnncv/kernel/sgemm.cu:13-100).  Nothing of either is reused.
//
// 128x128 tile per 256-thread workgroup, 4 waves of 64x64 (2x2 accumulators of
// v_mfma_f32_32x32x2_f32), K walked 16 at a time through two LDS buffers.
//  * A (M x K, K contiguous) is kept in LDS as rows of four 16-byte chunks + one chunk of padding;
//    a lane reads one chunk (4 consecutive k of its row) per two MFMAs' worth of k.
//  * B (K x N, N contiguous) is kept k-major exactly as it lies in memory, so the global loads are
//    coalesced along n and the MFMA operand read (one float per lane, lanes along n) is a
//    conflict-free 128-byte LDS row segment.
//  * MFMA k-slot h of lane-half h takes k = 4*(2*kk + h) + j for both operands.
//  * The accumulator layout puts 32 consecutive n in 32 lanes, so the C read-modify-write moves
//    128 contiguous bytes per half wave.
#include "common.hpp"

namespace nncv_hip {

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int GBK = 16;
constexpr int kARow = 80;  // bytes: 16 floats + 4 pad

// GBM x GBN tile per workgroup (128x128 for large problems, 64x64 when that is what it takes to
// give each of the 256 CUs a workgroup); waves are arranged 2x2.
template <int GBM, int GBN>
__global__ __launch_bounds__(256) void gemm_nn_f32_kernel(const float* __restrict__ A, const float* __restrict__ B,
                                                          float* __restrict__ C, int M, int N, int K) {
  constexpr int kBRow = (GBN + 4) * 4;  // bytes: GBN floats + 4 pad (keeps 16-byte alignment)
  constexpr int TM = GBM / 64, TN = GBN / 64;
  constexpr int WTM = GBM / 2, WTN = GBN / 2;  // wave tile
  constexpr int BROWS = 256 / (GBN / 4);       // B rows covered by one pass of the loader
  __shared__ __align__(16) unsigned char sA[2][GBM * kARow];
  __shared__ __align__(16) unsigned char sB[2][GBK * kBRow];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave & 1, wn = wave >> 1;
  const int m0 = blockIdx.y * GBM, n0 = blockIdx.x * GBN;

  // loader mapping. A: GBM rows x 4 chunks, TM per thread (rows ar + 64 i).
  const int ack = tid & 3, ar = tid >> 2;
  // B: 16 rows x GBN/4 float4, TN per thread (rows br + BROWS i).
  const int bc4 = tid % (GBN / 4), br = tid / (GBN / 4);

  floatx4 ra[TM], rb[TN];
  auto load = [&](int k0) {
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int m = m0 + ar + 64 * i, k = k0 + ack * 4;
      ra[i] = (m < M && k < K) ? *reinterpret_cast<const floatx4*>(A + (long long)m * K + k) : floatx4{0, 0, 0, 0};
    }
#pragma unroll
    for (int i = 0; i < TN; ++i) {
      const int kb = k0 + br + BROWS * i, n = n0 + bc4 * 4;
      rb[i] = (kb < K && n < N) ? *reinterpret_cast<const floatx4*>(B + (long long)kb * N + n) : floatx4{0, 0, 0, 0};
    }
  };
  auto store = [&](int buf) {
#pragma unroll
    for (int i = 0; i < TM; ++i) *reinterpret_cast<floatx4*>(sA[buf] + (ar + 64 * i) * kARow + ack * 16) = ra[i];
#pragma unroll
    for (int i = 0; i < TN; ++i) *reinterpret_cast<floatx4*>(sB[buf] + (br + BROWS * i) * kBRow + bc4 * 16) = rb[i];
  };

  floatx16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  const int nk = (K + GBK - 1) / GBK;
  load(0);
  store(0);
  __syncthreads();
  const int lrow = lane & 31, lh = lane >> 5;
  for (int kt = 0; kt < nk; ++kt) {
    const bool more = kt + 1 < nk;
    if (more) load((kt + 1) * GBK);
    const unsigned char* pa = sA[kt & 1] + (wm * WTM + lrow) * kARow;
    const unsigned char* pb = sB[kt & 1] + (wn * WTN + lrow) * 4;
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      const int chunk = 2 * kk + lh;
      floatx4 fa[TM];
      float fb[TN][4];
#pragma unroll
      for (int i = 0; i < TM; ++i) fa[i] = *reinterpret_cast<const floatx4*>(pa + i * 32 * kARow + chunk * 16);
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int e = 0; e < 4; ++e) fb[j][e] = *reinterpret_cast<const float*>(pb + (chunk * 4 + e) * kBRow + j * 32 * 4);
#pragma unroll
      for (int e = 0; e < 4; ++e)
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i][e], fb[j][e], acc[i][j], 0, 0, 0);
    }
    if (more) store((kt + 1) & 1);
    __syncthreads();
  }

  // D[i][j]: lane holds column n = lane%32, rows m = 8g + 4*(lane/32) + e
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int n = n0 + wn * WTN + j * 32 + lrow;
      if (n >= N) continue;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int m = m0 + wm * WTM + i * 32 + 8 * (v >> 2) + 4 * lh + (v & 3);
        if (m < M) {
          float* c = C + (long long)m * N + n;
          *c = *c + acc[i][j][v];
        }
      }
    }
}

void launch_gemm_nn_f32(const float* A, const float* B, float* C, int M, int N, int K, hipStream_t s) {
  NNCV_REQUIRE(M > 0 && N > 0 && K > 0, "matmul: empty operand");
  NNCV_REQUIRE(K % 4 == 0 && N % 4 == 0, "matmul: K and N must be multiples of 4 (16-byte rows)");
  ProfScope prof("gemm_nn_f32", 2.0 * M * N * K, 4.0 * ((double)M * K + (double)K * N + 2.0 * M * N), s);
  const long long big = (long long)((N + 127) / 128) * ((M + 127) / 128);
  if (big >= 256) {
    dim3 grid((N + 127) / 128, (M + 127) / 128);
    hipLaunchKernelGGL((gemm_nn_f32_kernel<128, 128>), grid, dim3(256), 0, s, A, B, C, M, N, K);
  } else {
    dim3 grid((N + 63) / 64, (M + 63) / 64);
    hipLaunchKernelGGL((gemm_nn_f32_kernel<64, 64>), grid, dim3(256), 0, s, A, B, C, M, N, K);
  }
  NNCV_HIP_CHECK(hipGetLastError());
}

}  // namespace nncv_hip
