// fp32 row-major C += A.B on gfx950 MFMA — the linalg.matmul of
// tests/MatMulOptimization/MatMulDeafult.mlir:6-9, which the reference lowers with 16/8/k8 tiles
// and 8x8x8 vector contracts (ModernTile.cpp:289-296, PrepareModernVec.cpp:43-48) and for which
// its unfinished CUDA kernel intended a 128x128x8 shared-memory tiling
// (src/libnncv/kernel/sgemm.cu:13-100).  Nothing of either is reused.
//
// Workgroup tile GBM x GBN = 128x128 (four waves of 64x64, 2x2 accumulators of v_mfma_f32_32x32x2_f32) for
// large problems, 64x64 (four waves of 32x32) when that is what it takes to give each of the 256 CUs a
// workgroup; K walked 16 at a time through two LDS buffers.
//  * A 1024^3 product is 256 tiles of 64x64 with 512 dependent 64-cycle MFMAs per wave: one wave per SIMD and
//    nothing to hide its loads, stores and barriers behind.  Small grids therefore run KG = 2 or 4 "K groups"
//    per workgroup (512 / 1024 threads): group g takes every KG-th K tile through LDS buffers of its own, the
//    groups' partial tiles meet in LDS at the end and all threads add them to C in whole 256-byte rows.
//    The order of that sum is fixed (group 0, 1, ...), so results do not change from run to run.
//  * A (M x K, K contiguous) is kept in LDS as rows of four 16-byte chunks + one chunk of padding;
//    a lane reads one chunk (4 consecutive k of its row) per two MFMAs' worth of k.
//  * B (K x N, N contiguous) is kept k-major exactly as it lies in memory, so the global loads are
//    coalesced along n and the MFMA operand read (one float per lane, lanes along n) is a
//    conflict-free 128-byte LDS row segment.
//  * MFMA k-slot h of lane-half h takes k = 4*(2*kk + h) + j for both operands.
//  * VEC: K and N multiples of 4 and 16-byte aligned operands -> 16-byte global loads; otherwise element
//    loads with a bounds check each (any M, N, K; linalg.matmul puts no condition on them).
#include "common.hpp"

namespace nncv_hip {

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));


// K tile of a round: 16 without K groups; 32 with them (a round then ends at a barrier of up to sixteen waves that all
// start the next one by waiting for their first operands: fewer, longer rounds)
constexpr int gemm_bk(int kg) { return kg > 1 ? 32 : 16; }
constexpr int gemm_arow(int kg) { return (gemm_bk(kg) + 4) * 4; }  // bytes of an A row in LDS: the K tile + 16 bytes of padding
constexpr int gemm_group_lds(int gbm, int gbn, int kg) { return 2 * gbm * gemm_arow(kg) + 2 * gemm_bk(kg) * (gbn + 4) * 4; }
constexpr int gemm_lds(int gbm, int gbn, int kg) {
  const int tiles = kg * gemm_group_lds(gbm, gbn, kg), red = kg > 1 ? kg * gbm * gbn * 4 : 0;
  return tiles > red ? tiles : red;
}

template <int GBM, int GBN, int KG, bool VEC>
__global__ __launch_bounds__(256 * KG) void gemm_nn_f32_kernel(const float* __restrict__ A, const float* __restrict__ B,
                                                               float* __restrict__ C, int M, int N, int K) {
  constexpr int GBK = gemm_bk(KG), kARow = gemm_arow(KG);
  constexpr int kBRow = (GBN + 4) * 4;  // bytes: GBN floats + 4 pad (keeps 16-byte alignment)
  constexpr int TM = GBM / 64, TN = GBN / 64;
  constexpr int KQ = GBK / 16;  // 16-wide K quarters of a tile: the loader and the MFMA loop walk them one by one
  constexpr int WTM = GBM / 2, WTN = GBN / 2;  // wave tile
  constexpr int BROWS = 256 / (GBN / 4);       // B rows covered by one pass of the loader
  static_assert(KG == 1 || (GBM == 64 && GBN == 64), "K groups go with the 64x64 tile");
  extern __shared__ __align__(16) unsigned char smem[];
  const int grp = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 8);
  const int tid = threadIdx.x & 255, lane = tid & 63, wave = tid >> 6;
  unsigned char* sA = smem + grp * gemm_group_lds(GBM, GBN, KG);  // [2][GBM * kARow]
  unsigned char* sB = sA + 2 * GBM * kARow;                   // [2][GBK * kBRow]
  const int wm = wave & 1, wn = wave >> 1;
  const int m0 = blockIdx.y * GBM, n0 = blockIdx.x * GBN;

  // loader mapping. A: GBM rows x 4 chunks, TM per thread (rows ar + 64 i).
  const int ack = tid & 3, ar = tid >> 2;
  // B: 16 rows x GBN/4 float4, TN per thread (rows br + BROWS i).
  const int bc4 = tid % (GBN / 4), br = tid / (GBN / 4);

  floatx4 ra[KQ][TM], rb[KQ][TN];
  auto load = [&](int k00) {
#pragma unroll
    for (int q = 0; q < KQ; ++q) {
      const int k0 = k00 + 16 * q;
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const int m = m0 + ar + 64 * i, k = k0 + ack * 4;
        if constexpr (VEC) {
          ra[q][i] = (m < M && k < K) ? *reinterpret_cast<const floatx4*>(A + (long long)m * K + k) : floatx4{0, 0, 0, 0};
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) ra[q][i][e] = (m < M && k + e < K) ? A[(long long)m * K + k + e] : 0.0f;
        }
      }
#pragma unroll
      for (int i = 0; i < TN; ++i) {
        const int kb = k0 + br + BROWS * i, n = n0 + bc4 * 4;
        if constexpr (VEC) {
          rb[q][i] = (kb < K && n < N) ? *reinterpret_cast<const floatx4*>(B + (long long)kb * N + n) : floatx4{0, 0, 0, 0};
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) rb[q][i][e] = (kb < K && n + e < N) ? B[(long long)kb * N + n + e] : 0.0f;
        }
      }
    }
  };
  auto store = [&](int buf) {
#pragma unroll
    for (int q = 0; q < KQ; ++q) {
#pragma unroll
      for (int i = 0; i < TM; ++i) *reinterpret_cast<floatx4*>(sA + buf * GBM * kARow + (ar + 64 * i) * kARow + q * 64 + ack * 16) = ra[q][i];
#pragma unroll
      for (int i = 0; i < TN; ++i)
        *reinterpret_cast<floatx4*>(sB + buf * GBK * kBRow + (16 * q + br + BROWS * i) * kBRow + bc4 * 16) = rb[q][i];
    }
  };

  // K groups: the four values of C this thread adds to at the end are requested now
  floatx4 cpre = {0, 0, 0, 0};
  if constexpr (KG > 1 && VEC) {
    const int e = threadIdx.x;
    if (e < 64 * 16) {
      const int gm = m0 + (e >> 4), gn = n0 + (e & 15) * 4;
      if (gm < M && gn + 3 < N) cpre = *reinterpret_cast<const floatx4*>(C + (long long)gm * N + gn);
    }
  }
  floatx16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  // K tile kt of group g in round r is r * KG + g; a group past the end of K loads zeros (same barriers for all)
  const int nk = (K + GBK - 1) / GBK, rounds = (nk + KG - 1) / KG;
  load(grp * GBK);
  store(0);
  __syncthreads();
  const int lrow = lane & 31, lh = lane >> 5;
  for (int r = 0; r < rounds; ++r) {
    const bool more = r + 1 < rounds;
    if (more) load(((r + 1) * KG + grp) * GBK);
    const unsigned char* pa = sA + (r & 1) * GBM * kARow + (wm * WTM + lrow) * kARow;
    const unsigned char* pb = sB + (r & 1) * GBK * kBRow + (wn * WTN + lrow) * 4;
#pragma unroll
    for (int kk = 0; kk < 2 * KQ; ++kk) {
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
    if (more) store((r + 1) & 1);
    __syncthreads();
  }

  if constexpr (KG > 1) {
    // partial tiles [group][64][64] in LDS (the operand buffers are free after the last barrier), then every thread
    // sums KG values for four consecutive n and adds them to C: 16 lanes per 256-byte row
    float* red = reinterpret_cast<float*>(smem);
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int m = wm * 32 + 8 * (v >> 2) + 4 * lh + (v & 3);
      red[(grp * 64 + m) * 64 + wn * 32 + lrow] = acc[0][0][v];
    }
    __syncthreads();
    const int t = threadIdx.x;
    for (int e = t; e < 64 * 16; e += 256 * KG) {
      const int m = e >> 4, nq = (e & 15) * 4;
      floatx4 sum = *reinterpret_cast<const floatx4*>(red + m * 64 + nq);
#pragma unroll
      for (int g = 1; g < KG; ++g) {
        const floatx4 p = *reinterpret_cast<const floatx4*>(red + (g * 64 + m) * 64 + nq);
        sum += p;
      }
      const int gm = m0 + m, gn = n0 + nq;
      if (gm >= M) continue;
      float* c = C + (long long)gm * N + gn;
      if (VEC && gn + 3 < N) {
        floatx4 cv = e == t ? cpre : *reinterpret_cast<floatx4*>(c);  // the thread's first element is the prefetched one
        cv += sum;
        *reinterpret_cast<floatx4*>(c) = cv;
      } else {
#pragma unroll
        for (int q = 0; q < 4; ++q)
          if (gn + q < N) c[q] += sum[q];
      }
    }
    return;
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

template <int GBM, int GBN, int KG, bool VEC>
static void launch_gemm_cfg(const float* A, const float* B, float* C, int M, int N, int K, hipStream_t s) {
  auto kern = gemm_nn_f32_kernel<GBM, GBN, KG, VEC>;
  constexpr int smem = gemm_lds(GBM, GBN, KG);
  static const bool attr = [&] {
    NNCV_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, smem));
    return true;
  }();
  (void)attr;
  dim3 grid((N + GBN - 1) / GBN, (M + GBM - 1) / GBM);
  hipLaunchKernelGGL(kern, grid, dim3(256 * KG), smem, s, A, B, C, M, N, K);
}

void launch_gemm_nn_f32(const float* A, const float* B, float* C, int M, int N, int K, hipStream_t s) {
  NNCV_REQUIRE(M > 0 && N > 0 && K > 0, "matmul: empty operand");
  ProfScope prof("gemm_nn_f32", 2.0 * M * N * K, 4.0 * ((double)M * K + (double)K * N + 2.0 * M * N), s);
  const bool vec = K % 4 == 0 && N % 4 == 0 && (reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B) | reinterpret_cast<uintptr_t>(C)) % 16 == 0;
  const long long big = (long long)((N + 127) / 128) * ((M + 127) / 128);
  const long long small = (long long)((N + 63) / 64) * ((M + 63) / 64);
  // K groups while the 64x64 grid leaves SIMDs with one wave (or none) and K is long enough to share
  const int kg = big >= 256 ? 1 : (small <= 384 && K >= 256) ? 4 : (small <= 768 && K >= 128) ? 2 : 1;
  if (big >= 256) {
    if (vec) launch_gemm_cfg<128, 128, 1, true>(A, B, C, M, N, K, s);
    else launch_gemm_cfg<128, 128, 1, false>(A, B, C, M, N, K, s);
  } else if (kg == 4) {
    if (vec) launch_gemm_cfg<64, 64, 4, true>(A, B, C, M, N, K, s);
    else launch_gemm_cfg<64, 64, 4, false>(A, B, C, M, N, K, s);
  } else if (kg == 2) {
    if (vec) launch_gemm_cfg<64, 64, 2, true>(A, B, C, M, N, K, s);
    else launch_gemm_cfg<64, 64, 2, false>(A, B, C, M, N, K, s);
  } else {
    if (vec) launch_gemm_cfg<64, 64, 1, true>(A, B, C, M, N, K, s);
    else launch_gemm_cfg<64, 64, 1, false>(A, B, C, M, N, K, s);
  }
  NNCV_HIP_CHECK(hipGetLastError());
}

}  // namespace nncv_hip
