// CPU baseline of the convolution, shaped like what nncv's HostWParallel pipeline emits for
// linalg.conv_2d_nchw_fchw: the (image, filter) space is split across OpenMP threads
// (convert-linalg-to-parallel-loops + convert-scf-to-openmp, DnnModelLowering.cpp:541-556) and
// the innermost spatial loop is vectorised 8 wide with AVX2 FMAs (the vector size the
// ModernTile/ModernVec passes pick for AVX2, Conv2dNCHWFCHWTileVec.cpp:51-60).
//
// Test infrastructure only: it is timed by bench.py's cpu_baseline leg and checked against the
// scalar oracle in tests/; nothing that ships links it.  fp32 accumulation in the reference's
// loop order (c, r, s innermost-to-outermost per output element), so results differ from the
// fp64-accumulating oracle by ordinary fp32 rounding.
#include <immintrin.h>
#include <omp.h>

#include <cstring>
#include <vector>

extern "C" int hwp_num_threads() { return omp_get_max_threads(); }
// number of OpenMP threads of the following calls (the reference's `-num-threads`, default 4: main.cpp:231)
extern "C" void hwp_set_num_threads(int n) { if (n > 0) omp_set_num_threads(n); }

// y[N][F][OH][OW] = conv(x[N][C][H][W] with a zero halo of `pad`, w[F][C][R][S]), stride `stride`.
extern "C" int hwp_conv2d_nchw_fchw(const float* x, const float* w, float* y, int N, int C, int H, int W, int F, int R, int S,
                                    int stride, int pad) {
  const int OH = (H + 2 * pad - R) / stride + 1, OW = (W + 2 * pad - S) / stride + 1;
  if (OH <= 0 || OW <= 0) return 1;
  const __m256i lane_off = _mm256_mullo_epi32(_mm256_setr_epi32(0, 1, 2, 3, 4, 5, 6, 7), _mm256_set1_epi32(stride));
#pragma omp parallel for collapse(2) schedule(static)
  for (int n = 0; n < N; ++n)
    for (int f = 0; f < F; ++f) {
      float* out = y + ((size_t)n * F + f) * OH * OW;
      std::memset(out, 0, sizeof(float) * OH * OW);
      for (int c = 0; c < C; ++c) {
        const float* xin = x + ((size_t)n * C + c) * H * W;
        for (int r = 0; r < R; ++r)
          for (int s = 0; s < S; ++s) {
            const float wv = w[(((size_t)f * C + c) * R + r) * S + s];
            const __m256 wvec = _mm256_set1_ps(wv);
            // output columns whose input column ox*stride - pad + s lies inside the image
            int ox0 = pad - s > 0 ? (pad - s + stride - 1) / stride : 0;
            int ox1 = (W - 1 + pad - s) / stride;  // inclusive
            if (ox1 > OW - 1) ox1 = OW - 1;
            for (int oy = 0; oy < OH; ++oy) {
              const int iy = oy * stride - pad + r;
              if (iy < 0 || iy >= H) continue;
              const float* xrow = xin + (size_t)iy * W + (s - pad);
              float* orow = out + (size_t)oy * OW;
              int ox = ox0;
              if (stride == 1) {
                for (; ox + 8 <= ox1 + 1; ox += 8)
                  _mm256_storeu_ps(orow + ox, _mm256_fmadd_ps(wvec, _mm256_loadu_ps(xrow + ox), _mm256_loadu_ps(orow + ox)));
              } else {
                for (; ox + 8 <= ox1 + 1; ox += 8) {
                  const __m256 xv = _mm256_i32gather_ps(xrow + (size_t)ox * stride, lane_off, 4);
                  _mm256_storeu_ps(orow + ox, _mm256_fmadd_ps(wvec, xv, _mm256_loadu_ps(orow + ox)));
                }
              }
              for (; ox <= ox1; ++ox) orow[ox] += wv * xrow[(size_t)ox * stride];
            }
          }
      }
    }
  return 0;
}
