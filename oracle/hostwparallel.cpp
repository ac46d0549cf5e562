// CPU baselines of the convolution for bench.py, two of them:
//
//  hwp_conv2d_nchw_fchw      this repository's OWN OpenMP x AVX2 routine: (image, filter) pairs across all threads,
//                            the output row 8 wide in AVX2 FMAs.  It is NOT the reference's schedule -- the
//                            reference tiles linalg.conv_2d_nchw_fchw with sequential scf.for only
//                            (ModernTile.cpp:330-331: the scf.forall form "is not impl yet") -- and it is faster
//                            than that schedule; it is the stronger CPU baseline of the two.
//  hwp_conv2d_ref_schedule   the reference's tile order, sequential: level 1 {0, Ft, OH, 8} with Ft the largest of
//                            1024..1 below F that divides F, level 2 {1, 8, 1, 8}, level 3 {0,0,0,0, 8, 1, 1}
//                            (ModernTile.cpp:126-136, :184-199), i.e. for f0 . for ow0 . for n . for f step 8 .
//                            for oh . for c step 8 . for kh . for kw, an [8 filters x 8 columns] block of 8-wide
//                            FMAs innermost (ModernVec.cpp:54-62); strided layers tile oh and ow to 1
//                            (ModernTile.cpp:203-209) and run scalar.  The halo is materialised first, as the
//                            reference's tensor.pad is.
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

// The reference's schedule (see the head of the file): one thread, its tile order.
extern "C" int hwp_conv2d_ref_schedule(const float* x, const float* w, float* y, int N, int C, int H, int W, int F, int R, int S,
                                       int stride, int pad) {
  const int OH = (H + 2 * pad - R) / stride + 1, OW = (W + 2 * pad - S) / stride + 1;
  if (OH <= 0 || OW <= 0) return 1;
  const int HP = H + 2 * pad, WP = W + 2 * pad + 8;  // + 8: the 8-wide loads of a last, partial column tile stay inside
  std::vector<float> xp((size_t)N * C * HP * WP, 0.0f);
  for (int n = 0; n < N; ++n)
    for (int c = 0; c < C; ++c)
      for (int iy = 0; iy < H; ++iy)
        std::memcpy(&xp[(((size_t)n * C + c) * HP + iy + pad) * WP + pad], x + (((size_t)n * C + c) * H + iy) * W, sizeof(float) * W);
  std::memset(y, 0, sizeof(float) * (size_t)N * F * OH * OW);
  int Ft = 1;
  for (int cand : {1024, 512, 256, 128, 64, 32, 16, 8, 4, 2, 1})
    if (cand < F && F % cand == 0) { Ft = cand; break; }
  if (stride != 1) {
    // oh and ow tiled to 1: a scalar multiply-add per (filter, channel, tap) in the same loop order
    for (int f0 = 0; f0 < F; f0 += Ft)
      for (int ow = 0; ow < OW; ++ow)
        for (int n = 0; n < N; ++n)
          for (int f = f0; f < f0 + Ft && f < F; ++f)
            for (int oh = 0; oh < OH; ++oh) {
              float acc = 0.0f;
              for (int c = 0; c < C; ++c)
                for (int r = 0; r < R; ++r)
                  for (int s = 0; s < S; ++s)
                    acc += xp[(((size_t)n * C + c) * HP + oh * stride + r) * WP + ow * stride + s] * w[(((size_t)f * C + c) * R + r) * S + s];
              y[(((size_t)n * F + f) * OH + oh) * OW + ow] = acc;
            }
    return 0;
  }
  for (int f0 = 0; f0 < F; f0 += Ft)
    for (int ow0 = 0; ow0 < OW; ow0 += 8) {
      const int wcols = OW - ow0 < 8 ? OW - ow0 : 8;
      for (int n = 0; n < N; ++n)
        for (int f = f0; f < f0 + Ft; f += 8) {
          const int nf = F - f < 8 ? F - f : 8;
          for (int oh = 0; oh < OH; ++oh) {
            __m256 acc[8];
            for (int i = 0; i < 8; ++i) acc[i] = _mm256_setzero_ps();
            for (int c0 = 0; c0 < C; c0 += 8)
              for (int r = 0; r < R; ++r)
                for (int s = 0; s < S; ++s)
                  for (int c = c0; c < c0 + 8 && c < C; ++c) {
                    const __m256 xv = _mm256_loadu_ps(&xp[(((size_t)n * C + c) * HP + oh + r) * WP + ow0 + s]);
                    for (int i = 0; i < nf; ++i)
                      acc[i] = _mm256_fmadd_ps(_mm256_set1_ps(w[(((size_t)(f + i) * C + c) * R + r) * S + s]), xv, acc[i]);
                  }
            for (int i = 0; i < nf; ++i) {
              float tmp[8];
              _mm256_storeu_ps(tmp, acc[i]);
              std::memcpy(y + (((size_t)n * F + f + i) * OH + oh) * OW + ow0, tmp, sizeof(float) * wcols);
            }
          }
        }
    }
  return 0;
}
