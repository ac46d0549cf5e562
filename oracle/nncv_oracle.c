/*
 * nncv_oracle.c — CPU restatement of the arithmetic of nncv's ResNet-18 /
 * conv / matmul hot path.  TEST INFRASTRUCTURE ONLY: nothing that ships may
 * link, load or call this file; it exists so that the HIP kernels can be
 * checked against an independent, obviously-correct scalar implementation.
 *
 * The reference has no callable conv/GEMM function: the path is what its
 * compiler emits for the linalg ops in tests/Nets/Res18.mlir.  Every function
 * below therefore restates the *closed form of the op* and cites the line of
 * the reference that fixes its semantics.
 *
 * Numerics: storage is fp32 everywhere (as in Res18.mlir); contractions
 * (conv, matmul, pooling sum) accumulate in fp64 and round once, which is the
 * correctly-rounded value any fp32 summation order of the reference's
 * HostWParallel object approximates.  Element-wise ops follow the reference's
 * fp32 op order exactly.
 *
 * Pinning status (checked in tests/test_oracle_*.py):
 *   conv / matmul / pooling / BN / ReLU / FC : torch-CPU functional ops as an
 *       independent library routine, brute force on tiny shapes, the
 *       closed-form fixture of tests/SplitParams (output == 15.0) and of
 *       tests/ConvOptimization/conv2dNchwWinograd.mlir (filter == 0.1).
 *   Winograd F(4x4,3x3) : the algebraic identity winograd == direct conv.
 *   resnet18 forward : torch-CPU functional composition on seeded weights.
 *   Parity unpinned (no build of the reference object is possible): the
 *   exact fp32 summation order / last-ulp results of the HostWParallel object.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define IDX4(n, c, h, w, C, H, W) ((((int64_t)(n) * (C) + (c)) * (H) + (h)) * (W) + (w))

/* linalg.conv_2d_nchw_fchw, dilation 1 (tests/Nets/Res18.mlir:124, :157):
 *   out[n,f,y,x] += sum_{c,r,s} in[n,c,y*sh+r,x*sw+s] * w[f,c,r,s]
 * `in` is already padded (the reference pads with tensor.pad, :118-122).
 * Accumulates into `out` like the named op accumulates into `outs`. */
void orc_conv2d_nchw_fchw(const float* in, const float* w, float* out, int N, int C, int H, int W,
                          int F, int R, int S, int sh, int sw) {
  const int OH = (H - R) / sh + 1, OW = (W - S) / sw + 1;
#pragma omp parallel
  {
    double* acc = (double*)malloc(sizeof(double) * (size_t)OH * OW);
#pragma omp for collapse(2) schedule(dynamic)
    for (int n = 0; n < N; ++n)
      for (int f = 0; f < F; ++f) {
        for (int i = 0; i < OH * OW; ++i) acc[i] = 0.0;
        for (int c = 0; c < C; ++c)
          for (int r = 0; r < R; ++r)
            for (int s = 0; s < S; ++s) {
              const double wv = (double)w[((((int64_t)f * C + c) * R + r) * S) + s];
              for (int y = 0; y < OH; ++y) {
                const float* ip = in + IDX4(n, c, y * sh + r, s, C, H, W);
                double* ap = acc + (size_t)y * OW;
                for (int x = 0; x < OW; ++x) ap[x] += (double)ip[x * sw] * wv;
              }
            }
        float* op = out + IDX4(n, f, 0, 0, F, OH, OW);
        for (int i = 0; i < OH * OW; ++i) op[i] = (float)((double)op[i] + acc[i]);
      }
    free(acc);
  }
}

/* linalg.matmul (tests/MatMulOptimization/MatMulDeafult.mlir:7): C += A.B, row-major. */
void orc_matmul(const float* a, const float* b, float* c, int M, int N, int K) {
#pragma omp parallel
  {
    double* acc = (double*)malloc(sizeof(double) * (size_t)N);
#pragma omp for schedule(static)
    for (int i = 0; i < M; ++i) {
      for (int j = 0; j < N; ++j) acc[j] = 0.0;
      for (int k = 0; k < K; ++k) {
        const double av = (double)a[(int64_t)i * K + k];
        const float* bp = b + (int64_t)k * N;
        for (int j = 0; j < N; ++j) acc[j] += av * (double)bp[j];
      }
      for (int j = 0; j < N; ++j)
        c[(int64_t)i * N + j] = (float)((double)c[(int64_t)i * N + j] + acc[j]);
    }
    free(acc);
  }
}

/* tensor.pad on the two spatial dims with a constant (Res18.mlir:118-122 zero; :144-148 -inf). */
void orc_pad_nchw(const float* in, float* out, int N, int C, int H, int W, int pad, float value) {
  const int PH = H + 2 * pad, PW = W + 2 * pad;
  for (int64_t i = 0; i < (int64_t)N * C * PH * PW; ++i) out[i] = value;
  for (int nc = 0; nc < N * C; ++nc)
    for (int y = 0; y < H; ++y)
      memcpy(out + ((int64_t)nc * PH + y + pad) * PW + pad, in + ((int64_t)nc * H + y) * W,
             sizeof(float) * (size_t)W);
}

/* BatchNorm generic body (Res18.mlir:127-136): operands (x, gamma, beta, mean, var);
 *   t = truncf(1e-5 : f64); d = var + t; r = rsqrt(d); ((x - mean) * r) * gamma + beta
 * math.rsqrt lowers to 1/sqrt in fp32. */
void orc_batchnorm_nchw(const float* x, const float* gamma, const float* beta, const float* mean,
                        const float* var, float* y, int N, int C, int HW) {
  const float eps = (float)1e-5;
  for (int n = 0; n < N; ++n)
    for (int c = 0; c < C; ++c) {
      const float d = var[c] + eps;
      const float r = 1.0f / sqrtf(d);
      const float* xp = x + ((int64_t)n * C + c) * HW;
      float* yp = y + ((int64_t)n * C + c) * HW;
      for (int i = 0; i < HW; ++i) {
        const float a = xp[i] - mean[c];
        const float b = a * r;
        const float m = b * gamma[c];
        yp[i] = m + beta[c];
      }
    }
}

/* ReLU generic body (Res18.mlir:137-142): cmpf ugt x, 0 ; select -> NaN passes through. */
void orc_relu(const float* x, float* y, int64_t n) {
  for (int64_t i = 0; i < n; ++i) y[i] = (x[i] > 0.0f || isnan(x[i])) ? x[i] : 0.0f;
}

/* residual add generic (Res18.mlir:193-197): (bn_out, identity) -> bn_out + identity */
void orc_add(const float* a, const float* b, float* y, int64_t n) {
  for (int64_t i = 0; i < n; ++i) y[i] = a[i] + b[i];
}

static inline float maximumf_nan(float a, float b) { /* arith.maximumf: NaN-propagating */
  if (isnan(a)) return a;
  if (isnan(b)) return b;
  return a > b ? a : b;
}

/* linalg.pooling_nchw_max (Res18.mlir:151) on a pre-padded input, out pre-filled (-inf, :149). */
void orc_maxpool_nchw(const float* in, float* out, int N, int C, int H, int W, int KH, int KW,
                      int sh, int sw) {
  const int OH = (H - KH) / sh + 1, OW = (W - KW) / sw + 1;
  for (int nc = 0; nc < N * C; ++nc)
    for (int y = 0; y < OH; ++y)
      for (int x = 0; x < OW; ++x) {
        float m = out[((int64_t)nc * OH + y) * OW + x];
        for (int r = 0; r < KH; ++r)
          for (int s = 0; s < KW; ++s)
            m = maximumf_nan(m, in[((int64_t)nc * H + y * sh + r) * W + x * sw + s]);
        out[((int64_t)nc * OH + y) * OW + x] = m;
      }
}

/* linalg.pooling_nchw_sum over the whole HxW window, then one divf by H*W
 * (Res18.mlir:609-614): sum first, one divide. */
void orc_global_avgpool_nchw(const float* in, float* out, int N, int C, int H, int W) {
  const float div = (float)(H * W);
  for (int nc = 0; nc < N * C; ++nc) {
    double s = 0.0;
    for (int i = 0; i < H * W; ++i) s += (double)in[(int64_t)nc * H * W + i];
    out[nc] = (float)s / div;
  }
}

/* FC head (Res18.mlir:617-628): transpose W[1000,512] -> [512,1000]; matmul into zeros; + bias. */
void orc_fc(const float* x, const float* w, const float* bias, float* y, int N, int IN, int OUT) {
  for (int n = 0; n < N; ++n)
    for (int o = 0; o < OUT; ++o) {
      double s = 0.0;
      for (int k = 0; k < IN; ++k) s += (double)x[(int64_t)n * IN + k] * (double)w[(int64_t)o * IN + k];
      y[(int64_t)n * OUT + o] = (float)s + bias[o];
    }
}

/* ------------------------------------------------------------------------------------------
 * Winograd F(4x4,3x3).  Structure follows the reference's rewrite
 * (OptimizeConv2dUsingWinograd.cpp:41-83 filter fold, :173-284 conv rewrite;
 * TileAndDecoWinogradPass.cpp:149-232 input, :357-413 output) with the F(6,3) matrices replaced
 * by the textbook F(4,3) set (Lavin & Gray, points 0, +-1, +-2, inf).  Ragged edge tiles are
 * zero-padded (TileAndDecoWinogradPass.cpp:97-99, :208-211) and the result is sliced back
 * (OptimizeConv2dUsingWinograd.cpp:272-278).  Transforms are evaluated in fp64.
 * Layouts (t = 6*i + j):  U[t][F][C],  V[t][tiles][C],  M[t][tiles][F],
 * tiles = N * ceil(OH/4) * ceil(OW/4), tile index = (n*TH + ty)*TW + tx.
 * ------------------------------------------------------------------------------------------ */
static const double WBT[6][6] = {{4, 0, -5, 0, 1, 0},  {0, -4, -4, 1, 1, 0}, {0, 4, -4, -1, 1, 0},
                                 {0, -2, -1, 2, 1, 0}, {0, 2, -1, -2, 1, 0}, {0, 4, 0, -5, 0, 1}};
static const double WG[6][3] = {{1.0 / 4, 0, 0},
                                {-1.0 / 6, -1.0 / 6, -1.0 / 6},
                                {-1.0 / 6, 1.0 / 6, -1.0 / 6},
                                {1.0 / 24, 1.0 / 12, 1.0 / 6},
                                {1.0 / 24, -1.0 / 12, 1.0 / 6},
                                {0, 0, 1}};
static const double WAT[4][6] = {
    {1, 1, 1, 1, 1, 0}, {0, 1, -1, 2, -2, 0}, {0, 1, 1, 4, 4, 0}, {0, 1, -1, 8, -8, 1}};

/* U[i,j] = sum_{p,q} G[i,p] g[f,c,p,q] G[j,q]  (OptimizeConv2dUsingWinograd.cpp:57-70) */
void orc_wino43_filter_transform(const float* w, double* U, int F, int C) {
  for (int f = 0; f < F; ++f)
    for (int c = 0; c < C; ++c) {
      const float* g = w + ((int64_t)f * C + c) * 9;
      for (int i = 0; i < 6; ++i)
        for (int j = 0; j < 6; ++j) {
          double s = 0.0;
          for (int p = 0; p < 3; ++p)
            for (int q = 0; q < 3; ++q) s += WG[i][p] * (double)g[p * 3 + q] * WG[j][q];
          U[((int64_t)(i * 6 + j) * F + f) * C + c] = s;
        }
    }
}

/* V = B^T d B per 6x6 tile of the zero-padded (pad) input; tiles step 4. `in` is UNPADDED
 * [N,C,H,W]; the halo is supplied as zeros. */
void orc_wino43_input_transform(const float* in, double* V, int N, int C, int H, int W, int pad) {
  const int OH = H + 2 * pad - 2, OW = W + 2 * pad - 2;
  const int TH = (OH + 3) / 4, TW = (OW + 3) / 4;
  const int64_t tiles = (int64_t)N * TH * TW;
  for (int n = 0; n < N; ++n)
    for (int ty = 0; ty < TH; ++ty)
      for (int tx = 0; tx < TW; ++tx)
        for (int c = 0; c < C; ++c) {
          double d[6][6], t[6][6];
          for (int y = 0; y < 6; ++y)
            for (int x = 0; x < 6; ++x) {
              const int iy = ty * 4 + y - pad, ix = tx * 4 + x - pad;
              d[y][x] = (iy >= 0 && iy < H && ix >= 0 && ix < W) ? (double)in[IDX4(n, c, iy, ix, C, H, W)] : 0.0;
            }
          for (int i = 0; i < 6; ++i)
            for (int x = 0; x < 6; ++x) {
              double s = 0.0;
              for (int y = 0; y < 6; ++y) s += WBT[i][y] * d[y][x];
              t[i][x] = s;
            }
          const int64_t tile = ((int64_t)n * TH + ty) * TW + tx;
          for (int i = 0; i < 6; ++i)
            for (int j = 0; j < 6; ++j) {
              double s = 0.0;
              for (int x = 0; x < 6; ++x) s += t[i][x] * WBT[j][x];
              V[((int64_t)(i * 6 + j) * tiles + tile) * C + c] = s;
            }
        }
}

/* M[t] = V[t] . U[t]^T   (linalg.batch_matmul, OptimizeConv2dUsingWinograd.cpp:227-248) */
void orc_wino43_batched_gemm(const double* V, const double* U, double* M, int64_t tiles, int C, int F) {
#pragma omp parallel for collapse(2) schedule(static)
  for (int t = 0; t < 36; ++t)
    for (int64_t p = 0; p < tiles; ++p)
      for (int f = 0; f < F; ++f) {
        const double* v = V + ((int64_t)t * tiles + p) * C;
        const double* u = U + ((int64_t)t * F + f) * C;
        double s = 0.0;
        for (int c = 0; c < C; ++c) s += v[c] * u[c];
        M[((int64_t)t * tiles + p) * F + f] = s;
      }
}

/* Y = A^T M A per tile, sliced to [N,F,OH,OW]; out += Y (accumulating like the conv it replaces). */
void orc_wino43_output_transform(const double* M, float* out, int N, int F, int OH, int OW) {
  const int TH = (OH + 3) / 4, TW = (OW + 3) / 4;
  const int64_t tiles = (int64_t)N * TH * TW;
  for (int n = 0; n < N; ++n)
    for (int ty = 0; ty < TH; ++ty)
      for (int tx = 0; tx < TW; ++tx)
        for (int f = 0; f < F; ++f) {
          const int64_t tile = ((int64_t)n * TH + ty) * TW + tx;
          double m[6][6], t[4][6];
          for (int i = 0; i < 6; ++i)
            for (int j = 0; j < 6; ++j) m[i][j] = M[((int64_t)(i * 6 + j) * tiles + tile) * F + f];
          for (int a = 0; a < 4; ++a)
            for (int j = 0; j < 6; ++j) {
              double s = 0.0;
              for (int i = 0; i < 6; ++i) s += WAT[a][i] * m[i][j];
              t[a][j] = s;
            }
          for (int a = 0; a < 4; ++a)
            for (int b = 0; b < 4; ++b) {
              const int y = ty * 4 + a, x = tx * 4 + b;
              if (y >= OH || x >= OW) continue;
              double s = 0.0;
              for (int j = 0; j < 6; ++j) s += t[a][j] * WAT[b][j];
              float* o = out + IDX4(n, f, y, x, F, OH, OW);
              *o = (float)((double)*o + s);
            }
        }
}

/* Whole 3x3 stride-1 conv through the Winograd route (for the identity test). */
void orc_conv3x3_winograd43(const float* in, const float* w, float* out, int N, int C, int H, int W,
                            int F, int pad) {
  const int OH = H + 2 * pad - 2, OW = W + 2 * pad - 2;
  const int64_t tiles = (int64_t)N * ((OH + 3) / 4) * ((OW + 3) / 4);
  double* U = (double*)malloc(sizeof(double) * 36 * (size_t)F * C);
  double* V = (double*)malloc(sizeof(double) * 36 * (size_t)tiles * C);
  double* M = (double*)malloc(sizeof(double) * 36 * (size_t)tiles * F);
  orc_wino43_filter_transform(w, U, F, C);
  orc_wino43_input_transform(in, V, N, C, H, W, pad);
  orc_wino43_batched_gemm(V, U, M, tiles, C, F);
  orc_wino43_output_transform(M, out, N, F, OH, OW);
  free(U); free(V); free(M);
}

/* ------------------------------------------------------------------------------------------
 * ResNet-18 forward as emitted by torch-mlir (tests/Nets/Res18.mlir, whole file).
 * `params` is the flat fp32 blob of a -split-params model.bin in the canonical tensor order:
 * torchvision state_dict order without num_batches_tracked; each BN contributes
 * weight(gamma), bias(beta), running_mean, running_var.  102 tensors, 11 699 112 elements.
 * ------------------------------------------------------------------------------------------ */
typedef struct { const float *w, *g, *b, *m, *v; } conv_bn_t;

static const float* take(const float** p, int64_t n) { const float* r = *p; *p += n; return r; }

static conv_bn_t take_conv_bn(const float** p, int F, int C, int R) {
  conv_bn_t cb;
  cb.w = take(p, (int64_t)F * C * R * R);
  cb.g = take(p, F); cb.b = take(p, F); cb.m = take(p, F); cb.v = take(p, F);
  return cb;
}

/* pad -> conv -> BN (Res18.mlir:152-178 pattern); returns malloc'd [N,F,OH,OW] */
static float* conv_bn(const float* x, int N, int C, int H, int W, conv_bn_t cb, int F, int R,
                      int stride, int pad, int* OHo, int* OWo) {
  const int PH = H + 2 * pad, PW = W + 2 * pad;
  const int OH = (PH - R) / stride + 1, OW = (PW - R) / stride + 1;
  float* xp = (float*)malloc(sizeof(float) * (size_t)N * C * PH * PW);
  orc_pad_nchw(x, xp, N, C, H, W, pad, 0.0f);
  float* y = (float*)calloc((size_t)N * F * OH * OW, sizeof(float));
  orc_conv2d_nchw_fchw(xp, cb.w, y, N, C, PH, PW, F, R, R, stride, stride);
  free(xp);
  orc_batchnorm_nchw(y, cb.g, cb.b, cb.m, cb.v, y, N, F, OH * OW);
  *OHo = OH; *OWo = OW;
  return y;
}

int64_t orc_resnet18_num_params(void) { return 11699112; }

/* Optional taps: if `tap_layer` >= 0 the activation after that residual stage (0: after maxpool,
 * 1..4: after layer1..layer4) is copied to `tap` (NCHW). */
int orc_resnet18_forward(const float* x, int N, int H, int W, const float* params, float* logits,
                         int tap_layer, float* tap) {
  const float* p = params;
  int oh, ow;
  /* stem: pad3, conv7x7 s2, BN, ReLU (Res18.mlir:118-142) */
  conv_bn_t stem = take_conv_bn(&p, 64, 3, 7);
  float* a = conv_bn(x, N, 3, H, W, stem, 64, 7, 2, 3, &oh, &ow);
  orc_relu(a, a, (int64_t)N * 64 * oh * ow);
  /* maxpool 3x3 s2 on -inf padded (Res18.mlir:144-151) */
  {
    const int PH = oh + 2, PW = ow + 2, OH = (PH - 3) / 2 + 1, OW = (PW - 3) / 2 + 1;
    float* ap = (float*)malloc(sizeof(float) * (size_t)N * 64 * PH * PW);
    orc_pad_nchw(a, ap, N, 64, oh, ow, 1, -INFINITY);
    float* y = (float*)malloc(sizeof(float) * (size_t)N * 64 * OH * OW);
    for (int64_t i = 0; i < (int64_t)N * 64 * OH * OW; ++i) y[i] = -INFINITY;
    orc_maxpool_nchw(ap, y, N, 64, PH, PW, 3, 3, 2, 2);
    free(ap); free(a);
    a = y; oh = OH; ow = OW;
  }
  if (tap_layer == 0) memcpy(tap, a, sizeof(float) * (size_t)N * 64 * oh * ow);
  int C = 64;
  static const int widths[4] = {64, 128, 256, 512};
  for (int L = 0; L < 4; ++L) {
    const int F = widths[L];
    for (int blk = 0; blk < 2; ++blk) {
      const int stride = (L > 0 && blk == 0) ? 2 : 1;
      const int down = (stride != 1 || C != F);
      conv_bn_t c1 = take_conv_bn(&p, F, C, 3);
      conv_bn_t c2 = take_conv_bn(&p, F, F, 3);
      conv_bn_t ds; memset(&ds, 0, sizeof ds);
      if (down) ds = take_conv_bn(&p, F, C, 1);
      int h1, w1, h2, w2;
      float* y1 = conv_bn(a, N, C, oh, ow, c1, F, 3, stride, 1, &h1, &w1);
      orc_relu(y1, y1, (int64_t)N * F * h1 * w1);
      float* y2 = conv_bn(y1, N, F, h1, w1, c2, F, 3, 1, 1, &h2, &w2);
      free(y1);
      float* idn = a;
      if (down) { /* 1x1 s2 on the unpadded block input (Res18.mlir:297), BN (:299-309) */
        int hd, wd;
        idn = conv_bn(a, N, C, oh, ow, ds, F, 1, stride, 0, &hd, &wd);
        free(a);
      }
      orc_add(y2, idn, y2, (int64_t)N * F * h2 * w2); /* (bn_out, identity) :193, :310 */
      orc_relu(y2, y2, (int64_t)N * F * h2 * w2);
      free(idn);
      a = y2; C = F; oh = h2; ow = w2;
    }
    if (tap_layer == L + 1) memcpy(tap, a, sizeof(float) * (size_t)N * C * oh * ow);
  }
  /* head (Res18.mlir:609-628) */
  float* pooled = (float*)malloc(sizeof(float) * (size_t)N * 512);
  orc_global_avgpool_nchw(a, pooled, N, 512, oh, ow);
  free(a);
  const float* fw = take(&p, 1000 * 512);
  const float* fb = take(&p, 1000);
  orc_fc(pooled, fw, fb, logits, N, 512, 1000);
  free(pooled);
  return (p - params) == orc_resnet18_num_params() ? 0 : -1;
}
