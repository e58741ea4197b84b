/*
 * TEST INFRASTRUCTURE: CPU restatement of the reference's unfold / fold for
 * the 2-D convolution (opzoo/Convolution/Convolution.cpp:13-90) and of the
 * products the operator builds from them (opzoo/Convolution/Convolution.py:
 * 17-57).  Plain C, fp32, no fused multiply-add.  Only tests, the smoke check
 * and the benchmark's CPU-baseline leg may load this file's library.
 *
 * Pins (tests/test_conv_oracle.py): im2col / col2im bit-exact against the
 * compiled reference (oracle/_ref/libref_conv.so); col2im is the adjoint of
 * im2col; the assembled convolution and its three gradients against
 * torch.nn.functional.conv2d and its autograd on the CPU (a library routine;
 * the reference's own test compares with mx.gluon.nn.Conv2D the same way,
 * opzoo/Convolution/test_conv.py:9-48, at its shape and tolerance).
 */
#include <stddef.h>
#include <string.h>

/* opzoo/Convolution/Convolution.cpp:13-45 */
void oracle_im2col_f32(int n, const float* im, int H, int W, int KH, int KW, int pad_h, int pad_w,
                       int stride_h, int stride_w, int dil_h, int dil_w, int OH, int OW, float* col) {
  for (int index = 0; index < n; ++index) {
    int t = index;
    const int ow = t % OW; t /= OW;
    const int oh = t % OH; t /= OH;
    const int kw = t % KW; t /= KW;
    const int kh = t % KH; t /= KH;
    const int c = t;
    const int ih = -pad_h + kh * dil_h + stride_h * oh;
    const int iw = -pad_w + kw * dil_w + stride_w * ow;
    col[index] = (ih >= 0 && ih < H && iw >= 0 && iw < W) ? im[(c * H + ih) * W + iw] : 0.0f;
  }
}

/* opzoo/Convolution/Convolution.cpp:47-90 */
void oracle_col2im_f32(int n, const float* col, int H, int W, int KH, int KW, int pad_h, int pad_w,
                       int stride_h, int stride_w, int dil_h, int dil_w, int OH, int OW, float* im) {
  const int ext_w = (KW - 1) * dil_w + 1, ext_h = (KH - 1) * dil_h + 1;
  for (int index = 0; index < n; ++index) {
    float val = 0.0f;
    const int w_im = index % W + pad_w;
    const int h_im = (index / W) % H + pad_h;
    const int c = index / (W * H);
    const int w0 = (w_im < ext_w) ? 0 : (w_im - ext_w) / stride_w + 1;
    const int w1 = (w_im / stride_w + 1 < OW) ? w_im / stride_w + 1 : OW;
    const int h0 = (h_im < ext_h) ? 0 : (h_im - ext_h) / stride_h + 1;
    const int h1 = (h_im / stride_h + 1 < OH) ? h_im / stride_h + 1 : OH;
    for (int oh = h0; oh < h1; ++oh)
      for (int ow = w0; ow < w1; ++ow) {
        int hk = h_im - oh * stride_h, wk = w_im - ow * stride_w;
        if (hk % dil_h == 0 && wk % dil_w == 0) {
          hk /= dil_h; wk /= dil_w;
          val += col[(((c * KH + hk) * KW + wk) * OH + oh) * OW + ow];
        }
      }
    im[index] = val;
  }
}

/* out[M, N] = a[M, K] x b[K, N], fp32 accumulation in k order (the framework
 * product the reference calls, Convolution.py:31,50,56, is not part of the
 * reference's sources; any order is within the parity tolerance). */
static void matmul(const float* a, const float* b, float* out, int M, int K, int N) {
  for (int i = 0; i < M; ++i) {
    float* o = out + (size_t)i * N;
    memset(o, 0, sizeof(float) * N);
    for (int k = 0; k < K; ++k) {
      const float av = a[(size_t)i * K + k];
      const float* br = b + (size_t)k * N;
      for (int j = 0; j < N; ++j) o[j] += av * br[j];
    }
  }
}

/* Convolution.py:17-34: per image im2col, weight[D, C*KH*KW] x col, + bias. */
void oracle_conv2d_forward_f32(const float* x, const float* w, const float* bias, int N, int C, int H, int W,
                               int D, int KH, int KW, int pad_h, int pad_w, int stride_h, int stride_w,
                               int dil_h, int dil_w, int OH, int OW, float* col /* [C*KH*KW*OH*OW] */,
                               float* y) {
  const int K = C * KH * KW, ohw = OH * OW;
  for (int i = 0; i < N; ++i) {
    oracle_im2col_f32(K * ohw, x + (size_t)i * C * H * W, H, W, KH, KW, pad_h, pad_w, stride_h, stride_w,
                      dil_h, dil_w, OH, OW, col);
    float* yi = y + (size_t)i * D * ohw;
    matmul(w, col, yi, D, K, ohw);
    if (bias != NULL)
      for (int d = 0; d < D; ++d)
        for (int j = 0; j < ohw; ++j) yi[(size_t)d * ohw + j] += bias[d];
  }
}

/* Convolution.py:36-57: dx = col2im(weight' x dy), dw = sum over images of
 * dy x col(x)', db = sum of dy.  scratch holds two [C*KH*KW*OH*OW] buffers. */
void oracle_conv2d_backward_f32(const float* dy, const float* x, const float* w, int N, int C, int H, int W,
                                int D, int KH, int KW, int pad_h, int pad_w, int stride_h, int stride_w,
                                int dil_h, int dil_w, int OH, int OW, float* scratch, float* dx, float* dw,
                                float* db) {
  const int K = C * KH * KW, ohw = OH * OW;
  float* col = scratch;
  float* colx = scratch + (size_t)K * ohw;
  memset(dw, 0, sizeof(float) * (size_t)D * K);
  if (db != NULL) memset(db, 0, sizeof(float) * D);
  for (int i = 0; i < N; ++i) {
    const float* dyi = dy + (size_t)i * D * ohw;
    /* col[k, j] = sum_d w[d, k] * dy[d, j] */
    for (int k = 0; k < K; ++k) {
      float* o = col + (size_t)k * ohw;
      memset(o, 0, sizeof(float) * ohw);
      for (int d = 0; d < D; ++d) {
        const float wv = w[(size_t)d * K + k];
        const float* dr = dyi + (size_t)d * ohw;
        for (int j = 0; j < ohw; ++j) o[j] += wv * dr[j];
      }
    }
    oracle_col2im_f32(C * H * W, col, H, W, KH, KW, pad_h, pad_w, stride_h, stride_w, dil_h, dil_w, OH, OW,
                      dx + (size_t)i * C * H * W);
    oracle_im2col_f32(K * ohw, x + (size_t)i * C * H * W, H, W, KH, KW, pad_h, pad_w, stride_h, stride_w,
                      dil_h, dil_w, OH, OW, colx);
    for (int d = 0; d < D; ++d) {
      const float* dr = dyi + (size_t)d * ohw;
      for (int k = 0; k < K; ++k) {
        const float* cr = colx + (size_t)k * ohw;
        float s = 0.0f;
        for (int j = 0; j < ohw; ++j) s += dr[j] * cr[j];
        dw[(size_t)d * K + k] += s;
      }
      if (db != NULL) {
        float s = 0.0f;
        for (int j = 0; j < ohw; ++j) s += dr[j];
        db[d] += s;
      }
    }
  }
}
