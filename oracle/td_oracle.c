/*
 * td_oracle.c — CPU restatement of tiny-dnn's training hot path.
 *
 * TEST INFRASTRUCTURE ONLY: this file is the checker for the HIP library. It
 * is never linked into the product; only tests, the smoke check and the
 * benchmark's cpu_baseline leg load it.
 *
 * Every function follows the reference's scalar ("internal" engine) loops and
 * cites the file:line it restates (paths relative to the tiny-dnn tree).
 * float_t = float (tiny_dnn/config.h:88-92). Summation order inside one
 * sample is the reference's; across samples weight gradients are summed in
 * sample order 0..N-1, which is what edge::merge_grads does
 * (tiny_dnn/node.h:89-103). OpenMP is used only over loops whose iterations
 * are independent in the reference too, so results do not depend on the
 * thread count.
 *
 * Pinning (what fixes each function independently of this file; all checked
 * in tests/test_oracle_*.py):
 *   conv fwd/bwd   reference KATs test/test_convolutional_layer.h:82-252,
 *                  float64 brute-force definition, torch.nn.functional.conv2d
 *                  and its autograd, compiled reference (oracle/_ref)
 *   fc fwd/bwd     KATs test/test_fully_connected_layer.h:48-118, numpy matmul,
 *                  compiled reference
 *   max-pool       KATs test/test_max_pooling_layer.h:25-281, compiled reference
 *   ave-pool       KATs test/test_average_pooling_layer.h:14-71, numeric
 *                  gradient check, compiled reference
 *   activations    closed forms, numeric gradient check, compiled reference
 *   losses         closed forms, softmax∘CE identity dz = y - t
 *   optimizers     two-step KATs test/test_optimizers.h:15-190, compiled reference
 *   net step       compiled reference network<sequential>::fit on the same
 *                  seeded arrays (committed fixture tests/golden/lenet_step.npz)
 */
#include "td_oracle.h"

#include <float.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------ shapes */

/* tiny_dnn/util/util.h:329-344 (conv_out_length) */
static int conv_out_length(int in_length, int window, int stride, int dilation, int pad_same) {
  int output_length = pad_same ? in_length : in_length - dilation * window + dilation;
  return (output_length + stride - 1) / stride;
}

/* tiny_dnn/util/util.h:346-363 (pool_out_length): float division then floor/ceil */
static int pool_out_length(int in_length, int window, int stride, int ceil_mode, int pad_same) {
  int output_length = pad_same ? in_length : in_length - window + 1;
  float tmp         = (float)(output_length + stride - 1) / (float)stride;
  return (int)(ceil_mode ? ceilf(tmp) : floorf(tmp));
}

int tdo_conv_out_w(const tdo_conv_desc *d) {
  return conv_out_length(d->in_w, d->k_w, d->w_stride, d->w_dilation, d->pad_same);
}
int tdo_conv_out_h(const tdo_conv_desc *d) {
  return conv_out_length(d->in_h, d->k_h, d->h_stride, d->h_dilation, d->pad_same);
}
/* tiny_dnn/layers/convolutional_layer.h:470-475 (in_length) */
int tdo_conv_padded_w(const tdo_conv_desc *d) {
  return d->pad_same ? d->in_w + d->k_w - 1 : d->in_w;
}
int tdo_conv_padded_h(const tdo_conv_desc *d) {
  return d->pad_same ? d->in_h + d->k_h - 1 : d->in_h;
}
int tdo_pool_out_w(const tdo_pool_desc *d) {
  return pool_out_length(d->in_w, d->pool_w, d->stride_w, d->ceil_mode, d->pad_same);
}
int tdo_pool_out_h(const tdo_pool_desc *d) {
  return pool_out_length(d->in_h, d->pool_h, d->stride_h, d->ceil_mode, d->pad_same);
}

/* connection_table::is_connected(x = outc, y = inc) = connected_[y*cols + x]
 * (tiny_dnn/core/params/conv_params.h:52-56), rows = in_c, cols = out_c */
static inline int tbl_connected(const tdo_conv_desc *d, int outc, int inc) {
  return d->tbl == NULL ? 1 : (d->tbl[(size_t)inc * d->out_c + outc] != 0);
}

/* vectorize::dot, generic (non-SIMD) instantiation: detail::dot_product<scalar_generic>
 * (tiny_dnn/util/product.h:321-364) keeps four running sums over i%4 and adds them as
 * (r0+r1)+(r2+r3); the size%4 tail goes into r0 first. */
static inline float dot4(const float *f1, const float *f2, size_t size) {
  float r0 = 0.0f, r1 = 0.0f, r2 = 0.0f, r3 = 0.0f;
  const size_t n4 = size / 4, n1 = size % 4;
  for (size_t i = 0; i < n4; ++i) {
    r0 = f1[i * 4 + 0] * f2[i * 4 + 0] + r0;
    r1 = f1[i * 4 + 1] * f2[i * 4 + 1] + r1;
    r2 = f1[i * 4 + 2] * f2[i * 4 + 2] + r2;
    r3 = f1[i * 4 + 3] * f2[i * 4 + 3] + r3;
  }
  const size_t idx = n4 * 4;
  for (size_t i = 0; i < n1; ++i) r0 = f1[idx + i] * f2[idx + i] + r0;
  r0 = r0 + r1;
  r2 = r2 + r3;
  r0 = r0 + r2;
  return r0;
}

/* ------------------------------------------------------------- convolution */

/* Conv2dPadding::copy_and_pad_input, tiny_dnn/core/params/conv_params.h:106-133:
 * offset (k_w/2, k_h/2), zero elsewhere. */
static float *pad_input(const tdo_conv_desc *d, int batch, const float *x) {
  const int pw = tdo_conv_padded_w(d), ph = tdo_conv_padded_h(d);
  const size_t psz = (size_t)pw * ph * d->in_c;
  const size_t isz = (size_t)d->in_w * d->in_h * d->in_c;
  float *buf       = (float *)calloc(psz * (size_t)batch, sizeof(float));
  if (!buf) return NULL;
  const int ox = d->pad_same ? d->k_w / 2 : 0, oy = d->pad_same ? d->k_h / 2 : 0;
#pragma omp parallel for schedule(static)
  for (int s = 0; s < batch; s++)
    for (int c = 0; c < d->in_c; c++)
      for (int y = 0; y < d->in_h; y++)
        memcpy(buf + psz * s + ((size_t)ph * c + y + oy) * pw + ox,
               x + isz * s + ((size_t)d->in_h * c + y) * d->in_w, sizeof(float) * d->in_w);
  return buf;
}

/* kernels::conv2d_op_internal (forward), tiny_dnn/core/kernels/conv2d_op_internal.h:13-74;
 * out_data is zero-filled by Conv2dOp::compute (tiny_dnn/core/kernels/conv2d_op.h:35). */
int tdo_conv2d_fwd(const tdo_conv_desc *d, int batch, const float *x, const float *w,
                   const float *b, float *y) {
  const int iw = tdo_conv_padded_w(d), ih = tdo_conv_padded_h(d);
  const int ow = tdo_conv_out_w(d), oh = tdo_conv_out_h(d);
  const int id = d->in_c, od = d->out_c, kw = d->k_w, kh = d->k_h;
  const size_t psz = (size_t)iw * ih * id, osz = (size_t)ow * oh * od;
  /* padding::same pads by the undilated window (convolutional_layer.h:470-474), so with a
   * dilation the loop below would read past the padded rows, as the reference does: there is
   * no defined result to restate. */
  if (d->pad_same && (d->w_dilation != 1 || d->h_dilation != 1)) return -2;
  float *xp = pad_input(d, batch, x);
  if (!xp) return -1;
#pragma omp parallel for schedule(static)
  for (int s = 0; s < batch; s++) {
    const float *in = xp + psz * s;
    float *a        = y + osz * s;
    for (int o = 0; o < od; o++) {
      float *pa = a + (size_t)oh * ow * o;
      for (int i = 0; i < oh * ow; i++) pa[i] = 0.0f;
      for (int inc = 0; inc < id; inc++) {
        if (!tbl_connected(d, o, inc)) continue;
        const float *pw  = w + (size_t)kw * kh * (id * o + inc);
        const float *pin = in + (size_t)iw * ih * inc;
        float *pout      = pa;
        for (int yy = 0; yy < oh; yy++) {
          const float *pin_line = pin;
          for (int xx = 0; xx < ow; xx++) {
            const float *pin_element = pin_line;
            const float *pw_element  = pw;
            float sum                = 0.0f;
            for (int wy = 0; wy < kh; wy++) {
              for (int wx = 0; wx < kw; wx++)
                sum += pw_element[wx] * pin_element[wx * d->w_dilation];
              pw_element += kw;
              pin_element += iw * d->h_dilation;
            }
            pout[xx] += sum;
            pin_line += d->w_stride;
          }
          pout += ow;
          pin += (size_t)iw * d->h_stride;
        }
      }
      if (d->has_bias)
        for (int i = 0; i < oh * ow; i++) pa[i] += b[o];
    }
  }
  free(xp);
  return 0;
}

/* Conv2dGradOp::compute + kernels::conv2d_op_internal (backward),
 * tiny_dnn/core/kernels/conv2d_grad_op.h:22-50, conv2d_op_internal.h:78-181,
 * then Conv2dPadding::copy_and_unpad_delta (conv_params.h:140-166).
 * Like the reference, the backward pass ignores the dilation fields. */
int tdo_conv2d_bwd(const tdo_conv_desc *d, int batch, const float *x, const float *w,
                   const float *dy, float *dx, float *dw, float *db) {
  const int iw = tdo_conv_padded_w(d), ih = tdo_conv_padded_h(d);
  const int ow = tdo_conv_out_w(d), oh = tdo_conv_out_h(d);
  const int id = d->in_c, od = d->out_c, kw = d->k_w, kh = d->k_h;
  const size_t psz = (size_t)iw * ih * id, osz = (size_t)ow * oh * od;
  const size_t isz = (size_t)d->in_w * d->in_h * id;
  float *xp        = pad_input(d, batch, x);
  float *dxp       = (float *)calloc(psz * (size_t)batch, sizeof(float)); /* fill_tensor(prev_delta,0) */
  if (!xp || !dxp) {
    free(xp);
    free(dxp);
    return -1;
  }

  /* propagate delta to previous layer: scatter, conv2d_op_internal.h:91-127 */
#pragma omp parallel for schedule(static)
  for (int s = 0; s < batch; s++) {
    for (int inc = 0; inc < id; inc++) {
      for (int outc = 0; outc < od; outc++) {
        if (!tbl_connected(d, outc, inc)) continue;
        const float *pw         = w + (size_t)kw * kh * (id * outc + inc);
        const float *pdelta_src = dy + osz * s + (size_t)oh * ow * outc;
        float *pdelta_dst       = dxp + psz * s + (size_t)iw * ih * inc;
        for (int yy = 0; yy < oh; yy++) {
          for (int xx = 0; xx < ow; xx++) {
            const float *ppw        = pw;
            const float ppdelta_src = pdelta_src[yy * ow + xx];
            float *ppdelta_dst = pdelta_dst + (size_t)yy * d->h_stride * iw + xx * d->w_stride;
            for (int wy = 0; wy < kh; wy++)
              for (int wx = 0; wx < kw; wx++) ppdelta_dst[wy * iw + wx] += *ppw++ * ppdelta_src;
          }
        }
      }
    }
  }
  /* unpad (identity copy for padding::valid) */
  {
    const int ox = d->pad_same ? kw / 2 : 0, oy = d->pad_same ? kh / 2 : 0;
#pragma omp parallel for schedule(static)
    for (int s = 0; s < batch; s++)
      for (int c = 0; c < id; c++)
        for (int yy = 0; yy < d->in_h; yy++)
          memcpy(dx + isz * s + ((size_t)d->in_h * c + yy) * d->in_w,
                 dxp + psz * s + ((size_t)ih * c + yy + oy) * iw + ox, sizeof(float) * d->in_w);
  }

  /* accumulate dw: conv2d_op_internal.h:130-169, merged over samples in order */
  if (dw) {
#pragma omp parallel for schedule(dynamic) collapse(2)
    for (int inc = 0; inc < id; inc++) {
      for (int outc = 0; outc < od; outc++) {
        for (int wy = 0; wy < kh; wy++) {
          for (int wx = 0; wx < kw; wx++) {
            const size_t widx = (size_t)kw * kh * (id * outc + inc) + (size_t)wy * kw + wx;
            if (!tbl_connected(d, outc, inc)) {
              dw[widx] = 0.0f;
              continue;
            }
            float merged = 0.0f;
            for (int s = 0; s < batch; s++) {
              float dst          = 0.0f;
              const float *prevo = xp + psz * s + ((size_t)ih * inc + wy) * iw + wx;
              const float *delta = dy + osz * s + (size_t)oh * ow * outc;
              if (d->w_stride > 1) {
                for (int yy = 0; yy < oh; yy++) {
                  const size_t prevo_idx = (size_t)yy * iw * d->h_stride;
                  const size_t delta_idx = (size_t)yy * ow;
                  for (int xx = 0; xx < ow; xx++)
                    dst += prevo[prevo_idx + (size_t)xx * d->w_stride] * delta[delta_idx + xx];
                }
              } else {
                for (int yy = 0; yy < oh; yy++) {
                  dst += dot4(prevo + (size_t)yy * iw * d->h_stride, delta + (size_t)yy * ow,
                              (size_t)ow);
                }
              }
              /* dW[sample] starts at 0 (clear_grads), merge_grads: copy sample 0, add the rest */
              merged = (s == 0) ? (0.0f + dst) : merged + (0.0f + dst);
            }
            dw[widx] = merged;
          }
        }
      }
    }
  }

  /* accumulate db: conv2d_op_internal.h:172-179 */
  if (db && d->has_bias) {
    for (int outc = 0; outc < od; outc++) {
      float merged = 0.0f;
      for (int s = 0; s < batch; s++) {
        const float *delta = dy + osz * s + (size_t)oh * ow * outc;
        float acc          = 0.0f;
        for (int i = 0; i < oh * ow; i++) acc += delta[i];
        merged = (s == 0) ? acc : merged + acc;
      }
      db[outc] = merged;
    }
  }
  free(xp);
  free(dxp);
  return 0;
}

/* -------------------------------------------------------- fully connected */

/* kernels::fully_connected_op_internal (forward),
 * tiny_dnn/core/kernels/fully_connected_op_internal.h:15-36 */
int tdo_fc_fwd(int in, int out, int has_bias, int batch, const float *x, const float *w,
               const float *b, float *y) {
#pragma omp parallel for schedule(static)
  for (int s = 0; s < batch; s++) {
    const float *xi = x + (size_t)in * s;
    float *yo       = y + (size_t)out * s;
    for (int i = 0; i < out; i++) yo[i] = 0.0f;
    /* same per-output summation order (c ascending); loop interchange keeps
     * every out[i] a left-to-right sum over c */
    for (int c = 0; c < in; c++) {
      const float *wr = w + (size_t)c * out;
      const float xc  = xi[c];
      for (int i = 0; i < out; i++) yo[i] += wr[i] * xc;
    }
    if (has_bias)
      for (int i = 0; i < out; i++) yo[i] += b[i];
  }
  return 0;
}

/* FullyConnectedGradOp::compute + kernels::fully_connected_op_internal (backward),
 * tiny_dnn/core/kernels/fully_connected_grad_op.h:22-52,
 * fully_connected_op_internal.h:38-71 */
int tdo_fc_bwd(int in, int out, int has_bias, int batch, const float *x, const float *w,
               const float *dy, float *dx, float *dw, float *db) {
#pragma omp parallel for schedule(static)
  for (int s = 0; s < batch; s++) {
    const float *d = dy + (size_t)out * s;
    for (int c = 0; c < in; c++) {
      const float *wr = w + (size_t)c * out;
      dx[(size_t)in * s + c] = 0.0f + dot4(d, wr, (size_t)out);
    }
  }
  if (dw) {
#pragma omp parallel for schedule(static)
    for (int c = 0; c < in; c++) {
      float *dwr = dw + (size_t)c * out;
      for (int s = 0; s < batch; s++) {
        const float *d = dy + (size_t)out * s;
        const float xc = x[(size_t)in * s + c];
        if (s == 0)
          for (int r = 0; r < out; r++) dwr[r] = 0.0f + d[r] * xc;
        else
          for (int r = 0; r < out; r++) dwr[r] += 0.0f + d[r] * xc;
      }
    }
  }
  if (db && has_bias) {
    for (int r = 0; r < out; r++) {
      float merged = 0.0f;
      for (int s = 0; s < batch; s++) merged = (s == 0) ? dy[r] : merged + dy[(size_t)out * s + r];
      db[r] = merged;
    }
  }
  return 0;
}

/* ------------------------------------------------------------ max pooling */

/* kernels::maxpool_op_internal, tiny_dnn/core/kernels/maxpool_op_internal.h:16-40,
 * windows from max_pooling_layer::connect_kernel/init_connection
 * (tiny_dnn/layers/max_pooling_layer.h:195-235): clipped at right/bottom,
 * scanned dy-major; strict '>' so the first maximum wins and NaN never wins. */
int tdo_maxpool_fwd(const tdo_pool_desc *d, int batch, const float *x, float *y,
                    int64_t *argmax) {
  const int ow = tdo_pool_out_w(d), oh = tdo_pool_out_h(d);
  const size_t isz = (size_t)d->in_w * d->in_h * d->in_c, osz = (size_t)ow * oh * d->in_c;
#pragma omp parallel for schedule(static)
  for (int s = 0; s < batch; s++) {
    const float *in = x + isz * s;
    for (int c = 0; c < d->in_c; c++)
      for (int oy = 0; oy < oh; oy++)
        for (int ox = 0; ox < ow; ox++) {
          int dxmax = d->in_w - ox * d->stride_w;
          int dymax = d->in_h - oy * d->stride_h;
          if (dxmax > d->pool_w) dxmax = d->pool_w;
          if (dymax > d->pool_h) dymax = d->pool_h;
          float max_value = -FLT_MAX; /* numeric_limits<float>::lowest() */
          int64_t idx     = 0;
          for (int wy = 0; wy < dymax; wy++)
            for (int wx = 0; wx < dxmax; wx++) {
              const int64_t j = ((int64_t)d->in_h * c + oy * d->stride_h + wy) * d->in_w +
                                ox * d->stride_w + wx;
              if (in[j] > max_value) {
                max_value = in[j];
                idx       = j;
              }
            }
          const size_t o = ((size_t)oh * c + oy) * ow + ox;
          if (argmax) argmax[osz * s + o] = idx;
          y[osz * s + o] = max_value;
        }
  }
  return 0;
}

/* in2out as left by init_connection: the LAST window (c, oy, ox ascending) that
 * touches an input element; elements no window touches keep 0
 * (max_pooling_layer.h:218,224-225). */
static int64_t *build_in2out(const tdo_pool_desc *d) {
  const int ow = tdo_pool_out_w(d), oh = tdo_pool_out_h(d);
  const size_t isz = (size_t)d->in_w * d->in_h * d->in_c;
  int64_t *in2out  = (int64_t *)calloc(isz, sizeof(int64_t));
  if (!in2out) return NULL;
  for (int c = 0; c < d->in_c; c++)
    for (int oy = 0; oy < oh; oy++)
      for (int ox = 0; ox < ow; ox++) {
        int dxmax = d->in_w - ox * d->stride_w;
        int dymax = d->in_h - oy * d->stride_h;
        if (dxmax > d->pool_w) dxmax = d->pool_w;
        if (dymax > d->pool_h) dymax = d->pool_h;
        for (int wy = 0; wy < dymax; wy++)
          for (int wx = 0; wx < dxmax; wx++)
            in2out[((size_t)d->in_h * c + oy * d->stride_h + wy) * d->in_w + ox * d->stride_w +
                   wx] = ((int64_t)oh * c + oy) * ow + ox;
      }
  return in2out;
}

/* MaxPoolGradOp::compute + kernels::maxpool_grad_op_internal,
 * tiny_dnn/core/kernels/maxpool_grad_op.h:22-46, maxpool_op_internal.h:42-57 */
int tdo_maxpool_bwd(const tdo_pool_desc *d, int batch, const float *dy, const int64_t *argmax,
                    float *dx) {
  const int ow = tdo_pool_out_w(d), oh = tdo_pool_out_h(d);
  const size_t isz = (size_t)d->in_w * d->in_h * d->in_c, osz = (size_t)ow * oh * d->in_c;
  int64_t *in2out  = build_in2out(d);
  if (!in2out) return -1;
#pragma omp parallel for schedule(static)
  for (int s = 0; s < batch; s++)
    for (size_t i = 0; i < isz; i++) {
      const int64_t outi = in2out[i];
      dx[isz * s + i]    = (argmax[osz * s + outi] == (int64_t)i) ? dy[osz * s + outi] : 0.0f;
    }
  free(in2out);
  return 0;
}

/* -------------------------------------------------------- average pooling */

/* Connection lists of average_pooling_layer::init_connection/connect_kernel
 * (tiny_dnn/layers/average_pooling_layer.h:270-304) in creation order. */
typedef struct {
  int n_pairs;   /* total (in,out) pairs */
  int *pair_in;  /* creation order: c, y, x, dy, dx */
  int *pair_out;
  int *chan_start; /* [in_c+1] ranges of pairs per channel (weight2io) */
  int *in_first_out; /* in2wo[idx][0].second, or -1 */
} avepool_conn;

static int avepool_build(const tdo_pool_desc *d, avepool_conn *cn) {
  const int ow = tdo_pool_out_w(d), oh = tdo_pool_out_h(d);
  const size_t isz = (size_t)d->in_w * d->in_h * d->in_c;
  size_t cap       = 0;
  for (int y = 0; y < d->in_h - d->pool_h + 1; y += d->stride_h)
    for (int x = 0; x < d->in_w - d->pool_w + 1; x += d->stride_w) cap += (size_t)d->pool_w * d->pool_h;
  cap *= (size_t)d->in_c;
  cn->pair_in      = (int *)malloc(sizeof(int) * (cap ? cap : 1));
  cn->pair_out     = (int *)malloc(sizeof(int) * (cap ? cap : 1));
  cn->chan_start   = (int *)malloc(sizeof(int) * (d->in_c + 1));
  cn->in_first_out = (int *)malloc(sizeof(int) * (isz ? isz : 1));
  if (!cn->pair_in || !cn->pair_out || !cn->chan_start || !cn->in_first_out) return -1;
  for (size_t i = 0; i < isz; i++) cn->in_first_out[i] = -1;
  int n = 0;
  for (int c = 0; c < d->in_c; c++) {
    cn->chan_start[c] = n;
    for (int y = 0; y < d->in_h - d->pool_h + 1; y += d->stride_h)
      for (int x = 0; x < d->in_w - d->pool_w + 1; x += d->stride_w) {
        int dymax = d->in_h - y, dxmax = d->in_w - x;
        if (dymax > d->pool_h) dymax = d->pool_h;
        if (dxmax > d->pool_w) dxmax = d->pool_w;
        const int dstx = x / d->stride_w, dsty = y / d->stride_h;
        if (dstx >= ow || dsty >= oh) continue; /* out_.get_index would be out of range */
        const int outidx = (oh * c + dsty) * ow + dstx;
        for (int wy = 0; wy < dymax; wy++)
          for (int wx = 0; wx < dxmax; wx++) {
            const int inidx = (d->in_h * c + y + wy) * d->in_w + x + wx;
            cn->pair_in[n]  = inidx;
            cn->pair_out[n] = outidx;
            if (cn->in_first_out[inidx] < 0) cn->in_first_out[inidx] = outidx;
            n++;
          }
      }
  }
  cn->chan_start[d->in_c] = n;
  cn->n_pairs             = n;
  return 0;
}

static void avepool_free(avepool_conn *cn) {
  free(cn->pair_in);
  free(cn->pair_out);
  free(cn->chan_start);
  free(cn->in_first_out);
}

/* tiny_average_pooling_kernel, tiny_dnn/layers/average_pooling_layer.h:25-55:
 * value = (sum over window) * (W[c]*scale) + b[c], scale = 1/(pool_w*pool_h) (:203) */
int tdo_avepool_fwd(const tdo_pool_desc *d, int batch, const float *x, const float *w,
                    const float *b, float *y) {
  if ((d->in_w % d->pool_w) || (d->in_h % d->pool_h)) return -2; /* pooling_size_mismatch */
  const int ow = tdo_pool_out_w(d), oh = tdo_pool_out_h(d);
  const size_t isz = (size_t)d->in_w * d->in_h * d->in_c, osz = (size_t)ow * oh * d->in_c;
  const float scale = 1.0f / (float)(d->pool_w * d->pool_h);
  avepool_conn cn;
  if (avepool_build(d, &cn)) return -1;
#pragma omp parallel for schedule(static)
  for (int s = 0; s < batch; s++) {
    const float *in = x + isz * s;
    float *out      = y + osz * s;
    /* out2wi[idx] lists the window inputs in creation order: accumulate per output */
    for (size_t i = 0; i < osz; i++) out[i] = 0.0f;
    for (int p = 0; p < cn.n_pairs; p++) out[cn.pair_out[p]] += in[cn.pair_in[p]];
    for (int c = 0; c < d->in_c; c++) {
      const float weight = w[c] * scale;
      const float bias   = b[c];
      for (int i = 0; i < oh * ow; i++) {
        float v = out[(size_t)oh * ow * c + i];
        v *= weight;
        v += bias;
        out[(size_t)oh * ow * c + i] = v;
      }
    }
  }
  avepool_free(&cn);
  return 0;
}

/* tiny_average_pooling_back_kernel, tiny_dnn/layers/average_pooling_layer.h:58-106 */
int tdo_avepool_bwd(const tdo_pool_desc *d, int batch, const float *x, const float *w,
                    const float *dy, float *dx, float *dw, float *db) {
  if ((d->in_w % d->pool_w) || (d->in_h % d->pool_h)) return -2;
  const int ow = tdo_pool_out_w(d), oh = tdo_pool_out_h(d);
  const int inarea = d->in_w * d->in_h;
  const size_t isz = (size_t)inarea * d->in_c, osz = (size_t)ow * oh * d->in_c;
  const float scale = 1.0f / (float)(d->pool_w * d->pool_h);
  avepool_conn cn;
  if (avepool_build(d, &cn)) return -1;
  for (size_t i = 0; i < isz; i++)
    if (cn.in_first_out[i] < 0) { /* in2wo[idx][0] on an empty list: undefined in the reference */
      avepool_free(&cn);
      return -3;
    }
#pragma omp parallel for schedule(static)
  for (int s = 0; s < batch; s++) {
    const float *curr = dy + osz * s;
    float *prev       = dx + isz * s;
    for (int c = 0; c < d->in_c; c++) {
      const float weight = w[c] * scale;
      for (int j = 0; j < inarea; j++) {
        const size_t idx = (size_t)inarea * c + j;
        prev[idx]        = weight * curr[cn.in_first_out[idx]];
      }
    }
  }
  for (int c = 0; c < d->in_c; c++) {
    float mw = 0.0f, mb = 0.0f;
    for (int s = 0; s < batch; s++) {
      const float *in   = x + isz * s;
      const float *curr = dy + osz * s;
      float diff        = 0.0f;
      for (int p = cn.chan_start[c]; p < cn.chan_start[c + 1]; p++)
        diff += in[cn.pair_in[p]] * curr[cn.pair_out[p]];
      const float gw = 0.0f + diff * scale;
      float dsum     = 0.0f;
      for (int i = 0; i < oh * ow; i++) dsum += curr[(size_t)oh * ow * c + i];
      const float gb = 0.0f + dsum;
      mw             = (s == 0) ? gw : mw + gw;
      mb             = (s == 0) ? gb : mb + gb;
    }
    if (dw) dw[c] = mw;
    if (db) db[c] = mb;
  }
  avepool_free(&cn);
  return 0;
}

/* ------------------------------------------------------------ activations */

/* activation_layer::forward_propagation, tiny_dnn/activations/activation_layer.h:74-79;
 * tanh_layer.h:24-28, relu_layer.h:25-29, softmax_layer.h:24-34, sigmoid_layer.h:24-28 */
void tdo_act_default_params(int kind, float *p) {
  p[0] = p[1] = 0.0f;
  switch (kind) {
    case TDO_ACT_LEAKY_RELU: p[0] = 0.01f; break;                 /* epsilon, leaky_relu_layer.h:25 */
    case TDO_ACT_ELU: p[0] = 1.0f; break;                         /* alpha, elu_layer.h:18 */
    case TDO_ACT_SELU: p[0] = 1.05070f; p[1] = 1.67326f; break;   /* lambda, alpha, selu_layer.h:26-27 */
    case TDO_ACT_SOFTPLUS: p[0] = 1.0f; p[1] = 20.0f; break;      /* beta, threshold, softplus_layer.h:26-27 */
  }
}

int tdo_act_fwd(int kind, int batch, int len, const float *x, float *y) {
  float p[2];
  tdo_act_default_params(kind, p);
  return tdo_act_fwd_p(kind, p, batch, len, x, y);
}

int tdo_act_bwd(int kind, int batch, int len, const float *x, const float *y, const float *dy,
                float *dx) {
  float p[2];
  tdo_act_default_params(kind, p);
  return tdo_act_bwd_p(kind, p, batch, len, x, y, dy, dx);
}

/* forward_activation of leaky_relu_layer.h:74-78, elu_layer.h:37-42, selu_layer.h:82-88,
 * softplus_layer.h:84-90, softsign_layer.h:24-28 (computed in double: `1.0 + std::abs`),
 * asinh_layer.h:24-28, tanh_p1m2_layer.h:24-30, beside the four kinds above */
int tdo_act_fwd_p(int kind, const float *p, int batch, int len, const float *x, float *y) {
  if (kind < TDO_ACT_TANH || kind > TDO_ACT_TANH_P1M2) return -2;
  const float p0 = p[0], p1 = p[1];
#pragma omp parallel for schedule(static)
  for (int s = 0; s < batch; s++) {
    const float *xi = x + (size_t)len * s;
    float *yo       = y + (size_t)len * s;
    switch (kind) {
      case TDO_ACT_TANH:
        for (int j = 0; j < len; j++) yo[j] = tanhf(xi[j]);
        break;
      case TDO_ACT_RELU:
        for (int j = 0; j < len; j++) yo[j] = xi[j] > 0.0f ? xi[j] : 0.0f; /* std::max(0,x) */
        break;
      case TDO_ACT_SIGMOID:
        for (int j = 0; j < len; j++) yo[j] = 1.0f / (1.0f + expf(-xi[j]));
        break;
      case TDO_ACT_SOFTMAX: {
        float alpha = xi[0];
        for (int j = 1; j < len; j++)
          if (alpha < xi[j]) alpha = xi[j]; /* std::max_element */
        float denominator = 0.0f;
        for (int j = 0; j < len; j++) {
          yo[j] = expf(xi[j] - alpha);
          denominator += yo[j];
        }
        for (int j = 0; j < len; j++) yo[j] /= denominator;
      } break;
      case TDO_ACT_LEAKY_RELU:
        for (int j = 0; j < len; j++) yo[j] = xi[j] > 0.0f ? xi[j] : p0 * xi[j];
        break;
      case TDO_ACT_ELU:
        for (int j = 0; j < len; j++) yo[j] = xi[j] < 0.0f ? (p0 * (expf(xi[j]) - 1.0f)) : xi[j];
        break;
      case TDO_ACT_SELU:
        for (int j = 0; j < len; j++)
          yo[j] = p0 * (xi[j] > 0.0f ? xi[j] : p1 * (expf(xi[j]) - 1.0f));
        break;
      case TDO_ACT_SOFTPLUS:
        for (int j = 0; j < len; j++) {
          const float betain = p0 * xi[j];
          yo[j] = (betain > p1) ? xi[j] : (1 / p0) * log1pf(expf(betain));
        }
        break;
      case TDO_ACT_SOFTSIGN:
        for (int j = 0; j < len; j++) yo[j] = (float)(xi[j] / (1.0 + fabsf(xi[j])));
        break;
      case TDO_ACT_ASINH:
        for (int j = 0; j < len; j++) yo[j] = asinhf(xi[j]);
        break;
      case TDO_ACT_TANH_P1M2:
        for (int j = 0; j < len; j++) {
          const float ep = expf(xi[j]);
          yo[j] = ep / (ep + (1.0f / ep));
        }
        break;
    }
  }
  return 0;
}

/* activation_layer::back_propagation, activation_layer.h:81-91; tanh_layer.h:30-38,
 * relu_layer.h:31-39, softmax_layer.h:36-55 (full Jacobian row dotted with dy),
 * sigmoid_layer.h:30-38 */
/* ... and backward_activation of leaky_relu_layer.h:80-88, elu_layer.h:44-52,
 * selu_layer.h:90-99 (uses x; the product runs in double because of the literal 1.0),
 * softplus_layer.h:92-102, softsign_layer.h:30-40 (uses x, double), asinh_layer.h:30-38,
 * tanh_p1m2_layer.h:32-40 */
int tdo_act_bwd_p(int kind, const float *p, int batch, int len, const float *x, const float *y,
                  const float *dy, float *dx) {
  if (kind < TDO_ACT_TANH || kind > TDO_ACT_TANH_P1M2) return -2;
  if ((kind == TDO_ACT_SELU || kind == TDO_ACT_SOFTSIGN) && !x) return -2;
  const float p0 = p[0], p1 = p[1];
#pragma omp parallel for schedule(static)
  for (int s = 0; s < batch; s++) {
    const float *xi = x ? x + (size_t)len * s : NULL;
    const float *yo = y + (size_t)len * s;
    const float *d  = dy + (size_t)len * s;
    float *o        = dx + (size_t)len * s;
    switch (kind) {
      case TDO_ACT_TANH:
        for (int j = 0; j < len; j++) o[j] = d[j] * (1.0f - yo[j] * yo[j]);
        break;
      case TDO_ACT_RELU:
        for (int j = 0; j < len; j++) o[j] = d[j] * (yo[j] > 0.0f ? 1.0f : 0.0f);
        break;
      case TDO_ACT_SIGMOID:
        for (int j = 0; j < len; j++) o[j] = d[j] * yo[j] * (1.0f - yo[j]);
        break;
      case TDO_ACT_SOFTMAX: {
        float *df = (float *)malloc(sizeof(float) * (size_t)(len ? len : 1));
        for (int j = 0; j < len; j++) {
          for (int k = 0; k < len; k++)
            df[k] = (k == j) ? yo[j] * (1.0f - yo[j]) : -yo[k] * yo[j];
          o[j] = dot4(d, df, (size_t)len); /* vectorize::dot(&dy[0], &df[0], len) */
        }
        free(df);
      } break;
      case TDO_ACT_LEAKY_RELU:
        for (int j = 0; j < len; j++) o[j] = d[j] * (yo[j] > 0.0f ? 1.0f : p0);
        break;
      case TDO_ACT_ELU:
        for (int j = 0; j < len; j++) o[j] = d[j] * (yo[j] > 0.0f ? 1.0f : (p0 + yo[j]));
        break;
      case TDO_ACT_SELU:
        for (int j = 0; j < len; j++)
          o[j] = (float)(d[j] * p0 * (xi[j] > 0.0f ? 1.0 : (double)(p1 * expf(xi[j]))));
        break;
      case TDO_ACT_SOFTPLUS:
        for (int j = 0; j < len; j++) {
          const float betaout = p0 * yo[j];
          const float exp_bo  = expf(betaout);
          o[j] = (betaout > p1) ? d[j] : d[j] * (exp_bo - 1) / exp_bo;
        }
        break;
      case TDO_ACT_SOFTSIGN:
        for (int j = 0; j < len; j++) {
          const double dd = 1.0 + fabsf(xi[j]);
          o[j] = (float)(d[j] / (dd * dd));
        }
        break;
      case TDO_ACT_ASINH:
        for (int j = 0; j < len; j++) o[j] = d[j] / coshf(yo[j]);
        break;
      case TDO_ACT_TANH_P1M2:
        for (int j = 0; j < len; j++) o[j] = d[j] * (2 * yo[j] * (1.0f - yo[j]));
        break;
    }
  }
  return 0;
}

/* ------------------------------------------------------------------ losses */

/* ------------------------------------------------- batch normalization, dropout */

/* tiny_dnn/util/math_functions.h:25-37 and 68-79: per channel, the samples' runs are added one
 * after the other onto one float (std::accumulate), then divided by (float)batch*spatial */
static void moments_mean(int channels, int spatial, int batch, const float *in, float *mean) {
  for (int j = 0; j < channels; j++) mean[j] = 0.0f;
  for (int i = 0; i < batch; i++)
    for (int j = 0; j < channels; j++) {
      const float *p = in + ((size_t)i * channels + j) * spatial;
      float r = mean[j];
      for (int k = 0; k < spatial; k++) r = r + p[k];
      mean[j] = r;
    }
  const float denom = (float)batch * spatial;
  for (int j = 0; j < channels; j++) mean[j] = mean[j] / denom;
}

/* tiny_dnn/util/math_functions.h:39-61: sum of pow(x - mean, 2) over max(1, batch*spatial - 1) */
static void moments_variance(int channels, int spatial, int batch, const float *in,
                             const float *mean, float *variance) {
  for (int j = 0; j < channels; j++) variance[j] = 0.0f;
  for (int i = 0; i < batch; i++)
    for (int j = 0; j < channels; j++) {
      const float *p = in + ((size_t)i * channels + j) * spatial;
      const float ex = mean[j];
      float r = variance[j];
      /* the unqualified pow(x - ex, float_t{2.0}) of the reference is the C library's
       * pow(double, double): the square and the addition are carried out in double and
       * rounded to float once per element */
      for (int k = 0; k < spatial; k++) {
        const double d = (double)(p[k] - ex);
        r = (float)((double)r + d * d);
      }
      variance[j] = r;
    }
  float denom = (float)((size_t)batch * spatial) - 1.0f;
  if (denom < 1.0f) denom = 1.0f;
  for (int j = 0; j < channels; j++) variance[j] = variance[j] / denom;
}

/* batch_normalization_layer.h:127-169 */
int tdo_batchnorm_fwd(int channels, int spatial, int batch, float eps, int train, const float *x,
                      float *mean, float *variance, float *stddev, float *y) {
  if (channels < 0 || spatial < 0 || batch < 0) return -1;
  if (train) {
    moments_mean(channels, spatial, batch, x, mean);
    moments_variance(channels, spatial, batch, x, mean, variance);
  }
  for (int j = 0; j < channels; j++) stddev[j] = sqrtf(variance[j] + eps);
  for (int i = 0; i < batch; i++)
    for (int j = 0; j < channels; j++) {
      const float m = mean[j];
      for (int k = 0; k < spatial; k++) {
        const size_t idx = ((size_t)i * channels + j) * spatial + k;
        y[idx] = (x[idx] - m) / stddev[j];
      }
    }
  return 0;
}

/* batch_normalization_layer.h:87-125 */
int tdo_batchnorm_bwd(int channels, int spatial, int batch, const float *y, const float *dy,
                      const float *stddev, float *dx) {
  if (channels < 0 || spatial < 0 || batch < 0) return -1;
  const size_t total = (size_t)batch * channels * spatial;
  float *prod = (float *)malloc(sizeof(float) * (total ? total : 1));
  float *m_prod = (float *)malloc(sizeof(float) * (channels ? channels : 1));
  float *m_dy = (float *)malloc(sizeof(float) * (channels ? channels : 1));
  if (!prod || !m_prod || !m_dy) { free(prod); free(m_prod); free(m_dy); return -1; }
  for (size_t i = 0; i < total; i++) prod[i] = y[i] * dy[i];
  moments_mean(channels, spatial, batch, prod, m_prod);
  moments_mean(channels, spatial, batch, dy, m_dy);
  for (int i = 0; i < batch; i++)
    for (int j = 0; j < channels; j++)
      for (int k = 0; k < spatial; k++) {
        const size_t idx = ((size_t)i * channels + j) * spatial + k;
        float v = dy[idx] - m_dy[j] - m_prod[j] * y[idx];
        dx[idx] = v / stddev[j];
      }
  free(prod); free(m_prod); free(m_dy);
  return 0;
}

/* batch_normalization_layer.h:171-177 */
void tdo_batchnorm_update_moving(int channels, float momentum, const float *mean_cur,
                                 const float *var_cur, float *mean, float *variance) {
  for (int i = 0; i < channels; i++) {
    mean[i]     = momentum * mean[i] + (1 - momentum) * mean_cur[i];
    variance[i] = momentum * variance[i] + (1 - momentum) * var_cur[i];
  }
}

/* dropout_layer.h:84-117 */
int tdo_dropout_fwd(int batch, int len, int train, float scale, const unsigned char *mask,
                    const float *x, float *y) {
  if (batch < 0 || len < 0) return -1;
  const size_t total = (size_t)batch * len;
  for (size_t i = 0; i < total; i++) y[i] = train ? mask[i] * scale * x[i] : x[i];
  return 0;
}

/* dropout_layer.h:62-82 */
int tdo_dropout_bwd(int batch, int len, const unsigned char *mask, const float *dy, float *dx) {
  if (batch < 0 || len < 0) return -1;
  const size_t total = (size_t)batch * len;
  for (size_t i = 0; i < total; i++) dx[i] = mask[i] * dy[i];
  return 0;
}

/* MT19937 (Matsumoto & Nishimura 1998) as std::mt19937 specifies it: seeding by the linear
 * recurrence 1812433253, tempering (11, 7/0x9d2c5680, 15/0xefc60000, 18) */
void tdo_mt_seed(unsigned int *state, unsigned int seed) {
  state[0] = seed;
  for (unsigned int i = 1; i < 624; i++) state[i] = 1812433253u * (state[i - 1] ^ (state[i - 1] >> 30)) + i;
  state[624] = 624;
}

static unsigned int mt_next(unsigned int *mt) {
  if (mt[624] >= 624) {
    for (int k = 0; k < 624; k++) {
      const unsigned int yv = (mt[k] & 0x80000000u) | (mt[(k + 1) % 624] & 0x7fffffffu);
      mt[k] = mt[(k + 397) % 624] ^ (yv >> 1) ^ ((yv & 1u) ? 0x9908b0dfu : 0u);
    }
    mt[624] = 0;
  }
  unsigned int v = mt[mt[624]++];
  v ^= v >> 11;
  v ^= (v << 7) & 0x9d2c5680u;
  v ^= (v << 15) & 0xefc60000u;
  v ^= v >> 18;
  return v;
}

/* util/random.h:67-69 with libstdc++'s uniform_real_distribution<float>(0,1): one 32-bit draw
 * converted to float, divided by 2^32, and clamped below 1 */
void tdo_dropout_mask(unsigned int *state, float rate, size_t n, unsigned char *mask) {
  for (size_t i = 0; i < n; i++) {
    float u = (float)mt_next(state) / 4294967296.0f;
    if (u >= 1.0f) u = nextafterf(1.0f, 0.0f);
    mask[i] = u <= rate ? 1 : 0;
  }
}



/* gradient<E> for a mini-batch, tiny_dnn/lossfunctions/loss_function.h:191-218; * mse::df :28-36, cross_entropy::df :120-128, cross_entropy_multiclass::df :143-150 */
int tdo_loss_grad(int kind, int batch, int len, const float *y, const float *t, float *dy) {
  const size_t n = (size_t)batch * len;
  switch (kind) {
    case TDO_LOSS_MSE: {
      const float factor = 2.0f / (float)len;
      for (size_t i = 0; i < n; i++) dy[i] = factor * (y[i] - t[i]);
    } break;
    case TDO_LOSS_CE_MULTICLASS:
      for (size_t i = 0; i < n; i++) dy[i] = -t[i] / y[i];
      break;
    case TDO_LOSS_CE:
      for (size_t i = 0; i < n; i++) dy[i] = (y[i] - t[i]) / (y[i] * (1.0f - y[i]));
      break;
    default: return -2;
  }
  return 0;
}

/* E::f summed over the batch (network::get_loss, tiny_dnn/network.h:486-533) */
float tdo_loss_value(int kind, int batch, int len, const float *y, const float *t) {
  float total = 0.0f;
  for (int s = 0; s < batch; s++) {
    const float *ys = y + (size_t)len * s, *ts = t + (size_t)len * s;
    float d = 0.0f;
    switch (kind) {
      case TDO_LOSS_MSE:
        for (int i = 0; i < len; i++) d += (ys[i] - ts[i]) * (ys[i] - ts[i]);
        d /= (float)len;
        break;
      case TDO_LOSS_CE_MULTICLASS:
        for (int i = 0; i < len; i++) d += -ts[i] * logf(ys[i]);
        break;
      case TDO_LOSS_CE:
        for (int i = 0; i < len; i++)
          d += -ts[i] * logf(ys[i]) - (1.0f - ts[i]) * logf(1.0f - ys[i]);
        break;
    }
    total += d;
  }
  return total;
}

/* -------------------------------------------------------------- optimizers */

/* defaults of the reference constructors, tiny_dnn/optimizers/optimizer.h */
void tdo_opt_default(tdo_opt *o, int kind) {
  memset(o, 0, sizeof(*o));
  o->kind = kind;
  switch (kind) {
    case TDO_OPT_SGD: o->alpha = 0.01f; o->lambda = 0.0f; break;                 /* :183 */
    case TDO_OPT_MOMENTUM:
    case TDO_OPT_NESTEROV: o->alpha = 0.01f; o->lambda = 0.0f; o->mu = 0.9f; break; /* :203,:229 */
    case TDO_OPT_ADAM:                                                            /* :104-110 */
      o->alpha = 0.001f; o->b1 = 0.9f; o->b2 = 0.999f; o->b1_t = 0.9f; o->b2_t = 0.999f;
      o->eps = 1e-8f;
      break;
    case TDO_OPT_ADAGRAD: o->alpha = 0.01f; o->eps = 1e-8f; break;                /* :58 */
    case TDO_OPT_RMSPROP: o->alpha = 0.0001f; o->mu = 0.99f; o->eps = 1e-8f; break; /* :79 */
    case TDO_OPT_ADAMAX:                                                          /* :146-151 */
      o->alpha = 0.002f; o->b1 = 0.9f; o->b2 = 0.999f; o->b1_t = 0.9f; o->eps = 1e-8f;
      break;
  }
}

/* optimizer::update, tiny_dnn/optimizers/optimizer.h: gradient_descent :185-188,
 * momentum :205-213, adam :112-127 (eps inside the sqrt; b1_t,b2_t advance once per
 * call), adagrad :60-66, RMSprop :81-88, adamax :153-165 (alpha/(1.0-b1_t) in double),
 * nesterov_momentum :231-239 */
int tdo_opt_update(tdo_opt *o, size_t n, const float *g, float *w, float *s0, float *s1) {
  switch (o->kind) {
    case TDO_OPT_SGD:
      for (size_t i = 0; i < n; i++) w[i] = w[i] - o->alpha * (g[i] + o->lambda * w[i]);
      break;
    case TDO_OPT_MOMENTUM:
      for (size_t i = 0; i < n; i++) {
        const float V = o->mu * s0[i] - o->alpha * (g[i] + w[i] * o->lambda);
        w[i] += V;
        s0[i] = V;
      }
      break;
    case TDO_OPT_NESTEROV:
      for (size_t i = 0; i < n; i++) {
        const float V = o->mu * s0[i] - o->alpha * (g[i] + w[i] * o->lambda);
        w[i] += (-o->mu) * s0[i] + (1 + o->mu) * V;
        s0[i] = V;
      }
      break;
    case TDO_OPT_ADAM:
      for (size_t i = 0; i < n; i++) {
        s0[i] = o->b1 * s0[i] + (1.0f - o->b1) * g[i];
        s1[i] = o->b2 * s1[i] + (1.0f - o->b2) * g[i] * g[i];
        w[i] -= o->alpha * (s0[i] / (1.0f - o->b1_t)) / sqrtf((s1[i] / (1.0f - o->b2_t)) + o->eps);
      }
      o->b1_t *= o->b1;
      o->b2_t *= o->b2;
      break;
    case TDO_OPT_ADAGRAD:
      for (size_t i = 0; i < n; i++) {
        s0[i] += g[i] * g[i];
        w[i] -= o->alpha * g[i] / (sqrtf(s0[i]) + o->eps);
      }
      break;
    case TDO_OPT_RMSPROP:
      for (size_t i = 0; i < n; i++) {
        s0[i] = o->mu * s0[i] + (1 - o->mu) * g[i] * g[i];
        w[i] -= o->alpha * g[i] / sqrtf(s0[i] + o->eps);
      }
      break;
    case TDO_OPT_ADAMAX:
      for (size_t i = 0; i < n; i++) {
        s0[i]         = o->b1 * s0[i] + (1.0f - o->b1) * g[i];
        const float a = o->b2 * s1[i], bb = fabsf(g[i]);
        s1[i]         = a < bb ? bb : a; /* std::max */
        w[i] = (float)((double)w[i] -
                       ((double)o->alpha / (1.0 - (double)o->b1_t)) * (double)(s0[i] / (s1[i] + o->eps)));
      }
      o->b1_t *= o->b1;
      break;
    default: return -2;
  }
  return 0;
}

/* layer::update_weight for one trainable tensor, tiny_dnn/layers/layer.h:663-682:
 * diff = merged * rcp_batch_size, then optimizer->update(diff, W).
 * rcp_batch_size = 1 / ith_in_node(i)->get_data()->size() where i is the WEIGHT edge;
 * set_sample_count (layer.h:699-718) never grows the data tensor of a trainable edge, so
 * that size is 1 and the summed (not averaged) gradient reaches the optimizer. The
 * compiled reference confirms it (network<sequential>::fit matches bit for bit only with
 * a divisor of 1). `weight_edge_samples` is that size; callers restating the reference
 * pass 1. */
int tdo_update_weight(tdo_opt *o, size_t n, int weight_edge_samples, const float *merged,
                      float *w, float *s0, float *s1) {
  float *g = (float *)malloc(sizeof(float) * (n ? n : 1));
  if (!g) return -1;
  const float rcp_batch_size = 1.0f / (float)weight_edge_samples;
  for (size_t i = 0; i < n; i++) g[i] = merged[i] * rcp_batch_size;
  const int rc = tdo_opt_update(o, n, g, w, s0, s1);
  free(g);
  return rc;
}

/* ----------------------------------------------------- sequential network */

typedef struct {
  tdo_layer spec;
  size_t in_size, out_size, w_size, b_size;
  float *w, *b, *dw, *db, *s0w, *s1w, *s0b, *s1b;
  float *out;  /* [max_batch][out_size] */
  float *dout; /* gradient wrt out */
  float *dx;   /* gradient wrt in */
  int64_t *argmax;
  /* batch-norm: moving mean / variance, this batch's moments, stddev; dropout: mask */
  float *bn_mean, *bn_var, *bn_mean_cur, *bn_var_cur, *bn_stddev;
  unsigned char *mask;
} net_layer;

struct tdo_net {
  int n_layers, max_batch;
  net_layer *l;
  float *x; /* copy of the current input batch */
  int test_phase; /* 0: net_phase::train */
};

static int layer_sizes(net_layer *L) {
  const tdo_layer *s = &L->spec;
  switch (s->kind) {
    case TDO_L_CONV:
      L->in_size  = (size_t)s->conv.in_w * s->conv.in_h * s->conv.in_c;
      L->out_size = (size_t)tdo_conv_out_w(&s->conv) * tdo_conv_out_h(&s->conv) * s->conv.out_c;
      L->w_size   = (size_t)s->conv.k_w * s->conv.k_h * s->conv.in_c * s->conv.out_c;
      L->b_size   = s->conv.has_bias ? (size_t)s->conv.out_c : 0;
      break;
    case TDO_L_FC:
      L->in_size = (size_t)s->fc_in;
      L->out_size = (size_t)s->fc_out;
      L->w_size = (size_t)s->fc_in * s->fc_out;
      L->b_size = s->fc_bias ? (size_t)s->fc_out : 0;
      break;
    case TDO_L_MAXPOOL:
    case TDO_L_AVEPOOL:
      L->in_size  = (size_t)s->pool.in_w * s->pool.in_h * s->pool.in_c;
      L->out_size = (size_t)tdo_pool_out_w(&s->pool) * tdo_pool_out_h(&s->pool) * s->pool.in_c;
      L->w_size   = s->kind == TDO_L_AVEPOOL ? (size_t)s->pool.in_c : 0;
      L->b_size   = L->w_size;
      break;
    case TDO_L_ACT: /* size inherited from the previous layer, filled by the caller */
    case TDO_L_DROPOUT:
      L->w_size = L->b_size = 0;
      break;
    case TDO_L_BATCHNORM:
      L->in_size = L->out_size = (size_t)s->bn_channels * s->bn_spatial;
      L->w_size = L->b_size = 0;
      break;
    default: return -2;
  }
  return 0;
}

static float *fzalloc(size_t n) { return (float *)calloc(n ? n : 1, sizeof(float)); }

tdo_net *tdo_net_create(const tdo_layer *layers, int n_layers, int max_batch) {
  tdo_net *net = (tdo_net *)calloc(1, sizeof(tdo_net));
  if (!net) return NULL;
  net->n_layers  = n_layers;
  net->max_batch = max_batch;
  net->l         = (net_layer *)calloc((size_t)n_layers, sizeof(net_layer));
  for (int i = 0; i < n_layers; i++) {
    net_layer *L = &net->l[i];
    L->spec      = layers[i];
    if (layers[i].kind == TDO_L_ACT || layers[i].kind == TDO_L_DROPOUT) {
      if (i == 0) {
        tdo_net_destroy(net);
        return NULL;
      }
      L->in_size = L->out_size = net->l[i - 1].out_size;
    }
    if (layer_sizes(L) || (i > 0 && L->in_size != net->l[i - 1].out_size)) {
      tdo_net_destroy(net);
      return NULL;
    }
    L->w = fzalloc(L->w_size); L->dw = fzalloc(L->w_size);
    L->s0w = fzalloc(L->w_size); L->s1w = fzalloc(L->w_size);
    L->b = fzalloc(L->b_size); L->db = fzalloc(L->b_size);
    L->s0b = fzalloc(L->b_size); L->s1b = fzalloc(L->b_size);
    L->out  = fzalloc(L->out_size * (size_t)max_batch);
    L->dout = fzalloc(L->out_size * (size_t)max_batch);
    L->dx   = fzalloc(L->in_size * (size_t)max_batch);
    if (layers[i].kind == TDO_L_MAXPOOL)
      L->argmax = (int64_t *)calloc(L->out_size * (size_t)max_batch, sizeof(int64_t));
    if (layers[i].kind == TDO_L_BATCHNORM) {
      const size_t c = (size_t)layers[i].bn_channels;
      L->bn_mean = fzalloc(c); L->bn_var = fzalloc(c); L->bn_mean_cur = fzalloc(c);
      L->bn_var_cur = fzalloc(c); L->bn_stddev = fzalloc(c);
    }
    if (layers[i].kind == TDO_L_DROPOUT)
      L->mask = (unsigned char *)calloc(L->out_size * (size_t)max_batch + 1, 1);
  }
  net->x = fzalloc(net->l[0].in_size * (size_t)max_batch);
  return net;
}

void tdo_net_destroy(tdo_net *net) {
  if (!net) return;
  for (int i = 0; i < net->n_layers; i++) {
    net_layer *L = &net->l[i];
    free(L->w); free(L->b); free(L->dw); free(L->db);
    free(L->s0w); free(L->s1w); free(L->s0b); free(L->s1b);
    free(L->out); free(L->dout); free(L->dx); free(L->argmax);
    free(L->bn_mean); free(L->bn_var); free(L->bn_mean_cur); free(L->bn_var_cur); free(L->bn_stddev);
    free(L->mask);
  }
  free(net->l);
  free(net->x);
  free(net);
}

void tdo_net_set_phase(tdo_net *net, int train) { net->test_phase = !train; }
unsigned char *tdo_net_dropout_mask(tdo_net *net, int i) { return net->l[i].mask; }
float *tdo_net_bn_stat(tdo_net *net, int i, int which) { return which ? net->l[i].bn_var : net->l[i].bn_mean; }
int tdo_net_num_layers(const tdo_net *net) { return net->n_layers; }
size_t tdo_net_in_size(const tdo_net *net) { return net->l[0].in_size; }
size_t tdo_net_out_size(const tdo_net *net) { return net->l[net->n_layers - 1].out_size; }
size_t tdo_net_weight_size(const tdo_net *net, int i) { return net->l[i].w_size; }
size_t tdo_net_bias_size(const tdo_net *net, int i) { return net->l[i].b_size; }
size_t tdo_net_layer_out_size(const tdo_net *net, int i) { return net->l[i].out_size; }
float *tdo_net_weight(tdo_net *net, int i) { return net->l[i].w; }
float *tdo_net_bias(tdo_net *net, int i) { return net->l[i].b; }
const float *tdo_net_layer_out(const tdo_net *net, int i) { return net->l[i].out; }
const float *tdo_net_layer_dx(const tdo_net *net, int i) { return net->l[i].dx; }
const float *tdo_net_layer_dw(const tdo_net *net, int i) { return net->l[i].dw; }
const float *tdo_net_layer_db(const tdo_net *net, int i) { return net->l[i].db; }
const int64_t *tdo_net_layer_argmax(const tdo_net *net, int i) { return net->l[i].argmax; }

/* sequential::forward, tiny_dnn/nodes.h:288-303 */
int tdo_net_forward(tdo_net *net, int batch, const float *x) {
  if (batch > net->max_batch || batch < 1) return -2;
  memcpy(net->x, x, sizeof(float) * net->l[0].in_size * (size_t)batch);
  const float *in = net->x;
  for (int i = 0; i < net->n_layers; i++) {
    net_layer *L = &net->l[i];
    int rc       = 0;
    switch (L->spec.kind) {
      case TDO_L_CONV: rc = tdo_conv2d_fwd(&L->spec.conv, batch, in, L->w, L->b, L->out); break;
      case TDO_L_FC:
        rc = tdo_fc_fwd(L->spec.fc_in, L->spec.fc_out, L->spec.fc_bias, batch, in, L->w, L->b, L->out);
        break;
      case TDO_L_MAXPOOL: rc = tdo_maxpool_fwd(&L->spec.pool, batch, in, L->out, L->argmax); break;
      case TDO_L_AVEPOOL: rc = tdo_avepool_fwd(&L->spec.pool, batch, in, L->w, L->b, L->out); break;
      case TDO_L_ACT:
        rc = tdo_act_fwd_p(L->spec.act, L->spec.act_p, batch, (int)L->out_size, in, L->out);
        break;
      case TDO_L_BATCHNORM: { /* batch_normalization_layer.h:127-169 */
        const int train = !net->test_phase;
        rc = tdo_batchnorm_fwd(L->spec.bn_channels, L->spec.bn_spatial, batch, L->spec.bn_eps, train, in,
                               train ? L->bn_mean_cur : L->bn_mean, train ? L->bn_var_cur : L->bn_var,
                               L->bn_stddev, L->out);
      } break;
      case TDO_L_DROPOUT: /* dropout_layer.h:84-117 */
        rc = tdo_dropout_fwd(batch, (int)L->out_size, !net->test_phase,
                             1.0f / (1.0f - L->spec.dropout_rate), L->mask, in, L->out);
        break;
    }
    if (rc) return rc;
    in = L->out;
  }
  return 0;
}

/* network::train_onebatch, tiny_dnn/network.h:911-926: fprop, bprop (loss gradient then
 * sequential::backward, nodes.h:276-286), nodes::update_weights (nodes.h:103-107) which
 * visits layers front to back and, inside a layer, weight before bias (layer.h:663-682). */
int tdo_net_train_step(tdo_net *net, tdo_opt *opt, int loss_kind, int batch, const float *x,
                       const float *t, int do_update) {
  int rc = tdo_net_forward(net, batch, x);
  if (rc) return rc;
  const int n    = net->n_layers;
  net_layer *last = &net->l[n - 1];
  rc = tdo_loss_grad(loss_kind, batch, (int)last->out_size, last->out, t, last->dout);
  if (rc) return rc;
  for (int i = n - 1; i >= 0; i--) {
    net_layer *L    = &net->l[i];
    const float *in = i == 0 ? net->x : net->l[i - 1].out;
    switch (L->spec.kind) {
      case TDO_L_CONV:
        rc = tdo_conv2d_bwd(&L->spec.conv, batch, in, L->w, L->dout, L->dx, L->dw, L->db);
        break;
      case TDO_L_FC:
        rc = tdo_fc_bwd(L->spec.fc_in, L->spec.fc_out, L->spec.fc_bias, batch, in, L->w, L->dout,
                        L->dx, L->dw, L->db);
        break;
      case TDO_L_MAXPOOL: rc = tdo_maxpool_bwd(&L->spec.pool, batch, L->dout, L->argmax, L->dx); break;
      case TDO_L_AVEPOOL:
        rc = tdo_avepool_bwd(&L->spec.pool, batch, in, L->w, L->dout, L->dx, L->dw, L->db);
        break;
      case TDO_L_ACT:
        rc = tdo_act_bwd_p(L->spec.act, L->spec.act_p, batch, (int)L->out_size, in, L->out, L->dout,
                           L->dx);
        break;
      case TDO_L_BATCHNORM: /* batch_normalization_layer.h:87-125 */
        rc = tdo_batchnorm_bwd(L->spec.bn_channels, L->spec.bn_spatial, batch, L->out, L->dout, L->bn_stddev,
                               L->dx);
        break;
      case TDO_L_DROPOUT: /* dropout_layer.h:62-82 */
        rc = tdo_dropout_bwd(batch, (int)L->out_size, L->mask, L->dout, L->dx);
        break;
    }
    if (rc) return rc;
    if (i > 0) memcpy(net->l[i - 1].dout, L->dx, sizeof(float) * L->in_size * (size_t)batch);
  }
  if (!do_update) return 0;
  for (int i = 0; i < n; i++) {
    net_layer *L = &net->l[i];
    if (L->w_size) {
      rc = tdo_update_weight(opt, L->w_size, 1, L->dw, L->w, L->s0w, L->s1w);
      if (rc) return rc;
    }
    if (L->b_size) {
      rc = tdo_update_weight(opt, L->b_size, 1, L->db, L->b, L->s0b, L->s1b);
      if (rc) return rc;
    }
    /* layer::update_weight ends in post_update (layer.h:681): batch_normalization_layer.h:171-177 */
    if (L->spec.kind == TDO_L_BATCHNORM)
      tdo_batchnorm_update_moving(L->spec.bn_channels, L->spec.bn_momentum, L->bn_mean_cur, L->bn_var_cur,
                                  L->bn_mean, L->bn_var);
  }
  return 0;
}
