// tiny_net.hip — the whole train step of a small net in three launches, the optimizer's included.
//
// A net whose activations of one sample fit in LDS (LeNet-5: 15 k floats) spends its step in
// launches, not in arithmetic: 24 kernels of 3-10 us on tensors of a few kilobytes. Here one
// workgroup takes one sample through the chain that has to run in order: forward through every
// layer with all layer outputs kept in LDS, the loss gradient, and the input gradients backward
// through every layer, reading the filters through the caches. Layer outputs, input gradients
// and max-pool records are also written to the net's tensors in memory, so a caller sees what
// the layer-by-layer path leaves. Nothing in that chain waits for a weight gradient, so those
// are a second launch of many small workgroups, (piece of a layer's work) x (sample), that read
// the layer's input and output gradient back from memory. What adds over the batch leaves that
// kernel as one slice per sample ([sample][tensor], the layout of the reference's own
// per-sample gradients, tiny_dnn/layers/layer.h:699-718). When the step ends with an update,
// the optimizer's kernel adds the slices up on its way (the split sums it also takes from the
// layer-by-layer step); a step that stops at the gradients adds them to the gradient tensors in
// sample order, the order of edge::merge_grads (tiny_dnn/node.h:89-103), with a kernel of its own.
//
// The arithmetic of each layer follows the reference's scalar kernels: convolution sums the
// taps of one input channel, then adds channel sums in channel order, then the bias
// (conv2d_op_internal.h:13-74); pooling scans windows row by row (maxpool_op_internal.h:16-40,
// average_pooling_layer.h:25-106). Sums that one thread would walk alone for too long (a bias
// gradient, a first layer's weight gradient, a fully-connected output) are split over a group
// of neighbouring lanes and added with butterfly shuffles, a fixed tree.
// Built with -ffp-contract=off like the other scalar kernels.
#include <cfloat>

#include "tiny_net.h"

namespace tdh {

namespace {

constexpr int TN_THREADS = 1024;

__device__ __forceinline__ float tn_act_fwd(int act, float p0, float x) {
  switch (act) {
    case TDH_ACT_TANH: return tanhf(x);
    case TDH_ACT_RELU: return x > 0.0f ? x : 0.0f;
    case TDH_ACT_SIGMOID: return 1.0f / (1.0f + expf(-x));
    case TDH_ACT_LEAKY_RELU: return x > 0.0f ? x : p0 * x;
    default: return x;
  }
}
// the factor of the activation's backward pass, from its OUTPUT (tanh_layer.h:30-38,
// relu_layer.h:31-39, sigmoid_layer.h:30-38, leaky_relu_layer.h:80-88)
__device__ __forceinline__ float tn_act_bwd(int act, float p0, float y, float dy) {
  switch (act) {
    case TDH_ACT_TANH: return dy * (1.0f - y * y);
    case TDH_ACT_RELU: return dy * (y > 0.0f ? 1.0f : 0.0f);
    case TDH_ACT_SIGMOID: return dy * y * (1.0f - y);
    case TDH_ACT_LEAKY_RELU: return dy * (y > 0.0f ? 1.0f : p0);
    default: return dy;
  }
}

// sum over the `group` (a power of two <= 64) neighbouring lanes that hold the pieces of one value
__device__ __forceinline__ float group_sum(float v, int group) {
  for (int off = group >> 1; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}
// lanes per value, so that `values` of them make at least two rounds of the workgroup busy
// and no lane's share of `length` terms is empty
__device__ __forceinline__ int group_for(int values, int length) {
  int g = 64;
  while (g > 1 && (values * g > 2 * TN_THREADS || g > length)) g >>= 1;
  return g;
}

// A barrier for data that went through LDS only: the waves wait for their own LDS traffic and
// meet, while their stores to memory stay in flight (__syncthreads would also wait for those,
// a microsecond per layer here). Wherever one thread reads memory another thread of the
// workgroup wrote, __syncthreads stays.
__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// memory -> LDS with eight reads in flight per thread
template <int NT>
__device__ __forceinline__ void fill_lds(float *dst, const float *__restrict__ src, const int n) {
  for (int base = 0; base < n; base += 8 * NT) {
    float v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int i = base + j * NT + static_cast<int>(threadIdx.x);
      v[j] = src[i < n ? i : 0];
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int i = base + j * NT + static_cast<int>(threadIdx.x);
      if (i < n) dst[i] = v[j];
    }
  }
}

// Every function below copies the sizes it needs out of the plan (uniform values: scalar
// registers) before its loops, and is inlined into the kernel so that `in`, `out`, `dy`, `dx`
// stay LDS addresses.
#define TN_INLINE __device__ __forceinline__

// ------------------------------------------------------------------ forward
TN_INLINE void conv_fwd(const TinyLayer *__restrict__ Lp, const float *in, float *out, float *__restrict__ gout) {
  const int C = Lp->C, H = Lp->H, W = Lp->W, K = Lp->K, OH = Lp->OH, OW = Lp->OW, R = Lp->R, S = Lp->S;
  const int sh = Lp->sh, sw = Lp->sw, ph = Lp->ph, pw = Lp->pw, has_bias = Lp->has_bias;
  const FastDiv d_plane = Lp->d_oplane, d_ow = Lp->d_ow;
  const float *__restrict__ w = Lp->w;
  const float *__restrict__ b = Lp->b;
  const uint8_t *__restrict__ tbl = Lp->tbl;
  const int plane = OH * OW, total = K * plane, taps = R * S;
  for (int o = threadIdx.x; o < total; o += TN_THREADS) {
    uint32_t co, r, oy, ox;
    d_plane.divmod(o, co, r);
    d_ow.divmod(r, oy, ox);
    const int y0 = static_cast<int>(oy) * sh - ph, x0 = static_cast<int>(ox) * sw - pw;
    const int wy0 = max(0, -y0), wy1 = min(R, H - y0), wx0 = max(0, -x0), wx1 = min(S, W - x0);
    float acc = 0.0f;
    for (int ci = 0; ci < C; ++ci) {
      if (tbl && !tbl[ci * K + co]) continue;
      const float *wp = w + static_cast<size_t>(co * C + ci) * taps;
      const float *ip = in + ci * H * W + y0 * W + x0;
      float sum = 0.0f;
      for (int wy = wy0; wy < wy1; ++wy)
        for (int wx = wx0; wx < wx1; ++wx) sum += wp[wy * S + wx] * ip[wy * W + wx];
      acc += sum;
    }
    if (has_bias) acc += b[co];
    out[o]  = acc;
    gout[o] = acc;
  }
}

// fully_connected_op_internal.h:15-36: out[i] = sum_c W[c*out + i] * in[c] + b[i]; the sum over
// c is split over a group of lanes
TN_INLINE void fc_fwd(const TinyLayer *__restrict__ Lp, const float *in, float *out, float *__restrict__ gout) {
  const int n_out = Lp->out_size, n_in = Lp->in_size, has_bias = Lp->has_bias;
  const float *__restrict__ w = Lp->w;
  const float *__restrict__ b = Lp->b;
  const int g = group_for(n_out, n_in), total = n_out * g, gs = __ffs(g) - 1;
  for (int base = 0; base < total; base += TN_THREADS) {
    const int it = base + threadIdx.x, i = it >> gs, part = it & (g - 1);
    float sum = 0.0f;
    if (it < total)
      for (int c = part; c < n_in; c += g) sum += w[static_cast<size_t>(c) * n_out + i] * in[c];
    sum = group_sum(sum, g);
    if (it < total && part == 0) {
      if (has_bias) sum += b[i];
      out[i]  = sum;
      gout[i] = sum;
    }
  }
}

// max_pooling_layer.h:195-222 + maxpool_op_internal.h:16-40: windows clipped at the edges,
// strict '>' from lowest(), the record is the flat CHW input index (0 when nothing wins)
TN_INLINE void maxpool_fwd(const TinyLayer *__restrict__ Lp, const float *in, float *out, float *__restrict__ gout,
                           int32_t *__restrict__ gargmax) {
  const int C = Lp->C, H = Lp->H, W = Lp->W, OH = Lp->OH, OW = Lp->OW, R = Lp->R, S = Lp->S, sh = Lp->sh, sw = Lp->sw;
  const FastDiv d_plane = Lp->d_oplane, d_ow = Lp->d_ow;
  const int total = C * OH * OW;
  for (int o = threadIdx.x; o < total; o += TN_THREADS) {
    uint32_t c, r, oy, ox;
    d_plane.divmod(o, c, r);
    d_ow.divmod(r, oy, ox);
    const int x0 = ox * sw, y0 = oy * sh;
    const int dxmax = min(S, W - x0), dymax = min(R, H - y0);
    float best = -FLT_MAX;
    int idx    = 0;
    for (int wy = 0; wy < dymax; ++wy)
      for (int wx = 0; wx < dxmax; ++wx) {
        const int j   = (H * c + y0 + wy) * W + x0 + wx;
        const float v = in[j];
        if (v > best) {
          best = v;
          idx  = j;
        }
      }
    out[o]     = best;
    gout[o]    = best;
    gargmax[o] = idx;
  }
}

// average_pooling_layer.h:25-55: value = sum(window) * (W[c] * scale) + b[c]
TN_INLINE void avepool_fwd(const TinyLayer *__restrict__ Lp, const float *in, float *out, float *__restrict__ gout) {
  const int C = Lp->C, H = Lp->H, W = Lp->W, OH = Lp->OH, OW = Lp->OW, R = Lp->R, S = Lp->S, sh = Lp->sh, sw = Lp->sw;
  const FastDiv d_plane = Lp->d_oplane, d_ow = Lp->d_ow;
  const float scale = Lp->scale;
  const float *__restrict__ w = Lp->w;
  const float *__restrict__ b = Lp->b;
  const int total = C * OH * OW;
  for (int o = threadIdx.x; o < total; o += TN_THREADS) {
    uint32_t c, r, oy, ox;
    d_plane.divmod(o, c, r);
    d_ow.divmod(r, oy, ox);
    const int x0 = ox * sw, y0 = oy * sh;
    float value  = 0.0f;
    if (x0 + S <= W && y0 + R <= H)
      for (int wy = 0; wy < R; ++wy)
        for (int wx = 0; wx < S; ++wx) value += in[(c * H + y0 + wy) * W + x0 + wx];
    const float weight = w[c] * scale;
    value *= weight;
    value += b[c];
    out[o]  = value;
    gout[o] = value;
  }
}

TN_INLINE void act_fwd(const TinyLayer *__restrict__ Lp, const float *in, float *out, float *__restrict__ gout) {
  const int n = Lp->out_size, act = Lp->act;
  const float p0 = Lp->p0;
  for (int o = threadIdx.x; o < n; o += TN_THREADS) {
    const float v = tn_act_fwd(act, p0, in[o]);
    out[o]  = v;
    gout[o] = v;
  }
}

// softmax_layer.h:24-34 on one row, by the first wave
TN_INLINE void softmax_fwd(const TinyLayer *__restrict__ Lp, const float *in, float *out, float *__restrict__ gout) {
  if (threadIdx.x >= 64) return;
  const int lane = threadIdx.x, len = Lp->out_size;
  float m = -FLT_MAX;
  for (int j = lane; j < len; j += 64) m = fmaxf(m, in[j]);
  for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
  float s = 0.0f;
  for (int j = lane; j < len; j += 64) {
    const float e = expf(in[j] - m);
    out[j]        = e;
    s += e;
  }
  for (int off = 32; off > 0; off >>= 1) s += __shfl_xor(s, off, 64);
  for (int j = lane; j < len; j += 64) {
    const float v = out[j] / s;
    out[j]  = v;
    gout[j] = v;
  }
}

// ------------------------------------------------------------------ backward
// conv2d_op_internal.h:91-127 as a gather: dX[ci][iy][ix] = sum over connected co and taps of
// W[co][ci][wy][wx] * dY[co][oy][ox] with iy = oy*sh + wy - ph, ix = ox*sw + wx - pw
TN_INLINE void conv_bwd_dx(const TinyLayer *__restrict__ Lp, const float *dy, float *dx, float *__restrict__ gdx) {
  const int C = Lp->C, H = Lp->H, W = Lp->W, K = Lp->K, OH = Lp->OH, OW = Lp->OW, R = Lp->R, S = Lp->S;
  const int sh = Lp->sh, sw = Lp->sw, ph = Lp->ph, pw = Lp->pw;
  const FastDiv d_plane = Lp->d_iplane, d_w = Lp->d_w;
  const float *__restrict__ w = Lp->w;
  const uint8_t *__restrict__ tbl = Lp->tbl;
  const int total = C * H * W, taps = R * S, oplane = OH * OW;
  const bool unit = sh == 1 && sw == 1;
  for (int e = threadIdx.x; e < total; e += TN_THREADS) {
    uint32_t ci, r, iy, ix;
    d_plane.divmod(e, ci, r);
    d_w.divmod(r, iy, ix);
    float acc = 0.0f;
    if (unit) {
      // oy = iy + ph - wy in [0, OH): wy from max(0, iy+ph-OH+1) to min(R-1, iy+ph)
      const int ty = iy + ph, tx = ix + pw;
      const int wy0 = max(0, ty - OH + 1), wy1 = min(R - 1, ty), wx0 = max(0, tx - OW + 1), wx1 = min(S - 1, tx);
      for (int co = 0; co < K; ++co) {
        if (tbl && !tbl[ci * K + co]) continue;
        const float *wp = w + static_cast<size_t>(co * C + ci) * taps;
        const float *dp = dy + co * oplane + ty * OW + tx;
        for (int wy = wy0; wy <= wy1; ++wy)
          for (int wx = wx0; wx <= wx1; ++wx) acc += wp[wy * S + wx] * dp[-wy * OW - wx];
      }
    } else {
      for (int co = 0; co < K; ++co) {
        if (tbl && !tbl[ci * K + co]) continue;
        const float *wp = w + static_cast<size_t>(co * C + ci) * taps;
        const float *dp = dy + co * oplane;
        for (int wy = 0; wy < R; ++wy) {
          const int ty = static_cast<int>(iy) + ph - wy;
          if (ty < 0) break;
          const int oy = ty / sh;
          if (oy * sh != ty || oy >= OH) continue;
          for (int wx = 0; wx < S; ++wx) {
            const int tx = static_cast<int>(ix) + pw - wx;
            if (tx < 0) break;
            const int ox = tx / sw;
            if (ox * sw == tx && ox < OW) acc += wp[wy * S + wx] * dp[oy * OW + ox];
          }
        }
      }
    }
    dx[e] = acc;
    if (gdx) gdx[e] = acc;
  }
}

// fully_connected_op_internal.h:38-71
TN_INLINE void fc_bwd_dx(const TinyLayer *__restrict__ Lp, const float *dy, float *dx, float *__restrict__ gdx) {
  const int n_out = Lp->out_size, n_in = Lp->in_size;
  const float *__restrict__ w = Lp->w;
  for (int c = threadIdx.x; c < n_in; c += TN_THREADS) {
    const float *wr = w + static_cast<size_t>(c) * n_out;
    float acc = 0.0f;
    int i = 0;
    for (; i + 8 <= n_out; i += 8) {   // eight reads in flight
      float wv[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) wv[j] = wr[i + j];
#pragma unroll
      for (int j = 0; j < 8; ++j) acc += dy[i + j] * wv[j];
    }
    for (; i < n_out; ++i) acc += dy[i] * wr[i];
    dx[c] = acc;
    if (gdx) gdx[c] = acc;
  }
}
// dW[c][i] = in[c] * dy[i] for the elements [base, base + count), db = dy with base 0
template <int NT>
TN_INLINE void fc_bwd_param(const TinyLayer *__restrict__ Lp, const float *in, const float *dy,
                            float *__restrict__ gw, float *__restrict__ gb, const int base, const int count) {
  const int nb = Lp->nb;
  const FastDiv d_out = Lp->d_out;
  for (int e = base + threadIdx.x; e < base + count; e += NT) {
    uint32_t c, i;
    d_out.divmod(e, c, i);
    gw[e] = in[c] * dy[i];
  }
  if (base == 0)
    for (int i = threadIdx.x; i < nb; i += NT) gb[i] = dy[i];
}

// maxpool_op_internal.h:42-57: an input takes the gradient of the LAST window that contains it
// when that window's record names it
TN_INLINE void maxpool_bwd(const TinyLayer *__restrict__ Lp, const float *dy, const int32_t *gargmax, float *dx,
                           float *__restrict__ gdx) {
  const int C = Lp->C, H = Lp->H, W = Lp->W, OH = Lp->OH, OW = Lp->OW, R = Lp->R, S = Lp->S, sh = Lp->sh, sw = Lp->sw;
  const FastDiv d_plane = Lp->d_iplane, d_w = Lp->d_w;
  const int total = C * H * W;
  for (int e = threadIdx.x; e < total; e += TN_THREADS) {
    uint32_t c, r, yy, xx;
    d_plane.divmod(e, c, r);
    d_w.divmod(r, yy, xx);
    const int ox = min(OW - 1, static_cast<int>(xx) / sw), oy = min(OH - 1, static_cast<int>(yy) / sh);
    const bool covered = (static_cast<int>(xx) < ox * sw + S) && (static_cast<int>(yy) < oy * sh + R);
    const int outi = covered ? (OH * c + oy) * OW + ox : 0;
    const float v  = (gargmax[outi] == e) ? dy[outi] : 0.0f;
    dx[e] = v;
    if (gdx) gdx[e] = v;
  }
}

// average_pooling_layer.h:58-106
TN_INLINE void avepool_bwd_dx(const TinyLayer *__restrict__ Lp, const float *dy, float *dx, float *__restrict__ gdx) {
  const int C = Lp->C, H = Lp->H, W = Lp->W, OH = Lp->OH, OW = Lp->OW, R = Lp->R, S = Lp->S, sh = Lp->sh, sw = Lp->sw;
  const FastDiv d_plane = Lp->d_iplane, d_w = Lp->d_w;
  const float scale = Lp->scale;
  const float *__restrict__ w = Lp->w;
  const int total = C * H * W;
  const bool two = R == 2 && S == 2 && sh == 2 && sw == 2;
  for (int e = threadIdx.x; e < total; e += TN_THREADS) {
    uint32_t c, r, iy, ix;
    d_plane.divmod(e, c, r);
    d_w.divmod(r, iy, ix);
    int ox, oy;
    if (two) {
      ox = static_cast<int>(ix) < 2 ? 0 : static_cast<int>(ix) >> 1;
      oy = static_cast<int>(iy) < 2 ? 0 : static_cast<int>(iy) >> 1;
    } else {
      ox = static_cast<int>(ix) < S ? 0 : (static_cast<int>(ix) - S + sw) / sw;
      oy = static_cast<int>(iy) < R ? 0 : (static_cast<int>(iy) - R + sh) / sh;
    }
    const float weight = w[c] * scale;
    const float v      = weight * dy[(c * OH + oy) * OW + ox];
    dx[e] = v;
    if (gdx) gdx[e] = v;
  }
}
template <int NT>
TN_INLINE void avepool_bwd_param(const TinyLayer *__restrict__ Lp, const float *in, const float *dy,
                                 float *__restrict__ gw, float *__restrict__ gb) {
  const int C = Lp->C, H = Lp->H, W = Lp->W, OH = Lp->OH, OW = Lp->OW, R = Lp->R, S = Lp->S, sh = Lp->sh, sw = Lp->sw;
  const FastDiv d_ow = Lp->d_ow;
  const float scale = Lp->scale;
  const int oplane = OH * OW;
  int g = 64;
  while (g > 1 && (C * g > NT || g > oplane)) g >>= 1;
  const int items = C * g, gs = __ffs(g) - 1;
  for (int base = 0; base < items; base += NT) {
    const int it = base + threadIdx.x, c = it >> gs, part = it & (g - 1);
    float sw_ = 0.0f, sb = 0.0f;
    if (it < items)
      for (int o = part; o < oplane; o += g) {
        uint32_t oy, ox;
        d_ow.divmod(o, oy, ox);
        const int x0 = ox * sw, y0 = oy * sh;
        const float dv = dy[c * oplane + o];
        sb += dv;
        if (x0 + S <= W && y0 + R <= H)
          for (int wy = 0; wy < R; ++wy)
            for (int wx = 0; wx < S; ++wx) sw_ += in[(c * H + y0 + wy) * W + x0 + wx] * dv;
      }
    sw_ = group_sum(sw_, g);
    sb  = group_sum(sb, g);
    if (it < items && part == 0) {
      gw[c] = sw_ * scale;
      gb[c] = sb;
    }
  }
}

TN_INLINE void act_bwd(const TinyLayer *__restrict__ Lp, const float *y, const float *dy, float *dx,
                       float *__restrict__ gdx) {
  const int n = Lp->out_size, act = Lp->act;
  const float p0 = Lp->p0;
  for (int e = threadIdx.x; e < n; e += TN_THREADS) {
    const float v = tn_act_bwd(act, p0, y[e], dy[e]);
    dx[e] = v;
    if (gdx) gdx[e] = v;
  }
}


// ---- the convolutions' fast forms -------------------------------------------------------
__device__ __forceinline__ int wave_index() { return __builtin_amdgcn_readfirstlane(threadIdx.x >> 6); }
constexpr int TN_WAVES = TN_THREADS / 64;

// dX of a stride-1 convolution reads dY from a copy with a frame of zeros,
// [K][H + R - 1][W + S - 1] with dY[co][0][0] at row R-1-ph, column S-1-pw, so that every tap of
// every input pixel reads inside the copy and the loops hold no bounds test: the tap (wy, wx) of
// input pixel (iy, ix) is the copy's element (iy + R-1 - wy, ix + S-1 - wx).
template <int NT, typename Src>
TN_INLINE void stage_framed_dy(const TinyLayer *__restrict__ Lp, const Src *dy, float *framed) {
  const int K = Lp->K, H = Lp->H, W = Lp->W, OH = Lp->OH, OW = Lp->OW, R = Lp->R, S = Lp->S;
  const int PW = W + S - 1, PP = (H + R - 1) * PW, oy0 = R - 1 - Lp->ph, ox0 = S - 1 - Lp->pw;
  const FastDiv d_pplane = Lp->d_pplane, d_pw = Lp->d_pw;
  for (int e = threadIdx.x; e < K * PP; e += NT) {
    uint32_t co, r, py, px;
    d_pplane.divmod(e, co, r);
    d_pw.divmod(r, py, px);
    const int oy = static_cast<int>(py) - oy0, ox = static_cast<int>(px) - ox0;
    const bool in = static_cast<unsigned>(oy) < static_cast<unsigned>(OH) && static_cast<unsigned>(ox) < static_cast<unsigned>(OW);
    const float v = dy[in ? (co * OH + oy) * OW + ox : 0];
    framed[e] = in ? v : 0.0f;
  }
}
// the rows [py_lo, py_hi] of the copy only (a workgroup that computes a few rows of dX)
template <int NT, typename Src>
TN_INLINE void stage_framed_rows(const TinyLayer *__restrict__ Lp, const Src *dy, float *framed, const int py_lo,
                                 const int py_hi) {
  const int K = Lp->K, H = Lp->H, W = Lp->W, OH = Lp->OH, OW = Lp->OW, R = Lp->R, S = Lp->S;
  const int PW = W + S - 1, PP = (H + R - 1) * PW, oy0 = R - 1 - Lp->ph, ox0 = S - 1 - Lp->pw;
  const FastDiv d_pw = Lp->d_pw;
  const int cells = (py_hi - py_lo + 1) * PW;
  for (int co = 0; co < K; ++co)
    for (int idx = threadIdx.x; idx < cells; idx += NT) {
      uint32_t q, px;
      d_pw.divmod(idx, q, px);
      const int py = py_lo + static_cast<int>(q);
      const int oy = py - oy0, ox = static_cast<int>(px) - ox0;
      const bool in = static_cast<unsigned>(oy) < static_cast<unsigned>(OH) && static_cast<unsigned>(ox) < static_cast<unsigned>(OW);
      const float v = dy[in ? (co * OH + oy) * OW + ox : 0];
      framed[co * PP + py * PW + static_cast<int>(px)] = in ? v : 0.0f;
    }
}
__host__ __device__ inline int conv_framed_floats(const TinyLayer &L) {
  return L.K * (L.H + L.R - 1) * (L.W + L.S - 1);
}

// A wave's 64 lanes are 64 pixels of one block of NB channels, so every filter value a wave needs
// is the same for all its lanes: it comes through the scalar cache straight from the weight
// tensor, W[co][ci][tap], and enters the multiply-add as a scalar operand; LDS carries one
// 4-byte read per tap, the pixel. (Filters staged in LDS and read 16 bytes per lane and tap make
// LDS the bound: it serves the four SIMDs together.) Windows of 3x3 and 5x5 are unrolled; other
// sizes take the general loops further up. Waves without an item of their own take a part
// of the summed-over channels of somebody else's; the parts meet in `scratch`.
// how many parts (1, 2 or 4) when there are `items` items and `channels` channels to sum over
// (loads through a pointer to the constant address space with a wave-uniform address are scalar
// loads; the filters are not written while these kernels run)
typedef const float __attribute__((address_space(4))) *ScalarFloats;
TN_INLINE int scalar_parts(const int items, const int channels, const int waves) {
  int parts = 1;
  while (parts < 4 && 2 * parts * items <= waves && 2 * parts <= channels) parts <<= 1;
  return parts;
}
// channels of a block: three when that divides the count and four does not
__host__ __device__ inline int scalar_block(const int channels) {
  return channels == 1 ? 1 : ((channels % 3 == 0 && (channels & 3) != 0) ? 3 : 4);
}

template <int R, int S, bool PAD, int NB, bool TBL>
TN_INLINE void conv_fwd_scalar(const TinyLayer *__restrict__ Lp, const float *in, float *out, float *__restrict__ gout,
                               float *scratch) {
  const int C = Lp->C, H = Lp->H, W = Lp->W, K = Lp->K, OH = Lp->OH, OW = Lp->OW;
  const int sh = Lp->sh, sw = Lp->sw, ph = Lp->ph, pw = Lp->pw, has_bias = Lp->has_bias;
  const FastDiv d_ow = Lp->d_ow;
  const float *__restrict__ w = Lp->w;
  const float *__restrict__ b = Lp->b;
  const uint8_t *__restrict__ tbl = Lp->tbl;
  constexpr int taps = R * S;
  const int plane = OH * OW, chunks = (plane + 63) >> 6, blocks = (K + NB - 1) / NB, items = blocks * chunks;
  const int parts = scalar_parts(items, C, TN_WAVES), Ch = (C + parts - 1) / parts, total = items * parts;
  const int lane = threadIdx.x & 63;
  for (int it0 = 0; it0 < total; it0 += TN_WAVES) {
    const int item = it0 + wave_index();
    const bool active = item < total;
    const int it = active ? item : 0;
    const int cp = it / items, rem = it - cp * items, blk = rem / chunks, chunk = rem - blk * chunks, co0 = blk * NB;
    const int p = (chunk << 6) + lane;
    const bool live = p < plane;
    uint32_t oy, ox;
    d_ow.divmod(live ? p : 0, oy, ox);
    const int y0 = static_cast<int>(oy) * sh - ph, x0 = static_cast<int>(ox) * sw - pw;
    int cob[NB];
#pragma unroll
    for (int q = 0; q < NB; ++q) cob[q] = min(co0 + q, K - 1);
    float acc[NB];
#pragma unroll
    for (int q = 0; q < NB; ++q) acc[q] = 0.0f;
    const int c_lo = cp * Ch, c_hi = active ? min(C, c_lo + Ch) : c_lo;
    for (int ci = c_lo; ci < c_hi; ++ci) {
      const float *ip = in + ci * H * W + y0 * W + x0;
      ScalarFloats wq[NB];
#pragma unroll
      for (int q = 0; q < NB; ++q) wq[q] = (ScalarFloats)(w + static_cast<size_t>(cob[q] * C + ci) * taps);
      float sum[NB];
#pragma unroll
      for (int q = 0; q < NB; ++q) sum[q] = 0.0f;
#pragma unroll
      for (int wy = 0; wy < R; ++wy) {
#pragma unroll
        for (int wx = 0; wx < S; ++wx) {
          float v;
          if (PAD) {
            const bool ok = static_cast<unsigned>(y0 + wy) < static_cast<unsigned>(H) &&
                            static_cast<unsigned>(x0 + wx) < static_cast<unsigned>(W);
            v = ip[ok ? wy * W + wx : -(y0 * W + x0)];
            v = ok ? v : 0.0f;
          } else {
            v = ip[wy * W + wx];
          }
#pragma unroll
          for (int q = 0; q < NB; ++q) sum[q] = __builtin_fmaf(wq[q][wy * S + wx], v, sum[q]);
        }
      }
#pragma unroll
      for (int q = 0; q < NB; ++q)
        if (!TBL || tbl[ci * K + cob[q]]) acc[q] += sum[q];
    }
    if (parts > 1) {
      if (active && cp > 0) {
#pragma unroll
        for (int q = 0; q < NB; ++q) scratch[(((cp - 1) * items + rem) * NB + q) * 64 + lane] = acc[q];
      }
      lds_barrier();
      if (active && cp == 0)
        for (int o = 1; o < parts; ++o) {
#pragma unroll
          for (int q = 0; q < NB; ++q) acc[q] += scratch[(((o - 1) * items + rem) * NB + q) * 64 + lane];
        }
      lds_barrier();
    }
    if (active && cp == 0 && live) {
#pragma unroll
      for (int q = 0; q < NB; ++q)
        if (co0 + q < K) {
          const float v = has_bias ? acc[q] + b[co0 + q] : acc[q];
          out[(co0 + q) * plane + p]  = v;
          gout[(co0 + q) * plane + p] = v;
        }
    }
  }
}
template <int R, int S, bool PAD>
TN_INLINE void conv_fwd_scalar_any(const TinyLayer *__restrict__ Lp, const float *in, float *out,
                                   float *__restrict__ gout, float *scratch) {
  // (a connection table makes every channel sum conditional: a version of its own, so that the
  // loops of a net without one stay free of branches)
  const bool tbl = Lp->tbl != nullptr;
  if (scalar_block(Lp->K) == 3) {
    if (tbl) conv_fwd_scalar<R, S, PAD, 3, true>(Lp, in, out, gout, scratch);
    else conv_fwd_scalar<R, S, PAD, 3, false>(Lp, in, out, gout, scratch);
  } else {
    if (tbl) conv_fwd_scalar<R, S, PAD, 4, true>(Lp, in, out, gout, scratch);
    else conv_fwd_scalar<R, S, PAD, 4, false>(Lp, in, out, gout, scratch);
  }
}

// dX from the zero-framed dY (stage_framed_dy); the waves of a workgroup of NT threads take the
// items [item0, item1) of items * parts in turn (item = part * items + block * chunks + chunk);
// dx (LDS) may be NULL
template <int R, int S, int NB, int NT, bool TBL>
TN_INLINE void conv_bwd_dx_scalar(const TinyLayer *__restrict__ Lp, const float *framed, float *dx,
                                  float *__restrict__ gdx, float *scratch, const int item0, const int item1,
                                  const int parts) {
  const int C = Lp->C, H = Lp->H, W = Lp->W, K = Lp->K;
  const FastDiv d_w = Lp->d_w;
  const float *__restrict__ w = Lp->w;
  const uint8_t *__restrict__ tbl = Lp->tbl;
  constexpr int taps = R * S;
  const int plane = H * W, chunks = (plane + 63) >> 6, blocks = (C + NB - 1) / NB, items = blocks * chunks;
  const int PW = W + S - 1, PP = (H + R - 1) * PW, Kh = (K + parts - 1) / parts;
  const int lane = threadIdx.x & 63;
  for (int it0 = item0; it0 < item1; it0 += NT / 64) {
    const int item = it0 + wave_index();
    const bool active = item < item1;
    const int it = active ? item : item0;
    const int kp = it / items, rem = it - kp * items, blk = rem / chunks, chunk = rem - blk * chunks, ci0 = blk * NB;
    const int p = (chunk << 6) + lane;
    const bool live = p < plane;
    uint32_t iy, ix;
    d_w.divmod(live ? p : 0, iy, ix);
    const float *dp0 = framed + (static_cast<int>(iy) + R - 1) * PW + static_cast<int>(ix);
    int cib[NB];
#pragma unroll
    for (int q = 0; q < NB; ++q) cib[q] = min(ci0 + q, C - 1);
    float acc[NB];
#pragma unroll
    for (int q = 0; q < NB; ++q) acc[q] = 0.0f;
    const int c_lo = kp * Kh, c_hi = active ? min(K, c_lo + Kh) : c_lo;
    for (int co = c_lo; co < c_hi; ++co) {
      const float *dp = dp0 + co * PP;
      ScalarFloats wq[NB];
#pragma unroll
      for (int q = 0; q < NB; ++q) wq[q] = (ScalarFloats)(w + static_cast<size_t>(co * C + cib[q]) * taps);
      float sum[NB];
#pragma unroll
      for (int q = 0; q < NB; ++q) sum[q] = 0.0f;
#pragma unroll
      for (int wy = 0; wy < R; ++wy) {
        const float *row = dp - wy * PW;
#pragma unroll
        for (int wx = 0; wx < S; ++wx) {
          const float v = row[S - 1 - wx];
#pragma unroll
          for (int q = 0; q < NB; ++q) sum[q] = __builtin_fmaf(wq[q][wy * S + wx], v, sum[q]);
        }
      }
#pragma unroll
      for (int q = 0; q < NB; ++q)
        if (!TBL || tbl[cib[q] * K + co]) acc[q] += sum[q];
    }
    if (parts > 1) {
      if (active && kp > 0) {
#pragma unroll
        for (int q = 0; q < NB; ++q) scratch[(((kp - 1) * items + rem) * NB + q) * 64 + lane] = acc[q];
      }
      lds_barrier();
      if (active && kp == 0)
        for (int o = 1; o < parts; ++o) {
#pragma unroll
          for (int q = 0; q < NB; ++q) acc[q] += scratch[(((o - 1) * items + rem) * NB + q) * 64 + lane];
        }
      lds_barrier();
    }
    if (active && kp == 0 && live) {
#pragma unroll
      for (int q = 0; q < NB; ++q)
        if (ci0 + q < C) {
          if (dx) dx[(ci0 + q) * plane + p] = acc[q];
          if (gdx) gdx[(ci0 + q) * plane + p] = acc[q];
        }
    }
  }
}
// whole-wave items of the scalar dX
__host__ __device__ inline int conv_dx_scalar_items(const TinyLayer &L) {
  const int nb = scalar_block(L.C);
  return ((L.C + nb - 1) / nb) * ((L.H * L.W + 63) >> 6);
}
template <int R, int S, int NT>
TN_INLINE void conv_bwd_dx_scalar_any(const TinyLayer *__restrict__ Lp, const float *framed, float *dx,
                                      float *__restrict__ gdx, float *scratch, const int item0, const int item1,
                                      const int parts) {
  const int nb = scalar_block(Lp->C);
  if (Lp->tbl) {
    if (nb == 1) conv_bwd_dx_scalar<R, S, 1, NT, true>(Lp, framed, dx, gdx, scratch, item0, item1, parts);
    else if (nb == 3) conv_bwd_dx_scalar<R, S, 3, NT, true>(Lp, framed, dx, gdx, scratch, item0, item1, parts);
    else conv_bwd_dx_scalar<R, S, 4, NT, true>(Lp, framed, dx, gdx, scratch, item0, item1, parts);
  } else {
    if (nb == 1) conv_bwd_dx_scalar<R, S, 1, NT, false>(Lp, framed, dx, gdx, scratch, item0, item1, parts);
    else if (nb == 3) conv_bwd_dx_scalar<R, S, 3, NT, false>(Lp, framed, dx, gdx, scratch, item0, item1, parts);
    else conv_bwd_dx_scalar<R, S, 4, NT, false>(Lp, framed, dx, gdx, scratch, item0, item1, parts);
  }
}

// ---------------------------------------------------------------- convolutions on the matrix cores
// out[m][p] = bias[m] + sum_k A[m][k] * in[koff[k] + poff(p)]: the forward pass of a stride-1
// convolution without padding (every tap of every output pixel lies inside the input) as a
// product of the filters with the patches of the input. v_mfma_f32_16x16x4_f32: lane
// (r = lane % 16, q = lane / 16) supplies A[row r][one k] and B[the same k][column r] and holds
// D[row 4 q + i][column r], i = 0..3; which four k an instruction adds up is free, and here step
// st of `steps` takes k = q * steps + st, so that a lane's operands of four steps in a row are
// 16 consecutive bytes of a filter row and of the offset table. A wave takes 16 channels x
// T tiles of 16 pixels at once (what bounds a tile is the chain of LDS reads in front of its
// first product, not the products: T tiles share that chain). `a` holds A as [M][pitch] with
// zeros from n_k on, `koff` the input offset of every k < 4 * steps, `bias` the bias or NULL,
// all in LDS (stage_mfma_operands); steps is a multiple of four.
typedef float tn_f4 __attribute__((ext_vector_type(4)));
constexpr int MFMA_AHEAD = 4;   // filter values a thread holds for the layer whose filters wait in registers
__host__ __device__ inline int mfma_steps(const int n_k) { return ((n_k + 15) >> 4) << 2; }
// (a row pitch of 4 * odd floats: sixteen rows read 16 bytes each from different banks, two rows a bank group)
__host__ __device__ inline int mfma_pitch(const int n_k) { return (4 * mfma_steps(n_k)) | 4; }
template <int T>
TN_INLINE void conv_mfma(const float *src, const float *a, const int *koff, const int M, const int n_k,
                         const int plane, const FastDiv d_row, const int src_pitch, const float *bias,
                         float *out, float *__restrict__ gout) {
  const int lane = threadIdx.x & 63, r = lane & 15, q = lane >> 4;
  const int steps = mfma_steps(n_k), pitch = mfma_pitch(n_k), groups = steps >> 2;
  const int m_tiles = (M + 15) >> 4, p_tiles = (plane + 15) >> 4, p_items = (p_tiles + T - 1) / T;
  const int total = m_tiles * p_items;
  const int k_left = n_k - q * steps;   // this lane's steps from k_left on are padding
  for (int it0 = 0; it0 < total; it0 += TN_WAVES) {
    const int item = it0 + wave_index();
    if (item >= total) break;     // (no barrier inside)
    const int mt = item / p_items, pi = item - mt * p_items;
    const int arow = min(mt * 16 + r, M - 1);
    const float *sp[T];
#pragma unroll
    for (int j = 0; j < T; ++j) {
      uint32_t py, px;
      d_row.divmod(min((pi * T + j) * 16 + r, plane - 1), py, px);
      sp[j] = src + static_cast<int>(py) * src_pitch + static_cast<int>(px);
    }
    const float4 *a4 = reinterpret_cast<const float4 *>(a + arow * pitch + q * steps);
    const int4 *k4 = reinterpret_cast<const int4 *>(koff + q * steps);
    tn_f4 acc[T];
#pragma unroll
    for (int j = 0; j < T; ++j) acc[j] = tn_f4{0.0f, 0.0f, 0.0f, 0.0f};
    float4 av = a4[0];
    int4 ko   = k4[0];
    for (int g = 0; g < groups; ++g) {
      float b[T][4];
#pragma unroll
      for (int j = 0; j < T; ++j) {
        b[j][0] = sp[j][ko.x]; b[j][1] = sp[j][ko.y]; b[j][2] = sp[j][ko.z]; b[j][3] = sp[j][ko.w];
      }
      const float4 ac = av;
      const int gn = min(g + 1, groups - 1);
      av = a4[gn];
      ko = k4[gn];
      // (a zero filter value times an infinity would be a NaN)
      const int st = 4 * g;
      const bool on0 = st < k_left, on1 = st + 1 < k_left, on2 = st + 2 < k_left, on3 = st + 3 < k_left;
#pragma unroll
      for (int j = 0; j < T; ++j) {
        acc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(ac.x, on0 ? b[j][0] : 0.0f, acc[j], 0, 0, 0);
        acc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(ac.y, on1 ? b[j][1] : 0.0f, acc[j], 0, 0, 0);
      }
#pragma unroll
      for (int j = 0; j < T; ++j) {
        acc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(ac.z, on2 ? b[j][2] : 0.0f, acc[j], 0, 0, 0);
        acc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(ac.w, on3 ? b[j][3] : 0.0f, acc[j], 0, 0, 0);
      }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = mt * 16 + 4 * q + i;
      if (m >= M) continue;
      const float bv = bias ? bias[m] : 0.0f;
#pragma unroll
      for (int j = 0; j < T; ++j) {
        const int p = (pi * T + j) * 16 + r;
        if (p < plane) {
          const float v = bias ? acc[j][i] + bv : acc[j][i];
          out[m * plane + p] = v;
          if (gout) gout[m * plane + p] = v;
        }
      }
    }
  }
}
// The operand and the offset table of the input gradient described at TinyLayer::mf_dx_w, from
// the filter values the thread still holds (mfma_filters_load: value j is element
// e0 + j * TN_THREADS + thread of the weight tensor), the rows' ends zeroed.
TN_INLINE void mfma_dx_operand_store(const TinyLayer *__restrict__ L, const float (&v)[MFMA_AHEAD], float *lds) {
  const int C = L->C, K = L->K, R = L->R, S = L->S, taps = R * S, nw = K * C * taps;
  const int n_k = K * R, pitch = mfma_pitch(n_k), k4 = 4 * mfma_steps(n_k), rows = C * S;
  const int PW = L->W + S - 1, PP = (L->H + R - 1) * PW;
  const uint8_t *__restrict__ tbl = L->tbl;
  float *a = lds + L->mf_dx_w;
  int *ko  = reinterpret_cast<int *>(lds + L->mf_dx_ko);
#pragma unroll
  for (int j = 0; j < MFMA_AHEAD; ++j) {
    const int e = j * TN_THREADS + threadIdx.x;
    if (e >= nw) continue;
    uint32_t pair, t, co, ci, wy, wx;
    L->d_taps.divmod(e, pair, t);
    L->d_c.divmod(pair, co, ci);
    L->d_s.divmod(t, wy, wx);
    a[(ci * S + wx) * pitch + co * R + wy] = (tbl && !tbl[ci * K + co]) ? 0.0f : v[j];
  }
  const int pad = pitch - n_k;
  for (int idx = threadIdx.x; idx < rows * pad; idx += TN_THREADS) {
    const int row = idx / pad;
    a[row * pitch + n_k + idx - row * pad] = 0.0f;
  }
  for (int k = threadIdx.x; k < k4; k += TN_THREADS) {
    const int co = k / R, wy = k - co * R;
    ko[k] = k < n_k ? co * PP + (R - 1 - wy) * PW : 0;
  }
}
// dX from D (TinyLayer::mf_dx_d): the filter columns' shifted sums, in column order
TN_INLINE void mfma_dx_gather(const TinyLayer *__restrict__ L, const float *d, float *dx, float *__restrict__ gdx) {
  const int C = L->C, H = L->H, W = L->W, S = L->S, PW = W + S - 1, cols = H * PW;
  const FastDiv d_iplane = L->d_iplane, d_w = L->d_w;
  for (int e = threadIdx.x; e < C * H * W; e += TN_THREADS) {
    uint32_t ci, r, iy, ix;
    d_iplane.divmod(e, ci, r);
    d_w.divmod(r, iy, ix);
    const float *row = d + (ci * S) * cols + iy * PW + ix + S - 1;
    float sum = 0.0f;
    for (int wx = 0; wx < S; ++wx) sum += row[wx * cols - wx];
    dx[e] = sum;
    if (gdx) gdx[e] = sum;
  }
}
// The operands above for a layer that has them, straight from the weight tensor. Every filter
// value is read once, in the tensor's own order ([co][(ci, tap)], which is A's); pairs of
// channels that a connection table leaves unconnected get a zero, and so do the ends of the
// rows. In two halves, so that the reads can be in flight while other layers run: the first
// asks for up to MFMA_AHEAD values a thread, the second puts them in LDS.
TN_INLINE void mfma_filters_load(const TinyLayer *__restrict__ L, const int e0, float (&v)[MFMA_AHEAD], float &bias) {
  const int nw = L->K * L->C * L->R * L->S;
#pragma unroll
  for (int j = 0; j < MFMA_AHEAD; ++j) v[j] = L->w[min(e0 + j * TN_THREADS + static_cast<int>(threadIdx.x), nw - 1)];
  // (the bias goes with the first piece: a value a thread, there are fewer channels than threads)
  bias = (e0 == 0 && L->has_bias) ? L->b[min(static_cast<int>(threadIdx.x), L->K - 1)] : 0.0f;
}
TN_INLINE void mfma_filters_store(const TinyLayer *__restrict__ L, const int e0, const float (&v)[MFMA_AHEAD],
                                  const float bias, float *lds) {
  const int K = L->K, taps = L->R * L->S, n_k = L->C * taps, nw = K * n_k, pitch = mfma_pitch(n_k);
  const uint8_t *__restrict__ tbl = L->tbl;
  float *fa = lds + L->mf_fwd_w;
#pragma unroll
  for (int j = 0; j < MFMA_AHEAD; ++j) {
    const int e = e0 + j * TN_THREADS + threadIdx.x;
    if (e >= nw) continue;
    uint32_t co, k, ci, t;
    L->d_nk.divmod(e, co, k);
    L->d_taps.divmod(k, ci, t);
    fa[co * pitch + k] = (tbl && !tbl[ci * K + co]) ? 0.0f : v[j];
  }
  if (e0 == 0 && L->has_bias && static_cast<int>(threadIdx.x) < K) lds[L->mf_fwd_b + threadIdx.x] = bias;
}
// everything else: the rows' zero ends and the offset table
TN_INLINE void mfma_tables(const TinyLayer *__restrict__ L, float *lds) {
  const int K = L->K, H = L->H, W = L->W, taps = L->R * L->S;
  const int n_k = L->C * taps, pitch = mfma_pitch(n_k), k4 = 4 * mfma_steps(n_k), pad = pitch - n_k;
  float *fa = lds + L->mf_fwd_w;
  int *ko   = reinterpret_cast<int *>(lds + L->mf_fwd_ko);
  for (int idx = threadIdx.x; idx < K * pad; idx += TN_THREADS) {
    const int row = idx / pad;
    fa[row * pitch + n_k + idx - row * pad] = 0.0f;
  }
  for (int k = threadIdx.x; k < k4; k += TN_THREADS) {
    uint32_t ci, t, wy, wx;
    L->d_taps.divmod(min(k, n_k - 1), ci, t);
    L->d_s.divmod(t, wy, wx);
    ko[k] = k < n_k ? static_cast<int>(ci) * H * W + static_cast<int>(wy) * W + static_cast<int>(wx) : 0;
  }
}
// every layer but the one whose filters travel in registers (`ahead`, or -1): when the kernel starts
TN_INLINE void stage_mfma_operands(const TinyPlan *__restrict__ plan, float *lds, const int ahead) {
  const int n = plan->n_mfma;
  for (int q = 0; q < n; ++q) {   // (the plan lists them: walking every layer is a scalar load and a wait each)
    const int li = plan->mfma_layers[q];
    if (li == ahead) continue;
    const TinyLayer *__restrict__ L = &plan->l[li];
    mfma_tables(L, lds);
    const int nw = L->K * L->C * L->R * L->S;
    for (int e0 = 0; e0 < nw; e0 += MFMA_AHEAD * TN_THREADS) {
      float v[MFMA_AHEAD], bias;
      mfma_filters_load(L, e0, v, bias);
      mfma_filters_store(L, e0, v, bias, lds);
    }
  }
}

// A convolution whose window is the whole input (one output pixel per channel, no padding) is a
// matrix-vector product: out[co] = sum_k W[co][k] in[k], dX[k] = sum_co W[co][k] dY[co]. Lanes
// run along k, so the filter rows are read in whole cache lines, and a lane asks for all the
// filter values of a round before it uses the first: what bounds these few kilobytes is the
// latency of a read, not its size.
__host__ __device__ inline bool conv_is_matvec(const TinyLayer &L) {
  return L.OH == 1 && L.OW == 1 && L.ph == 0 && L.pw == 0 && L.R == L.H && L.S == L.W;
}
// shapes the dX from a framed dY takes (whether it runs is the plan's dx_framed, set where LDS is laid out)
inline bool conv_dx_shape_is_framed(const TinyLayer &L) {
  return !conv_is_matvec(L) && L.sh == 1 && L.sw == 1 &&
         ((L.R == 5 && L.S == 5) || (L.R == 3 && L.S == 3));
}
// the same with 16-byte reads: no connection table, n_k a multiple of four, `in` 16-byte aligned.
// A group of lanes per output channel, as many as keep the whole workgroup busy in one round;
// the lanes of a group read neighbouring 16-byte pieces of the filter row, eight in flight each.
TN_INLINE void conv_fwd_matvec4(const TinyLayer *__restrict__ Lp, const float *in, float *out, float *__restrict__ gout) {
  const int K = Lp->K, has_bias = Lp->has_bias;
  const float *__restrict__ b = Lp->b;
  const int n_k4 = (Lp->C * Lp->R * Lp->S) >> 2;
  const float4 *__restrict__ w4 = reinterpret_cast<const float4 *>(Lp->w);
  const float4 *in4 = reinterpret_cast<const float4 *>(in);
  int g = 64;
  while (g > 1 && (K * g > TN_THREADS || 4 * g > n_k4)) g >>= 1;
  const int gs = __ffs(g) - 1, total = K * g;
  for (int base = 0; base < total; base += TN_THREADS) {
    const int it = base + threadIdx.x, part = it & (g - 1);
    const bool on = it < total;
    const int co = on ? it >> gs : 0;
    const float4 *wr = w4 + static_cast<size_t>(co) * n_k4;
    float sum = 0.0f;
    for (int k0 = 0; k0 < n_k4; k0 += 8 * g) {
      float4 a[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int k = k0 + g * j + part;
        a[j] = wr[k < n_k4 ? k : 0];
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int k = k0 + g * j + part;
        if (k < n_k4) {
          const float4 xv = in4[k];
          sum += (a[j].x * xv.x + a[j].y * xv.y) + (a[j].z * xv.z + a[j].w * xv.w);
        }
      }
    }
    sum = group_sum(sum, g);
    if (on && part == 0) {
      const float v = has_bias ? sum + b[co] : sum;
      out[co]  = v;
      gout[co] = v;
    }
  }
}
// dX[k] with 16-byte reads along k (same conditions): a thread takes four neighbouring k for one
// of `parts` ranges of output channels; the parts' sums meet in `scratch` and add up in order
TN_INLINE void conv_bwd_dx_matvec4(const TinyLayer *__restrict__ Lp, const float *dy, float *dx,
                                   float *__restrict__ gdx, float *scratch) {
  const int K = Lp->K, n_k = Lp->C * Lp->R * Lp->S, n_k4 = n_k >> 2;
  const float4 *__restrict__ w4 = reinterpret_cast<const float4 *>(Lp->w);
  int parts = 1;
  while (parts < 8 && 2 * parts * n_k4 <= TN_THREADS && 2 * parts * n_k <= TINY_SCRATCH_FLOATS) parts <<= 1;
  const int Kh = (K + parts - 1) / parts;
  for (int k0 = 0; k0 < n_k4; k0 += TN_THREADS / parts) {
    const int span = min(n_k4 - k0, TN_THREADS / parts);   // pieces of this trip
    const int part = threadIdx.x / span, kk = threadIdx.x - part * span;
    const bool on = part < parts;
    const int k = k0 + kk, c_lo = part * Kh, c_hi = on ? min(K, c_lo + Kh) : c_lo;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    int co = c_lo;
    for (; co + 4 <= c_hi; co += 4) {   // four rows in flight
      float4 wv[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) wv[j] = w4[static_cast<size_t>(co + j) * n_k4 + k];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float d = dy[co + j];
        acc.x += wv[j].x * d; acc.y += wv[j].y * d; acc.z += wv[j].z * d; acc.w += wv[j].w * d;
      }
    }
    for (; co < c_hi; ++co) {
      const float4 wv = w4[static_cast<size_t>(co) * n_k4 + k];
      const float d   = dy[co];
      acc.x += wv.x * d; acc.y += wv.y * d; acc.z += wv.z * d; acc.w += wv.w * d;
    }
    if (parts > 1) {
      if (on) reinterpret_cast<float4 *>(scratch)[part * span + kk] = acc;
      lds_barrier();
      if (part == 0)
        for (int q = 1; q < parts; ++q) {
          const float4 o = reinterpret_cast<const float4 *>(scratch)[q * span + kk];
          acc.x += o.x; acc.y += o.y; acc.z += o.z; acc.w += o.w;
        }
      lds_barrier();
    }
    if (part == 0) {
      const float r[4] = {acc.x, acc.y, acc.z, acc.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        dx[4 * k + j] = r[j];
        if (gdx) gdx[4 * k + j] = r[j];
      }
    }
  }
}
TN_INLINE void conv_fwd_matvec(const TinyLayer *__restrict__ Lp, const float *in, float *out, float *__restrict__ gout) {
  const int C = Lp->C, K = Lp->K, taps = Lp->R * Lp->S, has_bias = Lp->has_bias;
  const FastDiv d_taps = Lp->d_taps;
  const float *__restrict__ w = Lp->w;
  const float *__restrict__ b = Lp->b;
  const uint8_t *__restrict__ tbl = Lp->tbl;
  const int n_k = C * taps, lane = threadIdx.x & 63;
  constexpr int ROWS = 4;   // filter rows per wave and round, eight values of each per lane
  for (int co0 = wave_index(); co0 < K; co0 += ROWS * TN_WAVES) {
    float s[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) s[r] = 0.0f;
    for (int k0 = 0; k0 < n_k; k0 += 512) {
      float a[ROWS][8];
#pragma unroll
      for (int r = 0; r < ROWS; ++r) {
        const int co = co0 + r * TN_WAVES;
        const float *wr = w + static_cast<size_t>(co < K ? co : co0) * n_k;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int k = k0 + 64 * j + lane;
          a[r][j] = wr[k < n_k ? k : 0];
        }
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int k = k0 + 64 * j + lane;
        const bool ok = k < n_k;
        const float xv = in[ok ? k : 0];
        const int ci = d_taps.div(ok ? k : 0);
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
          const int co = co0 + r * TN_WAVES;
          const float v = a[r][j] * xv;
          if (ok && co < K && (!tbl || tbl[ci * K + co])) s[r] += v;
        }
      }
    }
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
      const int co = co0 + r * TN_WAVES;
      const float sum = group_sum(s[r], 64);
      if (lane == 0 && co < K) {
        const float v = has_bias ? sum + b[co] : sum;
        out[co]  = v;
        gout[co] = v;
      }
    }
  }
}
// dX[k]: the threads split into `parts` ranges of output channels when k leaves most of them
// idle; the parts' sums meet in `scratch` (parts * stride floats of LDS) and add up in order
TN_INLINE void conv_bwd_dx_matvec(const TinyLayer *__restrict__ Lp, const float *dy, float *dx, float *__restrict__ gdx,
                                  float *scratch) {
  const int C = Lp->C, K = Lp->K, taps = Lp->R * Lp->S;
  const FastDiv d_taps = Lp->d_taps;
  const float *__restrict__ w = Lp->w;
  const uint8_t *__restrict__ tbl = Lp->tbl;
  const int n_k = C * taps;
  const int parts = n_k <= 256 ? 4 : (n_k <= 512 ? 2 : 1), stride = TN_THREADS / parts;
  const int part = threadIdx.x / stride, kk = threadIdx.x - part * stride;
  const int Kh = (K + parts - 1) / parts, c_lo = part * Kh, c_hi = min(K, c_lo + Kh);
  for (int k0 = 0; k0 < n_k; k0 += stride) {
    const int k = k0 + kk;
    const bool ok = k < n_k;
    const int kc = ok ? k : 0, ci = d_taps.div(kc);
    float acc = 0.0f;
    int co = c_lo;
    for (; co + 8 <= c_hi; co += 8) {   // eight rows in flight
      float wv[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) wv[j] = w[static_cast<size_t>(co + j) * n_k + kc];
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if (!tbl || tbl[ci * K + co + j]) acc += wv[j] * dy[co + j];
    }
    for (; co < c_hi; ++co)
      if (!tbl || tbl[ci * K + co]) acc += w[static_cast<size_t>(co) * n_k + kc] * dy[co];
    if (parts > 1) {
      scratch[part * stride + kk] = acc;
      lds_barrier();
      if (part == 0) {
        for (int q = 1; q < parts; ++q) acc += scratch[q * stride + kk];
      }
      lds_barrier();
    }
    if (part == 0 && ok) {
      dx[k] = acc;
      if (gdx) gdx[k] = acc;
    }
  }
}

// lanes that share one weight's sum over output rows in the parameter-gradient kernel
__host__ __device__ inline int conv_param_group(const TinyLayer &L) {
  int g = 32;
  while (g > 1 && (32 * g > L.OH * L.OW || g > L.OH)) g >>= 1;   // 32 output pixels or more per lane
  return g;
}
// this sample's dW and db of a convolution (conv2d_op_internal.h:130-179): a group of lanes per
// weight; the lanes of a group take output rows in turn, a lane walks the pixels of its rows
// whose window element lies inside the input, and the group adds up with butterfly shuffles.
// (Lanes that take pixels in turn instead, neighbouring lanes on neighbouring words, run into no
// bank conflicts but pay more for the bookkeeping per pixel: 13.1 against 10.4 us for LeNet-5.)
// Units [base, base + count) of nw * group (weights x lanes); the bias gradient goes with base 0.
template <int NT>
TN_INLINE void conv_bwd_param_rows(const TinyLayer *__restrict__ Lp, const float *in, const float *dy,
                                   float *__restrict__ gw, const int base0, const int count) {
  const int H = Lp->H, W = Lp->W, K = Lp->K, OH = Lp->OH, OW = Lp->OW;
  const int sh = Lp->sh, sw = Lp->sw, ph = Lp->ph, pw = Lp->pw;
  const FastDiv d_taps = Lp->d_taps, d_s = Lp->d_s, d_c = Lp->d_c;
  const uint8_t *__restrict__ tbl = Lp->tbl;
  const int plane = OH * OW;
  const bool unit = sh == 1 && sw == 1;
  {
    const int g = conv_param_group(*Lp), gs = __ffs(g) - 1, end = base0 + count;
    for (int base = base0; base < end; base += NT) {
      const int it = base + threadIdx.x, idx = it >> gs, part = it & (g - 1);
      float sum = 0.0f;
      if (it < end) {
        uint32_t pair, tap, co, ci, wy, wx;
        d_taps.divmod(idx, pair, tap);
        d_c.divmod(pair, co, ci);
        d_s.divmod(tap, wy, wx);
        if (!tbl || tbl[ci * K + co]) {
          // iy = oy*sh + wy - ph in [0, H), ix = ox*sw + wx - pw in [0, W)
          const int yoff = static_cast<int>(wy) - ph, xoff = static_cast<int>(wx) - pw;
          int oy_lo, oy_hi, ox_lo, ox_hi;
          if (unit) {
            oy_lo = max(0, -yoff); oy_hi = min(OH, H - yoff);
            ox_lo = max(0, -xoff); ox_hi = min(OW, W - xoff);
          } else {
            oy_lo = yoff >= 0 ? 0 : (-yoff + sh - 1) / sh; oy_hi = min(OH, (H - 1 - yoff) / sh + 1);
            ox_lo = xoff >= 0 ? 0 : (-xoff + sw - 1) / sw; ox_hi = min(OW, (W - 1 - xoff) / sw + 1);
          }
          const float *ip = in + ci * H * W + yoff * W + xoff;
          const float *dp = dy + co * plane;
          for (int oy = oy_lo + part; oy < oy_hi; oy += g) {
            const float *ir = ip + oy * sh * W;
            const float *dr = dp + oy * OW;
            int ox = ox_lo;
            if (unit) {
              for (; ox + 4 <= ox_hi; ox += 4)
                sum += ir[ox] * dr[ox] + ir[ox + 1] * dr[ox + 1] + ir[ox + 2] * dr[ox + 2] + ir[ox + 3] * dr[ox + 3];
              for (; ox < ox_hi; ++ox) sum += ir[ox] * dr[ox];
            } else {
              for (; ox + 4 <= ox_hi; ox += 4)
                sum += ir[ox * sw] * dr[ox] + ir[(ox + 1) * sw] * dr[ox + 1] + ir[(ox + 2) * sw] * dr[ox + 2] +
                       ir[(ox + 3) * sw] * dr[ox + 3];
              for (; ox < ox_hi; ++ox) sum += ir[ox * sw] * dr[ox];
            }
          }
        }
      }
      sum = group_sum(sum, g);
      if (it < end && part == 0) gw[idx] = sum;
    }
  }
}
// the bias gradient of such a convolution, a job of its own (beside the first units of the weight
// gradient it made that workgroup the last of the launch to finish): every plane of dY, a group
// of lanes a channel
template <int NT>
TN_INLINE void conv_bwd_param_bias(const TinyLayer *__restrict__ Lp, const float *dy, float *__restrict__ gb) {
  const int nb = Lp->nb, plane = Lp->OH * Lp->OW;
  {
    int g = 64;
    while (g > 1 && (nb * g > 2 * NT || g > plane)) g >>= 1;
    const int total = nb * g, gs = __ffs(g) - 1;
    for (int base = 0; base < total; base += NT) {
      const int it = base + threadIdx.x, co = it >> gs, part = it & (g - 1);
      float sum = 0.0f;
      if (it < total)
        for (int p = part; p < plane; p += g) sum += dy[co * plane + p];
      sum = group_sum(sum, g);
      if (it < total && part == 0) gb[co] = sum;
    }
  }
}
// the same for a convolution that is a matrix-vector product: dW[co][k] = in[k] * dY[co] for
// the elements [base, base + count)
template <int NT>
TN_INLINE void conv_bwd_param_matvec(const TinyLayer *__restrict__ Lp, const float *in, const float *dy,
                                     float *__restrict__ gw, float *__restrict__ gb, const int base, const int count) {
  const int K = Lp->K, nb = Lp->nb;
  const FastDiv d_taps = Lp->d_taps, d_nk = Lp->d_nk;
  const uint8_t *__restrict__ tbl = Lp->tbl;
  for (int e = base + threadIdx.x; e < base + count; e += NT) {
    uint32_t co, k;
    d_nk.divmod(e, co, k);
    float v = in[k] * dy[co];
    if (tbl && !tbl[d_taps.div(k) * K + co]) v = 0.0f;
    gw[e] = v;
  }
  if (base == 0)
    for (int co = threadIdx.x; co < nb; co += NT) gb[co] = dy[co];
}

// One workgroup per sample. LDS: the sample's input, every layer's output, two gradient buffers,
// the staging area.
__global__ void __launch_bounds__(TN_THREADS)
tiny_net_step_kernel(const TinyPlan *__restrict__ plan, const int loss, const int softmax_xent,
                     const float *__restrict__ x, const float *__restrict__ t) {
  extern __shared__ float lds[];
  const int s = blockIdx.x, n = plan->n, in_size = plan->in_size;
  float *wl = lds + plan->lds_w;   // where partial sums of split layers meet (TINY_SCRATCH_FLOATS)
  // (one layer's filters for the matrix cores are asked for here, in front of the sample's input,
  // and put in LDS while the layer in front of that layer runs: no layer waits for them)
  const int ahead = plan->mf_ahead;
  float ahead_w[MFMA_AHEAD] = {0.0f, 0.0f, 0.0f, 0.0f}, ahead_b = 0.0f;
  if (ahead > 0) mfma_filters_load(&plan->l[ahead], 0, ahead_w, ahead_b);
  fill_lds<TN_THREADS>(lds, x + static_cast<size_t>(s) * in_size, in_size);
  stage_mfma_operands(plan, lds, ahead);
  lds_barrier();
  for (int li = 0; li < n; ++li) {
    const TinyLayer *__restrict__ L = &plan->l[li];
    if (li + 1 == ahead) {
      mfma_filters_store(&plan->l[ahead], 0, ahead_w, ahead_b, lds);
      mfma_tables(&plan->l[ahead], lds);
    }
    const int kind = L->kind, out_size = L->out_size;
    const float *in = lds + L->lds_in;
    float *out      = lds + L->lds_out;
    float *gout     = L->out + static_cast<size_t>(s) * out_size;
    switch (kind) {
      case TDH_L_CONV:
        if (conv_is_matvec(*L)) {
          if (!L->tbl && ((L->C * L->R * L->S) & 3) == 0 && (L->lds_in & 3) == 0) conv_fwd_matvec4(L, in, out, gout);
          else conv_fwd_matvec(L, in, out, gout);
        }
        else if (L->mf_fwd_w >= 0) {
          const float *fa = lds + L->mf_fwd_w, *fb = L->has_bias ? lds + L->mf_fwd_b : nullptr;
          const int *fk = reinterpret_cast<const int *>(lds + L->mf_fwd_ko);
          const int n_k = L->C * L->R * L->S, plane = L->OH * L->OW;
          // (several pixel tiles a wave when there are more tiles than waves)
          if (((L->K + 15) >> 4) * ((plane + 15) >> 4) > TN_WAVES) conv_mfma<4>(in, fa, fk, L->K, n_k, plane, L->d_ow, L->W, fb, out, gout);
          else conv_mfma<1>(in, fa, fk, L->K, n_k, plane, L->d_ow, L->W, fb, out, gout);
        }
        else if (L->R == 5 && L->S == 5 && L->ph == 0 && L->pw == 0) conv_fwd_scalar_any<5, 5, false>(L, in, out, gout, wl);
        else if (L->R == 5 && L->S == 5) conv_fwd_scalar_any<5, 5, true>(L, in, out, gout, wl);
        else if (L->R == 3 && L->S == 3 && L->ph == 0 && L->pw == 0) conv_fwd_scalar_any<3, 3, false>(L, in, out, gout, wl);
        else if (L->R == 3 && L->S == 3) conv_fwd_scalar_any<3, 3, true>(L, in, out, gout, wl);
        else conv_fwd(L, in, out, gout);
        break;
      case TDH_L_FC: fc_fwd(L, in, out, gout); break;
      case TDH_L_MAXPOOL: maxpool_fwd(L, in, out, gout, L->argmax + static_cast<size_t>(s) * out_size); break;
      case TDH_L_AVEPOOL: avepool_fwd(L, in, out, gout); break;
      default:
        if (L->act == TDH_ACT_SOFTMAX) softmax_fwd(L, in, out, gout);
        else act_fwd(L, in, out, gout);
        break;
    }
    lds_barrier();
  }
  // the loss gradient with respect to the net's output (loss_function.h:28-36, 120-150); with a
  // closing softmax and cross_entropy_multiclass the gradient with respect to the softmax's
  // INPUT in closed form, y * sum(t) - t, and the softmax layer's own backward pass is skipped
  float *ga = lds + plan->lds_g0, *gb = lds + plan->lds_g1;
  const TinyLayer *__restrict__ last = &plan->l[n - 1];
  const int n_out = last->out_size;
  const float *y  = lds + last->lds_out;
  const float *tr = t + static_cast<size_t>(s) * n_out;
  int first_bwd   = n - 1;
  if (softmax_xent) {
    float st = 0.0f;  // (every thread adds up the same few targets, in order)
    for (int j = 0; j < n_out; ++j) st += tr[j];
    float *gdz = last->dx + static_cast<size_t>(s) * n_out;
    for (int j = threadIdx.x; j < n_out; j += TN_THREADS) {
      const float v = fmaf(y[j], st, -tr[j]);
      ga[j]  = v;
      gdz[j] = v;
    }
    first_bwd = n - 2;
  } else {
    const float mse_factor = plan->mse_factor;
    float *gdl = plan->dloss + static_cast<size_t>(s) * n_out;
    for (int j = threadIdx.x; j < n_out; j += TN_THREADS) {
      float v;
      if (loss == TDH_LOSS_MSE) v = mse_factor * (y[j] - tr[j]);
      else if (loss == TDH_LOSS_CE_MULTICLASS) v = -tr[j] / y[j];
      else v = (y[j] - tr[j]) / (y[j] * (1.0f - y[j]));
      ga[j]  = v;
      gdl[j] = v;
    }
  }
  __syncthreads();   // (also: the max-pool records written to memory above are read back below)
  // input gradients only: the parameter-gradient kernel reads what this loop leaves in memory
  const int last_bwd = (plan->first_dx_as_job || plan->skip_first_dx) ? 1 : 0;
  for (int li = first_bwd; li >= last_bwd; --li) {
    const TinyLayer *__restrict__ L = &plan->l[li];
    const int kind = L->kind, in_sz = L->in_size;
    // (the layer in front of this one in memory order is the next to run: its operand goes into
    // the scratch area now, which this phase does not use when that is so; see tiny_build_jobs)
    if (li - 1 == ahead && ahead > 0 && plan->l[ahead].mf_dx_w >= 0) mfma_dx_operand_store(&plan->l[ahead], ahead_w, lds);
    float *gdx = L->dx ? L->dx + static_cast<size_t>(s) * in_sz : nullptr;
    switch (kind) {
      case TDH_L_CONV:
        if (conv_is_matvec(*L)) {
          if (!L->tbl && ((L->C * L->R * L->S) & 3) == 0) conv_bwd_dx_matvec4(L, ga, gb, gdx, wl);
          else conv_bwd_dx_matvec(L, ga, gb, gdx, wl);
        }
        else if (!L->dx_framed) conv_bwd_dx(L, ga, gb, gdx);
        else {
          float *framed = lds + plan->lds_pad;
          stage_framed_dy<TN_THREADS>(L, ga, framed);
          lds_barrier();
          const int items = conv_dx_scalar_items(*L), parts = scalar_parts(items, L->K, TN_WAVES);
          if (L->mf_dx_w >= 0) {
            // (the operand was written into the scratch area while the layer behind ran; D has every
            // position of H framed rows as a column, so a column's offset is its index)
            float *dd = lds + L->mf_dx_d;
            const int PW = L->W + L->S - 1, cols = L->H * PW;
            conv_mfma<2>(framed, lds + L->mf_dx_w, reinterpret_cast<const int *>(lds + L->mf_dx_ko), L->C * L->S,
                         L->K * L->R, cols, L->d_pw, PW, nullptr, dd, nullptr);
            lds_barrier();
            mfma_dx_gather(L, dd, gb, gdx);
          }
          else if (L->R == 5) conv_bwd_dx_scalar_any<5, 5, TN_THREADS>(L, framed, gb, gdx, wl, 0, items * parts, parts);
          else conv_bwd_dx_scalar_any<3, 3, TN_THREADS>(L, framed, gb, gdx, wl, 0, items * parts, parts);
        }
        break;
      case TDH_L_FC: fc_bwd_dx(L, ga, gb, gdx); break;
      case TDH_L_MAXPOOL: maxpool_bwd(L, ga, L->argmax + static_cast<size_t>(s) * L->out_size, gb, gdx); break;
      case TDH_L_AVEPOOL: avepool_bwd_dx(L, ga, gb, gdx); break;
      default: act_bwd(L, lds + L->lds_out, ga, gb, gdx); break;
    }
    lds_barrier();
    float *sw = ga;
    ga = gb;
    gb = sw;
  }
}

// The parameter gradients of one sample, a job per workgroup: the layer's input and the gradient
// of its output come back from memory into LDS (the step kernel wrote both), then the job's
// units run as they would in one workgroup.
constexpr int TP_THREADS = 256;
__global__ void __launch_bounds__(TP_THREADS)
tiny_net_param_kernel(const TinyPlan *__restrict__ plan, const float *__restrict__ x) {
  extern __shared__ float lds[];
  const TinyJob job = plan->jobs[blockIdx.y];
  const int s = blockIdx.x, n = plan->n, li = job.layer;
  const TinyLayer *__restrict__ L = &plan->l[li];
  const int in_sz = L->in_size, out_sz = L->out_size, kind = L->kind;
  const float *gin = (li == 0 ? x : plan->l[li - 1].out) + static_cast<size_t>(s) * in_sz;
  const float *gdy = (li == n - 1 ? plan->dloss : plan->l[li + 1].dx) + static_cast<size_t>(s) * out_sz;
  if (job.what == 1) {   // the first layer's dX from a framed dY: dY goes from memory straight into its frame
    float *framed = lds;
    float *gdx = L->dx + static_cast<size_t>(s) * in_sz;
    // the rows of the frame that this job's pixels read: its items are chunks of 64 pixels of
    // one block of channels, or else everything
    const int plane = L->H * L->W, chunks = (plane + 63) >> 6, last = job.base + job.count - 1;
    int py_lo = 0, py_hi = L->H + L->R - 2;
    if (job.base / chunks == last / chunks) {
      const int p_lo = (job.base % chunks) << 6, p_hi = min(plane - 1, ((last % chunks) << 6) + 63);
      py_lo = static_cast<int>(L->d_w.div(p_lo));
      py_hi = static_cast<int>(L->d_w.div(p_hi)) + L->R - 1;
    }
    stage_framed_rows<TP_THREADS>(L, gdy, framed, py_lo, py_hi);
    lds_barrier();
    if (L->R == 5) conv_bwd_dx_scalar_any<5, 5, TP_THREADS>(L, framed, nullptr, gdx, nullptr, job.base, job.base + job.count, 1);
    else conv_bwd_dx_scalar_any<3, 3, TP_THREADS>(L, framed, nullptr, gdx, nullptr, job.base, job.base + job.count, 1);
    return;
  }
  if (job.what == 2) {   // a convolution's bias gradient: dY alone
    fill_lds<TP_THREADS>(lds, gdy, out_sz);
    lds_barrier();
    conv_bwd_param_bias<TP_THREADS>(L, lds, L->gb + static_cast<size_t>(s) * L->nb);
    return;
  }
  float *in = lds, *dy = lds + ((in_sz + 3) & ~3);
  fill_lds<TP_THREADS>(in, gin, in_sz);
  // (a convolution's weight-gradient units name the output channels whose gradient planes they read)
  int dy_lo = 0, dy_n = out_sz;
  if (kind == TDH_L_CONV && !conv_is_matvec(*L)) {
    const int gs = __ffs(conv_param_group(*L)) - 1, plane = L->OH * L->OW;
    const int co_lo = static_cast<int>(L->d_nk.div(job.base >> gs));
    const int co_hi = static_cast<int>(L->d_nk.div((job.base + job.count - 1) >> gs));
    dy_lo = co_lo * plane;
    dy_n  = (co_hi - co_lo + 1) * plane;
  }
  fill_lds<TP_THREADS>(dy + dy_lo, gdy + dy_lo, dy_n);
  lds_barrier();
  float *gw = L->gw + static_cast<size_t>(s) * L->nw;
  float *gb = L->gb ? L->gb + static_cast<size_t>(s) * L->nb : nullptr;
  switch (kind) {
    case TDH_L_CONV:
      if (conv_is_matvec(*L)) conv_bwd_param_matvec<TP_THREADS>(L, in, dy, gw, gb, job.base, job.count);
      else conv_bwd_param_rows<TP_THREADS>(L, in, dy, gw, job.base, job.count);
      break;
    case TDH_L_FC: fc_bwd_param<TP_THREADS>(L, in, dy, gw, gb, job.base, job.count); break;
    case TDH_L_AVEPOOL: avepool_bwd_param<TP_THREADS>(L, in, dy, gw, gb); break;
    default: break;
  }
}

// g[i] += slice[0][i] + slice[1][i] + ... in sample order (edge::merge_grads, node.h:89-103)
__global__ void __launch_bounds__(256)
tiny_net_merge_kernel(const TinyMerge m, const int batch) {
  int j = 0;
  while (j + 1 < m.n && m.first_block[j + 1] <= static_cast<int>(blockIdx.x)) ++j;
  const int i = (static_cast<int>(blockIdx.x) - m.first_block[j]) * 256 + threadIdx.x;
  if (i >= m.len[j]) return;
  const float *p = m.slices[j] + i;
  float sum = p[0];
  for (int s = 1; s < batch; ++s) sum += p[static_cast<size_t>(s) * m.len[j]];
  m.g[j][i] += sum;
}

}  // namespace

int tiny_prepare() {
  static bool attr_set = false;
  if (!attr_set) {
    TDH_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&tiny_net_step_kernel),
                                hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(TINY_LDS_MAX_BYTES)));
    TDH_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&tiny_net_param_kernel),
                                hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(TINY_LDS_MAX_BYTES)));
    attr_set = true;
  }
  return TDH_OK;
}

int tiny_build_jobs(TinyPlan &P) {
  // units of work per layer and the units one workgroup takes: a lane's item for the grouped
  // sums, sixteen elements per lane for the element-wise products, a wave's item for the dX
  struct Piece { int layer, what, units, per_job; };
  Piece pieces[2 * TINY_MAX_LAYERS + 1];
  int n_pieces = 0;
  size_t lds = 0, framed = 0;
  for (int i = 0; i < P.n; ++i) {
    TinyLayer &L = P.l[i];
    L.dx_framed = L.kind == TDH_L_CONV && conv_dx_shape_is_framed(L) && L.dx != nullptr;
    if (L.dx_framed) {
      L.d_pplane = FastDiv(static_cast<uint32_t>((L.H + L.R - 1) * (L.W + L.S - 1)));
      L.d_pw     = FastDiv(static_cast<uint32_t>(L.W + L.S - 1));
    }
  }
  P.first_dx_as_job = P.l[0].dx_framed && P.n > 1 && !P.skip_first_dx;
  for (int i = 0; i < P.n; ++i) {
    const TinyLayer &L = P.l[i];
    if (i == 0 && P.first_dx_as_job) {
      pieces[n_pieces++] = {i, 1, conv_dx_scalar_items(L), TP_THREADS / 64};
      lds = std::max(lds, static_cast<size_t>(conv_framed_floats(L)));
    } else if (L.dx_framed) {
      framed = std::max(framed, static_cast<size_t>(conv_framed_floats(L)));
    }
    if (!L.nw) continue;
    lds = std::max(lds, static_cast<size_t>(((L.in_size + 3) & ~3) + ((L.out_size + 3) & ~3)));
    if (L.kind == TDH_L_CONV && !conv_is_matvec(L)) {
      pieces[n_pieces++] = {i, 0, L.nw * conv_param_group(L), TP_THREADS};
      if (L.nb) pieces[n_pieces++] = {i, 2, 1, 1};
    }
    else if (L.kind == TDH_L_CONV || L.kind == TDH_L_FC) pieces[n_pieces++] = {i, 0, L.nw, 16 * TP_THREADS};
    else pieces[n_pieces++] = {i, 0, 1, 1};
  }
  P.lds_pad = P.lds_floats;
  P.lds_floats += static_cast<int>(framed);
  // operands of the products that run on the matrix cores, while LDS has room for them
  P.n_mfma = 0;
  P.mf_ahead = -1;
  for (int i = 0; i < P.n; ++i) {
    TinyLayer &L = P.l[i];
    L.mf_fwd_w = L.mf_fwd_ko = L.mf_fwd_b = -1;
    // (few output channels leave most of a 16-row tile empty, and a short sum is over before
    // the operands of its first product have arrived: those stay with the scalar loops)
    if (L.kind != TDH_L_CONV || conv_is_matvec(L) || L.sh != 1 || L.sw != 1 || L.K < 8 ||
        L.C * L.R * L.S < 48)
      continue;
    const size_t room = TINY_LDS_MAX_BYTES / sizeof(float);
    const int taps = L.R * L.S;
    // (both areas start on 16 bytes: rows and offset tables are read four values at a time)
    if (L.ph == 0 && L.pw == 0) {
      const int n_k = L.C * taps;
      const size_t need = static_cast<size_t>(mfma_pitch(n_k)) * L.K + 4 * mfma_steps(n_k) + L.K;
      const int at = (P.lds_floats + 3) & ~3;
      if (at + need <= room) {
        L.mf_fwd_w = at; L.mf_fwd_ko = at + mfma_pitch(n_k) * L.K; L.mf_fwd_b = L.mf_fwd_ko + 4 * mfma_steps(n_k);
        P.lds_floats = at + static_cast<int>(need);
        P.mfma_layers[P.n_mfma++] = i;
        if (P.mf_ahead < 0 && i > 0 && L.K * n_k <= MFMA_AHEAD * TN_THREADS) P.mf_ahead = i;
      }
    }
  }
  for (int i = 0; i < P.n; ++i) P.l[i].mf_dx_w = P.l[i].mf_dx_ko = P.l[i].mf_dx_d = -1;
  if (P.mf_ahead > 0 && P.mf_ahead + 1 < P.n) {
    // the input gradient of that layer on the matrix cores: its operand goes into the scratch
    // area while the layer behind it runs its backward phase, which therefore must be one that
    // leaves that area alone (a pointwise activation or a pool), and D needs room of its own
    TinyLayer &L = P.l[P.mf_ahead];
    const TinyLayer &behind = P.l[P.mf_ahead + 1];
    // (not a closing softmax either: under cross_entropy_multiclass its backward phase is skipped)
    const bool quiet = (behind.kind == TDH_L_ACT && behind.act != TDH_ACT_SOFTMAX) || behind.kind == TDH_L_MAXPOOL ||
                       behind.kind == TDH_L_AVEPOOL;
    const int n_k = L.K * L.R, rows = L.C * L.S, cols = L.H * (L.W + L.S - 1);
    const size_t operand = static_cast<size_t>(mfma_pitch(n_k)) * rows + 4 * mfma_steps(n_k);
    const int at = (P.lds_floats + 3) & ~3;
    if (L.dx_framed && quiet && operand <= TINY_SCRATCH_FLOATS &&
        at + static_cast<size_t>(rows) * cols <= TINY_LDS_MAX_BYTES / sizeof(float)) {
      L.mf_dx_w  = P.lds_w;
      L.mf_dx_ko = P.lds_w + mfma_pitch(n_k) * rows;
      L.mf_dx_d  = at;
      P.lds_floats = at + rows * cols;
    }
  }
  for (int scale = 1;; scale *= 2) {
    int jobs = 0;
    for (int q = 0; q < n_pieces; ++q) jobs += ceil_div(pieces[q].units, pieces[q].per_job * scale);
    if (jobs > TINY_MAX_JOBS) continue;
    P.n_jobs = 0;
    for (int q = 0; q < n_pieces; ++q) {
      const int per = pieces[q].per_job * scale;
      for (int base = 0; base < pieces[q].units; base += per) {
        TinyJob &J = P.jobs[P.n_jobs++];
        J.layer = static_cast<int16_t>(pieces[q].layer);
        J.what  = static_cast<int16_t>(pieces[q].what);
        J.base  = base;
        J.count = std::min(per, pieces[q].units - base);
      }
    }
    break;
  }
  P.lds_job_floats = static_cast<int>(lds);
  return TDH_OK;
}

int launch_tiny_step(const TinyPlan &plan, const TinyPlan *dev_plan, int loss, int softmax_xent, int batch,
                     const float *x, const float *t) {
  ProfScope prof("tiny_net_step", plan.flop_per_sample * batch * (2.0 / 3.0), WORK_FLOP);
  TDH_LAUNCH(tiny_net_step_kernel, dim3(batch), dim3(TN_THREADS), plan.lds_floats * sizeof(float), ctx().stream,
             dev_plan, loss, softmax_xent, x, t);
  TDH_LAUNCH_CHECK();
  return TDH_OK;
}

int launch_tiny_params(const TinyPlan &plan, const TinyPlan *dev_plan, int batch, const float *x) {
  if (plan.n_jobs == 0) return TDH_OK;
  ProfScope prof("tiny_net_param_grads", plan.flop_per_sample * batch * (1.0 / 3.0), WORK_FLOP);
  // (x counts the samples: consecutive workgroups go to different XCDs, and this way each XCD
  // gets every job of the samples that fall to it rather than every sample of a few jobs)
  TDH_LAUNCH(tiny_net_param_kernel, dim3(batch, plan.n_jobs), dim3(TP_THREADS), plan.lds_job_floats * sizeof(float),
             ctx().stream, dev_plan, x);
  TDH_LAUNCH_CHECK();
  return TDH_OK;
}

int launch_tiny_merge(const TinyMerge &m, int batch) {
  if (m.n == 0) return TDH_OK;
  double bytes = 0.0;
  for (int j = 0; j < m.n; ++j) bytes += 4.0 * m.len[j] * (batch + 2);
  ProfScope prof("tiny_net_merge_grads", bytes, WORK_BYTE);
  TDH_LAUNCH(tiny_net_merge_kernel, dim3(m.first_block[m.n]), dim3(256), 0, ctx().stream, m, batch);
  TDH_LAUNCH_CHECK();
  return TDH_OK;
}

}  // namespace tdh
