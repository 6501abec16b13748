// pool.hip — max pooling (argmax record + gather backward) and tiny-dnn's trainable
// average pooling, forward and backward. All kernels stream each tensor once.
// Built with -ffp-contract=off (see elementwise.hip).
#include <cfloat>

#include "common.h"

namespace tdh {

namespace {

constexpr int PT = 256;

struct PoolGeom {
  int C, H, W, OH, OW, pw, ph, sw, sh;
  FastDiv div_ow, div_oh, div_c, div_w, div_h;
};

PoolGeom make_geom(const tdh_pool_desc *d) {
  PoolGeom g;
  g.C = d->in_c; g.H = d->in_h; g.W = d->in_w;
  g.OW = pool_out_length(d->in_w, d->pool_w, d->stride_w, d->ceil_mode, d->pad_same);
  g.OH = pool_out_length(d->in_h, d->pool_h, d->stride_h, d->ceil_mode, d->pad_same);
  g.pw = d->pool_w; g.ph = d->pool_h; g.sw = d->stride_w; g.sh = d->stride_h;
  g.div_ow = FastDiv(g.OW > 0 ? g.OW : 1); g.div_oh = FastDiv(g.OH > 0 ? g.OH : 1);
  g.div_c = FastDiv(g.C); g.div_w = FastDiv(g.W); g.div_h = FastDiv(g.H);
  return g;
}

// maxpool_op_internal.h:16-40 with the windows of max_pooling_layer::connect_kernel
// (max_pooling_layer.h:195-222): clipped at the right/bottom edge, scanned row by row,
// strict '>' from numeric_limits::lowest() so the first maximum wins, NaN never wins and
// an all-NaN window reports index 0.
__global__ void __launch_bounds__(PT)
maxpool_fwd_kernel(const float *__restrict__ x, float *__restrict__ y,
                   int32_t *__restrict__ argmax, const int total, const PoolGeom g,
                   float *__restrict__ act_out, const int act_kind) {
  const int o = blockIdx.x * PT + threadIdx.x;
  if (o >= total) return;
  uint32_t t, ox, oy, c, img;
  g.div_ow.divmod(o, t, ox);
  g.div_oh.divmod(t, t, oy);
  g.div_c.divmod(t, img, c);
  const int x0 = ox * g.sw, y0 = oy * g.sh;
  const int dxmax = min(g.pw, g.W - x0), dymax = min(g.ph, g.H - y0);
  const float *in = x + static_cast<size_t>(img) * g.C * g.H * g.W;
  float best      = -FLT_MAX;
  int idx         = 0;
  for (int wy = 0; wy < dymax; ++wy)
    for (int wx = 0; wx < dxmax; ++wx) {
      const int j   = (g.H * c + y0 + wy) * g.W + x0 + wx;
      const float v = in[j];
      if (v > best) {
        best = v;
        idx  = j;
      }
    }
  y[o] = best;
  if (argmax) argmax[o] = idx;
  if (act_out) act_out[o] = act_apply(act_kind, best);  // the activation layer that follows
}

// The same for the common geometry: 2x2 windows, stride 2, width a multiple of 4 and even
// height, 16-byte aligned tensors. A thread owns two neighbouring outputs, i.e. two input rows
// of four floats, read as 16-byte words; the window scan order (row by row, left to right) and
// the strict '>' are those of the general kernel.
// SUM: the input is a split reduction left to this kernel (sum.out is x): the thread adds up
// the eight values it reads, and writes them to x as the reduction kernel would have.
template <bool SUM>
__global__ void __launch_bounds__(PT)
maxpool2x2_fwd_kernel(const float *__restrict__ x, float *__restrict__ y,
                      int32_t *__restrict__ argmax, const int pairs, const int W, const int OW2,
                      const FastDiv div_ow2, const int rows_per_sample, float *__restrict__ act_out,
                      const int act_kind, const SplitSum sum) {
  const int t = blockIdx.x * PT + threadIdx.x;  // pair index: (plane*OH + oy)*OW2 + ox2
  if (t >= pairs) return;
  uint32_t row, ox2;
  div_ow2.divmod(t, row, ox2);                   // row = plane*OH + oy
  // input rows 2*row and 2*row+1 of the [planes*H][W] image, columns 4*ox2 .. 4*ox2+3
  const size_t at = static_cast<size_t>(2 * row) * W + 4 * ox2;
  float4 r0, r1;
  if (SUM) {
    float a[4], b[4];
    split_sum_values<4>(sum, at, a);
    split_sum_values<4>(sum, at + W, b);
    r0 = make_float4(a[0], a[1], a[2], a[3]);
    r1 = make_float4(b[0], b[1], b[2], b[3]);
  } else {
    r0 = *reinterpret_cast<const float4 *>(x + at);
    r1 = *reinterpret_cast<const float4 *>(x + at + W);
  }
  const float v[2][4] = {{r0.x, r0.y, r1.x, r1.y}, {r0.z, r0.w, r1.z, r1.w}};
  float best[2];
  int idx[2];
#pragma unroll
  for (int k = 0; k < 2; ++k) {
    best[k] = -FLT_MAX;
    int sel = -1;
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (v[k][j] > best[k]) {
        best[k] = v[k][j];
        sel     = j;
      }
    idx[k] = sel;
  }
  const size_t o = static_cast<size_t>(row) * (2 * OW2) + 2 * ox2;
  *reinterpret_cast<float2 *>(y + o) = make_float2(best[0], best[1]);
  if (act_out)
    *reinterpret_cast<float2 *>(act_out + o) =
      make_float2(act_apply(act_kind, best[0]), act_apply(act_kind, best[1]));
  if (argmax) {
    // flat CHW index inside the sample (rows_per_sample = C*H input rows a sample)
    int2 a;
    const int base = (static_cast<int>(2 * row) % rows_per_sample) * W + 4 * static_cast<int>(ox2);
    a.x = idx[0] < 0 ? 0 : base + (idx[0] >> 1) * W + (idx[0] & 1);
    a.y = idx[1] < 0 ? 0 : base + 2 + (idx[1] >> 1) * W + (idx[1] & 1);
    *reinterpret_cast<int2 *>(argmax + o) = a;
  }
}

// dx rows 2*row, 2*row+1, columns 4*ox2..4*ox2+3 from two outputs and their argmax records
// SUM: dy is a split reduction left to this kernel (sum.out is dy), as in the forward kernel
template <bool SUM>
__global__ void __launch_bounds__(PT)
maxpool2x2_bwd_kernel(const float *__restrict__ dy, const int32_t *__restrict__ argmax,
                      float *__restrict__ dx, const int pairs, const int W, const int OW2,
                      const FastDiv div_ow2, const int rows_per_sample, const ActGrad ag,
                      const SplitSum sum, const float *__restrict__ pooled_y) {
  const int t = blockIdx.x * PT + threadIdx.x;
  if (t >= pairs) return;
  uint32_t row, ox2;
  div_ow2.divmod(t, row, ox2);
  const size_t o  = static_cast<size_t>(row) * (2 * OW2) + 2 * ox2;
  float2 g;
  if (SUM) {
    float v[2];
    split_sum_values<2>(sum, o, v);
    g = make_float2(v[0], v[1]);
  } else {
    g = *reinterpret_cast<const float2 *>(dy + o);
  }
  const int2 a    = *reinterpret_cast<const int2 *>(argmax + o);
  const int base  = (static_cast<int>(2 * row) % rows_per_sample) * W + 4 * static_cast<int>(ox2);
  const size_t at = static_cast<size_t>(2 * row) * W + 4 * ox2;
  if (pooled_y) {
    // The activation in front of the pool: dx *= act'(its output), and the only element of a
    // window that gets a gradient is the one the pool passed on, so the pool's own output is
    // that activation output: a quarter of the reads. (A window none of whose elements exceeds
    // lowest() is recorded as element 0 of the sample, maxpool_op_internal.h:28-36: that element
    // gets the gradient if the window is the sample's first, and its own value decides.)
    const float2 pv = *reinterpret_cast<const float2 *>(pooled_y + o);
    float fx = act_grad_factor(ag.kind, pv.x);
    if (base == 0 && a.x == 0) fx = act_grad_factor(ag.kind, ag.y[at]);
    g.x *= fx;
    g.y *= act_grad_factor(ag.kind, pv.y);
  }
  float4 r0, r1;
  r0.x = a.x == base ? g.x : 0.0f;
  r0.y = a.x == base + 1 ? g.x : 0.0f;
  r0.z = a.y == base + 2 ? g.y : 0.0f;
  r0.w = a.y == base + 3 ? g.y : 0.0f;
  r1.x = a.x == base + W ? g.x : 0.0f;
  r1.y = a.x == base + W + 1 ? g.x : 0.0f;
  r1.z = a.y == base + W + 2 ? g.y : 0.0f;
  r1.w = a.y == base + W + 3 ? g.y : 0.0f;
  if (!pooled_y && ag.kind != TDH_ACT_NONE) {  // the activation layer in front of the pool: dx *= act'(its output)
    const float4 y0 = *reinterpret_cast<const float4 *>(ag.y + at);
    const float4 y1 = *reinterpret_cast<const float4 *>(ag.y + at + W);
    r0.x *= act_grad_factor(ag.kind, y0.x); r0.y *= act_grad_factor(ag.kind, y0.y);
    r0.z *= act_grad_factor(ag.kind, y0.z); r0.w *= act_grad_factor(ag.kind, y0.w);
    r1.x *= act_grad_factor(ag.kind, y1.x); r1.y *= act_grad_factor(ag.kind, y1.y);
    r1.z *= act_grad_factor(ag.kind, y1.z); r1.w *= act_grad_factor(ag.kind, y1.w);
  }
  float *p = dx + at;
  *reinterpret_cast<float4 *>(p)     = r0;
  *reinterpret_cast<float4 *>(p + W) = r1;
}

// maxpool_grad_op_internal (maxpool_op_internal.h:42-57). in2out[i] is the LAST window, in
// (c, oy, ox) creation order, that contains input i (max_pooling_layer.h:218), and 0 for
// inputs no window contains (strides larger than the window).
__global__ void __launch_bounds__(PT)
maxpool_bwd_kernel(const float *__restrict__ dy, const int32_t *__restrict__ argmax,
                   float *__restrict__ dx, const int total, const PoolGeom g, const ActGrad ag) {
  const int i = blockIdx.x * PT + threadIdx.x;
  if (i >= total) return;
  uint32_t t, xx, yy, c, img;
  g.div_w.divmod(i, t, xx);
  g.div_h.divmod(t, t, yy);
  g.div_c.divmod(t, img, c);
  const int ox = min(g.OW - 1, static_cast<int>(xx) / g.sw);
  const int oy = min(g.OH - 1, static_cast<int>(yy) / g.sh);
  const bool covered = (static_cast<int>(xx) < ox * g.sw + g.pw) &&
                       (static_cast<int>(yy) < oy * g.sh + g.ph);
  const int outi  = covered ? (g.OH * c + oy) * g.OW + ox : 0;
  const int local = (g.H * c + yy) * g.W + xx;  // flat CHW index inside the sample
  const size_t ob = static_cast<size_t>(img) * g.C * g.OH * g.OW;
  float v         = (argmax[ob + outi] == local) ? dy[ob + outi] : 0.0f;
  if (ag.kind != TDH_ACT_NONE) v *= act_grad_factor(ag.kind, ag.y[i]);
  dx[i] = v;
}

// tiny_average_pooling_kernel (average_pooling_layer.h:25-55). Window (oy,ox) exists when it
// lies fully inside the input (init_connection, :270-278); outputs without a window keep
// the empty sum. value = sum * (W[c]*scale) + b[c], in that order.
__global__ void __launch_bounds__(PT)
avepool_fwd_kernel(const float *__restrict__ x, const float *__restrict__ w,
                   const float *__restrict__ b, float *__restrict__ y, const int total,
                   const PoolGeom g, const float scale) {
  const int o = blockIdx.x * PT + threadIdx.x;
  if (o >= total) return;
  uint32_t t, ox, oy, c, img;
  g.div_ow.divmod(o, t, ox);
  g.div_oh.divmod(t, t, oy);
  g.div_c.divmod(t, img, c);
  const int x0 = ox * g.sw, y0 = oy * g.sh;
  float value  = 0.0f;
  if (x0 + g.pw <= g.W && y0 + g.ph <= g.H) {
    const float *in = x + (static_cast<size_t>(img) * g.C + c) * g.H * g.W;
    for (int wy = 0; wy < g.ph; ++wy)
      for (int wx = 0; wx < g.pw; ++wx) value += in[(y0 + wy) * g.W + x0 + wx];
  }
  const float weight = w[c] * scale;
  value *= weight;
  value += b[c];
  y[o] = value;
}

// prev_delta[idx] = (W[c]*scale) * curr_delta[first window containing idx]
// (average_pooling_layer.h:78-85; in2wo[idx][0] is the earliest created window)
__global__ void __launch_bounds__(PT)
avepool_bwd_dx_kernel(const float *__restrict__ dy, const float *__restrict__ w,
                      float *__restrict__ dx, const int total, const PoolGeom g,
                      const float scale, const ActGrad ag) {
  const int i = blockIdx.x * PT + threadIdx.x;
  if (i >= total) return;
  uint32_t t, xx, yy, c, img;
  g.div_w.divmod(i, t, xx);
  g.div_h.divmod(t, t, yy);
  g.div_c.divmod(t, img, c);
  const int ix = xx, iy = yy;
  const int ox = ix < g.pw ? 0 : (ix - g.pw + g.sw) / g.sw;
  const int oy = iy < g.ph ? 0 : (iy - g.ph + g.sh) / g.sh;
  const float weight = w[c] * scale;
  float v = weight * dy[((static_cast<size_t>(img) * g.C + c) * g.OH + oy) * g.OW + ox];
  // the gradient of the activation layer in front of the pool, folded in
  if (ag.kind != TDH_ACT_NONE) v *= act_grad_factor(ag.kind, ag.y[i]);
  dx[i] = v;
}

__device__ __forceinline__ float wave_sum_p(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

// One block per (sample, channel): partial[(img*C + c)*2 + {0,1}] =
//   { sum over windows of dy[o] * (sum of x in the window),  sum of dy[o] }
// (average_pooling_layer.h:87-104, the pair lists regrouped by output)
__global__ void __launch_bounds__(PT)
avepool_bwd_param_kernel(const float *__restrict__ x, const float *__restrict__ dy,
                         float *__restrict__ partial, const PoolGeom g) {
  __shared__ float sm[8];
  const int plane = blockIdx.x;  // img*C + c
  const float *in = x + static_cast<size_t>(plane) * g.H * g.W;
  const float *d  = dy + static_cast<size_t>(plane) * g.OH * g.OW;
  float sw_ = 0.0f, sb = 0.0f;
  for (int o = threadIdx.x; o < g.OH * g.OW; o += PT) {
    const int oy = o / g.OW, ox = o - oy * g.OW;
    const int x0 = ox * g.sw, y0 = oy * g.sh;
    const float dv = d[o];
    sb += dv;
    if (x0 + g.pw <= g.W && y0 + g.ph <= g.H) {
      float win = 0.0f;
      for (int wy = 0; wy < g.ph; ++wy)
        for (int wx = 0; wx < g.pw; ++wx) win += in[(y0 + wy) * g.W + x0 + wx];
      sw_ += win * dv;
    }
  }
  sw_ = wave_sum_p(sw_);
  sb  = wave_sum_p(sb);
  if ((threadIdx.x & 63) == 0) {
    sm[(threadIdx.x >> 6) * 2]     = sw_;
    sm[(threadIdx.x >> 6) * 2 + 1] = sb;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    partial[plane * 2]     = (sm[0] + sm[2]) + (sm[4] + sm[6]);
    partial[plane * 2 + 1] = (sm[1] + sm[3]) + (sm[5] + sm[7]);
  }
}

// dW[c] (+)= scale * sum_img partial_w, db[c] (+)= sum_img partial_b, samples in order
__global__ void __launch_bounds__(PT)
avepool_bwd_param_reduce_kernel(const float *__restrict__ partial, const int batch, const int C,
                                const float scale, float *__restrict__ dw,
                                float *__restrict__ db, const int accumulate) {
  const int c = blockIdx.x * PT + threadIdx.x;
  if (c >= C) return;
  float mw = 0.0f, mb = 0.0f;
  for (int s = 0; s < batch; ++s) {
    mw += partial[(s * C + c) * 2] * scale;
    mb += partial[(s * C + c) * 2 + 1];
  }
  if (dw) dw[c] = accumulate ? dw[c] + mw : mw;
  if (db) db[c] = accumulate ? db[c] + mb : mb;
}

// 2x2 windows at stride 2 that tile the input exactly, rows of whole 16-byte words
bool is_2x2_tiling(const PoolGeom &g) {
  return g.pw == 2 && g.ph == 2 && g.sw == 2 && g.sh == 2 && g.W % 4 == 0 && g.H % 2 == 0 &&
         g.OW * 2 == g.W && g.OH * 2 == g.H;
}
bool aligned8(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 7u) == 0; }
bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace

bool maxpool_scatters_from_fc(const tdh_pool_desc *d, PoolScatter *geom) {
  const PoolGeom g = make_geom(d);
  if (!is_2x2_tiling(g)) return false;
  geom->W = g.W; geom->OW = g.OW; geom->OH = g.OH;
  return true;
}

int maxpool_fwd(const tdh_pool_desc *d, int batch, const float *x, float *y, int32_t *argmax,
                float *act_out, int act_kind) {
  const PoolGeom g = make_geom(d);
  const long total = static_cast<long>(batch) * g.C * g.OH * g.OW;
  const bool fast  = is_2x2_tiling(g) && aligned16(x) && aligned8(y) && aligned8(argmax) && aligned8(act_out) &&
                    total / 2 < (1L << 31);
  // a split reduction left for the reader of x: taken by the 2x2 kernel, else finished first
  const size_t in_total = static_cast<size_t>(batch) * g.C * g.H * g.W;
  const bool take = ctx().split_sum_left && fast && total > 0 && left_split_sum().out == x &&
                    left_split_sum().stride == in_total;
  if (!take) TDH_TRY(finish_split_sum());
  if (total <= 0) return TDH_OK;
  if (take) {
    const SplitSum sum   = left_split_sum();
    ctx().split_sum_left = false;
    ProfScope prof(act_out ? "maxpool_fwd_act_sum" : "maxpool_fwd_sum",
                   4.0 * in_total * (sum.splits + 1) + (act_out ? 12.0 : 8.0) * total, WORK_BYTE);
    const int pairs = static_cast<int>(total / 2);
    TDH_LAUNCH(maxpool2x2_fwd_kernel<true>, dim3(ceil_div(pairs, PT)), dim3(PT), 0, ctx().stream, x, y, argmax,
               pairs, g.W, g.OW / 2, FastDiv(g.OW / 2), g.C * g.H, act_out, act_kind, sum);
    TDH_LAUNCH_CHECK();
    return TDH_OK;
  }
  ProfScope prof(act_out ? "maxpool_fwd_act" : "maxpool_fwd",
                 4.0 * batch * g.C * g.H * g.W + (act_out ? 12.0 : 8.0) * total, WORK_BYTE);
  if (fast) {
    const int pairs = static_cast<int>(total / 2);
    TDH_LAUNCH(maxpool2x2_fwd_kernel<false>, dim3(ceil_div(pairs, PT)), dim3(PT), 0, ctx().stream, x,
                       y, argmax, pairs, g.W, g.OW / 2, FastDiv(g.OW / 2), g.C * g.H, act_out, act_kind,
                       SplitSum());
    TDH_LAUNCH_CHECK();
    return TDH_OK;
  }
  TDH_LAUNCH(maxpool_fwd_kernel, dim3(ceil_div(total, PT)), dim3(PT), 0, ctx().stream, x,
                     y, argmax, static_cast<int>(total), g, act_out, act_kind);
  TDH_LAUNCH_CHECK();
  return TDH_OK;
}

int maxpool_bwd(const tdh_pool_desc *d, int batch, const float *dy, const int32_t *argmax,
                float *dx, ActGrad ag, const float *pooled_y) {
  const PoolGeom g = make_geom(d);
  const long total = static_cast<long>(batch) * g.C * g.H * g.W;
  const bool fast  = is_2x2_tiling(g) && aligned16(dx) && aligned8(dy) && aligned8(argmax) &&
                    total / 8 < (1L << 31) && (ag.kind == TDH_ACT_NONE || aligned16(ag.y));
  // a split reduction left for the reader of dy: taken by the 2x2 kernel, else finished first
  const size_t out_total = static_cast<size_t>(batch) * g.C * g.OH * g.OW;
  const bool take = ctx().split_sum_left && fast && total > 0 && g.OH > 0 && g.OW > 0 &&
                    left_split_sum().out == dy && left_split_sum().stride == out_total;
  if (!take) TDH_TRY(finish_split_sum());
  TDH_CHECK_ARG(g.OH > 0 && g.OW > 0, "maxpool backward: empty output");
  // (the pool's own output stands in for the activation output where a gradient lands)
  const float *py = (ag.kind != TDH_ACT_NONE && pooled_y && aligned8(pooled_y)) ? pooled_y : nullptr;
  if (take) {
    const SplitSum sum   = left_split_sum();
    ctx().split_sum_left = false;
    ProfScope prof(ag.kind != TDH_ACT_NONE ? "maxpool_bwd_act_sum" : "maxpool_bwd_sum",
                   4.0 * out_total * (sum.splits + 2 + (sum.ag.kind != TDH_ACT_NONE)) +
                     (ag.kind == TDH_ACT_NONE ? 4.0 : py ? 5.0 : 8.0) * total, WORK_BYTE);
    const int pairs = static_cast<int>(total / 8);
    TDH_LAUNCH(maxpool2x2_bwd_kernel<true>, dim3(ceil_div(pairs, PT)), dim3(PT), 0, ctx().stream, dy, argmax, dx,
               pairs, g.W, g.OW / 2, FastDiv(g.OW / 2), g.C * g.H, ag, sum, py);
    TDH_LAUNCH_CHECK();
    return TDH_OK;
  }
  ProfScope prof(ag.kind != TDH_ACT_NONE ? "maxpool_bwd_act" : "maxpool_bwd",
                 8.0 * batch * g.C * g.OH * g.OW + (ag.kind == TDH_ACT_NONE ? 4.0 : (fast && py) ? 5.0 : 8.0) * total, WORK_BYTE);
  if (fast) {
    const int pairs = static_cast<int>(total / 8);
    TDH_LAUNCH(maxpool2x2_bwd_kernel<false>, dim3(ceil_div(pairs, PT)), dim3(PT), 0, ctx().stream, dy,
                       argmax, dx, pairs, g.W, g.OW / 2, FastDiv(g.OW / 2), g.C * g.H, ag, SplitSum(), py);
    TDH_LAUNCH_CHECK();
    return TDH_OK;
  }
  TDH_LAUNCH(maxpool_bwd_kernel, dim3(ceil_div(total, PT)), dim3(PT), 0, ctx().stream, dy,
                     argmax, dx, static_cast<int>(total), g, ag);
  TDH_LAUNCH_CHECK();
  return TDH_OK;
}

// average_pooling_layer's constructor throws unless the input is a multiple of the window
// (average_pooling_layer.h:216-218)
static int check_avepool(const tdh_pool_desc *d) {
  TDH_CHECK_ARG(d->in_w % d->pool_w == 0 && d->in_h % d->pool_h == 0,
                "average pooling: input %dx%d is not a multiple of the window %dx%d", d->in_w,
                d->in_h, d->pool_w, d->pool_h);
  return TDH_OK;
}

int avepool_fwd(const tdh_pool_desc *d, int batch, const float *x, const float *w, const float *b,
                float *y) {
  TDH_TRY(check_avepool(d));
  const PoolGeom g = make_geom(d);
  const long total = static_cast<long>(batch) * g.C * g.OH * g.OW;
  if (total <= 0) return TDH_OK;
  const float scale = 1.0f / static_cast<float>(d->pool_w * d->pool_h);
  ProfScope prof("avepool_fwd", 4.0 * batch * g.C * g.H * g.W + 4.0 * total, WORK_BYTE);
  TDH_LAUNCH(avepool_fwd_kernel, dim3(ceil_div(total, PT)), dim3(PT), 0, ctx().stream, x,
                     w, b, y, static_cast<int>(total), g, scale);
  TDH_LAUNCH_CHECK();
  return TDH_OK;
}

size_t avepool_workspace_bytes(const tdh_pool_desc *d, int batch) {
  return ws_align(static_cast<size_t>(batch) * d->in_c * 2 * sizeof(float));
}

int avepool_bwd(const tdh_pool_desc *d, int batch, const float *x, const float *w, const float *dy,
                float *dx, float *dw, float *db, int accumulate, ActGrad ag) {
  TDH_TRY(check_avepool(d));
  const PoolGeom g = make_geom(d);
  // Every input element must lie in at least one window that maps to an existing output;
  // the reference dereferences in2wo[idx][0] unconditionally.
  for (int axis = 0; axis < 2; ++axis) {
    const int len = axis ? g.H : g.W, pool = axis ? g.ph : g.pw, stride = axis ? g.sh : g.sw;
    const int outs = axis ? g.OH : g.OW;
    for (int i = 0; i < len; ++i) {
      const int o = i < pool ? 0 : (i - pool + stride) / stride;
      const bool ok = o * stride <= i && o * stride + pool <= len && o < outs;
      TDH_CHECK_ARG(ok, "average pooling backward: input %s %d is covered by no window",
                    axis ? "row" : "column", i);
    }
  }
  const float scale = 1.0f / static_cast<float>(d->pool_w * d->pool_h);
  if (dx) {
    const long total = static_cast<long>(batch) * g.C * g.H * g.W;
    ProfScope prof(ag.kind != TDH_ACT_NONE ? "avepool_bwd_dx_act" : "avepool_bwd_dx",
                   4.0 * batch * g.C * g.OH * g.OW + (ag.kind != TDH_ACT_NONE ? 8.0 : 4.0) * total, WORK_BYTE);
    TDH_LAUNCH(avepool_bwd_dx_kernel, dim3(ceil_div(total, PT)), dim3(PT), 0, ctx().stream,
                       dy, w, dx, static_cast<int>(total), g, scale, ag);
    TDH_LAUNCH_CHECK();
  }
  if (dw || db) {
    void *ws = nullptr;
    TDH_TRY(ws_take(static_cast<size_t>(batch) * g.C * 2 * sizeof(float), &ws));
    ProfScope prof("avepool_bwd_param", 4.0 * batch * g.C * (g.H * g.W + g.OH * g.OW), WORK_BYTE);
    TDH_LAUNCH(avepool_bwd_param_kernel, dim3(batch * g.C), dim3(PT), 0, ctx().stream, x,
                       dy, static_cast<float *>(ws), g);
    TDH_LAUNCH_CHECK();
    TDH_LAUNCH(avepool_bwd_param_reduce_kernel, dim3(ceil_div(g.C, PT)), dim3(PT), 0,
                       ctx().stream, static_cast<const float *>(ws), batch, g.C, scale, dw, db,
                       accumulate);
    TDH_LAUNCH_CHECK();
  }
  return TDH_OK;
}

}  // namespace tdh
