// elementwise.hip — bandwidth-bound kernels: fills, activations and their gradients,
// loss gradients, optimizer updates and the fixed-order reductions used for bias
// gradients. One pass over each array, 16-byte accesses where alignment allows.
// Built with -ffp-contract=off so that a*b+c rounds twice, as in the scalar reference.
#include <algorithm>
#include <cfloat>
#include <vector>

#include "common.h"

namespace tdh {

namespace {

constexpr int EW_THREADS = 256;

inline int ew_blocks(size_t work_items) {
  const size_t want = ceil_div_sz(work_items, EW_THREADS);
  const size_t cap  = 256 * 16;  // enough waves to cover HBM latency on 256 CUs
  return static_cast<int>(want < 1 ? 1 : (want > cap ? cap : want));
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// out[i] = Op::apply(a[i], b[i], prm); n4 float4 groups when vec, scalar tail after
template <class Op, bool HAS_B>
__global__ void __launch_bounds__(EW_THREADS)
map_kernel(const float *__restrict__ a, const float *__restrict__ b, float *__restrict__ out,
           const size_t n4, const size_t n, const typename Op::Params prm) {
  const size_t stride = static_cast<size_t>(gridDim.x) * EW_THREADS;
  const size_t t0     = static_cast<size_t>(blockIdx.x) * EW_THREADS + threadIdx.x;
  for (size_t i = t0; i < n4; i += stride) {
    const float4 va = reinterpret_cast<const float4 *>(a)[i];
    float4 vb       = make_float4(0.f, 0.f, 0.f, 0.f);
    if (HAS_B) vb = reinterpret_cast<const float4 *>(b)[i];
    float4 r;
    r.x = Op::apply(va.x, vb.x, prm);
    r.y = Op::apply(va.y, vb.y, prm);
    r.z = Op::apply(va.z, vb.z, prm);
    r.w = Op::apply(va.w, vb.w, prm);
    reinterpret_cast<float4 *>(out)[i] = r;
  }
  for (size_t j = n4 * 4 + t0; j < n; j += stride)
    out[j] = Op::apply(a[j], HAS_B ? b[j] : 0.0f, prm);
}

template <class Op, bool HAS_B>
int launch_map(const float *a, const float *b, float *out, size_t n,
               const typename Op::Params &prm, const char *tag) {
  ProfScope prof(tag, (HAS_B ? 12.0 : 8.0) * n, WORK_BYTE);
  const bool vec  = aligned16(a) && aligned16(out) && (!HAS_B || aligned16(b));
  const size_t n4 = vec ? n / 4 : 0;
  TDH_LAUNCH((map_kernel<Op, HAS_B>), dim3(ew_blocks(vec ? n4 + 3 : n)), dim3(EW_THREADS),
                     0, ctx().stream, a, b, out, n4, n, prm);
  TDH_LAUNCH_CHECK();
  return TDH_OK;
}

struct NoParams {};

// forward activations: tanh_layer.h:24-28, relu_layer.h:25-29, sigmoid_layer.h:24-28
struct TanhFwd {
  typedef NoParams Params;
  static __device__ __forceinline__ float apply(float x, float, Params) { return tanhf(x); }
};
struct ReluFwd {
  typedef NoParams Params;
  static __device__ __forceinline__ float apply(float x, float, Params) {
    return x > 0.0f ? x : 0.0f;  // std::max(float_t(0), x): NaN maps to 0
  }
};
struct SigmoidFwd {
  typedef NoParams Params;
  static __device__ __forceinline__ float apply(float x, float, Params) {
    return 1.0f / (1.0f + expf(-x));
  }
};
// backward activations on the OUTPUT y: tanh_layer.h:30-38, relu_layer.h:31-39,
// sigmoid_layer.h:30-38.  a = y, b = dy
struct TanhBwd {
  typedef NoParams Params;
  static __device__ __forceinline__ float apply(float y, float dy, Params) {
    return dy * (1.0f - y * y);
  }
};
struct ReluBwd {
  typedef NoParams Params;
  static __device__ __forceinline__ float apply(float y, float dy, Params) {
    return dy * (y > 0.0f ? 1.0f : 0.0f);
  }
};
struct SigmoidBwd {
  typedef NoParams Params;
  static __device__ __forceinline__ float apply(float y, float dy, Params) {
    return dy * y * (1.0f - y);
  }
};
// parameterised and remaining pointwise activations; Params = the layer's constructor
// arguments. Forward: a = x. Backward: a = y (or x where the reference reads x), b = dy.
struct Act2 {
  float p0, p1;
};
struct LeakyReluFwd {  // leaky_relu_layer.h:74-78, p0 = epsilon
  typedef Act2 Params;
  static __device__ __forceinline__ float apply(float x, float, Params p) { return x > 0.0f ? x : p.p0 * x; }
};
struct LeakyReluBwd {  // leaky_relu_layer.h:80-88
  typedef Act2 Params;
  static __device__ __forceinline__ float apply(float y, float dy, Params p) { return dy * (y > 0.0f ? 1.0f : p.p0); }
};
struct EluFwd {  // elu_layer.h:37-42, p0 = alpha
  typedef Act2 Params;
  static __device__ __forceinline__ float apply(float x, float, Params p) {
    return x < 0.0f ? (p.p0 * (expf(x) - 1.0f)) : x;
  }
};
struct EluBwd {  // elu_layer.h:44-52
  typedef Act2 Params;
  static __device__ __forceinline__ float apply(float y, float dy, Params p) { return dy * (y > 0.0f ? 1.0f : (p.p0 + y)); }
};
struct SeluFwd {  // selu_layer.h:82-88, p0 = lambda, p1 = alpha
  typedef Act2 Params;
  static __device__ __forceinline__ float apply(float x, float, Params p) {
    return p.p0 * (x > 0.0f ? x : p.p1 * (expf(x) - 1.0f));
  }
};
struct SeluBwd {  // selu_layer.h:90-99: reads x; the product is a double one in the reference
  typedef Act2 Params;
  static __device__ __forceinline__ float apply(float x, float dy, Params p) {
    return static_cast<float>(dy * p.p0 * (x > 0.0f ? 1.0 : static_cast<double>(p.p1 * expf(x))));
  }
};
struct SoftplusFwd {  // softplus_layer.h:84-90, p0 = beta, p1 = threshold
  typedef Act2 Params;
  static __device__ __forceinline__ float apply(float x, float, Params p) {
    const float betain = p.p0 * x;
    return betain > p.p1 ? x : (1.0f / p.p0) * log1pf(expf(betain));
  }
};
struct SoftplusBwd {  // softplus_layer.h:92-102
  typedef Act2 Params;
  static __device__ __forceinline__ float apply(float y, float dy, Params p) {
    const float betaout = p.p0 * y;
    const float exp_bo  = expf(betaout);
    return betaout > p.p1 ? dy : dy * (exp_bo - 1.0f) / exp_bo;
  }
};
struct SoftsignFwd {  // softsign_layer.h:24-28 (double arithmetic: `1.0 + std::abs(x)`)
  typedef Act2 Params;
  static __device__ __forceinline__ float apply(float x, float, Params) {
    return static_cast<float>(x / (1.0 + fabsf(x)));
  }
};
struct SoftsignBwd {  // softsign_layer.h:30-40: reads x
  typedef Act2 Params;
  static __device__ __forceinline__ float apply(float x, float dy, Params) {
    const double d = 1.0 + fabsf(x);
    return static_cast<float>(dy / (d * d));
  }
};
struct AsinhFwd {  // asinh_layer.h:24-28
  typedef Act2 Params;
  static __device__ __forceinline__ float apply(float x, float, Params) { return asinhf(x); }
};
struct AsinhBwd {  // asinh_layer.h:30-38
  typedef Act2 Params;
  static __device__ __forceinline__ float apply(float y, float dy, Params) { return dy / coshf(y); }
};
struct TanhP1m2Fwd {  // tanh_p1m2_layer.h:24-30
  typedef Act2 Params;
  static __device__ __forceinline__ float apply(float x, float, Params) {
    const float ep = expf(x);
    return ep / (ep + (1.0f / ep));
  }
};
struct TanhP1m2Bwd {  // tanh_p1m2_layer.h:32-40
  typedef Act2 Params;
  static __device__ __forceinline__ float apply(float y, float dy, Params) { return dy * (2.0f * y * (1.0f - y)); }
};
// loss gradients: loss_function.h:28-36, :143-150, :120-128.  a = y, b = t
struct MseGrad {
  struct Params {
    float factor;
  };
  static __device__ __forceinline__ float apply(float y, float t, Params p) {
    return p.factor * (y - t);
  }
};
struct CeMultiGrad {
  typedef NoParams Params;
  static __device__ __forceinline__ float apply(float y, float t, Params) { return -t / y; }
};
struct CeGrad {
  typedef NoParams Params;
  static __device__ __forceinline__ float apply(float y, float t, Params) {
    return (y - t) / (y * (1.0f - y));
  }
};

__global__ void __launch_bounds__(EW_THREADS)
fill_zero_kernel(uint32_t *__restrict__ p, const size_t n4, const size_t n) {
  const size_t stride = static_cast<size_t>(gridDim.x) * EW_THREADS;
  const size_t t0     = static_cast<size_t>(blockIdx.x) * EW_THREADS + threadIdx.x;
  for (size_t i = t0; i < n4; i += stride) reinterpret_cast<uint4 *>(p)[i] = make_uint4(0, 0, 0, 0);
  for (size_t j = n4 * 4 + t0; j < n; j += stride) p[j] = 0u;
}

// plain device-to-device copy: one 16-byte load and store per lane and iteration
__global__ void __launch_bounds__(EW_THREADS)
copy_kernel(const uint32_t *__restrict__ src, uint32_t *__restrict__ dst, const size_t n4,
            const size_t n) {
  const size_t stride = static_cast<size_t>(gridDim.x) * EW_THREADS;
  const size_t t0     = static_cast<size_t>(blockIdx.x) * EW_THREADS + threadIdx.x;
  for (size_t i = t0; i < n4; i += stride)
    reinterpret_cast<uint4 *>(dst)[i] = reinterpret_cast<const uint4 *>(src)[i];
  for (size_t j = n4 * 4 + t0; j < n; j += stride) dst[j] = src[j];
}

// ------------------------------------------------------------------ softmax
// One wave64 per sample row; reductions by butterfly shuffles (every lane ends with the
// same value, summed in a fixed tree).
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}

// softmax_layer.h:24-34: y = exp(x - max) / sum
__global__ void __launch_bounds__(EW_THREADS)
softmax_fwd_kernel(const float *__restrict__ x, float *__restrict__ y, const int batch,
                   const int len) {
  const int row  = blockIdx.x * (EW_THREADS / 64) + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (row >= batch) return;
  const float *xr = x + static_cast<size_t>(row) * len;
  float *yr       = y + static_cast<size_t>(row) * len;
  float m         = -FLT_MAX;
  for (int j = lane; j < len; j += 64) m = fmaxf(m, xr[j]);
  m       = wave_max(m);
  float s = 0.0f;
  for (int j = lane; j < len; j += 64) {
    const float e = expf(xr[j] - m);
    yr[j]         = e;
    s += e;
  }
  s = wave_sum(s);
  for (int j = lane; j < len; j += 64) yr[j] = yr[j] / s;
}

// softmax_layer.h:36-55: dx_j = sum_k dy_k * df_k with df_j = y_j*(1 - y_j), df_k = -y_k*y_j,
// that is dx_j = dy_j*y_j*(1 - y_j) - y_j * sum_{k != j} dy_k*y_k. The reference adds the terms
// one by one, so a term that dwarfs the others (a saturated row: one y next to 1, the rest
// 1e-20) does not disturb the sums it is not part of. In one pass over the row the same is
// had by leaving the largest term t_m = dy_m*y_m out of the row sum (kept in double):
// sum_{k != m} is that sum itself, and sum_{k != j} = that sum - t_j + t_m for the others,
// where t_m dominates whatever the subtraction lost.
__global__ void __launch_bounds__(EW_THREADS)
softmax_bwd_kernel(const float *__restrict__ y, const float *__restrict__ dy,
                   float *__restrict__ dx, const int batch, const int len) {
  const int row  = blockIdx.x * (EW_THREADS / 64) + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (row >= batch) return;
  const float *yr  = y + static_cast<size_t>(row) * len;
  const float *dyr = dy + static_cast<size_t>(row) * len;
  // the largest |dy_k*y_k| of the row; of equal ones the first
  float big = -1.0f;
  int m     = len;
  for (int j = lane; j < len; j += 64) {
    const float t = fabsf(dyr[j] * yr[j]);
    if (t > big) { big = t; m = j; }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float ob = __shfl_xor(big, off, 64);
    const int om   = __shfl_xor(m, off, 64);
    if (ob > big || (ob == big && om < m)) { big = ob; m = om; }
  }
  double rest_m = 0.0;  // sum over k != m
  for (int j = lane; j < len; j += 64)
    if (j != m) rest_m += static_cast<double>(dyr[j]) * static_cast<double>(yr[j]);
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) rest_m += __shfl_xor(rest_m, off, 64);
  const double tm = m < len ? static_cast<double>(dyr[m]) * static_cast<double>(yr[m]) : 0.0;
  for (int j = lane; j < len; j += 64) {
    const float yj = yr[j], dj = dyr[j];
    const double own  = static_cast<double>(dj) * static_cast<double>(yj * (1.0f - yj));
    const double rest = j == m ? rest_m : rest_m - static_cast<double>(dj) * static_cast<double>(yj) + tm;
    dx[static_cast<size_t>(row) * len + j] = static_cast<float>(own - static_cast<double>(yj) * rest);
  }
}

// softmax backward of cross_entropy_multiclass::df (= -t/y) in closed form:
// dz_j = y_j * (-t_j/y_j + sum_k t_k) = y_j * sum(t) - t_j, as one fused multiply-add in every
// kernel that computes it (left to the compiler, one kernel fused it and another did not)
__global__ void __launch_bounds__(EW_THREADS)
softmax_xent_grad_kernel(const float *__restrict__ y, const float *__restrict__ t,
                         float *__restrict__ dz, const int batch, const int len) {
  const int row  = blockIdx.x * (EW_THREADS / 64) + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (row >= batch) return;
  const float *yr = y + static_cast<size_t>(row) * len;
  const float *tr = t + static_cast<size_t>(row) * len;
  float st        = 0.0f;
  for (int j = lane; j < len; j += 64) st += tr[j];
  st = wave_sum(st);
  for (int j = lane; j < len; j += 64) dz[static_cast<size_t>(row) * len + j] = fmaf(yr[j], st, -tr[j]);
}

// softmax forward and the gradient above in one pass over the row: the values and their order
// of evaluation are those of softmax_fwd_kernel followed by softmax_xent_grad_kernel
__global__ void __launch_bounds__(EW_THREADS)
softmax_fwd_xent_kernel(const float *__restrict__ x, const float *__restrict__ t,
                        float *__restrict__ y, float *__restrict__ dz, const int batch,
                        const int len) {
  const int row  = blockIdx.x * (EW_THREADS / 64) + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (row >= batch) return;
  const float *xr = x + static_cast<size_t>(row) * len;
  const float *tr = t + static_cast<size_t>(row) * len;
  float *yr       = y + static_cast<size_t>(row) * len;
  float *dr       = dz + static_cast<size_t>(row) * len;
  float m         = -FLT_MAX;
  for (int j = lane; j < len; j += 64) m = fmaxf(m, xr[j]);
  m       = wave_max(m);
  float s = 0.0f, st = 0.0f;
  for (int j = lane; j < len; j += 64) {
    const float e = expf(xr[j] - m);
    yr[j]         = e;
    s += e;
    st += tr[j];
  }
  s  = wave_sum(s);
  st = wave_sum(st);
  for (int j = lane; j < len; j += 64) {
    const float v = yr[j] / s;
    yr[j]         = v;
    dr[j]         = fmaf(v, st, -tr[j]);
  }
}

// --------------------------------------------------------------- optimizers
// tiny_dnn/optimizers/optimizer.h; g = merged * grad_scale is layer::update_weight's
// diff (tiny_dnn/layers/layer.h:668-673). Scalars that the reference derives once per
// call from its float members (1 - b1_t, ...) arrive precomputed in float.
struct OptScalars {
  float alpha, lambda, mu, b1, b2, eps, omb1, omb2, omb1t, omb2t, grad_scale;
  double adamax_lr;  // alpha / (1.0 - b1_t), evaluated in double as the reference does
};

template <int KIND>
__device__ __forceinline__ void opt_one(float g, float &w, float &s0, float &s1,
                                        const OptScalars &p) {
  g *= p.grad_scale;
  if (KIND == TDH_OPT_SGD) {  // :185-188
    w = w - p.alpha * (g + p.lambda * w);
  } else if (KIND == TDH_OPT_MOMENTUM) {  // :205-213
    const float V = p.mu * s0 - p.alpha * (g + w * p.lambda);
    w += V;
    s0 = V;
  } else if (KIND == TDH_OPT_NESTEROV) {  // :231-239
    const float V = p.mu * s0 - p.alpha * (g + w * p.lambda);
    w += (-p.mu) * s0 + (1 + p.mu) * V;
    s0 = V;
  } else if (KIND == TDH_OPT_ADAM) {  // :112-127, eps inside the square root
    s0 = p.b1 * s0 + p.omb1 * g;
    s1 = p.b2 * s1 + p.omb2 * g * g;
    w -= p.alpha * (s0 / p.omb1t) / sqrtf((s1 / p.omb2t) + p.eps);
  } else if (KIND == TDH_OPT_ADAGRAD) {  // :60-66
    s0 += g * g;
    w -= p.alpha * g / (sqrtf(s0) + p.eps);
  } else if (KIND == TDH_OPT_RMSPROP) {  // :81-88
    s0 = p.mu * s0 + (1 - p.mu) * g * g;
    w -= p.alpha * g / sqrtf(s0 + p.eps);
  } else if (KIND == TDH_OPT_ADAMAX) {  // :153-165
    s0 = p.b1 * s0 + p.omb1 * g;
    s1 = fmaxf(p.b2 * s1, fabsf(g));
    w  = static_cast<float>(static_cast<double>(w) -
                           p.adamax_lr * static_cast<double>(s0 / (s1 + p.eps)));
  }
}

template <int KIND, int NSTATE>
__global__ void __launch_bounds__(EW_THREADS)
opt_kernel(const float *__restrict__ g, float *__restrict__ w, float *__restrict__ s0,
           float *__restrict__ s1, const size_t n4, const size_t n, const OptScalars p) {
  const size_t stride = static_cast<size_t>(gridDim.x) * EW_THREADS;
  const size_t t0     = static_cast<size_t>(blockIdx.x) * EW_THREADS + threadIdx.x;
  for (size_t i = t0; i < n4; i += stride) {
    const float4 vg = reinterpret_cast<const float4 *>(g)[i];
    float4 vw       = reinterpret_cast<float4 *>(w)[i];
    float4 v0       = make_float4(0.f, 0.f, 0.f, 0.f), v1 = v0;
    if (NSTATE >= 1) v0 = reinterpret_cast<float4 *>(s0)[i];
    if (NSTATE >= 2) v1 = reinterpret_cast<float4 *>(s1)[i];
    opt_one<KIND>(vg.x, vw.x, v0.x, v1.x, p);
    opt_one<KIND>(vg.y, vw.y, v0.y, v1.y, p);
    opt_one<KIND>(vg.z, vw.z, v0.z, v1.z, p);
    opt_one<KIND>(vg.w, vw.w, v0.w, v1.w, p);
    reinterpret_cast<float4 *>(w)[i] = vw;
    if (NSTATE >= 1) reinterpret_cast<float4 *>(s0)[i] = v0;
    if (NSTATE >= 2) reinterpret_cast<float4 *>(s1)[i] = v1;
  }
  for (size_t j = n4 * 4 + t0; j < n; j += stride) {
    float ww = w[j], a = 0.0f, b = 0.0f;
    if (NSTATE >= 1) a = s0[j];
    if (NSTATE >= 2) b = s1[j];
    opt_one<KIND>(g[j], ww, a, b, p);
    w[j] = ww;
    if (NSTATE >= 1) s0[j] = a;
    if (NSTATE >= 2) s1[j] = b;
  }
}

template <int KIND, int NSTATE>
int launch_opt(size_t n, const float *g, float *w, float *s0, float *s1, const OptScalars &p) {
  static const char *const tags[] = {"opt_sgd", "opt_momentum", "opt_adam", "opt_adagrad",
                                     "opt_rmsprop", "opt_adamax", "opt_nesterov"};
  ProfScope prof(tags[KIND], (12.0 + 8.0 * NSTATE) * n, WORK_BYTE);
  const bool vec = aligned16(g) && aligned16(w) && (NSTATE < 1 || aligned16(s0)) &&
                   (NSTATE < 2 || aligned16(s1));
  const size_t n4 = vec ? n / 4 : 0;
  TDH_LAUNCH((opt_kernel<KIND, NSTATE>), dim3(ew_blocks(vec ? n4 + 3 : n)),
                     dim3(EW_THREADS), 0, ctx().stream, g, w, s0, s1, n4, n, p);
  TDH_LAUNCH_CHECK();
  return TDH_OK;
}

// The packed copies of element e = (co*C + ci)*rs + t of a convolution's weight tensor
__device__ __forceinline__ void opt_pack_store(const OptTensor &t, const uint32_t e, float v) {
  const uint32_t tap = e % t.rs, pair = e / t.rs;
  const uint32_t co = pair / t.C, ci = pair - co * t.C;
  if (t.tbl && !t.tbl[ci * t.Kc + co]) v = 0.0f;
  t.wp_fwd[(static_cast<size_t>(tap) * t.C + ci) * t.Kc + co] = v;
  t.wp_dx[(static_cast<size_t>(t.rs - 1 - tap) * t.Kc + co) * t.C + ci] = v;
}

// Multi-tensor form: block b works on tensor j = the table entry whose block range holds b.
template <int KIND, int NSTATE>
__global__ void __launch_bounds__(EW_THREADS)
opt_multi_kernel(const OptTensor *__restrict__ table, const int n_tensors, OptScalars p,
                 float b1_t, float b2_t, const float *powers_in, float *powers_out, const int advance,
                 const int zero_grad, const OptPending pend, const OptIndex idx) {
  if (powers_in) {
    b1_t = powers_in[0];
    b2_t = powers_in[1];
    // The device copy of the powers advances as n_tensors update() calls would
    // (optimizer.h:125-126), into the other of two buffers: nobody reads that one during this
    // launch, so no workgroup has to wait for another. advance: 1 = b1_t only (adamax), 2 = both.
    if (blockIdx.x == 0 && threadIdx.x == 0) {
      float q1 = b1_t, q2 = b2_t;
      for (int i = 0; i < n_tensors; ++i) {
        if (advance >= 1) q1 *= p.b1;
        if (advance == 2) q2 *= p.b2;
      }
      powers_out[0] = q1;
      powers_out[1] = q2;
    }
  }
  int j = 0, pj = -1;
  if (idx.n) {
    // first blocks ascend, and those past the last tensor compare false
#pragma unroll
    for (int k = 1; k < OPT_INDEX_MAX; ++k) j += idx.first_block[k] <= blockIdx.x ? 1 : 0;
    pj = idx.pend_of[j];
  } else {
    while (j + 1 < n_tensors && table[j + 1].first_block <= blockIdx.x) ++j;
  }
  const OptTensor t = table[j];
  // the reference multiplies b1_t by b1 after every update() call (optimizer.h:125-126)
  float p1 = b1_t, p2 = b2_t;
  for (int i = 0; i < j; ++i) {
    p1 *= p.b1;
    p2 *= p.b2;
  }
  p.omb1t     = 1.0f - p1;
  p.omb2t     = 1.0f - p2;
  p.adamax_lr = static_cast<double>(p.alpha) / (1.0 - static_cast<double>(p1));
  const uint32_t beg = (blockIdx.x - t.first_block) * t.block_elems;
  const uint32_t end = min(t.n, beg + t.block_elems);
  // tensors come from separate allocations (256-byte aligned): 16-byte accesses are safe
  const uint32_t end4 = beg + ((end - beg) & ~3u);
  // K-split partial slices of this gradient that nobody has added up yet: the summation tree of
  // splitk_reduce_block (eight 32-lane groups each add every eighth slice in order, the group
  // sums are added in group order), four consecutive elements a lane
  __shared__ float pending_sum[8][OPT_SUM_ELEMS_PER_BLOCK];
  if (!idx.n)
    for (int k = 0; k < pend.n; ++k)
      if (pend.sum[k].g == t.g) pj = k;
  // (the host hands over pending sums only for tensors with the small blocks; a tensor with
  // large blocks would index pending_sum out of bounds, so it is left alone here)
  if (t.block_elems != OPT_SUM_ELEMS_PER_BLOCK) pj = -1;
  if (pj >= 0) {
    const OptPendingSum ps = pend.sum[pj];
    constexpr uint32_t VEC = OPT_SUM_ELEMS_PER_BLOCK / 32;  // consecutive elements a lane adds up
    const uint32_t o = threadIdx.x & 31, grp = threadIdx.x >> 5, i0 = beg + VEC * o;
    float s4[VEC];
#pragma unroll
    for (uint32_t c = 0; c < VEC; ++c) s4[c] = 0.0f;
    if (VEC == 4 && i0 + 4 <= end && (ps.mn & 3u) == 0) {
      uint32_t z = grp;
      for (; z + 56 < ps.splits; z += 64) {
        float4 v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u)
          v[u] = *reinterpret_cast<const float4 *>(ps.partial + static_cast<size_t>(z + 8 * u) * ps.mn + i0);
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          s4[0] += v[u].x; s4[1 % VEC] += v[u].y; s4[2 % VEC] += v[u].z; s4[3 % VEC] += v[u].w;
        }
      }
      for (; z < ps.splits; z += 8) {
        const float4 v = *reinterpret_cast<const float4 *>(ps.partial + static_cast<size_t>(z) * ps.mn + i0);
        s4[0] += v.x; s4[1 % VEC] += v.y; s4[2 % VEC] += v.z; s4[3 % VEC] += v.w;
      }
    } else {
#pragma unroll
      for (uint32_t c = 0; c < VEC; ++c) {
        if (i0 + c >= end) break;
        const float *col = ps.partial + i0 + c;
        uint32_t z = grp;
        for (; z + 56 < ps.splits; z += 64) {  // eight slices per trip: the loads are issued together
          float v[8];
#pragma unroll
          for (int u = 0; u < 8; ++u) v[u] = col[static_cast<size_t>(z + 8 * u) * ps.mn];
#pragma unroll
          for (int u = 0; u < 8; ++u) s4[c] += v[u];
        }
        for (; z < ps.splits; z += 8) s4[c] += col[static_cast<size_t>(z) * ps.mn];
      }
    }
#pragma unroll
    for (uint32_t c = 0; c < VEC; ++c) pending_sum[grp][VEC * o + c] = s4[c];
    __syncthreads();
  }
  auto grad = [&](const uint32_t i, const float g) {
    if (pj < 0) return g;
    float tt = pending_sum[0][i - beg];
#pragma unroll
    for (int k = 1; k < 8; ++k) tt += pending_sum[k][i - beg];
    return tt + g;
  };
  for (uint32_t i = beg + threadIdx.x * 4; i < end4; i += EW_THREADS * 4) {
    float4 vg = *reinterpret_cast<const float4 *>(t.g + i);
    vg = make_float4(grad(i, vg.x), grad(i + 1, vg.y), grad(i + 2, vg.z), grad(i + 3, vg.w));
    float4 vw       = *reinterpret_cast<float4 *>(t.w + i);
    float4 v0       = make_float4(0.f, 0.f, 0.f, 0.f), v1 = v0;
    if (NSTATE >= 1) v0 = *reinterpret_cast<float4 *>(t.s0 + i);
    if (NSTATE >= 2) v1 = *reinterpret_cast<float4 *>(t.s1 + i);
    opt_one<KIND>(vg.x, vw.x, v0.x, v1.x, p);
    opt_one<KIND>(vg.y, vw.y, v0.y, v1.y, p);
    opt_one<KIND>(vg.z, vw.z, v0.z, v1.z, p);
    opt_one<KIND>(vg.w, vw.w, v0.w, v1.w, p);
    *reinterpret_cast<float4 *>(t.w + i) = vw;
    if (t.wp_fwd) {
      opt_pack_store(t, i, vw.x);
      opt_pack_store(t, i + 1, vw.y);
      opt_pack_store(t, i + 2, vw.z);
      opt_pack_store(t, i + 3, vw.w);
    }
    if (NSTATE >= 1) *reinterpret_cast<float4 *>(t.s0 + i) = v0;
    if (NSTATE >= 2) *reinterpret_cast<float4 *>(t.s1 + i) = v1;
    if (zero_grad) *reinterpret_cast<float4 *>(t.g + i) = make_float4(0.f, 0.f, 0.f, 0.f);
  }
  for (uint32_t i = end4 + threadIdx.x; i < end; i += EW_THREADS) {
    float ww = t.w[i], a = 0.0f, b = 0.0f;
    if (NSTATE >= 1) a = t.s0[i];
    if (NSTATE >= 2) b = t.s1[i];
    opt_one<KIND>(grad(i, t.g[i]), ww, a, b, p);
    t.w[i] = ww;
    if (t.wp_fwd) opt_pack_store(t, i, ww);
    if (NSTATE >= 1) t.s0[i] = a;
    if (NSTATE >= 2) t.s1[i] = b;
    if (zero_grad) t.g[i] = 0.0f;
  }
}

// ---------------------------------------------------------------- reductions
// Block-wide sum with a fixed shape: wave butterflies, then wave 0 adds the four wave
// totals in order. Every thread of the block must call it.
__device__ __forceinline__ float block_sum(float v, float *smem4) {
  v = wave_sum(v);
  if ((threadIdx.x & 63) == 0) smem4[threadIdx.x >> 6] = v;
  __syncthreads();
  const float r = (smem4[0] + smem4[1]) + (smem4[2] + smem4[3]);
  __syncthreads();
  return r;
}

// Bias gradient of a convolution: out[r] (+)= sum over images o and pixels of
// src[(o*rows + r)*cols + c]. Stage 1: workgroup (r, g) adds the planes of images
// o = g, g+G, ... in order, each plane with a fixed block-wide tree. Stage 2: one wave per
// row adds the G group sums with a fixed butterfly.
__device__ __forceinline__ void rowsum_stage1_block(const float *__restrict__ src, const int outer,
                                                    const int rows, const int cols, const int groups,
                                                    float *__restrict__ partial, const int r,
                                                    const int g, float *smem4) {
  float s = 0.0f;
  for (int o = g; o < outer; o += groups) {
    const float *p = src + (static_cast<size_t>(o) * rows + r) * cols;
    for (int i = threadIdx.x; i < cols; i += EW_THREADS) s += p[i];
  }
  s = block_sum(s, smem4);
  if (threadIdx.x == 0) partial[r * groups + g] = s;
}

__device__ __forceinline__ void rowsum_stage2_block(const float *__restrict__ partial, const int rows,
                                                    const int groups, float *__restrict__ out,
                                                    const int accumulate, const int block) {
  const int r    = block * (EW_THREADS / 64) + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (r >= rows) return;
  float s = 0.0f;
  for (int g = lane; g < groups; g += 64) s += partial[r * groups + g];
  s = wave_sum(s);
  if (lane == 0) out[r] = accumulate ? out[r] + s : s;
}

__global__ void __launch_bounds__(EW_THREADS)
rowsum_stage1_kernel(const float *__restrict__ src, const int outer, const int rows,
                     const int cols, const int groups, float *__restrict__ partial) {
  __shared__ float smem4[4];
  rowsum_stage1_block(src, outer, rows, cols, groups, partial, blockIdx.x, blockIdx.y, smem4);
}

__global__ void __launch_bounds__(EW_THREADS)
rowsum_stage2_kernel(const float *__restrict__ partial, const int rows, const int groups,
                     float *__restrict__ out, const int accumulate) {
  rowsum_stage2_block(partial, rows, groups, out, accumulate, blockIdx.x);
}

// The bias gradients of several layers in one pair of launches. Job j owns the workgroups
// [first1[j], first1[j+1]) of stage 1, numbered g*rows + r, and [first2[j], first2[j+1]) of
// stage 2; every job keeps the grouping and the order of additions of a launch of its own.
constexpr int ROWSUM_MULTI_MAX = 8;
struct RowsumJob {
  const float *src;
  float *partial, *out;
  int outer, rows, cols, groups, accumulate;
};
struct RowsumJobs {
  RowsumJob job[ROWSUM_MULTI_MAX];
  int first1[ROWSUM_MULTI_MAX + 1], first2[ROWSUM_MULTI_MAX + 1];
  int n;
};

__global__ void __launch_bounds__(EW_THREADS) rowsum_multi_stage1_kernel(const RowsumJobs jobs) {
  __shared__ float smem4[4];
  int j = 0;
  while (j + 1 < jobs.n && jobs.first1[j + 1] <= static_cast<int>(blockIdx.x)) ++j;
  const RowsumJob &q = jobs.job[j];
  const int b = static_cast<int>(blockIdx.x) - jobs.first1[j];
  const int g = b / q.rows, r = b - g * q.rows;
  rowsum_stage1_block(q.src, q.outer, q.rows, q.cols, q.groups, q.partial, r, g, smem4);
}

__global__ void __launch_bounds__(EW_THREADS) rowsum_multi_stage2_kernel(const RowsumJobs jobs) {
  int j = 0;
  while (j + 1 < jobs.n && jobs.first2[j + 1] <= static_cast<int>(blockIdx.x)) ++j;
  const RowsumJob &q = jobs.job[j];
  rowsum_stage2_block(q.partial, q.rows, q.groups, q.out, q.accumulate,
                      static_cast<int>(blockIdx.x) - jobs.first2[j]);
}

// out[c] (+)= sum_s src[s*cols + c] (fully_connected bias gradient). A workgroup owns 32
// columns; its eight row groups add rows g, g+8, ... and the group sums are added in order.
__global__ void __launch_bounds__(EW_THREADS)
colsum_kernel(const float *__restrict__ src, const int rows, const int cols,
              float *__restrict__ out, const int accumulate) {
  __shared__ float sm[8][32];
  const int cl = threadIdx.x & 31, g = threadIdx.x >> 5;
  const int c  = blockIdx.x * 32 + cl;
  float s = 0.0f;
  if (c < cols) {
    // eight loads in flight, added in row order (one at a time each add waits a trip to memory)
    int r = g;
    for (; r + 56 < rows; r += 64) {
      float v[8];
#pragma unroll
      for (int k = 0; k < 8; ++k) v[k] = src[static_cast<size_t>(r + 8 * k) * cols + c];
#pragma unroll
      for (int k = 0; k < 8; ++k) s += v[k];
    }
    for (; r < rows; r += 8) s += src[static_cast<size_t>(r) * cols + c];
  }
  sm[g][cl] = s;
  __syncthreads();
  if (g == 0 && c < cols) {
    float t = sm[0][cl];
#pragma unroll
    for (int i = 1; i < 8; ++i) t += sm[i][cl];
    out[c] = accumulate ? out[c] + t : t;
  }
}

}  // namespace

int launch_fill_zero(void *p, size_t bytes, const char *tag) {
  ProfScope prof(tag, static_cast<double>(bytes), WORK_BYTE);
  const size_t n  = bytes / 4;
  const size_t n4 = aligned16(p) ? n / 4 : 0;
  TDH_LAUNCH(fill_zero_kernel, dim3(ew_blocks(n4 ? n4 + 3 : n)), dim3(EW_THREADS), 0,
                     ctx().stream, static_cast<uint32_t *>(p), n4, n);
  TDH_LAUNCH_CHECK();
  return TDH_OK;
}

int launch_copy(void *dst, const void *src, size_t bytes) {
  ProfScope prof("copy", 2.0 * static_cast<double>(bytes), WORK_BYTE);
  const size_t n  = bytes / 4;
  const size_t n4 = (aligned16(dst) && aligned16(src)) ? n / 4 : 0;
  TDH_LAUNCH(copy_kernel, dim3(ew_blocks(n4 ? n4 + 3 : n)), dim3(EW_THREADS), 0, ctx().stream,
                     static_cast<const uint32_t *>(src), static_cast<uint32_t *>(dst), n4, n);
  TDH_LAUNCH_CHECK();
  return TDH_OK;
}

int launch_act_fwd(int kind, const float *p, int batch, int len, const float *x, float *y) {
  const size_t n = static_cast<size_t>(batch) * len;
  const Act2 prm{p[0], p[1]};
  switch (kind) {
    case TDH_ACT_LEAKY_RELU: return launch_map<LeakyReluFwd, false>(x, nullptr, y, n, prm, "act_fwd_leaky_relu");
    case TDH_ACT_ELU: return launch_map<EluFwd, false>(x, nullptr, y, n, prm, "act_fwd_elu");
    case TDH_ACT_SELU: return launch_map<SeluFwd, false>(x, nullptr, y, n, prm, "act_fwd_selu");
    case TDH_ACT_SOFTPLUS: return launch_map<SoftplusFwd, false>(x, nullptr, y, n, prm, "act_fwd_softplus");
    case TDH_ACT_SOFTSIGN: return launch_map<SoftsignFwd, false>(x, nullptr, y, n, prm, "act_fwd_softsign");
    case TDH_ACT_ASINH: return launch_map<AsinhFwd, false>(x, nullptr, y, n, prm, "act_fwd_asinh");
    case TDH_ACT_TANH_P1M2: return launch_map<TanhP1m2Fwd, false>(x, nullptr, y, n, prm, "act_fwd_tanh_p1m2");
    case TDH_ACT_TANH: return launch_map<TanhFwd, false>(x, nullptr, y, n, NoParams(), "act_fwd_tanh");
    case TDH_ACT_RELU: return launch_map<ReluFwd, false>(x, nullptr, y, n, NoParams(), "act_fwd_relu");
    case TDH_ACT_SIGMOID: return launch_map<SigmoidFwd, false>(x, nullptr, y, n, NoParams(), "act_fwd_sigmoid");
    case TDH_ACT_SOFTMAX: {
      ProfScope prof("act_fwd_softmax", 8.0 * n, WORK_BYTE);
      TDH_LAUNCH(softmax_fwd_kernel, dim3(ceil_div(batch, EW_THREADS / 64)),
                         dim3(EW_THREADS), 0, ctx().stream, x, y, batch, len);
      TDH_LAUNCH_CHECK();
      return TDH_OK;
    }
  }
  return set_error(TDH_ERR_INVALID, "activation kind %d is not supported", kind);
}

int launch_act_bwd(int kind, const float *p, int batch, int len, const float *x, const float *y,
                   const float *dy, float *dx) {
  const size_t n = static_cast<size_t>(batch) * len;
  const Act2 prm{p[0], p[1]};
  if ((kind == TDH_ACT_SELU || kind == TDH_ACT_SOFTSIGN) && x == nullptr)
    return set_error(TDH_ERR_INVALID, "the gradient of activation kind %d reads the layer input x", kind);
  switch (kind) {
    case TDH_ACT_LEAKY_RELU: return launch_map<LeakyReluBwd, true>(y, dy, dx, n, prm, "act_grad_leaky_relu");
    case TDH_ACT_ELU: return launch_map<EluBwd, true>(y, dy, dx, n, prm, "act_grad_elu");
    case TDH_ACT_SELU: return launch_map<SeluBwd, true>(x, dy, dx, n, prm, "act_grad_selu");
    case TDH_ACT_SOFTPLUS: return launch_map<SoftplusBwd, true>(y, dy, dx, n, prm, "act_grad_softplus");
    case TDH_ACT_SOFTSIGN: return launch_map<SoftsignBwd, true>(x, dy, dx, n, prm, "act_grad_softsign");
    case TDH_ACT_ASINH: return launch_map<AsinhBwd, true>(y, dy, dx, n, prm, "act_grad_asinh");
    case TDH_ACT_TANH_P1M2: return launch_map<TanhP1m2Bwd, true>(y, dy, dx, n, prm, "act_grad_tanh_p1m2");
    case TDH_ACT_TANH: return launch_map<TanhBwd, true>(y, dy, dx, n, NoParams(), "act_grad_tanh");
    case TDH_ACT_RELU: return launch_map<ReluBwd, true>(y, dy, dx, n, NoParams(), "act_grad_relu");
    case TDH_ACT_SIGMOID: return launch_map<SigmoidBwd, true>(y, dy, dx, n, NoParams(), "act_grad_sigmoid");
    case TDH_ACT_SOFTMAX: {
      ProfScope prof("act_grad_softmax", 12.0 * n, WORK_BYTE);
      TDH_LAUNCH(softmax_bwd_kernel, dim3(ceil_div(batch, EW_THREADS / 64)),
                         dim3(EW_THREADS), 0, ctx().stream, y, dy, dx, batch, len);
      TDH_LAUNCH_CHECK();
      return TDH_OK;
    }
  }
  return set_error(TDH_ERR_INVALID, "activation kind %d is not supported", kind);
}

int launch_loss_grad(int kind, int batch, int len, const float *y, const float *t, float *dy) {
  const size_t n = static_cast<size_t>(batch) * len;
  switch (kind) {
    case TDH_LOSS_MSE: {
      MseGrad::Params p;
      p.factor = 2.0f / static_cast<float>(len);
      return launch_map<MseGrad, true>(y, t, dy, n, p, "loss_grad_mse");
    }
    case TDH_LOSS_CE_MULTICLASS: return launch_map<CeMultiGrad, true>(y, t, dy, n, NoParams(), "loss_grad_ce_multiclass");
    case TDH_LOSS_CE: return launch_map<CeGrad, true>(y, t, dy, n, NoParams(), "loss_grad_ce");
  }
  return set_error(TDH_ERR_INVALID, "loss kind %d is not supported", kind);
}

int launch_softmax_fwd_xent(int batch, int len, const float *x, const float *t, float *y, float *dz) {
  ProfScope prof("softmax_fwd_xent_grad", 20.0 * batch * len, WORK_BYTE);
  TDH_LAUNCH(softmax_fwd_xent_kernel, dim3(ceil_div(batch, EW_THREADS / 64)), dim3(EW_THREADS),
                     0, ctx().stream, x, t, y, dz, batch, len);
  TDH_LAUNCH_CHECK();
  return TDH_OK;
}

int launch_softmax_xent_grad(int batch, int len, const float *y, const float *t, float *dz) {
  ProfScope prof("softmax_xent_grad", 12.0 * batch * len, WORK_BYTE);
  TDH_LAUNCH(softmax_xent_grad_kernel, dim3(ceil_div(batch, EW_THREADS / 64)),
                     dim3(EW_THREADS), 0, ctx().stream, y, t, dz, batch, len);
  TDH_LAUNCH_CHECK();
  return TDH_OK;
}

int launch_opt_update(tdh_opt *o, size_t n, const float *g, float grad_scale, float *w, float *s0,
                      float *s1) {
  OptScalars p;
  p.alpha = o->alpha; p.lambda = o->lambda; p.mu = o->mu; p.b1 = o->b1; p.b2 = o->b2;
  p.eps = o->eps;
  p.omb1 = 1.0f - o->b1; p.omb2 = 1.0f - o->b2;
  p.omb1t = 1.0f - o->b1_t; p.omb2t = 1.0f - o->b2_t;
  p.grad_scale = grad_scale;
  p.adamax_lr  = static_cast<double>(o->alpha) / (1.0 - static_cast<double>(o->b1_t));
  int rc = TDH_OK;
  const int nstate = (o->kind == TDH_OPT_SGD) ? 0
                     : (o->kind == TDH_OPT_ADAM || o->kind == TDH_OPT_ADAMAX) ? 2 : 1;
  if (n > 0) {
    if (nstate >= 1 && !s0) return set_error(TDH_ERR_INVALID, "optimizer %d needs state s0", o->kind);
    if (nstate >= 2 && !s1) return set_error(TDH_ERR_INVALID, "optimizer %d needs state s1", o->kind);
    switch (o->kind) {
      case TDH_OPT_SGD: rc = launch_opt<TDH_OPT_SGD, 0>(n, g, w, s0, s1, p); break;
      case TDH_OPT_MOMENTUM: rc = launch_opt<TDH_OPT_MOMENTUM, 1>(n, g, w, s0, s1, p); break;
      case TDH_OPT_NESTEROV: rc = launch_opt<TDH_OPT_NESTEROV, 1>(n, g, w, s0, s1, p); break;
      case TDH_OPT_ADAM: rc = launch_opt<TDH_OPT_ADAM, 2>(n, g, w, s0, s1, p); break;
      case TDH_OPT_ADAGRAD: rc = launch_opt<TDH_OPT_ADAGRAD, 1>(n, g, w, s0, s1, p); break;
      case TDH_OPT_RMSPROP: rc = launch_opt<TDH_OPT_RMSPROP, 1>(n, g, w, s0, s1, p); break;
      case TDH_OPT_ADAMAX: rc = launch_opt<TDH_OPT_ADAMAX, 2>(n, g, w, s0, s1, p); break;
      default: return set_error(TDH_ERR_INVALID, "optimizer kind %d is not supported", o->kind);
    }
  }
  if (rc != TDH_OK) return rc;
  // the reference advances the powers once per update() call, whatever the tensor size
  if (o->kind == TDH_OPT_ADAM) {
    o->b1_t *= o->b1;
    o->b2_t *= o->b2;
  } else if (o->kind == TDH_OPT_ADAMAX) {
    o->b1_t *= o->b1;
  }
  return TDH_OK;
}

// grouping depends on the shape only
static int rowsum_groups(int outer) { return outer < 64 ? outer : 64; }

size_t rowsum_workspace_bytes(int outer, int rows, int cols) {
  (void)cols;
  return ws_align(static_cast<size_t>(rows) * rowsum_groups(outer) * sizeof(float));
}

int launch_opt_update_multi(tdh_opt *o, const OptTensor *dev_table, int n_tensors,
                            int total_blocks, double total_params, float grad_scale,
                            int zero_grad, const float *powers_in, float *powers_out,
                            const OptPending *pending, const OptTensor *host_table) {
  if (n_tensors <= 0) return TDH_OK;
  OptPending pend;
  pend.n = 0;
  double pending_bytes = 0.0;
  if (pending) {
    pend = *pending;
    for (int k = 0; k < pend.n; ++k) pending_bytes += 4.0 * pend.sum[k].splits * pend.sum[k].mn;
  }
  OptIndex idx;
  idx.n = 0;
  if (host_table && n_tensors <= OPT_INDEX_MAX) {
    idx.n = n_tensors;
    for (int k = 0; k < OPT_INDEX_MAX; ++k) {
      idx.first_block[k] = k < n_tensors ? host_table[k].first_block : 0xffffffffu;
      idx.pend_of[k]     = -1;
      for (int q = 0; k < n_tensors && q < pend.n; ++q)  // (the last match, as the kernel's search)
        if (pend.sum[q].g == host_table[k].g) idx.pend_of[k] = static_cast<int8_t>(q);
    }
  }
  OptScalars p;
  p.alpha = o->alpha; p.lambda = o->lambda; p.mu = o->mu; p.b1 = o->b1; p.b2 = o->b2;
  p.eps = o->eps;
  p.omb1 = 1.0f - o->b1; p.omb2 = 1.0f - o->b2;
  p.omb1t = p.omb2t = 0.0f;
  p.grad_scale = grad_scale;
  p.adamax_lr  = 0.0;
  static const char *const tags[] = {"opt_sgd_multi", "opt_momentum_multi", "opt_adam_multi",
                                     "opt_adagrad_multi", "opt_rmsprop_multi", "opt_adamax_multi",
                                     "opt_nesterov_multi"};
  TDH_CHECK_ARG(o->kind >= 0 && o->kind <= TDH_OPT_NESTEROV, "optimizer kind %d is not supported",
                o->kind);
  const int advance = o->kind == TDH_OPT_ADAM ? 2 : o->kind == TDH_OPT_ADAMAX ? 1 : 0;
  const int nstate = (o->kind == TDH_OPT_SGD) ? 0
                     : (o->kind == TDH_OPT_ADAM || o->kind == TDH_OPT_ADAMAX) ? 2 : 1;
  // gradient read (+ cleared), weight read+write, states read+write
  ProfScope prof(tags[o->kind], (12.0 + 8.0 * nstate + (zero_grad ? 4.0 : 0.0)) * total_params + pending_bytes,
                 WORK_BYTE);
#define TDH_LAUNCH_MULTI(KIND, NS)                                                            \
  TDH_LAUNCH((opt_multi_kernel<KIND, NS>), dim3(total_blocks), dim3(EW_THREADS), 0,   \
                     ctx().stream, dev_table, n_tensors, p, o->b1_t, o->b2_t,                  \
                     powers_in, powers_out, advance, zero_grad, pend, idx)
  switch (o->kind) {
    case TDH_OPT_SGD: TDH_LAUNCH_MULTI(TDH_OPT_SGD, 0); break;
    case TDH_OPT_MOMENTUM: TDH_LAUNCH_MULTI(TDH_OPT_MOMENTUM, 1); break;
    case TDH_OPT_NESTEROV: TDH_LAUNCH_MULTI(TDH_OPT_NESTEROV, 1); break;
    case TDH_OPT_ADAM: TDH_LAUNCH_MULTI(TDH_OPT_ADAM, 2); break;
    case TDH_OPT_ADAGRAD: TDH_LAUNCH_MULTI(TDH_OPT_ADAGRAD, 1); break;
    case TDH_OPT_RMSPROP: TDH_LAUNCH_MULTI(TDH_OPT_RMSPROP, 1); break;
    case TDH_OPT_ADAMAX: TDH_LAUNCH_MULTI(TDH_OPT_ADAMAX, 2); break;
  }
#undef TDH_LAUNCH_MULTI
  TDH_LAUNCH_CHECK();
  for (int j = 0; j < n_tensors; ++j) {
    if (o->kind == TDH_OPT_ADAM) {
      o->b1_t *= o->b1;
      o->b2_t *= o->b2;
    } else if (o->kind == TDH_OPT_ADAMAX) {
      o->b1_t *= o->b1;
    }
  }
  return TDH_OK;
}

static std::vector<RowsumJob> &deferred_rowsums() {
  static std::vector<RowsumJob> jobs;
  return jobs;
}

int flush_deferred_rowsums(bool launch) {
  std::vector<RowsumJob> &all = deferred_rowsums();
  if (!launch) all.clear();
  for (size_t at = 0; at < all.size(); at += ROWSUM_MULTI_MAX) {
    RowsumJobs jobs;
    jobs.n = static_cast<int>(std::min<size_t>(ROWSUM_MULTI_MAX, all.size() - at));
    int b1 = 0, b2 = 0;
    double bytes = 0.0;
    for (int j = 0; j < jobs.n; ++j) {
      const RowsumJob &q = jobs.job[j] = all[at + j];
      jobs.first1[j] = b1;
      jobs.first2[j] = b2;
      b1 += q.rows * q.groups;
      b2 += ceil_div(q.rows, EW_THREADS / 64);
      bytes += 4.0 * q.outer * q.rows * q.cols;
    }
    jobs.first1[jobs.n] = b1;
    jobs.first2[jobs.n] = b2;
    ProfScope prof("bias_grad_rowsum_multi", bytes, WORK_BYTE);
    TDH_LAUNCH(rowsum_multi_stage1_kernel, dim3(b1), dim3(EW_THREADS), 0, ctx().stream, jobs);
    hipError_t e = hipGetLastError();
    if (e == hipSuccess) {
      TDH_LAUNCH(rowsum_multi_stage2_kernel, dim3(b2), dim3(EW_THREADS), 0, ctx().stream,
                         jobs);
      e = hipGetLastError();
    }
    if (e != hipSuccess) {
      all.clear();
      return set_error(TDH_ERR_HIP, "rowsum_multi kernels: %s", hipGetErrorString(e));
    }
  }
  all.clear();
  return TDH_OK;
}

int launch_rowsum(const float *src, int outer, int rows, int cols, float *out, int accumulate) {
  const int groups = rowsum_groups(outer);
  void *ws = nullptr;
  TDH_TRY(ws_take(static_cast<size_t>(rows) * groups * sizeof(float), &ws));
  if (ctx().defer_rowsum) {
    deferred_rowsums().push_back(
        RowsumJob{src, static_cast<float *>(ws), out, outer, rows, cols, groups, accumulate});
    return TDH_OK;
  }
  ProfScope prof("bias_grad_rowsum", 4.0 * outer * rows * cols, WORK_BYTE);
  TDH_LAUNCH(rowsum_stage1_kernel, dim3(rows, groups), dim3(EW_THREADS), 0, ctx().stream,
                     src, outer, rows, cols, groups, static_cast<float *>(ws));
  TDH_LAUNCH_CHECK();
  TDH_LAUNCH(rowsum_stage2_kernel, dim3(ceil_div(rows, EW_THREADS / 64)), dim3(EW_THREADS),
                     0, ctx().stream, static_cast<const float *>(ws), rows, groups, out, accumulate);
  TDH_LAUNCH_CHECK();
  return TDH_OK;
}

int launch_colsum(const float *src, int rows, int cols, float *out, int accumulate) {
  ProfScope prof("bias_grad_colsum", 4.0 * rows * cols, WORK_BYTE);
  TDH_LAUNCH(colsum_kernel, dim3(ceil_div(cols, 32)), dim3(EW_THREADS), 0,
                     ctx().stream, src, rows, cols, out, accumulate);
  TDH_LAUNCH_CHECK();
  return TDH_OK;
}

}  // namespace tdh
