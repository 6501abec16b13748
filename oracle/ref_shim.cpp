/*
 * ref_shim.cpp — C entry points over the UNMODIFIED tiny-dnn headers.
 *
 * TEST INFRASTRUCTURE ONLY. Built by oracle/Makefile against the reference
 * tree where it lies (-I$(REF)); nothing of the reference is copied. The
 * resulting libraries (oracle/_ref/) validate oracle/td_oracle.c and serve as
 * the "reference" CPU baseline of the benchmark. They are never loaded by the
 * product library.
 *
 * Each entry point drives real tiny-dnn objects through their public API:
 * layer::forward / layer::backward (tiny_dnn/layers/layer.h:464-507),
 * edge::merge_grads (tiny_dnn/node.h:89-103), optimizer::update
 * (tiny_dnn/optimizers/optimizer.h) and network<sequential>::fit
 * (tiny_dnn/network.h:368-386).
 *
 * Include order works around tiny_dnn/tiny_dnn.h:122 naming linear_layer
 * without including its header.
 */
#include <fstream>
#include <iostream>
#ifdef CNN_USE_OMP
#include <omp.h>
#endif

#include "tiny_dnn/util/util.h"
#include "tiny_dnn/layers/layer.h"
#include "tiny_dnn/layers/linear_layer.h"
#include "tiny_dnn/tiny_dnn.h"

#include <chrono>
#include <cstdint>
#include <cstring>
#include <memory>
#include <sstream>
#include <vector>

using namespace tiny_dnn;

namespace {

struct conv_desc {
  int32_t in_w, in_h, in_c, k_w, k_h, out_c, w_stride, h_stride, w_dilation, h_dilation, pad_same,
    has_bias;
  const uint8_t *tbl;
};
struct pool_desc {
  int32_t in_w, in_h, in_c, pool_w, pool_h, stride_w, stride_h, pad_same, ceil_mode;
};
struct opt_desc {
  int32_t kind;
  float alpha, lambda, mu, b1, b2, eps, b1_t, b2_t;
};
struct layer_desc {
  int32_t kind, act;
  conv_desc conv;
  pool_desc pool;
  int32_t fc_in, fc_out, fc_bias;
  float act_p[2];
  int32_t bn_channels, bn_spatial;
  float bn_eps, bn_momentum;
  float dropout_rate;
};

core::backend_t engine_of(int engine) {
  return engine == 0 ? core::backend_t::internal : core::default_engine();
}

tensor_t to_tensor(const float *p, int batch, size_t len) {
  tensor_t t(batch);
  for (int s = 0; s < batch; s++) t[s].assign(p + len * s, p + len * (s + 1));
  return t;
}

void from_tensor(const tensor_t &t, int batch, size_t len, float *p) {
  for (int s = 0; s < batch; s++) std::memcpy(p + len * s, t[s].data(), sizeof(float) * len);
}

std::unique_ptr<convolutional_layer> make_conv(const conv_desc &d, int engine) {
  core::connection_table tbl;
  if (d.tbl) {
    std::vector<char> flags(size_t(d.in_c) * d.out_c);
    for (size_t i = 0; i < flags.size(); i++) flags[i] = d.tbl[i] != 0;
    tbl = core::connection_table(reinterpret_cast<const bool *>(flags.data()), d.in_c, d.out_c);
  }
  return std::unique_ptr<convolutional_layer>(new convolutional_layer(
    d.in_w, d.in_h, d.k_w, d.k_h, d.in_c, d.out_c, tbl,
    d.pad_same ? padding::same : padding::valid, d.has_bias != 0, d.w_stride, d.h_stride,
    d.w_dilation, d.h_dilation, engine_of(engine)));
}

std::unique_ptr<max_pooling_layer> make_maxpool(const pool_desc &d, int engine) {
  return std::unique_ptr<max_pooling_layer>(new max_pooling_layer(
    d.in_w, d.in_h, d.in_c, d.pool_w, d.pool_h, d.stride_w, d.stride_h, d.ceil_mode != 0,
    d.pad_same ? padding::same : padding::valid, engine_of(engine)));
}

std::unique_ptr<average_pooling_layer> make_avepool(const pool_desc &d) {
  return std::unique_ptr<average_pooling_layer>(new average_pooling_layer(
    d.in_w, d.in_h, d.in_c, d.pool_w, d.pool_h, d.stride_w, d.stride_h, d.ceil_mode != 0,
    d.pad_same ? padding::same : padding::valid));
}

/* Loads the first wn/bn entries of the layer's weight/bias vectors and zero-fills the rest
 * (average_pooling_layer declares a weight vector of pool_w*pool_h*channels entries,
 * tiny_dnn/layers/average_pooling_layer.h:222-226, of which only the first `channels`
 * are ever read). */
void load_weights(layer &l, const float *w, size_t wn, const float *b, size_t bn) {
  l.setup(false);
  auto wv = l.weights();
  std::vector<float_t> flat;
  if (wv.size() > 0) {
    std::vector<float_t> part(wv[0]->size(), 0.0f);
    if (w) std::copy(w, w + std::min(wn, part.size()), part.begin());
    flat.insert(flat.end(), part.begin(), part.end());
  }
  if (wv.size() > 1) {
    std::vector<float_t> part(wv[1]->size(), 0.0f);
    if (b) std::copy(b, b + std::min(bn, part.size()), part.begin());
    flat.insert(flat.end(), part.begin(), part.end());
  }
  int idx = 0;
  l.load(flat, idx);
}

/* merged gradient of in-edge i: exactly what update_weight feeds to the optimizer
 * before the 1/batch scaling */
void merged_grad(layer &l, size_t edge_index, float *dst, size_t n = 0) {
  vec_t merged;
  l.inputs()[edge_index]->merge_grads(&merged);
  std::memcpy(dst, merged.data(), sizeof(float) * (n ? std::min(n, merged.size()) : merged.size()));
}

/* run forward then backward on one layer with `batch` samples */
void layer_fwd(layer &l, int batch, const float *x, size_t in_len, float *y, size_t out_len) {
  std::vector<const tensor_t *> out;
  l.forward({to_tensor(x, batch, in_len)}, out);
  if (y) from_tensor(*out[0], batch, out_len, y);
}

double layer_bwd(layer &l, int batch, const float *dy, size_t out_len, float *dx, size_t in_len) {
  std::vector<tensor_t> g{to_tensor(dy, batch, out_len)};
  /* layer::forward cleared the out-edge gradient only; start weight grads from zero as
   * update_weight/clear_grads leaves them */
  l.clear_grads();
  auto t0 = std::chrono::steady_clock::now();
  std::vector<tensor_t> in_grads = l.backward(g);
  auto t1 = std::chrono::steady_clock::now();
  if (dx) from_tensor(in_grads[0], batch, in_len, dx);
  return std::chrono::duration<double>(t1 - t0).count();
}

template <typename Act, typename... P>
int act_run(int batch, int len, const float *x, float *y, const float *dy, float *dx, P... prm) {
  Act a((size_t)len, prm...);
  layer_fwd(a, batch, x, len, y, len);
  if (dy) layer_bwd(a, batch, dy, len, dx, len);
  return 0;
}

template <typename Opt>
void run_updates(Opt &o, size_t n, const float *g, float *w, int steps) {
  vec_t W(w, w + n), G(g, g + n);
  for (int s = 0; s < steps; s++) o.update(G, W, false);
  std::memcpy(w, W.data(), sizeof(float) * n);
}

}  // namespace

extern "C" {

int tdr_num_threads() {
#ifdef CNN_USE_OMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* 1 when the build's default engine is the AVX one */
int tdr_default_engine_is_avx() { return core::default_engine() == core::backend_t::avx; }

int tdr_conv2d_fwd(const conv_desc *d, int engine, int batch, const float *x, const float *w,
                   const float *b, float *y) {
  try {
    auto l = make_conv(*d, engine);
    load_weights(*l, w, l->weights()[0]->size(), d->has_bias ? b : nullptr, d->out_c);
    layer_fwd(*l, batch, x, l->in_shape()[0].size(), y, l->out_shape()[0].size());
    return 0;
  } catch (const std::exception &) { return -1; }
}

/* returns seconds spent inside layer::backward (negative on error) */
double tdr_conv2d_bwd(const conv_desc *d, int engine, int batch, const float *x, const float *w,
                      const float *dy, float *dx, float *dw, float *db, int repeat) {
  try {
    auto l = make_conv(*d, engine);
    std::vector<float> zb(d->out_c, 0.0f);
    load_weights(*l, w, l->weights()[0]->size(), d->has_bias ? zb.data() : nullptr, d->out_c);
    const size_t in_len = l->in_shape()[0].size(), out_len = l->out_shape()[0].size();
    layer_fwd(*l, batch, x, in_len, nullptr, out_len);
    double best = 1e30;
    for (int r = 0; r < (repeat < 1 ? 1 : repeat); r++) {
      const double t = layer_bwd(*l, batch, dy, out_len, dx, in_len);
      if (t < best) best = t;
    }
    if (dw) merged_grad(*l, 1, dw);
    if (db && d->has_bias) merged_grad(*l, 2, db);
    return best;
  } catch (const std::exception &) { return -1.0; }
}

int tdr_fc_fwd(int in, int out, int has_bias, int engine, int batch, const float *x,
               const float *w, const float *b, float *y) {
  try {
    fully_connected_layer l(in, out, has_bias != 0, engine_of(engine));
    load_weights(l, w, size_t(in) * out, has_bias ? b : nullptr, out);
    layer_fwd(l, batch, x, in, y, out);
    return 0;
  } catch (const std::exception &) { return -1; }
}

double tdr_fc_bwd(int in, int out, int has_bias, int engine, int batch, const float *x,
                  const float *w, const float *dy, float *dx, float *dw, float *db, int repeat) {
  try {
    fully_connected_layer l(in, out, has_bias != 0, engine_of(engine));
    std::vector<float> zb(out, 0.0f);
    load_weights(l, w, size_t(in) * out, has_bias ? zb.data() : nullptr, out);
    layer_fwd(l, batch, x, in, nullptr, out);
    double best = 1e30;
    for (int r = 0; r < (repeat < 1 ? 1 : repeat); r++) {
      const double t = layer_bwd(l, batch, dy, out, dx, in);
      if (t < best) best = t;
    }
    if (dw) merged_grad(l, 1, dw);
    if (db && has_bias) merged_grad(l, 2, db);
    return best;
  } catch (const std::exception &) { return -1.0; }
}

int tdr_maxpool_fwd(const pool_desc *d, int engine, int batch, const float *x, float *y) {
  try {
    auto l = make_maxpool(*d, engine);
    layer_fwd(*l, batch, x, l->in_shape()[0].size(), y, l->out_shape()[0].size());
    return 0;
  } catch (const std::exception &) { return -1; }
}

/* forward on x (records the argmax inside the layer) then backward with dy */
int tdr_maxpool_fwd_bwd(const pool_desc *d, int engine, int batch, const float *x, float *y,
                        const float *dy, float *dx) {
  try {
    auto l = make_maxpool(*d, engine);
    const size_t in_len = l->in_shape()[0].size(), out_len = l->out_shape()[0].size();
    layer_fwd(*l, batch, x, in_len, y, out_len);
    layer_bwd(*l, batch, dy, out_len, dx, in_len);
    return 0;
  } catch (const std::exception &) { return -1; }
}

int tdr_avepool_fwd(const pool_desc *d, int batch, const float *x, const float *w,
                    const float *b, float *y) {
  try {
    auto l = make_avepool(*d);
    load_weights(*l, w, d->in_c, b, d->in_c);
    layer_fwd(*l, batch, x, l->in_shape()[0].size(), y, l->out_shape()[0].size());
    return 0;
  } catch (const std::exception &) { return -1; }
}

int tdr_avepool_bwd(const pool_desc *d, int batch, const float *x, const float *w,
                    const float *dy, float *dx, float *dw, float *db) {
  try {
    auto l = make_avepool(*d);
    std::vector<float> zb(d->in_c, 0.0f);
    load_weights(*l, w, d->in_c, zb.data(), d->in_c);
    const size_t in_len = l->in_shape()[0].size(), out_len = l->out_shape()[0].size();
    layer_fwd(*l, batch, x, in_len, nullptr, out_len);
    layer_bwd(*l, batch, dy, out_len, dx, in_len);
    if (dw) merged_grad(*l, 1, dw, d->in_c);
    if (db) merged_grad(*l, 2, db, d->in_c);
    return 0;
  } catch (const std::exception &) { return -1; }
}

/* kind: 0 tanh, 1 relu, 2 softmax, 3 sigmoid, 4 leaky_relu {epsilon}, 5 elu {alpha},
 * 6 selu {lambda, alpha}, 7 softplus {beta, threshold}, 8 softsign, 9 asinh, 10 tanh_p1m2;
 * p: the constructor parameters in braces; dy/dx may be NULL (forward only) */
int tdr_act_p(int kind, const float *p, int batch, int len, const float *x, float *y,
              const float *dy, float *dx) {
  try {
    switch (kind) {
      case 0: return act_run<tanh_layer>(batch, len, x, y, dy, dx);
      case 1: return act_run<relu_layer>(batch, len, x, y, dy, dx);
      case 2: return act_run<softmax_layer>(batch, len, x, y, dy, dx);
      case 3: return act_run<sigmoid_layer>(batch, len, x, y, dy, dx);
      case 4: return act_run<leaky_relu_layer>(batch, len, x, y, dy, dx, p[0]);
      case 5: return act_run<elu_layer>(batch, len, x, y, dy, dx, p[0]);
      case 6: return act_run<selu_layer>(batch, len, x, y, dy, dx, p[0], p[1]);
      case 7: return act_run<softplus_layer>(batch, len, x, y, dy, dx, p[0], p[1]);
      case 8: return act_run<softsign_layer>(batch, len, x, y, dy, dx);
      case 9: return act_run<asinh_layer>(batch, len, x, y, dy, dx);
      case 10: return act_run<tanh_p1m2_layer>(batch, len, x, y, dy, dx);
    }
    return -2;
  } catch (const std::exception &) { return -1; }
}
int tdr_act(int kind, int batch, int len, const float *x, float *y, const float *dy, float *dx) {
  const float none[2] = {0.0f, 0.0f};
  return kind <= 3 ? tdr_act_p(kind, none, batch, len, x, y, dy, dx) : -2;
}

/* batch_normalization_layer: forward in the given phase, then backward. In the train phase the
 * layer's batch moments come back in mean/variance; in the test phase mean/variance are set on
 * the layer first. stddev comes back as sqrt(variance + eps) (the layer keeps it private). */
int tdr_batchnorm(int channels, int spatial, int batch, float eps, int train, const float *x,
                  float *mean, float *variance, float *y, const float *dy, float *dx) {
  try {
    batch_normalization_layer bn((size_t)spatial, (size_t)channels, eps, 0.999f,
                                 train ? net_phase::train : net_phase::test);
    if (!train) {
      bn.set_mean(vec_t(mean, mean + channels));
      bn.set_variance(vec_t(variance, variance + channels));
    } else {
      bn.update_immidiately(true);  /* copies the batch moments into mean_/variance_, read by save() */
    }
    const size_t len = (size_t)channels * spatial;
    layer_fwd(bn, batch, x, len, y, len);
    if (train) {
      std::ostringstream os;
      bn.save(os);
      std::istringstream is(os.str());
      for (int i = 0; i < channels; i++) is >> mean[i];
      for (int i = 0; i < channels; i++) is >> variance[i];
    }
    if (dy) layer_bwd(bn, batch, dy, len, dx, len);
    return 0;
  } catch (const std::exception &) { return -1; }
}

/* batch_normalization_layer::post_update after one train-phase forward of x, starting from the
 * moving averages mean/variance (in and out) */
int tdr_batchnorm_post_update(int channels, int spatial, int batch, float eps, float momentum,
                              const float *x, float *mean, float *variance) {
  try {
    batch_normalization_layer bn((size_t)spatial, (size_t)channels, eps, momentum, net_phase::train);
    bn.set_mean(vec_t(mean, mean + channels));
    bn.set_variance(vec_t(variance, variance + channels));
    const size_t len = (size_t)channels * spatial;
    layer_fwd(bn, batch, x, len, nullptr, len);
    bn.post_update();
    std::ostringstream os;
    bn.save(os);
    std::istringstream is(os.str());
    for (int i = 0; i < channels; i++) is >> mean[i];
    for (int i = 0; i < channels; i++) is >> variance[i];
    return 0;
  } catch (const std::exception &) { return -1; }
}

/* dropout_layer in the train phase after set_random_seed(seed): forward (mask and y come back),
 * then backward. Meaningful with one worker thread only: the samples draw from one generator. */
int tdr_dropout(int len, int batch, float rate, unsigned int seed, const float *x,
                unsigned char *mask, float *y, const float *dy, float *dx) {
  try {
    dropout_layer dl((size_t)len, rate, net_phase::train);
    set_random_seed(seed);
    const int threads = omp_get_max_threads();
    omp_set_num_threads(1);  /* the samples share one generator: any other count races */
    layer_fwd(dl, batch, x, len, y, len);
    omp_set_num_threads(threads);
    for (int s = 0; s < batch; s++) {
      const std::vector<uint8_t> &m = dl.get_mask((size_t)s);
      std::memcpy(mask + (size_t)len * s, m.data(), len);
    }
    if (dy) layer_bwd(dl, batch, dy, len, dx, len);
    return 0;
  } catch (const std::exception &) { return -1; }
}

/* kind: 0 mse, 1 cross_entropy_multiclass, 2 cross_entropy */
int tdr_loss_grad(int kind, int batch, int len, const float *y, const float *t, float *dy) {
  std::vector<tensor_t> yy(batch), tt(batch), cost;
  for (int s = 0; s < batch; s++) {
    yy[s] = {vec_t(y + size_t(len) * s, y + size_t(len) * (s + 1))};
    tt[s] = {vec_t(t + size_t(len) * s, t + size_t(len) * (s + 1))};
  }
  std::vector<tensor_t> g;
  switch (kind) {
    case 0: g = gradient<mse>(yy, tt, cost); break;
    case 1: g = gradient<cross_entropy_multiclass>(yy, tt, cost); break;
    case 2: g = gradient<cross_entropy>(yy, tt, cost); break;
    default: return -2;
  }
  for (int s = 0; s < batch; s++) std::memcpy(dy + size_t(len) * s, g[s][0].data(), sizeof(float) * len);
  return 0;
}

/* `steps` consecutive optimizer::update(g, w) calls on one fresh optimizer object with
 * the hyper-parameters of *o (kinds as in td_oracle.h) */
int tdr_opt_updates(const opt_desc *o, size_t n, const float *g, float *w, int steps) {
  switch (o->kind) {
    case 0: { gradient_descent p; p.alpha = o->alpha; p.lambda = o->lambda; run_updates(p, n, g, w, steps); } break;
    case 1: { momentum p; p.alpha = o->alpha; p.lambda = o->lambda; p.mu = o->mu; run_updates(p, n, g, w, steps); } break;
    case 2: { adam p; p.alpha = o->alpha; p.b1 = o->b1; p.b2 = o->b2; p.b1_t = o->b1_t; p.b2_t = o->b2_t; run_updates(p, n, g, w, steps); } break;
    case 3: { adagrad p; p.alpha = o->alpha; run_updates(p, n, g, w, steps); } break;
    case 4: { RMSprop p; p.alpha = o->alpha; p.mu = o->mu; run_updates(p, n, g, w, steps); } break;
    case 5: { adamax p; p.alpha = o->alpha; p.b1 = o->b1; p.b2 = o->b2; p.b1_t = o->b1_t; run_updates(p, n, g, w, steps); } break;
    case 6: { nesterov_momentum p; p.alpha = o->alpha; p.lambda = o->lambda; p.mu = o->mu; run_updates(p, n, g, w, steps); } break;
    default: return -2;
  }
  return 0;
}

/* ---- whole network: network<sequential>::fit on caller-provided arrays ---- */

struct tdr_net {
  network<sequential> net;
  std::vector<layer_desc> spec;
};

tdr_net *tdr_net_create(const layer_desc *layers, int n_layers, int engine) {
  try {
    std::unique_ptr<tdr_net> h(new tdr_net());
    h->spec.assign(layers, layers + n_layers);
    for (int i = 0; i < n_layers; i++) {
      const layer_desc &s = layers[i];
      switch (s.kind) {
        case 0: {
          core::connection_table tbl;
          if (s.conv.tbl) {
            std::vector<char> flags(size_t(s.conv.in_c) * s.conv.out_c);
            for (size_t k = 0; k < flags.size(); k++) flags[k] = s.conv.tbl[k] != 0;
            tbl = core::connection_table(reinterpret_cast<const bool *>(flags.data()), s.conv.in_c,
                                         s.conv.out_c);
          }
          h->net << convolutional_layer(
            s.conv.in_w, s.conv.in_h, s.conv.k_w, s.conv.k_h, s.conv.in_c, s.conv.out_c, tbl,
            s.conv.pad_same ? padding::same : padding::valid, s.conv.has_bias != 0,
            s.conv.w_stride, s.conv.h_stride, s.conv.w_dilation, s.conv.h_dilation,
            engine_of(engine));
        } break;
        case 1:
          h->net << fully_connected_layer(s.fc_in, s.fc_out, s.fc_bias != 0, engine_of(engine));
          break;
        case 2:
          h->net << max_pooling_layer(s.pool.in_w, s.pool.in_h, s.pool.in_c, s.pool.pool_w,
                                      s.pool.pool_h, s.pool.stride_w, s.pool.stride_h,
                                      s.pool.ceil_mode != 0,
                                      s.pool.pad_same ? padding::same : padding::valid,
                                      engine_of(engine));
          break;
        case 3:
          h->net << average_pooling_layer(s.pool.in_w, s.pool.in_h, s.pool.in_c, s.pool.pool_w,
                                          s.pool.pool_h, s.pool.stride_w, s.pool.stride_h,
                                          s.pool.ceil_mode != 0,
                                          s.pool.pad_same ? padding::same : padding::valid);
          break;
        case 4:
          switch (s.act) {
            case 0: h->net << tanh_layer(); break;
            case 1: h->net << relu_layer(); break;
            case 2: h->net << softmax_layer(); break;
            case 3: h->net << sigmoid_layer(); break;
            case 4: h->net << leaky_relu_layer(s.act_p[0]); break;
            case 5: h->net << elu_layer(s.act_p[0]); break;
            case 6: h->net << selu_layer(s.act_p[0], s.act_p[1]); break;
            case 7: h->net << softplus_layer(s.act_p[0], s.act_p[1]); break;
            case 8: h->net << softsign_layer(); break;
            case 9: h->net << asinh_layer(); break;
            case 10: h->net << tanh_p1m2_layer(); break;
            default: return nullptr;
          }
          break;
        case 5:
          h->net << batch_normalization_layer(s.bn_spatial, s.bn_channels, s.bn_eps, s.bn_momentum);
          break;
        case 6:
          if (i == 0) return nullptr;
          h->net << dropout_layer(h->net[i - 1]->out_data_size(), s.dropout_rate);
          break;
        default: return nullptr;
      }
    }
    h->net.init_weight();
    return h.release();
  } catch (const std::exception &) { return nullptr; }
}

void tdr_net_destroy(tdr_net *h) { delete h; }

size_t tdr_net_param_size(tdr_net *h, int layer, int which) {
  auto w = h->net[layer]->weights();
  return size_t(which) < w.size() ? w[which]->size() : 0;
}

int tdr_net_set_param(tdr_net *h, int layer, int which, const float *src) {
  auto w = h->net[layer]->weights();
  if (size_t(which) >= w.size()) return -2;
  std::copy(src, src + w[which]->size(), w[which]->begin());
  return 0;
}

int tdr_net_get_param(tdr_net *h, int layer, int which, float *dst) {
  auto w = h->net[layer]->weights();
  if (size_t(which) >= w.size()) return -2;
  std::copy(w[which]->begin(), w[which]->end(), dst);
  return 0;
}

/* set_random_seed (util/random.h:58-60): dropout layers draw their masks from this generator */
void tdr_set_random_seed(unsigned seed) { set_random_seed(seed); }

/* moving mean (which = 0) / variance (1) of batch-norm layer `layer`, read back through the
 * layer's own save() (batch_normalization_layer.h:179-189; printed with 8 significant digits) */
int tdr_net_get_bn_stat(tdr_net *h, int layer, int which, float *dst, int channels) {
  try {
    std::stringstream ss;
    h->net[layer]->save(ss);
    std::vector<float> v;
    float f;
    while (ss >> f) v.push_back(f);
    if (v.size() != size_t(2 * channels)) return -2;
    std::copy(v.begin() + which * channels, v.begin() + (which + 1) * channels, dst);
    return 0;
  } catch (const std::exception &) { return -1; }
}

/* `steps` mini-batch steps on the same batch (fit over `steps` epochs of one batch) with one
 * optimizer object; returns seconds per step (negative on error). loss: 0 mse,
 * 1 cross_entropy_multiclass, 2 cross_entropy. */
double tdr_net_fit(tdr_net *h, const opt_desc *o, int loss, int batch, const float *x,
                   size_t in_len, const float *t, size_t out_len, int steps) {
  try {
    std::vector<vec_t> X(batch), T(batch);
    for (int s = 0; s < batch; s++) {
      X[s].assign(x + in_len * s, x + in_len * (s + 1));
      T[s].assign(t + out_len * s, t + out_len * (s + 1));
    }
    auto nop = []() {};
    /* the samples of a dropout layer share one generator: any thread count but one races */
    bool has_dropout = false;
    for (const layer_desc &s : h->spec) has_dropout = has_dropout || s.kind == 6;
    struct OneThread {
      int saved;
      bool on;
      explicit OneThread(bool o) : saved(omp_get_max_threads()), on(o) { if (on) omp_set_num_threads(1); }
      ~OneThread() { if (on) omp_set_num_threads(saved); }
    } one_thread(has_dropout);
    auto t0  = std::chrono::steady_clock::now();
    bool ok  = false;
#define TDR_FIT(OPT)                                                                   \
  switch (loss) {                                                                      \
    case 0: ok = h->net.fit<mse>(OPT, X, T, batch, steps, nop, nop); break;            \
    case 1: ok = h->net.fit<cross_entropy_multiclass>(OPT, X, T, batch, steps, nop, nop); break; \
    case 2: ok = h->net.fit<cross_entropy>(OPT, X, T, batch, steps, nop, nop); break;  \
    default: return -2.0;                                                              \
  }
    switch (o->kind) {
      case 0: { gradient_descent p; p.alpha = o->alpha; p.lambda = o->lambda; TDR_FIT(p) } break;
      case 1: { momentum p; p.alpha = o->alpha; p.lambda = o->lambda; p.mu = o->mu; TDR_FIT(p) } break;
      case 2: { adam p; p.alpha = o->alpha; p.b1 = o->b1; p.b2 = o->b2; p.b1_t = o->b1_t; p.b2_t = o->b2_t; TDR_FIT(p) } break;
      /* eps is private in these three; the callers keep the constructor's value */
      case 3: { adagrad p; p.alpha = o->alpha; TDR_FIT(p) } break;
      case 4: { RMSprop p; p.alpha = o->alpha; p.mu = o->mu; TDR_FIT(p) } break;
      case 5: { adamax p; p.alpha = o->alpha; p.b1 = o->b1; p.b2 = o->b2; p.b1_t = o->b1_t; TDR_FIT(p) } break;
      case 6: { nesterov_momentum p; p.alpha = o->alpha; p.lambda = o->lambda; p.mu = o->mu; TDR_FIT(p) } break;
      default: return -2.0;
    }
#undef TDR_FIT
    auto t1 = std::chrono::steady_clock::now();
    if (!ok) return -1.0;
    return std::chrono::duration<double>(t1 - t0).count() / steps;
  } catch (const std::exception &) { return -1.0; }
}

/* forward only, returns the network output for the batch */
int tdr_net_predict(tdr_net *h, int batch, const float *x, size_t in_len, float *y,
                    size_t out_len) {
  try {
    for (int s = 0; s < batch; s++) {
      vec_t in(x + in_len * s, x + in_len * (s + 1));
      vec_t out = h->net.predict(in);
      std::memcpy(y + out_len * s, out.data(), sizeof(float) * out_len);
    }
    return 0;
  } catch (const std::exception &) { return -1; }
}

/* network::save(std::ostream&) / load(std::istream&) of the weights as text
 * (tiny_dnn/network.h:762-771, layer::save/load tiny_dnn/layers/layer.h:361-385) */
int tdr_net_save_weights(tdr_net *h, const char *path) {
  try {
    std::ofstream os(path);
    h->net.save(os);
    return os.good() ? 0 : -1;
  } catch (const std::exception &) { return -1; }
}
int tdr_net_load_weights(tdr_net *h, const char *path) {
  try {
    std::ifstream is(path);
    if (!is.good()) return -1;
    h->net.load(is);
    return 0;
  } catch (const std::exception &) { return -1; }
}

/* network::save / load with cereal archives (tiny_dnn/network.h:676-728, to_archive /
 * from_archive :787-811): what = content_type (0 weights, 1 model, 2 weights_and_model),
 * format = file_format (0 binary, 1 portable_binary, 2 json). Only in the build without
 * CNN_NO_SERIALIZATION; -3 elsewhere. */
int tdr_net_save_archive(tdr_net *h, const char *path, int what, int format) {
#ifndef CNN_NO_SERIALIZATION
  try {
    h->net.save(path, static_cast<content_type>(what), static_cast<file_format>(format));
    return 0;
  } catch (const std::exception &) { return -1; }
#else
  (void)h; (void)path; (void)what; (void)format;
  return -3;
#endif
}
int tdr_net_load_archive(tdr_net *h, const char *path, int what, int format) {
#ifndef CNN_NO_SERIALIZATION
  try {
    h->net.load(path, static_cast<content_type>(what), static_cast<file_format>(format));
    return 0;
  } catch (const std::exception &) { return -1; }
#else
  (void)h; (void)path; (void)what; (void)format;
  return -3;
#endif
}

/* io/mnist_parser.h, io/cifar10_parser.h. out_images: [count][len] floats (may be NULL to
 * query), out_labels: [count] int64. Returns the number of items, -1 on nn_error. */
long tdr_parse_mnist_images(const char *path, float scale_min, float scale_max, int x_pad, int y_pad,
                            float *out_images, size_t *len) {
  try {
    std::vector<vec_t> images;
    parse_mnist_images(path, &images, scale_min, scale_max, x_pad, y_pad);
    if (len) *len = images.empty() ? 0 : images[0].size();
    if (out_images)
      for (size_t i = 0; i < images.size(); i++)
        std::memcpy(out_images + i * images[0].size(), images[i].data(), sizeof(float) * images[0].size());
    return (long)images.size();
  } catch (const std::exception &) { return -1; }
}
long tdr_parse_mnist_labels(const char *path, int64_t *out_labels) {
  try {
    std::vector<label_t> labels;
    parse_mnist_labels(path, &labels);
    if (out_labels)
      for (size_t i = 0; i < labels.size(); i++) out_labels[i] = (int64_t)labels[i];
    return (long)labels.size();
  } catch (const std::exception &) { return -1; }
}
long tdr_parse_cifar10(const char *path, float scale_min, float scale_max, int x_pad, int y_pad,
                       float *out_images, int64_t *out_labels, size_t *len) {
  try {
    std::vector<vec_t> images;
    std::vector<label_t> labels;
    parse_cifar10(path, &images, &labels, scale_min, scale_max, x_pad, y_pad);
    if (len) *len = images.empty() ? 0 : images[0].size();
    for (size_t i = 0; i < images.size(); i++) {
      if (out_images) std::memcpy(out_images + i * images[0].size(), images[i].data(), sizeof(float) * images[0].size());
      if (out_labels) out_labels[i] = (int64_t)labels[i];
    }
    return (long)images.size();
  } catch (const std::exception &) { return -1; }
}

}  // extern "C"
