/*
 * td_oracle.h — CPU restatement of tiny-dnn's training hot path (TEST INFRASTRUCTURE ONLY).
 *
 * This is the checker the HIP path is compared against. It is never linked
 * into, imported by or called from the product library. Only the test-suite,
 * the smoke check and the cpu_baseline leg of the benchmark may load it.
 *
 * All tensors are dense fp32, [batch][flat] with the reference's per-sample
 * CHW layout: index = (H*c + y)*W + x   (tiny_dnn/util/util.h:168-173).
 * Conv weights are OIHW, FC weights are [in][out] row-major.
 *
 * Weight/bias gradients are returned MERGED: the in-order sum over samples of
 * the per-sample gradients, i.e. what edge::merge_grads (tiny_dnn/node.h:89-103)
 * produces. layer::update_weight (tiny_dnn/layers/layer.h:663-682) multiplies it
 * by 1/size-of-the-weight-edge's-data-tensor, which is 1: the optimizer sees the
 * SUM over the batch, not the mean.
 *
 * Pinning status of each function (what fixes its behaviour independently of
 * this file) is listed in td_oracle.c above each definition and checked by
 * tests/test_oracle_*.py.
 */
#ifndef TD_ORACLE_H
#define TD_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct tdo_conv_desc {
  int32_t in_w, in_h, in_c;
  int32_t k_w, k_h, out_c;
  int32_t w_stride, h_stride;
  int32_t w_dilation, h_dilation;
  int32_t pad_same; /* 0 = padding::valid, 1 = padding::same */
  int32_t has_bias;
  const uint8_t *tbl; /* NULL or [in_c][out_c] connection table (1 = connected) */
} tdo_conv_desc;

typedef struct tdo_pool_desc {
  int32_t in_w, in_h, in_c;
  int32_t pool_w, pool_h;
  int32_t stride_w, stride_h;
  int32_t pad_same;
  int32_t ceil_mode;
} tdo_pool_desc;

enum { TDO_ACT_TANH = 0, TDO_ACT_RELU = 1, TDO_ACT_SOFTMAX = 2, TDO_ACT_SIGMOID = 3,
       TDO_ACT_LEAKY_RELU = 4, TDO_ACT_ELU = 5, TDO_ACT_SELU = 6, TDO_ACT_SOFTPLUS = 7,
       TDO_ACT_SOFTSIGN = 8, TDO_ACT_ASINH = 9, TDO_ACT_TANH_P1M2 = 10 };
enum { TDO_LOSS_MSE = 0, TDO_LOSS_CE_MULTICLASS = 1, TDO_LOSS_CE = 2 };
enum { TDO_OPT_SGD = 0, TDO_OPT_MOMENTUM = 1, TDO_OPT_ADAM = 2, TDO_OPT_ADAGRAD = 3,
       TDO_OPT_RMSPROP = 4, TDO_OPT_ADAMAX = 5, TDO_OPT_NESTEROV = 6 };

/* optimizer hyper-parameters + the scalar state the reference keeps in the
 * optimizer object (b1_t/b2_t advance once per update() call). */
typedef struct tdo_opt {
  int32_t kind;
  float alpha, lambda, mu, b1, b2, eps;
  float b1_t, b2_t;
} tdo_opt;

void tdo_opt_default(tdo_opt *o, int kind);

/* shape helpers */
int tdo_conv_out_w(const tdo_conv_desc *d);
int tdo_conv_out_h(const tdo_conv_desc *d);
int tdo_conv_padded_w(const tdo_conv_desc *d);
int tdo_conv_padded_h(const tdo_conv_desc *d);
int tdo_pool_out_w(const tdo_pool_desc *d);
int tdo_pool_out_h(const tdo_pool_desc *d);

/* convolution; x is UNPADDED [batch][in_c*in_h*in_w]; dx likewise */
int tdo_conv2d_fwd(const tdo_conv_desc *d, int batch, const float *x, const float *w,
                   const float *b, float *y);
int tdo_conv2d_bwd(const tdo_conv_desc *d, int batch, const float *x, const float *w,
                   const float *dy, float *dx, float *dw, float *db);

/* fully connected */
int tdo_fc_fwd(int in, int out, int has_bias, int batch, const float *x, const float *w,
               const float *b, float *y);
int tdo_fc_bwd(int in, int out, int has_bias, int batch, const float *x, const float *w,
               const float *dy, float *dx, float *dw, float *db);

/* max pooling; argmax holds the flat per-sample CHW input index */
int tdo_maxpool_fwd(const tdo_pool_desc *d, int batch, const float *x, float *y,
                    int64_t *argmax);
int tdo_maxpool_bwd(const tdo_pool_desc *d, int batch, const float *dy,
                    const int64_t *argmax, float *dx);

/* average pooling with trainable per-channel scale w[c] and bias b[c] */
int tdo_avepool_fwd(const tdo_pool_desc *d, int batch, const float *x, const float *w,
                    const float *b, float *y);
int tdo_avepool_bwd(const tdo_pool_desc *d, int batch, const float *x, const float *w,
                    const float *dy, float *dx, float *dw, float *db);

/* activations: len = per-sample vector length */
int tdo_act_fwd(int kind, int batch, int len, const float *x, float *y);
int tdo_act_bwd(int kind, int batch, int len, const float *x, const float *y,
                const float *dy, float *dx);
/* the same with the layer's constructor parameters p[2]: leaky-relu {epsilon}, elu {alpha},
 * selu {lambda, alpha}, softplus {beta, threshold}; ignored by the other kinds */
void tdo_act_default_params(int kind, float *p);
int tdo_act_fwd_p(int kind, const float *p, int batch, int len, const float *x, float *y);
int tdo_act_bwd_p(int kind, const float *p, int batch, int len, const float *x, const float *y,
                  const float *dy, float *dx);

/* batch normalization over [batch][channels][spatial] (batch_normalization_layer.h,
 * util/math_functions.h:25-96); train != 0 computes mean/variance from x, else reads them */
int tdo_batchnorm_fwd(int channels, int spatial, int batch, float eps, int train, const float *x,
                      float *mean, float *variance, float *stddev, float *y);
int tdo_batchnorm_bwd(int channels, int spatial, int batch, const float *y, const float *dy,
                      const float *stddev, float *dx);
void tdo_batchnorm_update_moving(int channels, float momentum, const float *mean_cur,
                                 const float *var_cur, float *mean, float *variance);
/* dropout (dropout_layer.h): mask [batch][len] of 0/1 */
int tdo_dropout_fwd(int batch, int len, int train, float scale, const unsigned char *mask,
                    const float *x, float *y);
int tdo_dropout_bwd(int batch, int len, const unsigned char *mask, const float *dy, float *dx);
/* The reference's generator (util/random.h:19-69): one std::mt19937, seeded with 1 unless
 * set_random_seed is called, and bernoulli(p) = uniform_real_distribution<float>(0,1) <= p.
 * state: 625 words (624 of MT19937 state, then the position); tdo_mt_seed fills it. */
void tdo_mt_seed(unsigned int *state, unsigned int seed);
/* mask[i] = bernoulli(rate) for n elements, advancing state */
void tdo_dropout_mask(unsigned int *state, float rate, size_t n, unsigned char *mask);

/* loss gradient for a mini-batch (no 1/batch factor, as in the reference) */
int tdo_loss_grad(int kind, int batch, int len, const float *y, const float *t, float *dy);
float tdo_loss_value(int kind, int batch, int len, const float *y, const float *t);

/* optimizer::update on an already merged+scaled gradient g (s0/s1: state vectors) */
int tdo_opt_update(tdo_opt *o, size_t n, const float *g, float *w, float *s0, float *s1);
/* layer::update_weight for one tensor: g = merged * (1/weight_edge_samples), then update.
 * In the reference weight_edge_samples is always 1 (see td_oracle.c). */
int tdo_update_weight(tdo_opt *o, size_t n, int weight_edge_samples, const float *merged,
                      float *w, float *s0, float *s1);

/* ---- sequential network (one train step = fprop, loss grad, bprop, update) ---- */
enum { TDO_L_CONV = 0, TDO_L_FC = 1, TDO_L_MAXPOOL = 2, TDO_L_AVEPOOL = 3, TDO_L_ACT = 4,
       TDO_L_BATCHNORM = 5, TDO_L_DROPOUT = 6 };

typedef struct tdo_layer {
  int32_t kind;
  int32_t act; /* TDO_L_ACT: activation kind */
  tdo_conv_desc conv;
  tdo_pool_desc pool;
  int32_t fc_in, fc_out, fc_bias;
  float act_p[2]; /* TDO_L_ACT: parameters of the kinds that have them */
  int32_t bn_channels, bn_spatial; /* TDO_L_BATCHNORM: [batch][channels][spatial] */
  float bn_eps, bn_momentum;
  float dropout_rate;              /* TDO_L_DROPOUT (shape inherited from the layer in front) */
} tdo_layer;

typedef struct tdo_net tdo_net;

tdo_net *tdo_net_create(const tdo_layer *layers, int n_layers, int max_batch);
/* network::set_netphase (tiny_dnn/network.h:438-442): train != 0 is net_phase::train (the
 * state of a new net, and what fit sets); batch-norm and dropout layers behave by it */
void tdo_net_set_phase(tdo_net *net, int train);
/* the mask [max_batch][len] the next forward pass of dropout layer i applies (the caller draws
 * it, tdo_dropout_mask); which = 0 / 1: moving mean / variance of batch-norm layer i */
unsigned char *tdo_net_dropout_mask(tdo_net *net, int i);
float *tdo_net_bn_stat(tdo_net *net, int i, int which);
void tdo_net_destroy(tdo_net *net);
int tdo_net_num_layers(const tdo_net *net);
size_t tdo_net_in_size(const tdo_net *net);
size_t tdo_net_out_size(const tdo_net *net);
/* per layer: weight count, bias count, out size */
size_t tdo_net_weight_size(const tdo_net *net, int layer);
size_t tdo_net_bias_size(const tdo_net *net, int layer);
size_t tdo_net_layer_out_size(const tdo_net *net, int layer);
float *tdo_net_weight(tdo_net *net, int layer);
float *tdo_net_bias(tdo_net *net, int layer);
/* after a step: layer outputs [batch][out], merged dW/db, dX (grad wrt layer input) */
const float *tdo_net_layer_out(const tdo_net *net, int layer);
const float *tdo_net_layer_dx(const tdo_net *net, int layer);
const float *tdo_net_layer_dw(const tdo_net *net, int layer);
const float *tdo_net_layer_db(const tdo_net *net, int layer);
const int64_t *tdo_net_layer_argmax(const tdo_net *net, int layer);
int tdo_net_forward(tdo_net *net, int batch, const float *x);
/* full step; returns 0 on success. do_update = 0 leaves weights untouched */
int tdo_net_train_step(tdo_net *net, tdo_opt *opt, int loss_kind, int batch, const float *x,
                       const float *t, int do_update);

#ifdef __cplusplus
}
#endif
#endif
