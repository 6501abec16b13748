/*
 * tdh.h — C ABI of libtdh.so: tiny-dnn's training hot path on one AMD Instinct
 * MI355X (gfx950), hand-written HIP.
 *
 * The entry points are what tiny-dnn's operator layer binds for this path: each
 * one replaces the body of an OpKernel::compute (or of the free function the
 * reference calls in its place) and is cited next to its declaration (paths
 * relative to the tiny-dnn tree).
 *
 * Conventions
 *  - Every tensor argument is a DEVICE pointer obtained from tdh_malloc, dense
 *    fp32, [batch][flat] with tiny-dnn's per-sample CHW layout
 *    index = (H*c + y)*W + x  (tiny_dnn/util/util.h:168-173). Conv weights are
 *    OIHW, fully-connected weights [in][out] row-major.
 *  - Convolution inputs/gradients are UNPADDED; padding::same is applied
 *    implicitly by the kernels (the reference copies into padded buffers,
 *    tiny_dnn/core/params/conv_params.h:106-166).
 *  - Weight/bias gradients are produced already reduced over the batch (the sum
 *    over samples that edge::merge_grads computes, tiny_dnn/node.h:89-103) in a
 *    fixed order: the same inputs always give the same bits.
 *  - All work is queued on one library-owned stream; calls return without
 *    waiting for the GPU except tdh_sync, tdh_memcpy_d2h and tdh_event_elapsed_ms.
 *  - Every function returns TDH_OK (0) or a negative tdh_status; the message for
 *    the last failure on the calling thread is tdh_last_error(). The C++ host
 *    layer turns failures into tiny_dnn::nn_error, the reference's convention
 *    (tiny_dnn/util/nn_error.h:19-26).
 *  - Single caller thread (the reference's training thread); not re-entrant.
 */
#ifndef TDH_H
#define TDH_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum tdh_status {
  TDH_OK                = 0,
  TDH_ERR_INVALID       = -1, /* bad argument / unsupported shape */
  TDH_ERR_HIP           = -2, /* a HIP runtime call failed */
  TDH_ERR_NOT_INIT      = -3, /* tdh_init has not been called */
  TDH_ERR_UNSUPPORTED   = -4, /* valid in the reference but not built here */
  TDH_ERR_OOM           = -5
} tdh_status;

/* activation_layer subclasses (tiny_dnn/activations/) */
enum { TDH_ACT_TANH = 0, TDH_ACT_RELU = 1, TDH_ACT_SOFTMAX = 2, TDH_ACT_SIGMOID = 3,
       TDH_ACT_LEAKY_RELU = 4, TDH_ACT_ELU = 5, TDH_ACT_SELU = 6, TDH_ACT_SOFTPLUS = 7,
       TDH_ACT_SOFTSIGN = 8, TDH_ACT_ASINH = 9, TDH_ACT_TANH_P1M2 = 10, TDH_ACT_NONE = -1 };
/* loss functions (tiny_dnn/lossfunctions/loss_function.h) */
enum { TDH_LOSS_MSE = 0, TDH_LOSS_CE_MULTICLASS = 1, TDH_LOSS_CE = 2 };
/* optimizers (tiny_dnn/optimizers/optimizer.h) */
enum { TDH_OPT_SGD = 0, TDH_OPT_MOMENTUM = 1, TDH_OPT_ADAM = 2, TDH_OPT_ADAGRAD = 3,
       TDH_OPT_RMSPROP = 4, TDH_OPT_ADAMAX = 5, TDH_OPT_NESTEROV = 6 };
/* layer kinds of a sequential network */
enum { TDH_L_CONV = 0, TDH_L_FC = 1, TDH_L_MAXPOOL = 2, TDH_L_AVEPOOL = 3, TDH_L_ACT = 4,
       TDH_L_BATCHNORM = 5, TDH_L_DROPOUT = 6 };

/* core::conv_params (tiny_dnn/core/params/conv_params.h:63-90) */
typedef struct tdh_conv_desc {
  int32_t in_w, in_h, in_c;
  int32_t k_w, k_h, out_c;
  int32_t w_stride, h_stride;
  int32_t w_dilation, h_dilation; /* forward only, as in the reference; backward needs 1 */
  int32_t pad_same;               /* 0 = padding::valid, 1 = padding::same */
  int32_t has_bias;
  const uint8_t *tbl;             /* HOST pointer: NULL or connection_table [in_c][out_c] */
} tdh_conv_desc;

/* core::maxpool_params (tiny_dnn/core/params/maxpool_params.h:17-34) and the
 * constructor arguments of average_pooling_layer */
typedef struct tdh_pool_desc {
  int32_t in_w, in_h, in_c;
  int32_t pool_w, pool_h;
  int32_t stride_w, stride_h;
  int32_t pad_same;
  int32_t ceil_mode;
} tdh_pool_desc;

/* Hyper-parameters plus the scalar state tiny-dnn keeps inside the optimizer
 * object: adam/adamax advance b1_t (and b2_t) once per update() call, i.e. once
 * per weight TENSOR (tiny_dnn/optimizers/optimizer.h:112-127,153-165). */
typedef struct tdh_opt {
  int32_t kind;
  float alpha, lambda, mu, b1, b2, eps;
  float b1_t, b2_t;
} tdh_opt;

typedef struct tdh_layer {
  int32_t kind;
  int32_t act; /* TDH_L_ACT: activation kind */
  tdh_conv_desc conv;
  tdh_pool_desc pool;
  int32_t fc_in, fc_out, fc_bias;
  float act_p[2]; /* TDH_L_ACT: constructor parameters of the kinds that have them (see tdh_act_fwd_p) */
  /* TDH_L_BATCHNORM: batch_normalization_layer(in_spatial_size, in_channels, epsilon, momentum)
   * (tiny_dnn/layers/batch_normalization_layer.h:54-72); tensors are [batch][channels][spatial] */
  int32_t bn_channels, bn_spatial;
  float bn_eps, bn_momentum;
  /* TDH_L_DROPOUT: dropout_layer(in_dim, dropout_rate) (tiny_dnn/layers/dropout_layer.h:32-39);
   * in_dim is the size of the layer in front */
  float dropout_rate;
} tdh_layer;

/* ------------------------------------------------------------ library state */
int tdh_init(int device);
int tdh_shutdown(void);
const char *tdh_last_error(void);
const char *tdh_version(void);
/* name, compute units and memory of the device selected by tdh_init */
int tdh_device_info(char *name, size_t name_len, int32_t *compute_units, size_t *global_mem_bytes);

/* ----------------------------------------------------------- device memory */
int tdh_malloc(void **dptr, size_t bytes);
int tdh_free(void *dptr);
int tdh_memcpy_h2d(void *dst, const void *src, size_t bytes);
int tdh_memcpy_d2h(void *dst, const void *src, size_t bytes); /* waits for queued work */
int tdh_memcpy_d2d(void *dst, const void *src, size_t bytes);
int tdh_fill_zero(void *dptr, size_t bytes);                  /* fill kernel, graph-safe */
int tdh_sync(void);

/* timing on the library stream */
int tdh_event_create(void **event);
int tdh_event_destroy(void *event);
int tdh_event_record(void *event);
int tdh_event_elapsed_ms(void *start, void *stop, float *ms); /* waits for `stop` */

/* Per-kernel timing of everything launched between begin and end: each launch carries
 * a pair of events that the runtime stamps with the begin and the end of that kernel's
 * execution, and is booked under a kernel tag with its algorithmic work (unit 0 = FLOP,
 * 1 = bytes); a tag's time is the sum over its kernels. A captured train step runs
 * eagerly while profiling is on, so whole-step throughput is measured with profiling
 * off. tdh_profile_end waits for the GPU; entries are then read back by index, ordered
 * by total time (largest first). */
int tdh_profile_begin(void);
int tdh_profile_end(int32_t *n_entries);
int tdh_profile_entry(int32_t index, char *tag, size_t tag_len, int64_t *launches,
                      double *total_ms, double *work_per_launch, int32_t *work_unit);
/* The tag of the index-th kernel launch of the profiled region, in dispatch order ("-" for a
 * launch outside any tag); TDH_ERR_INVALID (no error text) past the last one. It lets a trace
 * of the same run, which knows kernels only by symbol, be read tag by tag. */
int tdh_profile_launch(int32_t index, char *tag, size_t tag_len);
/* A mark in the kernel stream that a trace can find: three launches of the fill kernel on
 * `dptr` (which they clear), booked under the tag "profile_mark", never under the tag of a
 * workload's own fills. */
int tdh_profile_mark(void *dptr, size_t bytes);

/* shape helpers: conv_out_length / pool_out_length (tiny_dnn/util/util.h:329-363) */
int tdh_conv_out_w(const tdh_conv_desc *d);
int tdh_conv_out_h(const tdh_conv_desc *d);
int tdh_pool_out_w(const tdh_pool_desc *d);
int tdh_pool_out_h(const tdh_pool_desc *d);

/* ------------------------------------------------------------- convolution */
/* Conv2dOp::compute (tiny_dnn/core/kernels/conv2d_op.h:23-51,
 * conv2d_op_internal.h:13-74): y = conv(x, w) + b */
int tdh_conv2d_fwd(const tdh_conv_desc *d, int batch, const float *x, const float *w,
                   const float *b, float *y);
/* Conv2dGradOp::compute (tiny_dnn/core/kernels/conv2d_grad_op.h:22-50,
 * conv2d_op_internal.h:78-181). dx is overwritten; dw/db are overwritten
 * (accumulate = 0) or added to (accumulate = 1, the reference's += into gradients
 * that update_weight later clears). Any of dx, dw, db may be NULL to skip it. */
int tdh_conv2d_bwd(const tdh_conv_desc *d, int batch, const float *x, const float *w,
                   const float *dy, float *dx, float *dw, float *db, int accumulate);

/* tdh_conv2d_bwd for callers that cannot allocate (tight serving loops, harnesses that forbid
 * hipMalloc). It has no counterpart in the reference. It is refused (TDH_ERR_INVALID) while a
 * network step of this library is being captured or holds the scratch buffer, and
 * (TDH_ERR_UNSUPPORTED) for a descriptor with a connection table. Same
 * arguments, kernels and results as tdh_conv2d_bwd, but the kernels' scratch (split partial
 * sums, repacked filters) lies in a static 64 MiB device array that the library holds on every
 * device it is initialised on, and the call allocates and frees nothing. A shape whose scratch
 * need exceeds the array is refused with TDH_ERR_INVALID (the message states both sizes); use
 * tdh_conv2d_bwd for it. All calls on one GPU share that GPU's array: calls are ordered by the
 * library stream, two processes' or threads' calls that overlap on one GPU would race. */
int tdh_conv2d_bwd_static(const tdh_conv_desc *d, int batch, const float *x, const float *w,
                          const float *dy, float *dx, float *dw, float *db, int accumulate);

/* --------------------------------------------------------- fully connected */
/* FullyConnectedOp::compute (tiny_dnn/core/kernels/fully_connected_op.h:25-63,
 * fully_connected_op_internal.h:15-36) */
int tdh_fc_fwd(int in, int out, int has_bias, int batch, const float *x, const float *w,
               const float *b, float *y);
/* FullyConnectedGradOp::compute (tiny_dnn/core/kernels/fully_connected_grad_op.h:22-52,
 * fully_connected_op_internal.h:38-71) */
int tdh_fc_bwd(int in, int out, int has_bias, int batch, const float *x, const float *w,
               const float *dy, float *dx, float *dw, float *db, int accumulate);

/* ----------------------------------------------------------------- pooling */
/* MaxPoolOp::compute (tiny_dnn/core/kernels/maxpool_op.h:23-61,
 * maxpool_op_internal.h:16-40). argmax[batch][out] = flat per-sample CHW index of
 * the first maximum in (dy,dx) scan order (the reference's out2inmax, held as
 * int32 here). */
int tdh_maxpool_fwd(const tdh_pool_desc *d, int batch, const float *x, float *y,
                    int32_t *argmax);
/* MaxPoolGradOp::compute (tiny_dnn/core/kernels/maxpool_grad_op.h:22-46,
 * maxpool_op_internal.h:42-57) */
int tdh_maxpool_bwd(const tdh_pool_desc *d, int batch, const float *dy, const int32_t *argmax,
                    float *dx);
/* AvePoolOp: tiny_average_pooling_kernel (tiny_dnn/layers/average_pooling_layer.h:25-55);
 * w and b hold one trainable scale / bias per channel */
int tdh_avepool_fwd(const tdh_pool_desc *d, int batch, const float *x, const float *w,
                    const float *b, float *y);
/* AvePoolGradOp: tiny_average_pooling_back_kernel
 * (tiny_dnn/layers/average_pooling_layer.h:58-106) */
int tdh_avepool_bwd(const tdh_pool_desc *d, int batch, const float *x, const float *w,
                    const float *dy, float *dx, float *dw, float *db, int accumulate);

/* ------------------------------------------------- activations and losses */
/* activation_layer::forward_propagation / back_propagation
 * (tiny_dnn/activations/activation_layer.h:74-91; tanh_layer.h:24-38,
 * relu_layer.h:25-39, softmax_layer.h:24-55, sigmoid_layer.h:24-38).
 * len = per-sample vector length; the backward uses the layer OUTPUT y. */
int tdh_act_fwd(int kind, int batch, int len, const float *x, float *y);
int tdh_act_bwd(int kind, int batch, int len, const float *y, const float *dy, float *dx);
/* The same for every activation layer, with the layer's constructor parameters p[2]:
 * leaky_relu {epsilon} (leaky_relu_layer.h:74-88), elu {alpha} (elu_layer.h:37-52),
 * selu {lambda, alpha} (selu_layer.h:82-99), softplus {beta, threshold}
 * (softplus_layer.h:84-102), softsign (softsign_layer.h:24-40), asinh (asinh_layer.h:24-38),
 * tanh_p1m2 (tanh_p1m2_layer.h:24-40); p is ignored by the other kinds and NULL selects the
 * constructor defaults. The backward takes the layer input x as well, as the reference's
 * backward_activation does: selu and softsign read it (x may be NULL for the others).
 * tdh_act_fwd / tdh_act_bwd are these calls with p = NULL and x = NULL. */
void tdh_act_default_params(int kind, float *p);
int tdh_act_fwd_p(int kind, const float *p, int batch, int len, const float *x, float *y);
int tdh_act_bwd_p(int kind, const float *p, int batch, int len, const float *x, const float *y,
                  const float *dy, float *dx);
/* batch_normalization_layer (tiny_dnn/layers/batch_normalization_layer.h:127-169): tensors are
 * [batch][channels][spatial]. train != 0: mean and variance receive this batch's moments
 * (util/math_functions.h:25-96: variance over max(1, batch*spatial - 1)); train == 0: they are
 * read (the moving averages). stddev[c] = sqrt(variance[c] + eps) is written either way and is
 * what the backward pass divides by. y = (x - mean) / stddev. */
int tdh_batchnorm_fwd(int channels, int spatial, int batch, float eps, int train, const float *x,
                      float *mean, float *variance, float *stddev, float *y);
/* batch_normalization_layer::back_propagation (batch_normalization_layer.h:87-125):
 * dx = (dy - mean(dy) - mean(dy*y) * y) / stddev, means per channel over batch and space */
int tdh_batchnorm_bwd(int channels, int spatial, int batch, const float *y, const float *dy,
                      const float *stddev, float *dx);
/* batch_normalization_layer::post_update (batch_normalization_layer.h:171-177):
 * mean = momentum*mean + (1-momentum)*mean_cur, the same for the variance */
int tdh_batchnorm_update_moving(int channels, float momentum, const float *mean_cur,
                                const float *var_cur, float *mean, float *variance);
/* dropout_layer (tiny_dnn/layers/dropout_layer.h:84-117): mask is [batch][len] bytes of 0/1, drawn
 * by the caller as the reference draws it (bernoulli(rate) per element, sample after sample);
 * train != 0: y = mask * scale * x with scale = 1/(1-rate), else y = x (mask may be NULL).
 * Backward (dropout_layer.h:62-82): dx = mask * dy, without the scale. */
int tdh_dropout_fwd(int batch, int len, int train, float scale, const uint8_t *mask, const float *x,
                    float *y);
int tdh_dropout_bwd(int batch, int len, const uint8_t *mask, const float *dy, float *dx);
/* gradient<E> for a mini-batch (tiny_dnn/lossfunctions/loss_function.h:191-218) */
int tdh_loss_grad(int kind, int batch, int len, const float *y, const float *t, float *dy);
/* softmax_layer backward applied to cross_entropy_multiclass::df in one kernel:
 * dz = y * sum(t) - t  (= y - t for one-hot targets) */
int tdh_softmax_xent_grad(int batch, int len, const float *y, const float *t, float *dz);

/* -------------------------------------------------------------- optimizers */
/* layer::update_weight for one tensor (tiny_dnn/layers/layer.h:663-682) followed by
 * optimizer::update (tiny_dnn/optimizers/optimizer.h): g = merged_grad * grad_scale,
 * then the update of `kind`. tiny-dnn's own grad_scale is 1 (its rcp_batch_size is
 * taken from the weight edge, whose data tensor has one entry). s0/s1 are the
 * optimizer's per-weight state vectors (may be NULL where unused). *o is updated on
 * the host exactly as the reference updates b1_t/b2_t. */
int tdh_opt_update(tdh_opt *o, size_t n, const float *merged_grad, float grad_scale, float *w,
                   float *s0, float *s1);
void tdh_opt_default(tdh_opt *o, int kind);

/* ------------------------------------------------------ sequential network */
/* network<sequential>::fit / train_onebatch (tiny_dnn/network.h:840-926) with
 * every tensor resident on the device. */
typedef struct tdh_net tdh_net;

enum {
  TDH_NET_FUSE_ACT_GRAD = 1, /* fold activation gradients into the next layer's dX epilogue */
  TDH_NET_GRAPH         = 2, /* replay the step as a captured HIP graph */
  /* A net whose activations of one sample fit in a workgroup's local memory (LeNet-5) trains in
   * three launches: one workgroup per sample runs forward, the loss gradient and the input
   * gradients of every layer; a second launch computes every sample's weight and bias
   * gradients; the optimizer launch adds those up and updates (a step without an update adds
   * them to the gradient tensors in sample order instead, edge::merge_grads,
   * tiny_dnn/node.h:89-103). Every layer output, input gradient and max-pool record is still
   * written to memory. Nets that do not qualify (size, batch normalization, dropout, a softmax
   * that is not the closing layer of a cross_entropy_multiclass net) ignore the flag. */
  TDH_NET_SAMPLE_STEP   = 4,
  /* Training never reads the gradient with respect to the net's input, which the reference
   * computes like every other (layer::backward of the first layer fills the gradient of its
   * data edge, tiny_dnn/layers/layer.h:557-575). With this flag a net whose first layer is a
   * convolution or a fully-connected layer leaves that product out: tdh_net_layer_dx(net, 0)
   * returns NULL after a step, everything else is what it is without the flag. Other first
   * layers ignore the flag. */
  TDH_NET_NO_INPUT_GRAD = 8
};

int tdh_net_create(const tdh_layer *layers, int n_layers, int max_batch, int flags,
                   tdh_net **net);
int tdh_net_destroy(tdh_net *net);
size_t tdh_net_in_size(const tdh_net *net);
size_t tdh_net_out_size(const tdh_net *net);
size_t tdh_net_layer_out_size(const tdh_net *net, int layer);
/* which: 0 = weight, 1 = bias; of a batch-norm layer (which has neither) 2 = moving mean,
 * 3 = moving variance (batch_normalization_layer.h:171-202, one value per channel, not touched
 * by the optimizer); sizes in floats */
size_t tdh_net_param_size(const tdh_net *net, int layer, int which);
int tdh_net_set_param(tdh_net *net, int layer, int which, const float *host_src);
int tdh_net_get_param(tdh_net *net, int layer, int which, float *host_dst);
/* optimizer::reset() as network::fit calls it before training (tiny_dnn/network.h:856,
 * tiny_dnn/optimizers/optimizer.h:36-38): clears the per-weight state vectors */
int tdh_net_reset_optimizer(tdh_net *net);
/* network::set_netphase (tiny_dnn/network.h:438-442): train != 0 is net_phase::train, the
 * state of a new net. In the train phase a batch-norm layer normalises by the moments of the
 * batch and every update moves its running averages (post_update), a dropout layer applies
 * its mask; in the test phase batch-norm uses the running averages and dropout is the identity. */
int tdh_net_set_phase(tdh_net *net, int train);
/* The mask that the following passes of dropout layer `layer` apply: host bytes [batch][len] of
 * 0/1, drawn by the caller as the reference draws them (bernoulli(dropout_rate) per element,
 * sample after sample, tiny_dnn/layers/dropout_layer.h:99-102), once per train step. The copy
 * is queued on the library stream, behind the kernels of the step before. */
int tdh_net_set_dropout_mask(tdh_net *net, int layer, int batch, const uint8_t *host_mask);
/* nodes::update_weights (tiny_dnn/nodes.h:103-107): layer::update_weight of every layer, front
 * to back, weight before bias, on the gradients accumulated since the last update, which are
 * then cleared (tiny_dnn/layers/layer.h:663-682). What tdh_net_train_step does with
 * do_update != 0, as a call of its own (network::update_weights, tiny_dnn/network.h:209-213). */
int tdh_net_update_weights(tdh_net *net, tdh_opt *opt);
/* nodes::clear_grads (tiny_dnn/nodes.h:118-122): zeroes every weight and bias gradient */
int tdh_net_clear_grads(tdh_net *net);
/* device views valid until the net is destroyed */
float *tdh_net_param(tdh_net *net, int layer, int which);
/* the layer's output as the last pass left it, or NULL where that pass never wrote it to
 * memory: in a train step with TDH_NET_FUSE_ACT_GRAD a convolution kernel that also writes the
 * pointwise activation or computes the 2x2 max-pool behind the convolution keeps the
 * convolution's own output in registers (nothing in the backward pass reads it: the gradients
 * of tanh, relu and sigmoid are functions of their outputs); tdh_net_forward always writes it */
const float *tdh_net_layer_out(const tdh_net *net, int layer);
/* the gradient with respect to the layer's input as the last step left it, or NULL where
 * that step never wrote it to memory: with TDH_NET_FUSE_ACT_GRAD the gradient of a folded
 * activation's output only exists in registers, and the backward kernels of a first
 * convolution (few input channels, stride 1) in front of a 2x2 / stride-2 max-pool read the
 * pooled gradient and the argmax records instead of the pool's input gradient */
const float *tdh_net_layer_dx(const tdh_net *net, int layer);
const float *tdh_net_layer_grad(const tdh_net *net, int layer, int which);
const int32_t *tdh_net_layer_argmax(const tdh_net *net, int layer);
/* x: [batch][in_size], t: [batch][out_size], device pointers */
int tdh_net_forward(tdh_net *net, int batch, const float *x);
/* fprop, loss gradient, bprop and (do_update != 0) update_weights + clear_grads */
int tdh_net_train_step(tdh_net *net, tdh_opt *opt, int loss_kind, int batch, const float *x,
                       const float *t, int do_update);
/* n_steps (1 to 8) consecutive train steps with update, step s on the mini-batch x[s], t[s]
 * (arrays of device pointers, which may repeat): what the loop over mini-batches of
 * network::fit does (tiny_dnn/network.h:866-879, one train_once per mini-batch) when the
 * batches are on the device already. The results are those of n_steps calls of
 * tdh_net_train_step; with TDH_NET_GRAPH the steps are captured into one graph, so a replay
 * starts once for all of them (a few microseconds each time, which is a tenth of a LeNet-5
 * step). A net with a dropout layer in the train phase is refused: its masks change between
 * the steps (tdh_net_set_dropout_mask). */
int tdh_net_train_steps(tdh_net *net, tdh_opt *opt, int loss_kind, int batch, int n_steps,
                        const float *const *x, const float *const *t);

/* ------------------------------------------------ batches from host memory */
/* network::fit hands each mini-batch over as host vectors (tiny_dnn/network.h:866-879;
 * layer::set_in_data copies them into the first layer, tiny_dnn/layers/layer.h:230-251).
 * A feeder takes them ahead of time: tdh_feeder_stage hands a batch in pageable host memory to
 * a worker thread of the feeder, which copies it into a pinned slot and queues its upload on a
 * copy stream at once; tdh_feeder_acquire makes the library stream wait for the upload of the
 * oldest staged batch and returns the device pointers to hand to tdh_net_train_step /
 * tdh_net_forward. Up to two batches may be staged and not yet acquired (stage, stage, then
 * acquire, stage, step, acquire, stage, step ...: the upload of a batch then overlaps the step
 * before it; staging one batch ahead works as well), a third is refused with TDH_ERR_INVALID.
 * x: [batch][x_len], t: [batch][t_len] floats; x_host / t_host must stay valid and unchanged
 * until the tdh_feeder_acquire that returns that batch. Queue every piece of work that reads a
 * batch before acquiring the next one: its device slot is reused by the second stage call
 * after that. */
typedef struct tdh_feeder tdh_feeder;
int tdh_feeder_create(size_t x_len, size_t t_len, int max_batch, tdh_feeder **feeder);
int tdh_feeder_destroy(tdh_feeder *feeder);
int tdh_feeder_stage(tdh_feeder *feeder, int batch, const float *x_host, const float *t_host);
int tdh_feeder_acquire(tdh_feeder *feeder, const float **x_dev, const float **t_dev, int *batch);

#ifdef __cplusplus
}
#endif
#endif /* TDH_H */
