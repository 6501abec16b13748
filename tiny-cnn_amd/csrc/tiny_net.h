// tiny_net.h — plan of the workgroup-per-sample train step of a small net (tiny_net.hip);
// built by net.hip from a network's layers.
#pragma once

#include "common.h"

namespace tdh {

constexpr int TINY_MAX_LAYERS     = 16;
constexpr int TINY_MAX_TENSORS    = 2 * TINY_MAX_LAYERS;
constexpr size_t TINY_LDS_MAX_BYTES = 152u << 10;  // of a compute unit's 160 KiB
constexpr int TINY_SCRATCH_FLOATS = 4096;          // LDS where the partial sums of a split layer meet
constexpr int TINY_MAX_JOBS       = 256;           // pieces of the parameter-gradient kernel's work per sample

struct TinyLayer {
  int kind, act;               // TDH_L_*, TDH_ACT_* (activation layers)
  float p0;                    // leaky relu's slope
  int C, H, W, K, OH, OW;      // input channels / size, output channels / size (conv, pools)
  int R, S, sh, sw, ph, pw;    // window rows / columns, strides, padding in front
  int in_size, out_size, has_bias;
  float scale;                 // average pooling: 1 / (window elements)
  const float *w, *b;
  const uint8_t *tbl;          // conv connection table [C][K], or NULL
  float *out;                  // memory: this layer's output [batch][out_size]
  float *dx;                   // memory: gradient w.r.t. this layer's input [batch][in_size]
  int32_t *argmax;             // memory: max-pool records [batch][out_size]
  float *gw, *gb;              // memory: per-sample gradient slices [batch][nw], [batch][nb]
  int nw, nb;
  int lds_in, lds_out;         // where the layer's input and output live in LDS (floats)
  // divisions by the layer's sizes as multiply-high + shift
  FastDiv d_oplane, d_ow, d_iplane, d_w, d_taps, d_s, d_c, d_out, d_nk;
  // the unrolled input gradient of a stride-1 3x3 / 5x5 convolution reads dY from a zero-framed copy,
  // [K][H + R - 1][W + S - 1] floats in LDS; 0 when the layer takes the general loops
  int dx_framed;
  FastDiv d_pplane, d_pw;
  // A stride-1 convolution's forward product without padding on the matrix cores (conv_mfma in
  // tiny_net.hip): where in LDS the step kernel keeps the filters as [co][k] (k = (ci, tap), rows
  // padded with zeros), the input offset of every k and a copy of the bias; -1: the scalar loops
  int mf_fwd_w, mf_fwd_ko, mf_fwd_b;
  // The input gradient of the layer whose filters wait in registers (TinyPlan::mf_ahead), from the
  // framed dY, as the same kind of product with the filter columns folded into the rows:
  //   D[(ci, wx)][iy][px] = sum over (co, wy) of W[co][ci][wy][wx] * framed[co][iy + R-1-wy][px]
  // (C * S rows, K * R terms a sum, every position of H framed rows a column), then
  //   dX[ci][iy][ix] = sum over wx of D[(ci, wx)][iy][ix + S-1-wx].
  // mf_dx_w / mf_dx_ko: the operand [(ci, wx)][(co, wy)] and its offset table, written into the
  // scratch area in front of the phase; mf_dx_d: D. -1: the scalar loops.
  int mf_dx_w, mf_dx_ko, mf_dx_d;
};

// One workgroup's share of the parameter-gradient kernel for one sample: the units
// [base, base + count) of a layer's weight-gradient work (the bias gradient goes with base 0,
// except that of a convolution that is not a matrix-vector product, which is a job of its own),
// or, for the first layer, the wave items [base, base + count) of its input gradient.
struct TinyJob {
  int16_t layer, what;         // what: 0 = weight (/ bias) gradient, 1 = input gradient, 2 = bias gradient
  int base, count;
};

struct TinyPlan {
  TinyLayer l[TINY_MAX_LAYERS];
  int n, in_size;
  int lds_g0, lds_g1, lds_w, lds_pad, lds_floats;   // lds_pad: the zero-framed dY
  int n_mfma, mfma_layers[TINY_MAX_LAYERS];   // the layers with operands to stage for the matrix cores
  int mf_ahead;                // the layer (> 0) whose filters wait in registers until the layer in front of it runs, or -1
  float mse_factor;            // 2 / outputs
  float *dloss;                // memory: gradient w.r.t. the net's output [batch][out_size]
  double flop_per_sample;
  TinyJob jobs[TINY_MAX_JOBS];
  int n_jobs;
  int first_dx_as_job;         // the first layer's input gradient is among the jobs
  int skip_first_dx;           // nobody wants the gradient of the net's input: it is not computed
  int lds_job_floats;          // LDS of the parameter-gradient kernel
};

// the per-sample slices of every trainable tensor and the gradient tensor each is added to
struct TinyMerge {
  const float *slices[TINY_MAX_TENSORS];
  float *g[TINY_MAX_TENSORS];
  int len[TINY_MAX_TENSORS];
  int first_block[TINY_MAX_TENSORS + 1];
  int n;
};

// raises the kernel's LDS limit; once, outside any stream capture
int tiny_prepare();
// dev_plan: the plan in device memory (the kernel walks its layers by index, which a kernel
// argument passed by value would pay for with a private copy per thread); loss, softmax_xent:
// this step's loss and whether the closing softmax folds into it
int launch_tiny_step(const TinyPlan &plan, const TinyPlan *dev_plan, int loss, int softmax_xent, int batch,
                     const float *x, const float *t);
// Cuts the parameter-gradient work of the plan's layers into jobs, decides which layers' input
// gradients read a zero-framed dY and appends that area to the plan's LDS (lds_floats comes
// in as the floats in use so far; the caller checks the result against TINY_LDS_MAX_BYTES).
int tiny_build_jobs(TinyPlan &plan);
// every layer's per-sample weight and bias gradient slices (and the first layer's input
// gradient) from the outputs and gradients that launch_tiny_step left in memory
int launch_tiny_params(const TinyPlan &plan, const TinyPlan *dev_plan, int batch, const float *x);
int launch_tiny_merge(const TinyMerge &m, int batch);

}  // namespace tdh
