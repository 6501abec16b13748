// common.h — library context, error plumbing and small device helpers shared by
// every translation unit of libtdh.so.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "../../include/tdh.h"

namespace tdh {

// ---------------------------------------------------------------- context
struct Context {
  bool ready            = false;
  int device            = -1;
  hipStream_t stream    = nullptr;
  int compute_units     = 0;
  size_t global_mem     = 0;
  char name[256]        = {0};
  // grow-only scratch for split-K partial sums and staged reductions; every public op
  // reserves its whole need up front (ws_begin) and then carves pieces off (ws_take), so
  // the buffer never moves while an op is queueing kernels
  char *workspace       = nullptr;
  size_t workspace_size = 0;
  size_t workspace_off  = 0;
  bool ws_locked        = false;  // a network owns the reservation: ops must fit, never grow
  bool ws_keep          = false;  // ws_begin does not rewind: pieces handed out stay disjoint
  // a train step collects the split reductions of its weight gradients and the row sums of its
  // bias gradients and launches each kind once (flush_deferred_*)
  bool defer_reduce = false, defer_rowsum = false;
  // leave_split_sum: the caller of a convolution asks it to leave a split reduction to the
  // kernel that reads the result next; split_sum_left: one was left (left_split_sum())
  bool leave_split_sum = false, split_sum_left = false;
  // two more streams (default priority) for work that branches off the main one inside a
  // captured train step; created on first use
  hipStream_t side[2]   = {nullptr, nullptr};
};

// Runs the launches of a scope on another stream of the context.
struct StreamSwap {
  hipStream_t saved;
  explicit StreamSwap(hipStream_t s);
  ~StreamSwap();
};

Context &ctx();
int set_error(int code, const char *fmt, ...);
// Makes sure the scratch buffer holds `total` bytes and rewinds it. Growing frees and
// reallocates (hipFree waits for queued kernels), which is refused while ws_locked.
int ws_begin(size_t total);
// Next 256-byte aligned piece of the reserved scratch.
int ws_take(size_t bytes, void **out);
bool gemm_plan_override(int *cfg, int *splits, int M);
inline size_t ws_align(size_t bytes) { return (bytes + 255) & ~static_cast<size_t>(255); }

#define TDH_REQUIRE_INIT()                                                     \
  do {                                                                         \
    if (!::tdh::ctx().ready)                                                   \
      return ::tdh::set_error(TDH_ERR_NOT_INIT, "%s: tdh_init has not been called", __func__); \
  } while (0)

#define TDH_CHECK_ARG(cond, ...)                                               \
  do {                                                                         \
    if (!(cond)) return ::tdh::set_error(TDH_ERR_INVALID, __VA_ARGS__);         \
  } while (0)

#define TDH_HIP(call)                                                          \
  do {                                                                         \
    hipError_t e_ = (call);                                                    \
    if (e_ != hipSuccess)                                                      \
      return ::tdh::set_error(TDH_ERR_HIP, "%s:%d %s -> %s", __FILE__, __LINE__, #call, \
                              hipGetErrorString(e_));                          \
  } while (0)

#define TDH_LAUNCH_CHECK() TDH_HIP(hipGetLastError())

#define TDH_TRY(call)                                                          \
  do {                                                                         \
    int rc_ = (call);                                                          \
    if (rc_ != TDH_OK) return rc_;                                             \
  } while (0)

// ------------------------------------------------------- per-kernel timing
// When profiling is on (tdh_profile_begin), every kernel launch is bracketed by two
// events on the library stream and booked under a tag together with its algorithmic
// work (FLOP for the MFMA GEMMs, bytes for the bandwidth kernels). Off by default:
// launches then record nothing.
enum WorkUnit { WORK_FLOP = 0, WORK_BYTE = 1 };
struct ProfScope {
  ProfScope(const char *tag, double work, WorkUnit unit);
  // GEMM launches carry their shape in the tag: "name m=..,n=..,k=.."
  ProfScope(const char *tag, int m, int n, int k);
  ~ProfScope();
  int slot, outer;
};
bool profiling_active();
// The duration of a profiled scope comes from the dispatches themselves: while a scope is
// open, TDH_LAUNCH hands every launch a pair of events to hipExtLaunchKernelGGL, which stamps
// them with the begin and the end of that kernel's execution; a scope's duration is the sum
// over its launches. (Events recorded around a launch would add the latency of their own
// packets, a few microseconds per kernel, and idle time between two launches of a scope.)
void prof_launch_events(hipEvent_t *start, hipEvent_t *stop);  // nulls outside a scope
#define TDH_LAUNCH(kernel, grid, block, shmem, stream, ...)                                  \
  do {                                                                                       \
    if (::tdh::profiling_active()) {                                                         \
      hipEvent_t tdh_ev0_, tdh_ev1_;                                                         \
      ::tdh::prof_launch_events(&tdh_ev0_, &tdh_ev1_);                                       \
      hipExtLaunchKernelGGL(kernel, grid, block, shmem, stream, tdh_ev0_, tdh_ev1_, 0,       \
                            __VA_ARGS__);                                                    \
    } else {                                                                                 \
      hipLaunchKernelGGL(kernel, grid, block, shmem, stream, __VA_ARGS__);                   \
    }                                                                                        \
  } while (0)

// ---------------------------------------------------------------- helpers
inline int ceil_div(int a, int b) { return (a + b - 1) / b; }
inline size_t ceil_div_sz(size_t a, size_t b) { return (a + b - 1) / b; }

// Workgroups are handed to the eight XCDs (each with its own L2) round-robin in launch order.
// This renumbers a workgroup's linear id so that ids that are neighbours after the renumbering,
// which is how the kernels below give neighbouring pieces of one image to their workgroups, run
// on the same XCD and find each other's overlapping rows in its L2.
__device__ __forceinline__ int xcd_compact_id(const int id, const int total) {
  const int per = total >> 3;
  return id < (per << 3) ? (id & 7) * per + (id >> 3) : id;
}

// Division by a runtime constant as multiply-high + shift. Exact for 0 <= n < 2^31.
struct FastDiv {
  uint32_t d = 1, mul = 1, shift = 0;
  FastDiv() = default;
  explicit FastDiv(uint32_t divisor) : d(divisor) {
    shift = 0;
    while ((1u << shift) < d && shift < 31) ++shift;
    const uint64_t one = 1;
    mul = static_cast<uint32_t>(((one << 32) * ((one << shift) - d)) / d + 1);
  }
  __host__ __device__ __forceinline__ uint32_t div(uint32_t n) const {
#if defined(__HIP_DEVICE_COMPILE__)
    const uint32_t t = __umulhi(mul, n);
#else
    const uint32_t t = static_cast<uint32_t>((static_cast<uint64_t>(mul) * n) >> 32);
#endif
    return (t + n) >> shift;
  }
  __host__ __device__ __forceinline__ void divmod(uint32_t n, uint32_t &q, uint32_t &r) const {
    q = div(n);
    r = n - q * d;
  }
};

// shapes (tiny_dnn/util/util.h:329-363)
int conv_out_length(int in_length, int window, int stride, int dilation, int pad_same);
int pool_out_length(int in_length, int window, int stride, int ceil_mode, int pad_same);

// ------------------------------------------------- internal launchers (device ptrs)
// elementwise.hip
int launch_fill_zero(void *p, size_t bytes, const char *tag = "fill_zero");
int launch_copy(void *dst, const void *src, size_t bytes);  // bytes % 4 == 0
// p: two constructor parameters (never null); x may be null unless the kind's gradient reads it
int launch_act_fwd(int kind, const float *p, int batch, int len, const float *x, float *y);
int launch_act_bwd(int kind, const float *p, int batch, int len, const float *x, const float *y,
                   const float *dy, float *dx);
int launch_loss_grad(int kind, int batch, int len, const float *y, const float *t, float *dy);
int launch_softmax_xent_grad(int batch, int len, const float *y, const float *t, float *dz);
// softmax forward (y) and the gradient above (dz) in one launch
int launch_softmax_fwd_xent(int batch, int len, const float *x, const float *t, float *y, float *dz);
int launch_opt_update(tdh_opt *o, size_t n, const float *g, float grad_scale, float *w, float *s0,
                      float *s1);
// One launch for every trainable tensor of a network (update order = table order). Entry j
// sees the optimizer's bias-correction powers advanced j times, as j earlier update() calls
// would have left them; gradients are cleared after use when zero_grad is set.
struct OptTensor {
  float *g, *w, *s0, *s1;
  uint32_t n, first_block;
  uint32_t block_elems;  // elements a workgroup updates: OPT_MULTI_ELEMS_PER_BLOCK or OPT_SUM_ELEMS_PER_BLOCK
  // A convolution's OIHW weight tensor whose filters the stride-1 kernels read in their own
  // layout: the update also writes the new value into those copies (wp_fwd[t][ci][co],
  // wp_dx[rs-1-t][co][ci]; unconnected pairs of the connection table as zero). NULL: none.
  float *wp_fwd, *wp_dx;
  const uint8_t *tbl;
  uint32_t C, Kc, rs;
};
constexpr int OPT_MULTI_ELEMS_PER_BLOCK = 1024;  // one 16-byte access per thread: a pass of a small net is latency, not bandwidth
// powers_in / powers_out: both NULL, or two device floats each: {b1_t, b2_t} that the kernel reads
// instead of the host values, and where it leaves them advanced n_tensors times for the next
// update (graph replay: a captured launch's arguments are frozen, so two captures whose
// buffers are swapped take turns). They must not overlap.
// Sums of K-split partial slices ([splits][mn] floats each) that the multi-tensor update adds to
// a gradient tensor before it uses it, in the order of the split reduction kernel (eight
// interleaved groups of slices, the group sums in order): the gradient tensors of a train step
// whose weight-gradient kernels left their reductions to the optimizer. Such a tensor's table
// entry has block_elems == OPT_SUM_ELEMS_PER_BLOCK.
constexpr int OPT_SUM_ELEMS_PER_BLOCK = 128;
constexpr int OPT_PENDING_MAX         = 32;
struct OptPendingSum {
  const float *partial;
  const float *g;  // the gradient tensor (an OptTensor::g) the sum belongs to
  uint32_t splits, mn;
};
struct OptPending {
  OptPendingSum sum[OPT_PENDING_MAX];
  int n;
};
// What a workgroup of the multi-tensor update needs to find its tensor and that tensor's pending
// sum without walking the device table entry by entry (each step of such a walk is a memory
// latency, and a step of a small net is little more than a few of those): the first block of
// every tensor and the index of its pending sum, as kernel arguments. n == 0: no index (more
// tensors than OPT_INDEX_MAX, or no host copy of the table), the kernel walks and searches.
constexpr int OPT_INDEX_MAX = 32;
struct OptIndex {
  uint32_t first_block[OPT_INDEX_MAX];  // 0xffffffff past the last tensor
  int8_t pend_of[OPT_INDEX_MAX];        // index into OptPending::sum, or -1
  int n;
};
// host_table: the host copy of dev_table (for the index above), or NULL
int launch_opt_update_multi(tdh_opt *o, const OptTensor *dev_table, int n_tensors,
                            int total_blocks, double total_params, float grad_scale,
                            int zero_grad, const float *powers_in, float *powers_out,
                            const OptPending *pending = nullptr, const OptTensor *host_table = nullptr);
// conv.hip: the recorded split reductions in the optimizer's form (false: they do not all fit its
// form or number). They stay recorded: flush_deferred_reduces launches or forgets them.
bool peek_deferred_reduces(OptPending *out);
bool profiling_active();
// api.hip: the argument checks of the convolution entry points (backward: also what only the
// backward pass refuses)
int check_conv_desc(const tdh_conv_desc *d, int batch, bool backward);
// deterministic reductions: out[r] (+)= sum over `cols` contiguous values of row r,
// rows laid out as [outer][rows][cols] and summed over outer in order
int launch_rowsum(const float *src, int outer, int rows, int cols, float *out, int accumulate);
// launch what was recorded on the current stream (launch = false: forget it)
int flush_deferred_rowsums(bool launch = true);   // elementwise.hip
int flush_deferred_reduces(bool launch = true);   // conv.hip
// conv_dw_small.hip: dW (+ db) of a convolution with few input channels
bool conv_dw_small_applicable(int batch, int C, int Kc, int H, int W, int OH, int OW, int R, int S,
                              int sh, int sw, int dh, int dw, int ph, int pw);
size_t conv_dw_small_workspace_bytes(int batch, int C, int Kc, int H, int W, int OH, int OW, int R,
                                     int S, int sh, int sw, int dh, int dw, int ph, int pw);
// The output gradient of a convolution whose output feeds a 2x2 / stride-2 max-pool, given as
// what the pool's backward pass would read instead of as the tensor it would write:
//   dY[img][co][y][x] = argmax[img][co][y/2][x/2] == (co*OH + y)*OW + x ? g[img][co][y/2][x/2] : 0
struct PoolGather {
  const float *g        = nullptr;  // [batch][Cout][OH/2][OW/2] gradient of the pooled output
  const int32_t *argmax = nullptr;  // same shape: flat CHW index of each window's maximum
};
// (dy_pool set: dy is not read; the plan must pass conv_dw_small_reads_pooled)
int conv_dw_small_run(int batch, int C, int Kc, const float *x, const float *dy, float *dw_out,
                      float *db_out, int H, int W, int OH, int OW, int R, int S, int sh, int sw, int dh,
                      int dw, int ph, int pw, int accumulate, const PoolGather *dy_pool = nullptr,
                      int force_band = 0);
bool conv_dw_small_reads_pooled(int batch, int C, int Kc, int H, int W, int OH, int OW, int R, int S,
                                int sh, int sw, int dh, int dw, int ph, int pw);
// the weight-gradient kernel of this layer also produces the bias gradient when asked for both
bool conv_dw_gives_db(const tdh_conv_desc *d, int batch);
// norm.hip
size_t batchnorm_workspace_bytes(int channels, int batch);
int batchnorm_fwd(int channels, int spatial, int batch, float eps, int train, const float *x,
                  float *mean, float *variance, float *stddev, float *y);
int batchnorm_bwd(int channels, int spatial, int batch, const float *y, const float *dy,
                  const float *stddev, float *dx);
int batchnorm_update_moving(int channels, float momentum, const float *mean_cur,
                            const float *var_cur, float *mean, float *var);
int dropout_fwd(size_t total, int train, float scale, const uint8_t *mask, const float *x, float *y);
int dropout_bwd(size_t total, const uint8_t *mask, const float *dy, float *dx);
size_t rowsum_workspace_bytes(int outer, int rows, int cols);
// out[c] (+)= sum_s src[s*cols + c]
int launch_colsum(const float *src, int rows, int cols, float *out, int accumulate);

// activation-gradient factor fused into GEMM epilogues
struct ActGrad {
  int kind = TDH_ACT_NONE;  // TDH_ACT_TANH / RELU / SIGMOID or NONE
  const float *y = nullptr; // activation OUTPUT, same indexing as the GEMM result
};

// A split reduction that the kernel reading the result finishes: value i is
// part[i] + part[stride + i] + ... (in this order) (+ bias of i's channel plane) (* act'(y[i])),
// and whoever computes it also writes it to out[i]. The 2x2 max-pool kernels behind a
// stride-1 convolution take it (a reduction kernel of its own costs a launch on the chain
// every later layer waits for).
struct SplitSum {
  const float *part = nullptr;
  int splits = 0;
  size_t stride = 0;  // elements of one partial = elements of the result
  const float *bias = nullptr;
  int MC = 1;
  FastDiv div_plane;
  ActGrad ag;
  float *out = nullptr;
};
SplitSum &left_split_sum();  // meaningful while ctx().split_sum_left
int finish_split_sum();      // the reduction as a launch of its own, when nobody took it


// conv.hip / fc.hip
// prepacked: filters already packed by conv_pack_filters for this direction (and only then)
// A 2x2 / stride-2 max-pool layer (and the pointwise activation behind it) computed by the
// forward kernel of the layer in front of it
struct PoolFuse {
  float *out;
  int32_t *argmax;
  float *act_out;  // or null
  int act_kind;
};
int conv2d_fwd(const tdh_conv_desc *d, int batch, const float *x, const float *w, const float *b,
               float *y, const uint8_t *tbl_resident = nullptr, const float *prepacked = nullptr,
               float *act_out = nullptr, int act_kind = 0, const PoolFuse *pool = nullptr);
// dX, dW and db of this (first) convolution leave conv2d_bwd as one launch when all three are
// asked for together (pooled: the gradient is read through the max-pool behind the layer)
bool conv_bwd_one_launch(const tdh_conv_desc *d, int batch, bool pooled);
// the forward kernel of this convolution can also compute the max-pool layer `pool` behind it
bool conv_fwd_fuses_pool(const tdh_conv_desc *d, const tdh_pool_desc *pool, int batch, bool prepacked);
// ... and the pointwise activation of this kind behind that pool
bool conv_fwd_pool_applies_act(const tdh_conv_desc *d, int batch, bool prepacked, int act_kind);
// the forward kernel of this layer can leave `y` out (null) when it writes the activation layer
// or the pool behind the convolution itself
bool conv_fwd_out_optional(const tdh_conv_desc *d, int batch, bool prepacked);
// conv_fwd_small.hip
bool conv_fwd_small_applicable(int batch, int C, int Kc, int H, int W, int OH, int OW, int R, int S,
                               int sh, int sw, int dh, int dw, int ph, int pw);
int conv_fwd_small_run(int batch, int C, int Kc, const float *x, const float *w, const float *bias,
                       float *out, int H, int W, int OH, int OW, int R, int S, int sh, int sw, int dh,
                       int dw, int ph, int pw, float *act_out, int act_kind, const PoolFuse *pool);
// dy_pool: the output gradient is given through the max-pool behind the layer (dy is not read
// and may be null); only where conv_bwd_reads_pooled says so
int conv2d_bwd(const tdh_conv_desc *d, int batch, const float *x, const float *w, const float *dy,
               float *dx, float *dw, float *db, int accumulate, ActGrad dx_act,
               const uint8_t *tbl_resident = nullptr, const float *prepacked_dx = nullptr,
               const PoolGather *dy_pool = nullptr);
// the backward kernels of this layer (the two of a first layer: few input channels, stride 1)
// can read their output gradient through this 2x2 / stride-2 max-pool over the layer's output
bool conv_bwd_reads_pooled(const tdh_conv_desc *d, const tdh_pool_desc *pool, int batch);
// true when forward (flip = 0) / dX (flip = 1) of this layer reads packed filters
bool conv_uses_packed(const tdh_conv_desc *d, int batch, int flip);
bool conv_fwd_applies_act(const tdh_conv_desc *d, int batch, bool prepacked);
// packs w (masked by the device-resident connection table, if any) into wp[k_w*k_h*in_c*out_c]
int conv_pack_filters(const tdh_conv_desc *d, int flip, const float *w, const uint8_t *tbl_resident,
                      float *wp);
int fc_fwd(int in, int out, int has_bias, int batch, const float *x, const float *w,
           const float *b, float *y, float *act_out = nullptr, int act_kind = 0);
// The backward pass of a 2x2 / stride-2 max-pool layer in front of a fully-connected layer,
// done by that layer's dX epilogue: the gradient of pooled element n of sample m goes to the
// input position the argmax record names, zeros to the other three of its window.
struct PoolScatter {
  const int32_t *argmax = nullptr;  // [batch][C*OH*OW], flat CHW input index inside the sample
  float *dx = nullptr;              // [batch][C*H*W]
  int W = 0, OW = 0, OH = 0;        // input width, pooled width and height (H = 2*OH, W = 2*OW)
};
// (pool.hip) the layer is such a pool; fills the geometry
bool maxpool_scatters_from_fc(const tdh_pool_desc *d, PoolScatter *geom);
// the weight and bias gradients (db null: no bias) of another small fully-connected layer of
// the same batch that fc_bwd's one-launch kernel computes beside its own (both layers within
// fc_bwd_fuses)
struct FcGrads {
  int in, out;
  const float *x, *dy;
  float *dw, *db;
};
int fc_bwd(int in, int out, int has_bias, int batch, const float *x, const float *w,
           const float *dy, float *dx, float *dw, float *db, int accumulate, ActGrad dx_act,
           const PoolScatter *pool = nullptr, const FcGrads *also = nullptr);
// (fc.hip) the closing classifier, two fully-connected layers deep, in one launch up to the
// gradient of the first layer's output
bool fc_two_layer_tail_applies(int in, int hidden, int out, int batch);
int fc_two_layer_tail(int in, int hidden, int out, int has_bias1, int has_bias2, int batch, const float *x,
                      const float *w1, const float *b1, float *y1, float *a1, int act_kind, const float *w2,
                      const float *b2, float *y2, float *soft, const float *t, float *dz, float *dh,
                      float *partials, unsigned int *tickets);
size_t fc_two_layer_tail_partials(int in, int batch);
size_t fc_two_layer_tail_tickets(int batch);
// the one-launch backward kernel of this layer can also scatter dX through a max-pool
bool fc_bwd_scatters_pool(int in, int out, int batch);
// conv_s1.hip: stride-1 forward / dX with LDS halo tiles (3x3 and 5x5 windows)
bool conv_s1_applicable(int R, int S, int batch, int KC, int MC, int IH, int IW, int OH, int OW,
                        int ph, int pw);
size_t conv_s1_workspace_bytes(int R, int S, int batch, int C, int Kc, int flip, int IH, int IW,
                               int OH, int OW, int ph, int pw);
int conv_s1_run(int R, int S, int batch, int C, int Kc, int flip, const float *in, const float *w,
                const uint8_t *tbl_dev, const float *bias, float *out, int IH, int IW, int OH,
                int OW, int ph, int pw, ActGrad ag, const char *tag,
                const float *prepacked = nullptr, float *act_out = nullptr, int act_kind = 0,
                const PoolFuse *pool = nullptr);
// the forward kernel of this shape can also compute the 2x2 / stride-2 max-pool behind it (and
// a relu behind that pool); `out` may then be null
bool conv_s1_fuses_pool(int R, int S, int batch, int KC, int MC, int IH, int IW, int OH, int OW,
                        int ph, int pw);
// one pass over the reduction channels: the kernel's epilogue is the only writer of `out`
bool conv_s1_single_pass(int R, int S, int batch, int KC, int MC, int IH, int IW, int OH, int OW,
                         int ph, int pw);
int conv_s1_repack(int R, int S, int C, int Kc, int flip, const float *w, const uint8_t *tbl_dev,
                   float *wp);
// conv_dw.hip: stride-1 weight gradient from LDS-staged tiles (3x3 and 5x5 windows)
bool conv_dw_halo_applicable(int R, int S, int batch, int C, int Kc, int H, int W, int OH, int OW,
                             int ph, int pw);
size_t conv_dw_halo_workspace_bytes(int R, int S, int batch, int C, int Kc, int H, int W, int OH,
                                    int OW, int ph, int pw);
int conv_dw_halo_run(int R, int S, int batch, int C, int Kc, const float *x, const float *dy,
                     float *dw, int H, int W, int OH, int OW, int ph, int pw, int accumulate,
                     float *db = nullptr);
// workspace bytes the op may ask for (so a net can reserve it before graph capture)
size_t conv2d_workspace_bytes(const tdh_conv_desc *d, int batch);
size_t fc_workspace_bytes(int in, int out, int batch);
bool fc_bwd_fuses(int in, int out, int batch);
// The last fully-connected layer in front of softmax + cross_entropy_multiclass in one launch:
// y = x*W + b, soft = softmax(y), dz = dL/dy, dx = dz*W^T (times dx_act's factor); with
// soft == nullptr the loss is mse on y itself
bool fc_softmax_xent_applies(int in, int out, int batch);
int fc_softmax_xent(int in, int out, int has_bias, int batch, const float *x, const float *w,
                    const float *b, float *y, float *soft, const float *t, float *dz, float *dx,
                    ActGrad dx_act);

// pool.hip
// act_out: also writes act(y) there (tanh / relu / sigmoid), the activation layer behind the pool
int maxpool_fwd(const tdh_pool_desc *d, int batch, const float *x, float *y, int32_t *argmax,
                float *act_out = nullptr, int act_kind = TDH_ACT_NONE);
// pooled_y: the pool's forward output, or NULL (with an activation gradient folded in, ag, the 2x2
// kernel reads it instead of the activation output)
int maxpool_bwd(const tdh_pool_desc *d, int batch, const float *dy, const int32_t *argmax,
                float *dx, ActGrad ag = ActGrad(), const float *pooled_y = nullptr);
int avepool_fwd(const tdh_pool_desc *d, int batch, const float *x, const float *w, const float *b,
                float *y);
int avepool_bwd(const tdh_pool_desc *d, int batch, const float *x, const float *w, const float *dy,
                float *dx, float *dw, float *db, int accumulate, ActGrad ag = ActGrad());
size_t avepool_workspace_bytes(const tdh_pool_desc *d, int batch);

// forward of the three parameter-free pointwise activations (tanh_layer.h:24-28,
// relu_layer.h:25-29, sigmoid_layer.h:24-28), for kernels that apply one on their way out
__device__ __forceinline__ float act_apply(int kind, float x) {
  switch (kind) {
    case TDH_ACT_TANH: return tanhf(x);
    case TDH_ACT_RELU: return x > 0.0f ? x : 0.0f;
    case TDH_ACT_SIGMOID: return 1.0f / (1.0f + expf(-x));
    default: return x;
  }
}

__device__ __forceinline__ float act_grad_factor(int kind, float y) {
  switch (kind) {
    case TDH_ACT_TANH: return 1.0f - y * y;
    case TDH_ACT_RELU: return y > 0.0f ? 1.0f : 0.0f;
    case TDH_ACT_SIGMOID: return y * (1.0f - y);
    default: return 1.0f;
  }
}

// VEC consecutive values of one channel plane (i a multiple of VEC, VEC in {1, 2, 4})
template <int VEC>
__device__ __forceinline__ void split_sum_values(const SplitSum &s, const size_t i, float (&v)[VEC]) {
#pragma unroll
  for (int e = 0; e < VEC; ++e) v[e] = 0.0f;
  for (int z = 0; z < s.splits; ++z) {
    const float *p = s.part + z * s.stride + i;
    if (VEC == 4) {
      const float4 f = *reinterpret_cast<const float4 *>(p);
      v[0] += f.x; v[1 % VEC] += f.y; v[2 % VEC] += f.z; v[3 % VEC] += f.w;
    } else if (VEC == 2) {
      const float2 f = *reinterpret_cast<const float2 *>(p);
      v[0] += f.x; v[1 % VEC] += f.y;
    } else {
      v[0] += p[0];
    }
  }
  const float b = s.bias ? s.bias[s.div_plane.div(static_cast<uint32_t>(i)) % s.MC] : 0.0f;
#pragma unroll
  for (int e = 0; e < VEC; ++e) {
    v[e] += b;
    if (s.ag.kind != TDH_ACT_NONE) v[e] *= act_grad_factor(s.ag.kind, s.ag.y[i + e]);
  }
  if (VEC == 4)
    *reinterpret_cast<float4 *>(s.out + i) = make_float4(v[0], v[1 % VEC], v[2 % VEC], v[3 % VEC]);
  else if (VEC == 2)
    *reinterpret_cast<float2 *>(s.out + i) = make_float2(v[0], v[1 % VEC]);
  else
    s.out[i] = v[0];
}

}  // namespace tdh
