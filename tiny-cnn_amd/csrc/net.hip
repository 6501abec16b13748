// net.hip — a sequential network whose tensors never leave the device: the restatement of
// network<sequential>::train_onebatch (tiny_dnn/network.h:911-926) = fprop
// (nodes.h:288-303), loss gradient (loss_function.h:191-218), bprop (nodes.h:276-286) and
// update_weights (nodes.h:103-107, layer.h:663-682), queued on the library stream.
#include <algorithm>
#include <cstring>
#include <vector>

#include "common.h"
#include "tiny_net.h"

struct tdh_net {
  struct Layer {
    tdh_layer spec;
    std::vector<uint8_t> tbl;  // private copy of the connection table
    uint8_t *tbl_dev = nullptr;
    size_t in_size = 0, out_size = 0, w_size = 0, b_size = 0;
    float *w = nullptr, *b = nullptr, *dw = nullptr, *db = nullptr;
    float *s0w = nullptr, *s1w = nullptr, *s0b = nullptr, *s1b = nullptr;
    float *out  = nullptr;  // [max_batch][out_size]
    float *dout = nullptr;  // gradient w.r.t. out; the next layer's backward writes it
    int32_t *argmax = nullptr;
    bool grad_folded = false;  // activation whose backward runs in the next layer's dX epilogue
    // set where the optimizer table is built: the tensor's entry there has the small blocks
    // (OPT_SUM_ELEMS_PER_BLOCK) that let the optimizer kernel add up K-split partial slices
    bool w_sums_in_opt = false, b_sums_in_opt = false;
    // filters in the LDS-halo kernels' layout for forward / dX, packed on a side stream at the
    // start of a captured step (stride-1 conv layers of a TDH_NET_GRAPH net)
    float *wp_fwd = nullptr, *wp_dx = nullptr;  // kept current by the optimizer kernel
    // batch-norm: running averages, this batch's moments, sqrt(variance + eps); dropout: mask
    float *bn_mean = nullptr, *bn_var = nullptr, *bn_mean_cur = nullptr, *bn_var_cur = nullptr,
          *bn_stddev = nullptr;
    uint8_t *mask = nullptr;  // [max_batch][out_size]
  };
  std::vector<Layer> layers;
  int max_batch  = 0;
  int flags      = 0;
  bool test_phase = false;  // net_phase::test
  float *dx_in   = nullptr;  // gradient w.r.t. the network input
  tdh::OptTensor *opt_table = nullptr;  // device table of trainable tensors, update order
  std::vector<tdh::OptTensor> opt_table_host;  // (its host copy)
  bool packs_valid = false;  // wp_fwd / wp_dx of every layer match its weights
  int opt_tensors = 0, opt_blocks = 0;
  double opt_params = 0.0;
  // graph replay (TDH_NET_GRAPH): one captured train step, re-captured when its key changes
  // the powers as the captured optimizer kernels use them: two buffers of {b1_t, b2_t} (at 0 and
  // at 4); a step reads buffer powers_at and leaves the advanced powers in the other one
  float *dev_powers = nullptr;
  int powers_at = 0;
  // partial sums and tickets of the one-launch kernel of two closing fully-connected layers
  float *tail_partials = nullptr, *tail_tickets = nullptr;
  static constexpr int kMaxSteps = 8;   // train steps one captured graph may hold (tdh_net_train_steps)
  struct GraphKey {
    int batch = 0, loss = 0, do_update = 0, test_phase = 0;
    int powers_at = 0;                  // which buffer of the powers the (first) captured optimizer launch reads
    int n_steps = 1;
    const float *x[kMaxSteps] = {}, *t[kMaxSteps] = {};
    const void *scratch = nullptr;      // the library scratch buffer the captured kernels use
    tdh_opt hyper = {};                 // hyper-parameters only (powers zeroed)
  };
  // a few captured steps are kept, so that alternating input buffers (double-buffered
  // uploads) or batch sizes (the short last batch of an epoch) do not re-capture every step
  static constexpr int kGraphSlots = 8;
  struct GraphSlot {
    hipGraphExec_t exec = nullptr;
    GraphKey key;
    uint64_t last_use = 0;
    std::vector<uint8_t> dx_unwritten, out_unwritten;  // what the captured step leaves in the net's fields of those names
  } graphs[kGraphSlots];
  uint64_t graph_clock = 0;
  // per layer: the last step kept the gradient with respect to this layer's input in registers
  // or read it through a pool (tdh_net_layer_dx has nothing to show)
  std::vector<uint8_t> dx_unwritten;
  std::vector<uint8_t> out_unwritten;  // likewise for a layer's output
  float mirror_b1_t = 0.0f, mirror_b2_t = 0.0f;  // what the device copy of the powers holds
  size_t scratch = 0;        // largest per-op scratch need; with TDH_NET_GRAPH the sum over the
                             // layers, because branches of the captured step run side by side
  std::vector<hipEvent_t> events;  // fork/join points of the captured step
  std::vector<void *> allocs;
  // the one-workgroup-per-sample step of a small net (tiny_net.hip), when the net qualifies
  bool tiny_ok = false;
  tdh::TinyPlan tiny;
  tdh::TinyPlan *tiny_dev = nullptr;  // the same in device memory
  tdh::TinyMerge tiny_merge;
};

namespace tdh {

namespace {

int layer_sizes(tdh_net::Layer &L) {
  const tdh_layer &s = L.spec;
  switch (s.kind) {
    case TDH_L_CONV: {
      TDH_TRY(check_conv_desc(&s.conv, 1, /*backward=*/true));  // a net is there to be trained
      const int ow = conv_out_length(s.conv.in_w, s.conv.k_w, s.conv.w_stride, s.conv.w_dilation,
                                     s.conv.pad_same);
      const int oh = conv_out_length(s.conv.in_h, s.conv.k_h, s.conv.h_stride, s.conv.h_dilation,
                                     s.conv.pad_same);
      L.in_size  = static_cast<size_t>(s.conv.in_w) * s.conv.in_h * s.conv.in_c;
      L.out_size = static_cast<size_t>(ow) * oh * s.conv.out_c;
      L.w_size   = static_cast<size_t>(s.conv.k_w) * s.conv.k_h * s.conv.in_c * s.conv.out_c;
      L.b_size   = s.conv.has_bias ? s.conv.out_c : 0;
    } break;
    case TDH_L_FC:
      L.in_size = s.fc_in; L.out_size = s.fc_out;
      L.w_size = static_cast<size_t>(s.fc_in) * s.fc_out;
      L.b_size = s.fc_bias ? s.fc_out : 0;
      break;
    case TDH_L_MAXPOOL:
    case TDH_L_AVEPOOL: {
      const int ow = pool_out_length(s.pool.in_w, s.pool.pool_w, s.pool.stride_w, s.pool.ceil_mode,
                                     s.pool.pad_same);
      const int oh = pool_out_length(s.pool.in_h, s.pool.pool_h, s.pool.stride_h, s.pool.ceil_mode,
                                     s.pool.pad_same);
      L.in_size  = static_cast<size_t>(s.pool.in_w) * s.pool.in_h * s.pool.in_c;
      L.out_size = static_cast<size_t>(ow) * oh * s.pool.in_c;
      L.w_size   = s.kind == TDH_L_AVEPOOL ? s.pool.in_c : 0;
      L.b_size   = L.w_size;
    } break;
    case TDH_L_ACT:
    case TDH_L_DROPOUT: L.w_size = L.b_size = 0; break;
    case TDH_L_BATCHNORM:
      if (s.bn_channels <= 0 || s.bn_spatial <= 0)
        return set_error(TDH_ERR_INVALID, "batch-norm layer: %d channels x %d", s.bn_channels, s.bn_spatial);
      L.in_size = L.out_size = static_cast<size_t>(s.bn_channels) * s.bn_spatial;
      L.w_size = L.b_size = 0;
      break;
    default: return set_error(TDH_ERR_INVALID, "unknown layer kind %d", s.kind);
  }
  return TDH_OK;
}

int net_alloc(tdh_net *net, size_t floats, float **out, bool zero) {
  *out = nullptr;
  if (floats == 0) return TDH_OK;
  void *p = nullptr;
  if (hipMalloc(&p, floats * sizeof(float)) != hipSuccess) {
    (void)hipGetLastError();
    return set_error(TDH_ERR_OOM, "network: cannot allocate %zu bytes", floats * sizeof(float));
  }
  net->allocs.push_back(p);
  *out = static_cast<float *>(p);
  if (zero) TDH_TRY(launch_fill_zero(p, floats * sizeof(float)));
  return TDH_OK;
}

bool is_pointwise_act(int act) {
  return act == TDH_ACT_TANH || act == TDH_ACT_RELU || act == TDH_ACT_SIGMOID;
}

// Whether the captured step of this net branches (weight and bias gradients and filter
// packing beside the main chain): mid-sized steps only. With tiny kernels the cross-queue
// synchronisation costs more than it hides, and products that fill the chip for hundreds of
// microseconds only fight the main chain for its caches (measured: LeNet-style net 5 % slower,
// VGG-style 1 % slower with branches). In between, a branch point and a join cost a replayed
// step about 5 us each, and what a branch buys depends on how the kernels fill the chip. The
// CIFAR-10-shape net, us a step with / without branches: batch 16 138 / 149, 32 143 / 151,
// 64 140 / 151, 128 181 / 177, 256 288 / 285, 512 517 / 541. Up to batch 64 its kernels leave
// compute units idle that a branch fills; at 128 and 256 every kernel is about one full round
// of workgroups, two kernels side by side only take turns, and the step is the sum of its
// kernels either way; beyond, the rounds of one kernel overlap the tail of another again.
double net_forward_flop(const tdh_net *net, int batch) {
  double macs = 0.0;
  for (const tdh_net::Layer &L : net->layers) {
    if (L.spec.kind == TDH_L_CONV)
      macs += static_cast<double>(L.out_size) * L.spec.conv.in_c * L.spec.conv.k_w * L.spec.conv.k_h;
    else if (L.spec.kind == TDH_L_FC)
      macs += static_cast<double>(L.spec.fc_in) * L.spec.fc_out;
  }
  return 2.0 * batch * macs;
}
// TDH_NET_NO_INPUT_GRAD on a net whose first layer is one of the kinds that honour it
bool net_skips_input_grad(const tdh_net *net) {
  if (!(net->flags & TDH_NET_NO_INPUT_GRAD) || net->layers.empty()) return false;
  const int kind = net->layers[0].spec.kind;
  return kind == TDH_L_CONV || kind == TDH_L_FC;
}

bool net_forks(const tdh_net *net, int batch) {
  const double flop = net_forward_flop(net, batch);
  return flop >= 1e8 && flop <= 3e10 && !(flop >= 2.2e9 && flop < 1e10);
}
// A step too small to branch (LeNet-5 at batch 16) is a chain of launches of a few
// microseconds each, and what counts is how many there are; a larger step that does not
// branch gains the reduction launches it does not make (VGG-style stack: 5.40 -> 5.37 ms): it runs the branching step's
// launches one after the other, so that the split sums of all weight gradients go to the
// optimizer kernel and the row sums of all bias gradients leave as one pair of launches.
// (With the graph flag only: a net created with it reserves every layer's scratch side by side.)
bool net_defers_serially(const tdh_net *net, int batch) {
  return (net->flags & TDH_NET_GRAPH) && (net->flags & TDH_NET_FUSE_ACT_GRAD) &&
         !net_forks(net, batch);
}

// The plan of the one-workgroup-per-sample step (tiny_net.hip) for a net that qualifies: at most
// TINY_MAX_LAYERS layers of the kinds that kernel knows, every layer output of one sample and two
// gradient buffers within a workgroup's LDS, little arithmetic per sample, and room for the
// per-sample gradient slices. Leaves net->tiny_ok false otherwise: the layer-by-layer step runs.
int build_tiny_plan(tdh_net *net) {
  net->tiny_ok = false;
  const int n = static_cast<int>(net->layers.size());
  if (!(net->flags & TDH_NET_SAMPLE_STEP) || n > TINY_MAX_LAYERS || net->max_batch > 512) return TDH_OK;
  if (net_forward_flop(net, 1) > 4e6) return TDH_OK;
  TinyPlan &P = net->tiny;
  std::memset(&P, 0, sizeof(P));
  P.n       = n;
  P.in_size = static_cast<int>(net->layers[0].in_size);
  size_t lds = net->layers[0].in_size, gmax = net->layers[0].in_size, slice_floats = 0;
  int tensors = 0;
  for (int i = 0; i < n; ++i) {
    const tdh_net::Layer &L = net->layers[i];
    const tdh_layer &sp = L.spec;
    TinyLayer &T = P.l[i];
    T.kind = sp.kind;
    T.in_size = static_cast<int>(L.in_size); T.out_size = static_cast<int>(L.out_size);
    T.w = L.w; T.b = L.b; T.out = L.out;
    T.dx = i == 0 ? net->dx_in : net->layers[i - 1].dout;
    if (i == 0 && net_skips_input_grad(net)) {
      T.dx = nullptr;
      P.skip_first_dx = 1;
    }
    T.nw = static_cast<int>(L.w_size); T.nb = static_cast<int>(L.b_size);
    T.lds_in  = i == 0 ? 0 : P.l[i - 1].lds_out;
    // a pointwise activation overwrites its input: of the forward values the backward pass
    // of the step kernel reads only the outputs of activations (the gradients of tanh, relu,
    // sigmoid and leaky relu are functions of those), and the weight gradients read the
    // copies in memory
    // (unless that input is itself an activation's output)
    const bool in_place = i > 0 && sp.kind == TDH_L_ACT && sp.act != TDH_ACT_SOFTMAX &&
                          net->layers[i - 1].spec.kind != TDH_L_ACT;
    T.lds_out = in_place ? T.lds_in : static_cast<int>(lds);
    if (!in_place) lds += L.out_size;
    gmax = std::max(gmax, L.out_size);
    switch (sp.kind) {
      case TDH_L_CONV: {
        const tdh_conv_desc &d = sp.conv;
        T.C = d.in_c; T.H = d.in_h; T.W = d.in_w; T.K = d.out_c;
        T.OW = conv_out_length(d.in_w, d.k_w, d.w_stride, d.w_dilation, d.pad_same);
        T.OH = conv_out_length(d.in_h, d.k_h, d.h_stride, d.h_dilation, d.pad_same);
        T.R = d.k_h; T.S = d.k_w; T.sh = d.h_stride; T.sw = d.w_stride;
        T.ph = d.pad_same ? d.k_h / 2 : 0; T.pw = d.pad_same ? d.k_w / 2 : 0;
        T.has_bias = d.has_bias;
        T.tbl = d.tbl ? L.tbl_dev : nullptr;
        if (d.w_dilation != 1 || d.h_dilation != 1) return TDH_OK;
        P.flop_per_sample += 6.0 * L.out_size * d.in_c * d.k_w * d.k_h;
      } break;
      case TDH_L_FC:
        T.has_bias = sp.fc_bias;
        P.flop_per_sample += 6.0 * sp.fc_in * sp.fc_out;
        break;
      case TDH_L_MAXPOOL:
      case TDH_L_AVEPOOL: {
        const tdh_pool_desc &d = sp.pool;
        if (d.pad_same) return TDH_OK;
        if (sp.kind == TDH_L_AVEPOOL && (d.stride_w != d.pool_w || d.stride_h != d.pool_h)) return TDH_OK;
        T.C = d.in_c; T.H = d.in_h; T.W = d.in_w; T.K = d.in_c;
        T.OW = pool_out_length(d.in_w, d.pool_w, d.stride_w, d.ceil_mode, d.pad_same);
        T.OH = pool_out_length(d.in_h, d.pool_h, d.stride_h, d.ceil_mode, d.pad_same);
        T.R = d.pool_h; T.S = d.pool_w; T.sh = d.stride_h; T.sw = d.stride_w;
        T.scale = 1.0f / static_cast<float>(d.pool_w * d.pool_h);
        T.argmax = L.argmax;
        T.has_bias = sp.kind == TDH_L_AVEPOOL;
      } break;
      case TDH_L_ACT:
        T.act = sp.act; T.p0 = sp.act_p[0];
        if (sp.act == TDH_ACT_SOFTMAX) {
          if (i != n - 1) return TDH_OK;   // only as the closing layer (with cross_entropy_multiclass)
        } else if (sp.act != TDH_ACT_TANH && sp.act != TDH_ACT_RELU && sp.act != TDH_ACT_SIGMOID &&
                   sp.act != TDH_ACT_LEAKY_RELU) {
          return TDH_OK;
        }
        break;
      default: return TDH_OK;   // batch normalization, dropout: the layer-by-layer step
    }
    tensors += (L.w_size ? 1 : 0) + (L.b_size ? 1 : 0);
    slice_floats += (ceil_div_sz(L.w_size * static_cast<size_t>(net->max_batch), 4) * 4) +
                    (ceil_div_sz(L.b_size * static_cast<size_t>(net->max_batch), 4) * 4);   // (16-byte aligned slices)
  }
  P.lds_g0 = static_cast<int>(lds);
  P.lds_g1 = static_cast<int>(lds + gmax);
  lds += 2 * gmax;
  lds = (lds + 3) & ~static_cast<size_t>(3);   // (16-byte reads of the staged filters)
  P.lds_w = static_cast<int>(lds);
  lds += TINY_SCRATCH_FLOATS;
  P.lds_floats = static_cast<int>(lds);
  P.dloss      = net->layers[n - 1].dout;
  P.mse_factor = 2.0f / static_cast<float>(net->layers[n - 1].out_size);
  if (tensors > TINY_MAX_TENSORS || slice_floats > (64u << 20)) return TDH_OK;
  TDH_TRY(tiny_build_jobs(P));   // (adds the framed dY's LDS to the plan's)
  if (std::max(P.lds_floats, P.lds_job_floats) * sizeof(float) > TINY_LDS_MAX_BYTES) return TDH_OK;
  float *slices = nullptr;
  TDH_TRY(net_alloc(net, slice_floats, &slices, false));
  TinyMerge &M = net->tiny_merge;
  std::memset(&M, 0, sizeof(M));
  int blocks = 0;
  for (int i = 0; i < n; ++i) {
    tdh_net::Layer &L = net->layers[i];
    TinyLayer &T = P.l[i];
    for (int which = 0; which < 2; ++which) {
      const size_t len = which ? L.b_size : L.w_size;
      if (!len) continue;
      (which ? T.gb : T.gw) = slices;
      M.slices[M.n] = slices;
      M.g[M.n]      = which ? L.db : L.dw;
      M.len[M.n]    = static_cast<int>(len);
      M.first_block[M.n] = blocks;
      blocks += ceil_div(static_cast<int>(len), 256);
      ++M.n;
      slices += ceil_div_sz(len * static_cast<size_t>(net->max_batch), 4) * 4;
    }
  }
  M.first_block[M.n] = blocks;
  for (int i = 0; i < n; ++i) {
    TinyLayer &T = P.l[i];
    const auto fd = [](int v) { return FastDiv(static_cast<uint32_t>(v > 0 ? v : 1)); };
    T.d_oplane = fd(T.OH * T.OW); T.d_ow = fd(T.OW); T.d_iplane = fd(T.H * T.W); T.d_w = fd(T.W);
    T.d_taps = fd(T.R * T.S); T.d_s = fd(T.S); T.d_c = fd(T.C); T.d_out = fd(T.out_size);
    T.d_nk = fd(T.C * T.R * T.S);
  }
  float *dev = nullptr;
  TDH_TRY(net_alloc(net, ceil_div_sz(sizeof(TinyPlan), sizeof(float)), &dev, false));
  net->tiny_dev = reinterpret_cast<TinyPlan *>(dev);
  TDH_TRY(tdh_memcpy_h2d(net->tiny_dev, &P, sizeof(TinyPlan)));
  TDH_TRY(tiny_prepare());
  net->tiny_ok = true;
  return TDH_OK;
}

// whether this step runs as the one-workgroup-per-sample kernel
bool tiny_step_applies(const tdh_net *net, int loss_kind) {
  if (!net->tiny_ok || net->test_phase) return false;
  const tdh_layer &last = net->layers.back().spec;
  if (last.kind == TDH_L_ACT && last.act == TDH_ACT_SOFTMAX && loss_kind != TDH_LOSS_CE_MULTICLASS) return false;
  return loss_kind == TDH_LOSS_MSE || loss_kind == TDH_LOSS_CE_MULTICLASS || loss_kind == TDH_LOSS_CE;
}

bool layer_forks(const tdh_net::Layer &L) {
  return L.spec.kind == TDH_L_CONV || L.spec.kind == TDH_L_FC;
}

// Asks the convolution called inside the scope to leave a split reduction to the max-pool
// kernel that reads its result next (maxpool_fwd / maxpool_bwd take it or finish it).
struct LeaveSplitSum {
  Context &c;
  LeaveSplitSum(Context &cc, bool on) : c(cc) { c.leave_split_sum = on; }
  ~LeaveSplitSum() { c.leave_split_sum = false; }
};

// Where the gradient of a layer's input goes in a train step: the gradient buffer of the
// layer in front, or, when that layer is an activation whose gradient the producing kernel
// applies, the buffer in front of the activation.
struct DxTarget {
  float *dx;
  ActGrad fold;
};
DxTarget dx_target(tdh_net *net, int i) {
  DxTarget d;
  d.dx = i == 0 ? net->dx_in : net->layers[i - 1].dout;
  if (i >= 1 && net->layers[i - 1].grad_folded) {
    d.fold.kind = net->layers[i - 1].spec.act;
    d.fold.y    = net->layers[i - 1].out;
    d.dx        = i - 1 == 0 ? net->dx_in : net->layers[i - 2].dout;
  }
  return d;
}

// Max-pool layer r of a fusing net sits directly behind a first convolution (few input
// channels, stride 1) whose backward kernels read the pooled gradient and the argmax records
// themselves: the pool's backward pass does not run and its input gradient is never written.
bool pool_read_by_conv(tdh_net *net, int r, int batch) {
  if (!(net->flags & TDH_NET_FUSE_ACT_GRAD) || r < 1) return false;
  const tdh_net::Layer &conv = net->layers[r - 1];
  return conv.spec.kind == TDH_L_CONV && !conv.tbl_dev &&
         conv_bwd_reads_pooled(&conv.spec.conv, &net->layers[r].spec.pool, batch);
}

// The 2x2 max-pool in front of layer i (behind a folded activation, nothing folded into the pool
// itself) that the dX epilogue of layer i can route its gradient through: its index, or -1.
int pool_in_front(tdh_net *net, int i, PoolScatter *through) {
  if (!(net->flags & TDH_NET_FUSE_ACT_GRAD)) return -1;
  const int r = i - 1 - ((i >= 1 && net->layers[i - 1].grad_folded) ? 1 : 0);
  if (r < 0 || net->layers[r].spec.kind != TDH_L_MAXPOOL ||
      !maxpool_scatters_from_fc(&net->layers[r].spec.pool, through))
    return -1;
  const DxTarget behind = dx_target(net, r);
  if (behind.fold.kind != TDH_ACT_NONE) return -1;
  through->argmax = net->layers[r].argmax;
  through->dx     = behind.dx;
  return r;
}

// What a train step runs together with the loss gradient as one launch.
// layer: the fully-connected layer in front of the closing softmax under
// cross_entropy_multiclass, or a closing fully-connected layer under mse (forward, loss
// gradient and its own dX), or -1.
// first: the fully-connected layer two in front of it (a pointwise activation between them)
// when the same launch also covers that one's forward pass and leaves the gradient of its
// output, or -1.
struct TailPlan {
  int layer = -1, first = -1;
  DxTarget target;  // where the dX of `layer` goes (first < 0)
};
TailPlan plan_tail(tdh_net *net, int loss_kind, int batch) {
  TailPlan plan;
  const int n = static_cast<int>(net->layers.size());
  if (!(net->flags & TDH_NET_FUSE_ACT_GRAD)) return plan;
  int at = -1;
  if (loss_kind == TDH_LOSS_CE_MULTICLASS && n >= 2 && net->layers[n - 1].spec.kind == TDH_L_ACT &&
      net->layers[n - 1].spec.act == TDH_ACT_SOFTMAX)
    at = n - 2;
  else if (loss_kind == TDH_LOSS_MSE)
    at = n - 1;
  if (at < 0) return plan;
  const tdh_layer &fc = net->layers[at].spec;
  if (!(fc.kind == TDH_L_FC && fc_softmax_xent_applies(fc.fc_in, fc.fc_out, batch))) return plan;
  plan.layer  = at;
  plan.target = dx_target(net, at);
  if (at >= 2 && net->layers[at - 1].grad_folded && net->layers[at - 2].spec.kind == TDH_L_FC && net->tail_tickets) {
    const tdh_layer &a = net->layers[at - 2].spec;
    if (a.fc_out == fc.fc_in && fc_two_layer_tail_applies(a.fc_in, a.fc_out, fc.fc_out, batch)) {
      plan.first = at - 2;
    }
  }
  return plan;
}

// packed: the layers' wp_fwd hold the current filters in the stride-1 kernels' layout
// xent_t / xent_dz: the net ends in softmax and the step's loss is cross_entropy_multiclass: the
// last layer's kernel also writes the loss gradient with respect to the softmax input
// tail: its layer runs as fc_softmax_xent, which also writes the loss gradient (to xent_dz, from
// the targets xent_t) and the gradient of its input; with tail->first that layer, the activation
// behind it and tail->layer run as fc_two_layer_tail
// training: the pass is the first half of a train step: an output that only the kernel which
// computes it would read (a first convolution's, with the max-pool directly behind it in the
// same kernel) is not written
int forward(tdh_net *net, int batch, const float *x, bool packed = false, const float *xent_t = nullptr,
            float *xent_dz = nullptr, const TailPlan *tail = nullptr, bool training = false) {
  const float *in = x;
  const int n     = static_cast<int>(net->layers.size());
  net->out_unwritten.assign(n, 0);
  for (int i = 0; i < n; ++i) {
    tdh_net::Layer &L  = net->layers[i];
    const tdh_layer &s = L.spec;
    switch (s.kind) {
      case TDH_L_CONV:
        TDH_TRY(ws_begin(conv2d_workspace_bytes(&s.conv, batch)));
      {
        const float *wp = packed && L.wp_fwd && conv_uses_packed(&s.conv, batch, 0) ? L.wp_fwd : nullptr;
        const bool fuse = (net->flags & TDH_NET_FUSE_ACT_GRAD) != 0;
        auto pointwise = [&](int k) {
          return k < n && net->layers[k].spec.kind == TDH_L_ACT && is_pointwise_act(net->layers[k].spec.act);
        };
        // the layers behind the convolution that leave the same kernel: a pointwise activation,
        // then a 2x2 max-pool, then the activation behind the pool
        int last = i;
        float *act_out = nullptr;
        int act_kind   = TDH_ACT_NONE;
        if (fuse && pointwise(i + 1) && conv_fwd_applies_act(&s.conv, batch, wp != nullptr)) {
          last     = i + 1;
          act_out  = net->layers[last].out;
          act_kind = net->layers[last].spec.act;
        }
        PoolFuse pf{nullptr, nullptr, nullptr, TDH_ACT_NONE};
        if (fuse && !(pointwise(i + 1) && last == i) && last + 1 < n &&
            net->layers[last + 1].spec.kind == TDH_L_MAXPOOL &&
            conv_fwd_fuses_pool(&s.conv, &net->layers[last + 1].spec.pool, batch, wp != nullptr)) {
          ++last;
          pf.out    = net->layers[last].out;
          pf.argmax = net->layers[last].argmax;
          if (pointwise(last + 1) &&
              conv_fwd_pool_applies_act(&s.conv, batch, wp != nullptr, net->layers[last + 1].spec.act)) {
            ++last;
            pf.act_out  = net->layers[last].out;
            pf.act_kind = net->layers[last].spec.act;
          }
        }
        {
          // nothing behind the convolution left its kernel and a max-pool reads the result
          LeaveSplitSum leave(ctx(), fuse && last == i && i + 1 < n &&
                                         net->layers[i + 1].spec.kind == TDH_L_MAXPOOL);
          // (the backward pass reads the outputs of the layers that left the kernel, never the
          // convolution's own: the gradients of the pointwise activations are functions of y)
          const bool own_out = !(training && ((pf.out && !act_out) ||
                                              (act_out && conv_fwd_out_optional(&s.conv, batch, wp != nullptr))));
          if (!own_out) net->out_unwritten[i] = 1;
          TDH_TRY(conv2d_fwd(&s.conv, batch, in, L.w, L.b, own_out ? L.out : nullptr, L.tbl_dev, wp, act_out, act_kind,
                             pf.out ? &pf : nullptr));
        }
        i = last;
      }
        break;
      case TDH_L_FC:
        TDH_TRY(ws_begin(fc_workspace_bytes(s.fc_in, s.fc_out, batch)));
        if (tail && i == tail->first) {
          tdh_net::Layer &B = net->layers[i + 2];
          const bool softmax_behind = i + 2 == n - 2;
          TDH_TRY(fc_two_layer_tail(s.fc_in, s.fc_out, B.spec.fc_out, s.fc_bias, B.spec.fc_bias, batch, in, L.w,
                                    L.b, L.out, net->layers[i + 1].out, net->layers[i + 1].spec.act, B.w, B.b,
                                    B.out, softmax_behind ? net->layers[n - 1].out : nullptr, xent_t, xent_dz,
                                    L.dout, net->tail_partials,
                                    reinterpret_cast<unsigned int *>(net->tail_tickets)));
          i = n - 1;
        } else
        if (tail && i == tail->layer) {
          const bool softmax_behind = i == n - 2;
          TDH_TRY(fc_softmax_xent(s.fc_in, s.fc_out, s.fc_bias, batch, in, L.w, L.b, L.out,
                                  softmax_behind ? net->layers[n - 1].out : nullptr, xent_t, xent_dz,
                                  tail->target.dx, tail->target.fold));
          if (softmax_behind) ++i;
        } else
        if ((net->flags & TDH_NET_FUSE_ACT_GRAD) && i + 1 < n && net->layers[i + 1].spec.kind == TDH_L_ACT &&
            is_pointwise_act(net->layers[i + 1].spec.act)) {
          // the activation layer behind the product leaves the same kernel
          TDH_TRY(fc_fwd(s.fc_in, s.fc_out, s.fc_bias, batch, in, L.w, L.b, L.out, net->layers[i + 1].out,
                         net->layers[i + 1].spec.act));
          ++i;
        } else {
          TDH_TRY(fc_fwd(s.fc_in, s.fc_out, s.fc_bias, batch, in, L.w, L.b, L.out));
        }
        break;
      case TDH_L_MAXPOOL:
        if ((net->flags & TDH_NET_FUSE_ACT_GRAD) && i + 1 < n && net->layers[i + 1].spec.kind == TDH_L_ACT &&
            is_pointwise_act(net->layers[i + 1].spec.act)) {
          // the activation layer behind the pool leaves the same kernel
          TDH_TRY(maxpool_fwd(&s.pool, batch, in, L.out, L.argmax, net->layers[i + 1].out,
                              net->layers[i + 1].spec.act));
          ++i;
        } else {
          TDH_TRY(maxpool_fwd(&s.pool, batch, in, L.out, L.argmax));
        }
        break;
      case TDH_L_AVEPOOL: TDH_TRY(avepool_fwd(&s.pool, batch, in, L.w, L.b, L.out)); break;
      case TDH_L_BATCHNORM: {  // batch_normalization_layer.h:127-169
        const int train = !net->test_phase;
        TDH_TRY(ws_begin(batchnorm_workspace_bytes(s.bn_channels, batch)));
        TDH_TRY(batchnorm_fwd(s.bn_channels, s.bn_spatial, batch, s.bn_eps, train, in,
                              train ? L.bn_mean_cur : L.bn_mean, train ? L.bn_var_cur : L.bn_var, L.bn_stddev,
                              L.out));
      } break;
      case TDH_L_DROPOUT:      // dropout_layer.h:84-117
        TDH_TRY(dropout_fwd(L.out_size * static_cast<size_t>(batch), !net->test_phase,
                            1.0f / (1.0f - s.dropout_rate), L.mask, in, L.out));
        break;
      case TDH_L_ACT:
        if (xent_t && !(tail && tail->layer == n - 1) && i == n - 1 && s.act == TDH_ACT_SOFTMAX)
          TDH_TRY(launch_softmax_fwd_xent(batch, static_cast<int>(L.out_size), in, xent_t, L.out, xent_dz));
        else
          TDH_TRY(launch_act_fwd(s.act, s.act_p, batch, static_cast<int>(L.out_size), in, L.out));
        break;
    }
    in = net->layers[i].out;  // of the activation layer when one was fused
  }
  return finish_split_sum();  // (a max-pool has taken or finished it; this is for the error paths)
}

}  // namespace

}  // namespace tdh

using namespace tdh;

extern "C" {

int tdh_net_create(const tdh_layer *layers, int n_layers, int max_batch, int flags,
                   tdh_net **out) {
  TDH_REQUIRE_INIT();
  TDH_CHECK_ARG(layers && out && n_layers > 0 && max_batch > 0, "tdh_net_create: bad argument");
  *out = nullptr;
  tdh_net *net   = new tdh_net();
  net->max_batch = max_batch;
  net->flags     = flags;
  net->layers.resize(n_layers);
  int rc = TDH_OK;
  for (int i = 0; i < n_layers && rc == TDH_OK; ++i) {
    tdh_net::Layer &L = net->layers[i];
    L.spec            = layers[i];
    if (L.spec.kind == TDH_L_CONV && L.spec.conv.tbl) {
      L.tbl.assign(L.spec.conv.tbl,
                   L.spec.conv.tbl + static_cast<size_t>(L.spec.conv.in_c) * L.spec.conv.out_c);
      L.spec.conv.tbl = L.tbl.data();
    }
    if (L.spec.kind == TDH_L_ACT || L.spec.kind == TDH_L_DROPOUT) {
      if (i == 0) {
        rc = set_error(TDH_ERR_INVALID, "tdh_net_create: an activation or dropout layer cannot be the first layer");
        break;
      }
      if (L.spec.kind == TDH_L_DROPOUT && !(L.spec.dropout_rate >= 0.0f && L.spec.dropout_rate < 1.0f)) {
        rc = set_error(TDH_ERR_INVALID, "tdh_net_create: dropout rate %g", L.spec.dropout_rate);
        break;
      }
      L.in_size = L.out_size = net->layers[i - 1].out_size;
    }
    rc = layer_sizes(L);
    if (rc == TDH_OK && i > 0 && L.in_size != net->layers[i - 1].out_size)
      rc = set_error(TDH_ERR_INVALID, "tdh_net_create: layer %d expects %zu inputs, layer %d gives %zu",
                     i, L.in_size, i - 1, net->layers[i - 1].out_size);
    if (rc == TDH_OK && (L.in_size * max_batch >= (1ul << 31) || L.out_size * max_batch >= (1ul << 31)))
      rc = set_error(TDH_ERR_INVALID, "tdh_net_create: layer %d activations exceed 2^31 elements", i);
  }
  for (int i = 0; i < n_layers && rc == TDH_OK; ++i) {
    tdh_net::Layer &L = net->layers[i];
    const size_t act  = L.out_size * static_cast<size_t>(max_batch);
    if ((rc = net_alloc(net, L.w_size, &L.w, true))) break;
    if ((rc = net_alloc(net, L.w_size, &L.dw, true))) break;
    if ((rc = net_alloc(net, L.w_size, &L.s0w, true))) break;
    if ((rc = net_alloc(net, L.w_size, &L.s1w, true))) break;
    if ((rc = net_alloc(net, L.b_size, &L.b, true))) break;
    if ((rc = net_alloc(net, L.b_size, &L.db, true))) break;
    if ((rc = net_alloc(net, L.b_size, &L.s0b, true))) break;
    if ((rc = net_alloc(net, L.b_size, &L.s1b, true))) break;
    if ((rc = net_alloc(net, act, &L.out, true))) break;
    if ((rc = net_alloc(net, act, &L.dout, true))) break;
    if (L.spec.kind == TDH_L_MAXPOOL) {
      float *p = nullptr;
      if ((rc = net_alloc(net, act, &p, true))) break;
      L.argmax = reinterpret_cast<int32_t *>(p);
    }
    if (L.spec.kind == TDH_L_BATCHNORM) {
      const size_t c = static_cast<size_t>(L.spec.bn_channels);
      if ((rc = net_alloc(net, c, &L.bn_mean, true))) break;
      if ((rc = net_alloc(net, c, &L.bn_var, true))) break;
      if ((rc = net_alloc(net, c, &L.bn_mean_cur, true))) break;
      if ((rc = net_alloc(net, c, &L.bn_var_cur, true))) break;
      if ((rc = net_alloc(net, c, &L.bn_stddev, true))) break;
    }
    if (L.spec.kind == TDH_L_DROPOUT) {
      float *p = nullptr;
      if ((rc = net_alloc(net, ceil_div_sz(act, sizeof(float)), &p, true))) break;
      L.mask = reinterpret_cast<uint8_t *>(p);
    }
    if ((flags & TDH_NET_GRAPH) && L.spec.kind == TDH_L_CONV && L.spec.conv.w_stride == 1 &&
        L.spec.conv.h_stride == 1) {
      if ((rc = net_alloc(net, L.w_size, &L.wp_fwd, false))) break;
      if ((rc = net_alloc(net, L.w_size, &L.wp_dx, false))) break;
    }
    if (!L.tbl.empty()) {
      float *p = nullptr;
      if ((rc = net_alloc(net, ceil_div_sz(L.tbl.size(), sizeof(float)), &p, false))) break;
      L.tbl_dev = reinterpret_cast<uint8_t *>(p);
      if ((rc = tdh_memcpy_h2d(L.tbl_dev, L.tbl.data(), L.tbl.size()))) break;
    }
    size_t need = 0;
    if (L.spec.kind == TDH_L_CONV) need = conv2d_workspace_bytes(&L.spec.conv, max_batch);
    if (L.spec.kind == TDH_L_FC) need = fc_workspace_bytes(L.spec.fc_in, L.spec.fc_out, max_batch);
    if (L.spec.kind == TDH_L_AVEPOOL) need = avepool_workspace_bytes(&L.spec.pool, max_batch);
    if (L.spec.kind == TDH_L_BATCHNORM) need = batchnorm_workspace_bytes(L.spec.bn_channels, max_batch);
    if (flags & TDH_NET_GRAPH)  // three times: dX, dW and db are separate calls of the operator there
      net->scratch += 3 * ws_align(need);
    else if (need > net->scratch)
      net->scratch = need;
    // fold pointwise activation gradients into the following layer's backward kernel (the dX
    // epilogue of a conv / fc layer, the scatter of a max-pool, the dX kernel of an average pool)
    if ((flags & TDH_NET_FUSE_ACT_GRAD) && L.spec.kind == TDH_L_ACT &&
        is_pointwise_act(L.spec.act) && i + 1 < n_layers &&
        (layers[i + 1].kind == TDH_L_CONV || layers[i + 1].kind == TDH_L_FC ||
         layers[i + 1].kind == TDH_L_MAXPOOL || layers[i + 1].kind == TDH_L_AVEPOOL))
      L.grad_folded = true;
  }
  if (rc == TDH_OK)
    rc = net_alloc(net, net->layers[0].in_size * static_cast<size_t>(max_batch), &net->dx_in, true);
  if (rc == TDH_OK) {
    // nodes::update_weights order: layers front to back, weight before bias
    std::vector<OptTensor> table;
    uint32_t block = 0;
    for (auto &L : net->layers) {
      for (int which = 0; which < 2; ++which) {
        const size_t n = which ? L.b_size : L.w_size;
        if (!n) continue;
        OptTensor t;
        t.wp_fwd = t.wp_dx = nullptr;
        t.tbl = nullptr;
        t.C = t.Kc = t.rs = 1;
        if (!which && L.wp_fwd) {
          t.wp_fwd = L.wp_fwd;
          t.wp_dx  = L.wp_dx;
          t.tbl    = L.spec.conv.tbl ? L.tbl_dev : nullptr;
          t.C      = static_cast<uint32_t>(L.spec.conv.in_c);
          t.Kc     = static_cast<uint32_t>(L.spec.conv.out_c);
          t.rs     = static_cast<uint32_t>(L.spec.conv.k_w * L.spec.conv.k_h);
        }
        t.g  = which ? L.db : L.dw;
        t.w  = which ? L.b : L.w;
        t.s0 = which ? L.s0b : L.s0w;
        t.s1 = which ? L.s1b : L.s1w;
        t.n  = static_cast<uint32_t>(n);
        t.first_block = block;
        // weight gradients whose kernels may leave split sums to the optimizer: small blocks,
        // eight groups of lanes add the slices of OPT_SUM_ELEMS_PER_BLOCK elements
        // (and every tensor of a net that may run the workgroup-per-sample step, whose
        // per-sample slices take the same way)
        t.block_elems = (((L.spec.kind == TDH_L_CONV || L.spec.kind == TDH_L_FC) && (flags & TDH_NET_GRAPH)) ||
                         (flags & TDH_NET_SAMPLE_STEP))
                          ? OPT_SUM_ELEMS_PER_BLOCK : OPT_MULTI_ELEMS_PER_BLOCK;
        if (n > (1u << 22)) t.block_elems = OPT_MULTI_ELEMS_PER_BLOCK;  // (bandwidth matters there)
        (which ? L.b_sums_in_opt : L.w_sums_in_opt) = t.block_elems == OPT_SUM_ELEMS_PER_BLOCK;
        block += static_cast<uint32_t>(ceil_div_sz(n, t.block_elems));
        net->opt_params += static_cast<double>(n);
        table.push_back(t);
      }
    }
    net->opt_tensors = static_cast<int>(table.size());
    net->opt_blocks  = static_cast<int>(block);
    if (!table.empty()) {
      float *p = nullptr;
      rc = net_alloc(net, ceil_div_sz(table.size() * sizeof(OptTensor), sizeof(float)), &p, false);
      if (rc == TDH_OK) {
        net->opt_table = reinterpret_cast<OptTensor *>(p);
        rc = tdh_memcpy_h2d(net->opt_table, table.data(), table.size() * sizeof(OptTensor));
        net->opt_table_host = table;
      }
    }
  }
  if (rc == TDH_OK) rc = net_alloc(net, 8, &net->dev_powers, true);
  if (rc == TDH_OK && (flags & TDH_NET_FUSE_ACT_GRAD)) {
    // [fc, pointwise activation, fc] closes the net, or stands in front of a closing softmax
    int b = n_layers - 1;
    if (layers[b].kind == TDH_L_ACT && layers[b].act == TDH_ACT_SOFTMAX) --b;
    if (b >= 2 && layers[b].kind == TDH_L_FC && layers[b - 2].kind == TDH_L_FC && net->layers[b - 1].grad_folded &&
        fc_two_layer_tail_applies(layers[b - 2].fc_in, layers[b - 2].fc_out, layers[b].fc_out, max_batch)) {
      rc = net_alloc(net, fc_two_layer_tail_tickets(max_batch), &net->tail_tickets, true);
      if (rc == TDH_OK)
        rc = net_alloc(net, fc_two_layer_tail_partials(layers[b - 2].fc_in, max_batch), &net->tail_partials, false);
    }
  }
  if (rc == TDH_OK && (flags & TDH_NET_GRAPH)) {
    Context &c = ctx();
    for (hipStream_t &s : c.side)
      if (!s && hipStreamCreateWithFlags(&s, hipStreamNonBlocking) != hipSuccess)
        rc = set_error(TDH_ERR_HIP, "tdh_net_create: cannot create a side stream");
    // events: [0,n) gradient forks, 2n and 2n+1 joins, 2n+2 start of the step
    for (int i = 0; rc == TDH_OK && i < 2 * n_layers + 4; ++i) {
      hipEvent_t e = nullptr;
      if (hipEventCreateWithFlags(&e, hipEventDisableTiming) != hipSuccess)
        rc = set_error(TDH_ERR_HIP, "tdh_net_create: cannot create an event");
      else
        net->events.push_back(e);
    }
  }
  if (rc == TDH_OK) rc = build_tiny_plan(net);
  // reserve the scratch every layer may need, so that no op ever has to grow it
  if (rc == TDH_OK) rc = ws_begin(net->scratch);
  if (rc != TDH_OK) {
    for (hipEvent_t e : net->events) (void)hipEventDestroy(e);
    for (void *p : net->allocs) (void)hipFree(p);
    delete net;
    return rc;
  }
  *out = net;
  return TDH_OK;
}

int tdh_net_destroy(tdh_net *net) {
  TDH_REQUIRE_INIT();
  if (!net) return TDH_OK;
  TDH_HIP(hipStreamSynchronize(ctx().stream));
  for (auto &g : net->graphs)
    if (g.exec) TDH_HIP(hipGraphExecDestroy(g.exec));
  for (hipEvent_t e : net->events) TDH_HIP(hipEventDestroy(e));
  for (void *p : net->allocs) TDH_HIP(hipFree(p));
  delete net;
  return TDH_OK;
}

size_t tdh_net_in_size(const tdh_net *net) { return net->layers.front().in_size; }
size_t tdh_net_out_size(const tdh_net *net) { return net->layers.back().out_size; }
size_t tdh_net_layer_out_size(const tdh_net *net, int layer) {
  return (layer >= 0 && layer < static_cast<int>(net->layers.size())) ? net->layers[layer].out_size : 0;
}
size_t tdh_net_param_size(const tdh_net *net, int layer, int which) {
  if (layer < 0 || layer >= static_cast<int>(net->layers.size())) return 0;
  const tdh_net::Layer &L = net->layers[layer];
  if ((which == 2 || which == 3) && L.spec.kind == TDH_L_BATCHNORM) return static_cast<size_t>(L.spec.bn_channels);
  return which == 0 ? L.w_size : (which == 1 ? L.b_size : 0);
}
static float *net_param_ptr(tdh_net *net, int layer, int which) {
  if (layer < 0 || layer >= static_cast<int>(net->layers.size())) return nullptr;
  tdh_net::Layer &L = net->layers[layer];
  if (which == 2) return L.bn_mean;
  if (which == 3) return L.bn_var;
  return which == 0 ? L.w : (which == 1 ? L.b : nullptr);
}
float *tdh_net_param(tdh_net *net, int layer, int which) {
  if (net) net->packs_valid = false;  // the caller may write through the pointer
  return net ? net_param_ptr(net, layer, which) : nullptr;
}
int tdh_net_set_param(tdh_net *net, int layer, int which, const float *host_src) {
  TDH_REQUIRE_INIT();
  float *dst = tdh_net_param(net, layer, which);  // marks the packed filters stale
  const size_t n = tdh_net_param_size(net, layer, which);
  TDH_CHECK_ARG(n == 0 || (dst && host_src), "tdh_net_set_param: no such parameter");
  return tdh_memcpy_h2d(dst, host_src, n * sizeof(float));
}
int tdh_net_reset_optimizer(tdh_net *net) {
  TDH_REQUIRE_INIT();
  TDH_CHECK_ARG(net != nullptr, "tdh_net_reset_optimizer: null net");
  for (tdh_net::Layer &L : net->layers) {
    float *state[4]      = {L.s0w, L.s1w, L.s0b, L.s1b};
    const size_t size[4] = {L.w_size, L.w_size, L.b_size, L.b_size};
    for (int i = 0; i < 4; ++i)
      if (state[i] && size[i]) TDH_TRY(launch_fill_zero(state[i], size[i] * sizeof(float)));
  }
  return TDH_OK;
}
// layer::update_weight ends in post_update (layer.h:681): a batch-norm layer moves its running
// averages towards the moments of the batch (batch_normalization_layer.h:171-177)
static int post_update(tdh_net *net) {
  for (tdh_net::Layer &L : net->layers)
    if (L.spec.kind == TDH_L_BATCHNORM)
      TDH_TRY(batchnorm_update_moving(L.spec.bn_channels, L.spec.bn_momentum, L.bn_mean_cur, L.bn_var_cur,
                                      L.bn_mean, L.bn_var));
  return TDH_OK;
}

int tdh_net_update_weights(tdh_net *net, tdh_opt *opt) {
  TDH_REQUIRE_INIT();
  TDH_CHECK_ARG(net && opt, "tdh_net_update_weights: null argument");
  // the optimizer kernel keeps the packed filter copies of a graph net current, as in a step
  TDH_TRY(launch_opt_update_multi(opt, net->opt_table, net->opt_tensors, net->opt_blocks,
                                  net->opt_params, 1.0f, 1, nullptr, nullptr, nullptr, net->opt_table_host.data()));
  return post_update(net);
}
int tdh_net_set_phase(tdh_net *net, int train) {
  TDH_REQUIRE_INIT();
  TDH_CHECK_ARG(net != nullptr, "tdh_net_set_phase: null net");
  net->test_phase = !train;
  return TDH_OK;
}
int tdh_net_set_dropout_mask(tdh_net *net, int layer, int batch, const uint8_t *host_mask) {
  TDH_REQUIRE_INIT();
  TDH_CHECK_ARG(net && host_mask && layer >= 0 && layer < static_cast<int>(net->layers.size()) &&
                  net->layers[layer].spec.kind == TDH_L_DROPOUT && batch > 0 && batch <= net->max_batch,
                "tdh_net_set_dropout_mask: bad argument");
  tdh_net::Layer &L = net->layers[layer];
  return tdh_memcpy_h2d(L.mask, host_mask, L.out_size * static_cast<size_t>(batch));
}
int tdh_net_clear_grads(tdh_net *net) {
  TDH_REQUIRE_INIT();
  TDH_CHECK_ARG(net != nullptr, "tdh_net_clear_grads: null net");
  for (tdh_net::Layer &L : net->layers) {
    if (L.dw && L.w_size) TDH_TRY(launch_fill_zero(L.dw, L.w_size * sizeof(float)));
    if (L.db && L.b_size) TDH_TRY(launch_fill_zero(L.db, L.b_size * sizeof(float)));
  }
  return TDH_OK;
}
int tdh_net_get_param(tdh_net *net, int layer, int which, float *host_dst) {
  TDH_REQUIRE_INIT();
  const float *src = net_param_ptr(net, layer, which);
  const size_t n   = tdh_net_param_size(net, layer, which);
  TDH_CHECK_ARG(n == 0 || (src && host_dst), "tdh_net_get_param: no such parameter");
  return tdh_memcpy_d2h(host_dst, src, n * sizeof(float));
}
const float *tdh_net_layer_out(const tdh_net *net, int layer) {
  if (layer < 0 || layer >= static_cast<int>(net->layers.size())) return nullptr;
  if (static_cast<size_t>(layer) < net->out_unwritten.size() && net->out_unwritten[layer]) return nullptr;
  return net->layers[layer].out;
}
const float *tdh_net_layer_dx(const tdh_net *net, int layer) {
  if (layer < 0 || layer >= static_cast<int>(net->layers.size())) return nullptr;
  if (static_cast<size_t>(layer) < net->dx_unwritten.size() && net->dx_unwritten[layer]) return nullptr;
  return layer == 0 ? net->dx_in : net->layers[layer - 1].dout;
}
const float *tdh_net_layer_grad(const tdh_net *net, int layer, int which) {
  if (layer < 0 || layer >= static_cast<int>(net->layers.size())) return nullptr;
  return which == 0 ? net->layers[layer].dw : (which == 1 ? net->layers[layer].db : nullptr);
}
const int32_t *tdh_net_layer_argmax(const tdh_net *net, int layer) {
  return (layer >= 0 && layer < static_cast<int>(net->layers.size())) ? net->layers[layer].argmax : nullptr;
}

int tdh_net_forward(tdh_net *net, int batch, const float *x) {
  TDH_REQUIRE_INIT();
  TDH_CHECK_ARG(net && x && batch > 0 && batch <= net->max_batch, "tdh_net_forward: bad argument");
  return forward(net, batch, x);
}

// Queues one whole train step on the library stream. forked (only while the stream is being
// captured): the weight and bias gradients of every conv / fc layer branch off onto the side
// stream, because nothing before the optimizer waits for them; the main stream carries only
// the chain forward -> loss -> dX ... -> dX, and the two join in front of the optimizer. The
// kernels and their arguments are the same either way, so are the results.
static int enqueue_step(tdh_net *net, tdh_opt *opt, int loss_kind, int batch, const float *x,
                        const float *t, int do_update, const float *powers_in, float *powers_out,
                        bool forked = false) {
  if (tiny_step_applies(net, loss_kind)) {
    // a small net: one workgroup per sample runs forward, loss and the input gradients out of
    // LDS, a second launch computes every sample's weight and bias gradients, a third adds
    // those slices in sample order, the fourth is the optimizer (tiny_net.hip)
    const tdh_layer &closing = net->layers.back().spec;
    const int softmax_xent = closing.kind == TDH_L_ACT && closing.act == TDH_ACT_SOFTMAX;
    net->dx_unwritten.assign(net->layers.size(), 0);   // everything is written to memory as well
    if (net_skips_input_grad(net)) net->dx_unwritten[0] = 1;
    net->out_unwritten.assign(net->layers.size(), 0);
    TDH_TRY(launch_tiny_step(net->tiny, net->tiny_dev, loss_kind, softmax_xent, batch, x, t));
    TDH_TRY(launch_tiny_params(net->tiny, net->tiny_dev, batch, x));
    // the samples' slices: added to the gradient tensors in sample order by a launch of their
    // own when the step stops there; otherwise the optimizer adds them up as it does the split
    // sums of the layer-by-layer step (it clears the gradient tensors afterwards either way)
    const TinyMerge &M = net->tiny_merge;
    bool to_optimizer = do_update && M.n <= OPT_PENDING_MAX;
    OptPending pending;
    pending.n = 0;
    for (int j = 0; j < M.n && to_optimizer; ++j) {
      bool small_blocks = false;
      for (const tdh_net::Layer &L : net->layers)
        if ((M.g[j] == L.dw && L.w_sums_in_opt) || (M.g[j] == L.db && L.b_sums_in_opt)) small_blocks = true;
      to_optimizer = small_blocks;
      pending.sum[pending.n++] = {M.slices[j], M.g[j], static_cast<uint32_t>(batch), static_cast<uint32_t>(M.len[j])};
    }
    if (!to_optimizer) TDH_TRY(launch_tiny_merge(net->tiny_merge, batch));
    if (!do_update) return TDH_OK;
    TDH_TRY(launch_opt_update_multi(opt, net->opt_table, net->opt_tensors, net->opt_blocks, net->opt_params, 1.0f,
                                    1, powers_in, powers_out, to_optimizer ? &pending : nullptr,
                                    net->opt_table_host.data()));
    return post_update(net);
  }
  Context &c = ctx();
  struct KeepScratch {  // hands out disjoint scratch pieces for the whole backward pass
    Context &c;
    bool on;
    KeepScratch(Context &cc, bool o) : c(cc), on(o) {}
    void start() { if (on) { c.workspace_off = 0; c.ws_keep = true; } }
    ~KeepScratch() { c.ws_keep = false; }
  } keep(c, forked || (!forked && ((profiling_active() && (net->flags & TDH_NET_GRAPH) && net_forks(net, batch)) ||
                                   net_defers_serially(net, batch))));
  bool side_used[2] = {false, false};
  bool last_dw_on_main = false;  // the last split sums were left behind the side stream's work
  // The split reductions behind the weight-gradient kernels and the row sums of the bias
  // gradients of a branching step are collected and launched once each behind the last layer:
  // one launch per layer would sit at the end of its side stream's queue anyway, and every
  // launch there costs its own dispatch latency.
  struct Deferred {
    Context &c;
    explicit Deferred(Context &cc) : c(cc) {}
    ~Deferred() {
      c.defer_reduce = c.defer_rowsum = false;
      c.leave_split_sum = c.split_sum_left = false;
      flush_deferred_reduces(false);
      flush_deferred_rowsums(false);
    }
  } deferred(c);
  // the per-kernel timing pass of a net whose captured step branches launches what that step
  // launches (a branching step computes dX, dW and db of a layer separately)
  const bool small_defers = !forked && net_defers_serially(net, batch);
  const bool as_forked = !forked && ((profiling_active() && (net->flags & TDH_NET_GRAPH) && net_forks(net, batch)) ||
                                     small_defers);
  const int n   = static_cast<int>(net->layers.size());
  // the optimizer kernel keeps the packed filters of the stride-1 kernels current
  const bool packed = net->packs_valid;
  tdh_net::Layer &last = net->layers[n - 1];
  int first_bwd        = n - 1;
  int tail_done        = -1;     // this layer already has the gradient of its input
  int pool_done        = -1;     // a max-pool layer whose backward pass the layer behind it did
  PoolGather through_pool;       // a max-pool layer whose backward pass the convolution in front
  int through_pool_for = -1;     // does while it reads its output gradient: that convolution
  FcGrads also         = {};     // the closing layer's weight and bias gradients, left to ...
  int also_for         = -1;     // ... this layer's backward launch
  // softmax + cross_entropy_multiclass: one closed-form kernel instead of -t/y followed by
  // the full softmax Jacobian, and that kernel is the softmax layer's forward kernel
  const TailPlan plan = plan_tail(net, loss_kind, batch);
  tail_done           = plan.layer;
  if (loss_kind == TDH_LOSS_CE_MULTICLASS && last.spec.kind == TDH_L_ACT &&
      last.spec.act == TDH_ACT_SOFTMAX && n >= 2) {
    TDH_TRY(forward(net, batch, x, packed, t, net->layers[n - 2].dout, tail_done >= 0 ? &plan : nullptr, true));
    first_bwd = n - 2;
  } else if (tail_done >= 0) {
    // mse on a closing fully-connected layer: its kernel writes the loss gradient too
    TDH_TRY(forward(net, batch, x, packed, t, last.dout, &plan, true));
  } else {
    TDH_TRY(forward(net, batch, x, packed, nullptr, nullptr, nullptr, true));
    TDH_TRY(launch_loss_grad(loss_kind, batch, static_cast<int>(last.out_size), last.out, t,
                             last.dout));
  }
  keep.start();
  net->dx_unwritten.assign(n, 0);
  for (int i = 1; i < n; ++i)  // (a folded activation gradient never leaves the registers)
    net->dx_unwritten[i] = net->layers[i - 1].grad_folded ? 1 : 0;
  for (int i = first_bwd; i >= 0; --i) {
    tdh_net::Layer &L  = net->layers[i];
    const tdh_layer &s = L.spec;
    const float *in    = i == 0 ? x : net->layers[i - 1].out;
    const DxTarget target = dx_target(net, i);
    float *dx             = target.dx;
    const ActGrad fold    = target.fold;
    if (i == 0 && net_skips_input_grad(net)) {
      dx = nullptr;
      net->dx_unwritten[0] = 1;
    }
    if (i == tail_done) {
      // only the weight and bias gradients are left, and nothing before the optimizer reads
      // them: they leave with the backward launch of the fully-connected layer two in front
      // when that is the one-launch kernel, else as one launch, on the side stream when the
      // step branches
      if (plan.first >= 0 && !(plan.first == 0 && net_skips_input_grad(net)) && fc_bwd_fuses(s.fc_in, s.fc_out, batch) &&
          fc_bwd_fuses(net->layers[plan.first].spec.fc_in, net->layers[plan.first].spec.fc_out, batch)) {
        also = FcGrads{s.fc_in, s.fc_out, in, L.dout, L.dw, L.b_size ? L.db : nullptr};
        also_for = plan.first;
        continue;
      }
      TDH_TRY(ws_begin(fc_workspace_bytes(s.fc_in, s.fc_out, batch)));
      if (forked) {
        TDH_HIP(hipEventRecord(net->events[i], c.stream));
        TDH_HIP(hipStreamWaitEvent(c.side[0], net->events[i], 0));
        side_used[0] = true;
        StreamSwap on_side(c.side[0]);
        TDH_TRY(fc_bwd(s.fc_in, s.fc_out, s.fc_bias, batch, in, L.w, L.dout, nullptr, L.dw,
                       L.b_size ? L.db : nullptr, 1, ActGrad()));
      } else {
        TDH_TRY(fc_bwd(s.fc_in, s.fc_out, s.fc_bias, batch, in, L.w, L.dout, nullptr, L.dw,
                       L.b_size ? L.db : nullptr, 1, ActGrad()));
      }
      continue;
    }
    // a small fully-connected layer computes its three gradients in one launch on the main
    // chain: its weight and bias products are too small to be worth a branch
    const bool fc_one_launch = s.kind == TDH_L_FC && fc_bwd_fuses(s.fc_in, s.fc_out, batch);
    const bool fork = forked && layer_forks(L) && !fc_one_launch;
    if (fork) {
      // this layer's output gradient is complete here: let the side streams start from it
      TDH_HIP(hipEventRecord(net->events[i], c.stream));
      TDH_HIP(hipStreamWaitEvent(c.side[0], net->events[i], 0));
      side_used[0] = true;
      // the second side stream carries the bias gradient where that is a launch of its own
      const bool own_db = L.b_size && !(s.kind == TDH_L_CONV && conv_dw_gives_db(&s.conv, batch));
      if (own_db) {
        TDH_HIP(hipStreamWaitEvent(c.side[1], net->events[i], 0));
        side_used[1] = true;
      }
    }
    switch (s.kind) {
      case TDH_L_CONV:
        TDH_TRY(ws_begin((forked || as_forked ? 3 : 1) * conv2d_workspace_bytes(&s.conv, batch)));
      {
        const PoolGather *gp = i == through_pool_for ? &through_pool : nullptr;
        const float *wp = packed && L.wp_dx && conv_uses_packed(&s.conv, batch, 1) ? L.wp_dx : nullptr;
        // the layer that reads this dX next (behind a folded activation) is a max-pool: its
        // backward kernel can add up a split reduction of dX
        const int reader = i - 1 - ((i >= 1 && net->layers[i - 1].grad_folded) ? 1 : 0);
        const bool pool_reads = (net->flags & TDH_NET_FUSE_ACT_GRAD) && reader >= 0 &&
                                net->layers[reader].spec.kind == TDH_L_MAXPOOL;
        if (forked) {
          if (!fork) {
            LeaveSplitSum leave(c, pool_reads);
            TDH_TRY(conv2d_bwd(&s.conv, batch, in, L.w, L.dout, dx, L.dw, L.b_size ? L.db : nullptr, 1, fold,
                               L.tbl_dev, wp, gp));
            break;
          }
          const bool db_with_dw = L.b_size && conv_dw_gives_db(&s.conv, batch);
          if (i == 0 && dx && !wp && conv_bwd_one_launch(&s.conv, batch, gp != nullptr)) {
            // the net's first layer, all its gradients from one launch (on the main stream,
            // like the two launches below)
            c.defer_reduce = true;
            TDH_TRY(conv2d_bwd(&s.conv, batch, in, L.w, L.dout, dx, L.dw, L.b_size ? L.db : nullptr, 1, fold,
                               L.tbl_dev, nullptr, gp));
            c.defer_reduce = false;
            last_dw_on_main = true;
            break;
          }
          if (dx) {
            LeaveSplitSum leave(c, pool_reads);
            TDH_TRY(conv2d_bwd(&s.conv, batch, in, L.w, L.dout, dx, nullptr, nullptr, 1, fold, L.tbl_dev, wp, gp));
          }
          if (i == 0 && (db_with_dw || !L.b_size)) {
            // The net's first layer: nothing waits for its dX, and its two kernels share nothing
            // and each fills the chip. Side by side they took 53 us on the CIFAR net, one after
            // the other 33: the weight gradient follows on the main stream. (It does not wait
            // for the side stream: by then that stream's last kernel is about to end, and a
            // wait across streams is 5 us of a replayed step whether or not it has to wait.)
            c.defer_reduce = true;
            TDH_TRY(conv2d_bwd(&s.conv, batch, in, L.w, L.dout, nullptr, L.dw, db_with_dw ? L.db : nullptr, 1,
                               ActGrad(), L.tbl_dev, nullptr, gp));
            c.defer_reduce = false;
            last_dw_on_main = true;
            break;
          }
          {
            StreamSwap on_side(c.side[0]);
            c.defer_reduce = true;
            TDH_TRY(conv2d_bwd(&s.conv, batch, in, L.w, L.dout, nullptr, L.dw, db_with_dw ? L.db : nullptr, 1,
                               ActGrad(), L.tbl_dev, nullptr, gp));
            c.defer_reduce = false;
          }
          if (L.b_size && !db_with_dw) {
            StreamSwap on_side(c.side[1]);
            c.defer_rowsum = true;
            TDH_TRY(conv2d_bwd(&s.conv, batch, in, L.w, L.dout, nullptr, nullptr, L.db, 1, ActGrad(), L.tbl_dev, nullptr, gp));
            c.defer_rowsum = false;
          }
        } else if (as_forked) {
          // the launches of the captured, branching step, one after the other
          if (i == 0 && dx && !wp && conv_bwd_one_launch(&s.conv, batch, gp != nullptr)) {
            c.defer_reduce = true;
            TDH_TRY(conv2d_bwd(&s.conv, batch, in, L.w, L.dout, dx, L.dw, L.b_size ? L.db : nullptr, 1, fold,
                               L.tbl_dev, nullptr, gp));
            c.defer_reduce = false;
            break;
          }
          if (dx) {
            LeaveSplitSum leave(c, pool_reads);
            TDH_TRY(conv2d_bwd(&s.conv, batch, in, L.w, L.dout, dx, nullptr, nullptr, 1, fold, L.tbl_dev, wp, gp));
          }
          const bool db_with_dw = L.b_size && conv_dw_gives_db(&s.conv, batch);
          c.defer_reduce = true;
          TDH_TRY(conv2d_bwd(&s.conv, batch, in, L.w, L.dout, nullptr, L.dw, db_with_dw ? L.db : nullptr, 1,
                             ActGrad(), L.tbl_dev, nullptr, gp));
          c.defer_reduce = false;
          if (L.b_size && !db_with_dw) {
            c.defer_rowsum = small_defers;
            TDH_TRY(conv2d_bwd(&s.conv, batch, in, L.w, L.dout, nullptr, nullptr, L.db, 1, ActGrad(), L.tbl_dev, nullptr, gp));
            c.defer_rowsum = false;
          }
        } else {
          LeaveSplitSum leave(c, pool_reads);
          TDH_TRY(conv2d_bwd(&s.conv, batch, in, L.w, L.dout, dx, L.dw, L.b_size ? L.db : nullptr, 1,
                             fold, L.tbl_dev, wp, gp));
        }
      } break;
      case TDH_L_FC:
        TDH_TRY(ws_begin(fc_workspace_bytes(s.fc_in, s.fc_out, batch)));
        if (fork) {
          if (dx) TDH_TRY(fc_bwd(s.fc_in, s.fc_out, s.fc_bias, batch, in, L.w, L.dout, dx, nullptr, nullptr, 1, fold));
          {
            StreamSwap on_side(c.side[0]);
            c.defer_reduce = true;
            TDH_TRY(fc_bwd(s.fc_in, s.fc_out, s.fc_bias, batch, in, L.w, L.dout, nullptr, L.dw, nullptr, 1, ActGrad()));
            c.defer_reduce = false;
          }
          if (L.b_size) {
            StreamSwap on_side(c.side[1]);
            TDH_TRY(fc_bwd(s.fc_in, s.fc_out, s.fc_bias, batch, in, L.w, L.dout, nullptr, nullptr, L.db, 1, ActGrad()));
          }
        } else if (as_forked && !fc_one_launch) {
          // the launches of the captured, branching step, one after the other
          if (dx) TDH_TRY(fc_bwd(s.fc_in, s.fc_out, s.fc_bias, batch, in, L.w, L.dout, dx, nullptr, nullptr, 1, fold));
          c.defer_reduce = true;
          TDH_TRY(fc_bwd(s.fc_in, s.fc_out, s.fc_bias, batch, in, L.w, L.dout, nullptr, L.dw, nullptr, 1, ActGrad()));
          c.defer_reduce = false;
          if (L.b_size)
            TDH_TRY(fc_bwd(s.fc_in, s.fc_out, s.fc_bias, batch, in, L.w, L.dout, nullptr, nullptr, L.db, 1, ActGrad()));
        } else {
          // a 2x2 max-pool in front (behind a folded activation, nothing folded into the pool
          // itself): the one-launch kernel's dX epilogue also routes the gradient through it
          PoolScatter through;
          int reader = fc_one_launch && fc_bwd_scatters_pool(s.fc_in, s.fc_out, batch)
                         ? pool_in_front(net, i, &through) : -1;
          if (reader >= 0 && pool_read_by_conv(net, reader, batch)) reader = -1;  // (less to write)
          TDH_TRY(fc_bwd(s.fc_in, s.fc_out, s.fc_bias, batch, in, L.w, L.dout, dx, L.dw,
                         L.b_size ? L.db : nullptr, 1, fold, reader >= 0 ? &through : nullptr,
                         i == also_for ? &also : nullptr));
          if (reader >= 0) pool_done = reader;
        }
        break;
      case TDH_L_MAXPOOL:
        if (i == pool_done) break;  // the layer behind has written this layer's dX
        // a first convolution directly in front reads the pooled gradient and the argmax
        // records itself: its output gradient, four times their size, is never written
        if (pool_read_by_conv(net, i, batch)) {
          TDH_TRY(finish_split_sum());  // (the kernels read a finished gradient)
          net->dx_unwritten[i] = 1;
          through_pool = PoolGather{L.dout, L.argmax};
          through_pool_for = i - 1;
          break;
        }
        TDH_TRY(maxpool_bwd(&s.pool, batch, L.dout, L.argmax, dx, fold, L.out));
        break;
      case TDH_L_AVEPOOL:
        TDH_TRY(ws_begin(avepool_workspace_bytes(&s.pool, batch)));
        TDH_TRY(avepool_bwd(&s.pool, batch, in, L.w, L.dout, dx, L.dw, L.db, 1, fold));
        break;
      case TDH_L_ACT:
        if (!L.grad_folded)
          TDH_TRY(launch_act_bwd(s.act, s.act_p, batch, static_cast<int>(L.out_size), in, L.out, L.dout, dx));
        break;
      case TDH_L_BATCHNORM:  // batch_normalization_layer.h:87-125
        TDH_TRY(ws_begin(batchnorm_workspace_bytes(s.bn_channels, batch)));
        TDH_TRY(batchnorm_bwd(s.bn_channels, s.bn_spatial, batch, L.out, L.dout, L.bn_stddev, dx));
        if (fold.kind != TDH_ACT_NONE) return set_error(TDH_ERR_INVALID, "batch-norm behind a folded activation");
        break;
      case TDH_L_DROPOUT:    // dropout_layer.h:62-82
        TDH_TRY(dropout_bwd(L.out_size * static_cast<size_t>(batch), L.mask, L.dout, dx));
        if (fold.kind != TDH_ACT_NONE) return set_error(TDH_ERR_INVALID, "dropout behind a folded activation");
        break;
    }
  }
  TDH_TRY(finish_split_sum());  // (a max-pool has taken or finished it)
  // the split sums of the weight gradients: added up by the optimizer kernel when it runs next
  // and every tensor concerned has the small blocks for that, else by a launch of their own
  OptPending pending;
  pending.n = 0;
  bool to_optimizer = false;
  if ((side_used[0] || as_forked) && do_update && peek_deferred_reduces(&pending)) {
    to_optimizer = true;
    for (int k = 0; k < pending.n; ++k) {
      bool small_blocks = false;
      for (const tdh_net::Layer &L : net->layers)
        if ((pending.sum[k].g == L.dw && L.w_sums_in_opt) || (pending.sum[k].g == L.db && L.b_sums_in_opt))
          small_blocks = true;
      to_optimizer = to_optimizer && small_blocks;
    }
    if (to_optimizer) TDH_TRY(flush_deferred_reduces(false));  // (forgets them: the optimizer has them)
  }
  if (side_used[0] && !to_optimizer && !last_dw_on_main) {
    StreamSwap on_side(c.side[0]);
    TDH_TRY(flush_deferred_reduces());
  } else if ((as_forked || last_dw_on_main) && !to_optimizer) {
    if (last_dw_on_main && side_used[0]) {  // (the side stream's kernels wrote some of the slices)
      TDH_HIP(hipEventRecord(net->events[2 * n], c.side[0]));
      TDH_HIP(hipStreamWaitEvent(c.stream, net->events[2 * n], 0));
    }
    TDH_TRY(flush_deferred_reduces());
  }
  if (side_used[1]) {
    StreamSwap on_side(c.side[1]);
    TDH_TRY(flush_deferred_rowsums());
  } else if (small_defers) {
    TDH_TRY(flush_deferred_rowsums());
  }
  for (int k = 0; k < 2; ++k) {  // the optimizer (and the end of the capture) wait for the branches
    if (!side_used[k]) continue;
    TDH_HIP(hipEventRecord(net->events[2 * n + k], c.side[k]));
    TDH_HIP(hipStreamWaitEvent(c.stream, net->events[2 * n + k], 0));
  }
  if (!do_update) return TDH_OK;
  // nodes::update_weights visits layers front to back, weight before bias; the gradient
  // reaches the optimizer unscaled (rcp_batch_size is 1, see tdh_opt_update) and is then
  // cleared (layer.h:680)
  TDH_TRY(launch_opt_update_multi(opt, net->opt_table, net->opt_tensors, net->opt_blocks,
                                  net->opt_params, 1.0f, 1, powers_in, powers_out,
                                  to_optimizer ? &pending : nullptr, net->opt_table_host.data()));
  return post_update(net);
}

static bool same_key(const tdh_net::GraphKey &a, const tdh_net::GraphKey &b) {
  // field by field: a caller's tdh_opt may carry padding or unused fields it never wrote
  const tdh_opt &p = a.hyper, &q = b.hyper;
  return a.batch == b.batch && a.loss == b.loss && a.do_update == b.do_update && a.test_phase == b.test_phase &&
         a.powers_at == b.powers_at && a.n_steps == b.n_steps &&
         std::equal(a.x, a.x + a.n_steps, b.x) && std::equal(a.t, a.t + a.n_steps, b.t) && a.scratch == b.scratch && p.kind == q.kind && p.alpha == q.alpha &&
         p.lambda == q.lambda && p.mu == q.mu && p.b1 == q.b1 && p.b2 == q.b2 && p.eps == q.eps;
}

// n_steps train steps, step s on the batch (xs[s], ts[s]): launched one after the other, or
// captured into one graph and replayed
static int train_steps(tdh_net *net, tdh_opt *opt, int loss_kind, int batch, int n_steps, const float *const *xs,
                       const float *const *ts, int do_update) {
  const float *x = xs[0], *t = ts[0];
  // The filters in the stride-1 kernels' layout: packed here when the weights came from
  // outside (creation, tdh_net_set_param, a pointer handed out), by the optimizer kernel after
  // that.
  if ((net->flags & TDH_NET_GRAPH) && !net->packs_valid) {
    for (tdh_net::Layer &L : net->layers) {
      if (!L.wp_fwd) continue;
      TDH_TRY(conv_pack_filters(&L.spec.conv, 0, L.w, L.tbl_dev, L.wp_fwd));
      TDH_TRY(conv_pack_filters(&L.spec.conv, 1, L.w, L.tbl_dev, L.wp_dx));
    }
    net->packs_valid = true;
  }
  // per-kernel timing needs the launches themselves, not a replay
  if (!(net->flags & TDH_NET_GRAPH) || profiling_active()) {
    // (the timing pass of a branching step keeps every layer's scratch piece until the optimizer
    // has read the split sums: the buffer must not grow, and so move, on the way)
    for (int s = 0; s < n_steps; ++s) {
      if (net->flags & TDH_NET_GRAPH) TDH_TRY(ws_begin(net->scratch));
      TDH_TRY(enqueue_step(net, opt, loss_kind, batch, xs[s], ts[s], do_update, nullptr, nullptr));
    }
    return TDH_OK;
  }

  tdh_net::GraphKey key;
  key.batch = batch; key.loss = loss_kind; key.do_update = do_update;
  key.n_steps = n_steps;
  for (int s = 0; s < n_steps; ++s) { key.x[s] = xs[s]; key.t[s] = ts[s]; }
  key.test_phase = net->test_phase;
  // (only steps that advance the powers take turns between the two buffers)
  const bool powers_move = opt && do_update && (opt->kind == TDH_OPT_ADAM || opt->kind == TDH_OPT_ADAMAX);
  key.powers_at = powers_move ? net->powers_at : 0;
  if (opt) {
    key.hyper      = *opt;
    key.hyper.b1_t = key.hyper.b2_t = 0.0f;
  }
  TDH_TRY(ws_begin(net->scratch));  // may move the scratch buffer if another op outgrew it
  key.scratch = ctx().workspace;
  tdh_net::GraphSlot *slot = nullptr;
  for (auto &g : net->graphs)
    if (g.exec && same_key(key, g.key)) slot = &g;
  if (!slot) {
    for (auto &g : net->graphs)  // an empty slot, else the least recently used one
      if (!g.exec) {
        slot = &g;
        break;
      }
    if (!slot) {
      slot = &net->graphs[0];
      for (auto &g : net->graphs)
        if (g.last_use < slot->last_use) slot = &g;
    }
    if (slot->exec) {
      TDH_HIP(hipGraphExecDestroy(slot->exec));
      slot->exec = nullptr;
    }
    Context &c  = ctx();
    c.ws_locked = true;  // nothing may allocate while the stream is capturing
    hipGraph_t graph = nullptr;
    hipError_t e = hipStreamBeginCapture(c.stream, hipStreamCaptureModeThreadLocal);
    int rc = TDH_OK;
    if (e == hipSuccess) {
      tdh_opt capture_opt;
      if (opt) capture_opt = *opt;
      for (int s = 0; s < n_steps && rc == TDH_OK; ++s) {
        // (steps that advance the powers take turns between the two buffers inside the graph as well)
        const int at = powers_move ? (key.powers_at + s) & 1 : key.powers_at;
        rc = enqueue_step(net, opt ? &capture_opt : nullptr, loss_kind, batch, xs[s], ts[s], do_update,
                          net->dev_powers + 4 * at, net->dev_powers + 4 * (1 - at),
                          /*forked=*/net_forks(net, batch));
      }
      e = hipStreamEndCapture(c.stream, &graph);
    }
    c.ws_locked = false;
    if (rc != TDH_OK) {
      if (graph) (void)hipGraphDestroy(graph);
      return rc;
    }
    if (e != hipSuccess || !graph)
      return set_error(TDH_ERR_HIP, "tdh_net_train_step: graph capture failed: %s",
                       hipGetErrorString(e));
    e = hipGraphInstantiate(&slot->exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    if (e != hipSuccess) {
      slot->exec = nullptr;
      return set_error(TDH_ERR_HIP, "tdh_net_train_step: graph instantiation failed: %s",
                       hipGetErrorString(e));
    }
    slot->key = key;
    slot->dx_unwritten  = net->dx_unwritten;
    slot->out_unwritten = net->out_unwritten;
    net->mirror_b1_t = net->mirror_b2_t = -1.0f;  // forces the upload below
  }
  // the captured optimizer kernel reads the powers from device memory; bring that copy in
  // line with the caller's optimizer object whenever the two have drifted apart
  if (opt && do_update && (opt->b1_t != net->mirror_b1_t || opt->b2_t != net->mirror_b2_t)) {
    const float h[2] = {opt->b1_t, opt->b2_t};
    TDH_TRY(tdh_memcpy_h2d(net->dev_powers + 4 * key.powers_at, h, sizeof(h)));
  }
  slot->last_use = ++net->graph_clock;
  TDH_HIP(hipGraphLaunch(slot->exec, ctx().stream));
  net->dx_unwritten  = slot->dx_unwritten;
  net->out_unwritten = slot->out_unwritten;
  if (opt && do_update) {
    // advance the host object exactly as the eager path does
    for (int j = 0; j < net->opt_tensors * n_steps; ++j) {
      if (opt->kind == TDH_OPT_ADAM) {
        opt->b1_t *= opt->b1;
        opt->b2_t *= opt->b2;
      } else if (opt->kind == TDH_OPT_ADAMAX) {
        opt->b1_t *= opt->b1;
      }
    }
    net->mirror_b1_t = opt->b1_t;
    net->mirror_b2_t = opt->b2_t;
    if (powers_move) net->powers_at = (net->powers_at + n_steps) & 1;  // where the last step left them
  }
  return TDH_OK;
}

int tdh_net_train_step(tdh_net *net, tdh_opt *opt, int loss_kind, int batch, const float *x,
                       const float *t, int do_update) {
  TDH_REQUIRE_INIT();
  TDH_CHECK_ARG(net && x && t && batch > 0 && batch <= net->max_batch,
                "tdh_net_train_step: bad argument");
  TDH_CHECK_ARG(!do_update || opt, "tdh_net_train_step: update requested without an optimizer");
  return train_steps(net, opt, loss_kind, batch, 1, &x, &t, do_update);
}

int tdh_net_train_steps(tdh_net *net, tdh_opt *opt, int loss_kind, int batch, int n_steps,
                        const float *const *x, const float *const *t) {
  TDH_REQUIRE_INIT();
  TDH_CHECK_ARG(net && opt && x && t && batch > 0 && batch <= net->max_batch && n_steps >= 1 &&
                n_steps <= tdh_net::kMaxSteps, "tdh_net_train_steps: bad argument (1 to %d steps a call)",
                tdh_net::kMaxSteps);
  for (int s = 0; s < n_steps; ++s) TDH_CHECK_ARG(x[s] && t[s], "tdh_net_train_steps: null batch %d", s);
  // a dropout layer's masks are handed over once per step, between the steps
  for (const tdh_net::Layer &L : net->layers)
    TDH_CHECK_ARG(L.spec.kind != TDH_L_DROPOUT || net->test_phase,
                  "tdh_net_train_steps: a net with a dropout layer trains one step a call");
  return train_steps(net, opt, loss_kind, batch, n_steps, x, t, 1);
}

}  // extern "C"
