// conv_s1.hip — host side of the stride-1 convolution (forward and dX) on the LDS-halo MFMA
// kernel of conv_s1_inst.hip: tile choice, filter repacking, split-K reduction.
#include "conv_s1.h"

namespace tdh {

namespace {

// out = part[0] + part[1] + ... (in this order) (+ bias[m]) (* act'(y)); four elements per
// thread when a channel plane is a multiple of four
template <int VEC>
__global__ void __launch_bounds__(256)
s1_split_reduce_kernel(const SplitSum sum, float *__restrict__ act_out, const int act_kind) {
  const size_t i = (static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x) * VEC;
  if (i >= sum.stride) return;
  float v[VEC];
  split_sum_values<VEC>(sum, i, v);
  if (act_out) {
#pragma unroll
    for (int e = 0; e < VEC; ++e) act_out[i + e] = act_apply(act_kind, v[e]);
  }
}

int launch_split_reduce(const SplitSum &sum, int plane, float *act_out, int act_kind) {
  const size_t total = sum.stride;
  ProfScope prof("conv_s1_split_reduce", 4.0 * total * (sum.splits + 1 + (sum.ag.kind != TDH_ACT_NONE)),
                 WORK_BYTE);
  if (plane % 4 == 0)
    TDH_LAUNCH((s1_split_reduce_kernel<4>), dim3(static_cast<unsigned>(ceil_div_sz(total / 4, 256))), dim3(256), 0,
               ctx().stream, sum, act_out, act_kind);
  else
    TDH_LAUNCH((s1_split_reduce_kernel<1>), dim3(static_cast<unsigned>(ceil_div_sz(total, 256))), dim3(256), 0,
               ctx().stream, sum, act_out, act_kind);
  TDH_LAUNCH_CHECK();
  return TDH_OK;
}

// wp[t][kc][m]: forward (flip = 0): kc = ci, m = co, t as is; dX (flip = 1): kc = co, m = ci,
// tap reversed. An optional connection table zeroes unconnected (ci, co) pairs.
__global__ void __launch_bounds__(256)
repack_weights_kernel(const float *__restrict__ w, const uint8_t *__restrict__ tbl,
                      float *__restrict__ wp, const int C, const int Kc, const int rs,
                      const int flip) {
  const int e = blockIdx.x * 256 + threadIdx.x;
  if (e >= C * Kc * rs) return;
  // e indexes the OIHW source: ((co*C + ci)*rs + t)
  const int t = e % rs, pair = e / rs;
  const int co = pair / C, ci = pair - co * C;
  float v = w[e];
  if (tbl && !tbl[ci * Kc + co]) v = 0.0f;
  if (!flip)
    wp[(static_cast<size_t>(t) * C + ci) * Kc + co] = v;
  else
    wp[(static_cast<size_t>(rs - 1 - t) * Kc + co) * C + ci] = v;
}

int pow2_ceil(int v) {
  int p = 1;
  while (p < v) p <<= 1;
  return p;
}
int ilog2(int v) {
  int l = 0;
  while ((1 << l) < v) ++l;
  return l;
}

// Splits the reduction channels over grid.z when the tiles alone leave most of the chip idle.
void choose_split(S1Plan &p, int rs, long blocks) {
  const int kch     = s1_kch(rs, p.tm, p.tn);
  const int nchunks = ceil_div(p.args.KC, kch);
  int splits = 1;
  if (blocks < 384 && nchunks >= 4) {
    splits = static_cast<int>(std::min<long>(8, (512 + blocks - 1) / blocks));
    splits = std::min(splits, nchunks / 2);
    // still under half the chip: one chunk per workgroup
    if (blocks * splits <= 128) splits = static_cast<int>(std::min<long>(nchunks, 256 / blocks));
  } else if (blocks <= 128 && nchunks >= 2) {
    splits = 2;  // half the chip would idle: one chunk per workgroup is still the better deal
  }
  const int per      = ceil_div(nchunks, splits) * kch;
  p.splits           = ceil_div(p.args.KC, per);
  p.args.kc_split    = p.splits > 1 ? per : p.args.KC;
  p.args.part        = nullptr;
  p.args.part_stride = static_cast<size_t>(p.args.batch) * p.args.MC * p.args.OH * p.args.OW;
  p.grid.z           = p.splits;
}

// Shape-only choice of the tile geometry; ok = false sends the caller to the generic GEMM.
// Candidates run from the largest workgroup tile to the smallest; the first one that yields
// at least 256 workgroups wins, else the one with the most workgroups, and shapes that cannot
// even fill a quarter of the chip are left to the split-K GEMM.
S1Plan make_plan(int R, int S, int batch, int KC, int MC, int IH, int IW, int OH, int OW, int ph,
                 int pw) {
  S1Plan best;
  best.ok = false;
  if (!((R == 3 && S == 3) || (R == 5 && S == 5))) return best;
  if (MC < 16 || KC < 8 || OW < 4 || OH < 1 || pw > 4) return best;
  // offsets inside the input are 32-bit
  if (static_cast<long>(batch) * KC * IH * IW >= (1L << 31)) return best;
  static const int cand_wide[3][2]   = {{2, 2}, {2, 1}, {1, 1}};  // MC > 32
  static const int cand_narrow[3][2] = {{1, 4}, {1, 2}, {1, 1}};  // MC <= 32
  long best_blocks = 0;
  for (int ci = 0; ci < 3; ++ci) {
    S1Plan p;
    p.ok = false;
    p.tc = OW >= 48 ? 64 : OW >= 24 ? 32 : OW >= 12 ? 16 : 8;
    p.tm = MC > 32 ? cand_wide[ci][0] : cand_narrow[ci][0];
    p.tn = MC > 32 ? cand_wide[ci][1] : cand_narrow[ci][1];
    const int pix = 128 * p.tn;
    if (pix < p.tc) continue;
    int tr = pix / p.tc;
    if (tr > pow2_ceil(OH)) tr = pow2_ceil(OH);
    const int ti = pix / (tr * p.tc);
    ConvS1Args &a = p.args;
    a.batch = batch; a.KC = KC; a.MC = MC; a.IH = IH; a.IW = IW; a.OH = OH; a.OW = OW;
    a.ph = ph; a.pw = pw; a.pwa = (pw + 3) & ~3;
    a.TR = tr; a.TI = ti; a.log_tr = ilog2(tr); a.log_ti = ilog2(ti);
    a.tiles_x = ceil_div(OW, p.tc);
    a.tiles_y = ceil_div(OH, tr);
    const int nq     = (3 + p.tc + S - 1 + 3) / 4;
    const int planeq = ti * (tr + R - 1) * nq;
    a.div_rows = FastDiv((tr + R - 1) * nq);
    const int kch = s1_kch(R * S, p.tm, p.tn);
    if (ceil_div(planeq, 256 / kch) > s1_niq(R, S, p.tc, p.tm, p.tn)) continue;
    p.lds_bytes = sizeof(float) * kch * (4 * static_cast<size_t>(planeq) + R * S * 32 * p.tm);
    if (p.lds_bytes > 150 * 1024) continue;
    const long tiles  = static_cast<long>(a.tiles_x) * a.tiles_y * ceil_div(batch, ti);
    const long blocks = tiles * ceil_div(MC, 32 * p.tm);
    if (tiles > 2000000000L) continue;
    p.grid = dim3(static_cast<unsigned>(tiles), ceil_div(MC, 32 * p.tm), 1);
    p.ok   = true;
    choose_split(p, R * S, blocks);
    // short reductions have nothing to overlap their loads with inside a workgroup: ask for
    // more, smaller workgroups then
    if (blocks >= (KC * R * S < 256 ? 1024 : 256)) return p;
    if (blocks > best_blocks) {
      best_blocks = blocks;
      best        = p;
    }
  }
  if (best_blocks * (best.ok ? best.splits : 1) < 128) best.ok = false;
  return best;
}

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace

bool conv_s1_applicable(int R, int S, int batch, int KC, int MC, int IH, int IW, int OH, int OW,
                        int ph, int pw) {
  return make_plan(R, S, batch, KC, MC, IH, IW, OH, OW, ph, pw).ok;
}

bool conv_s1_single_pass(int R, int S, int batch, int KC, int MC, int IH, int IW, int OH, int OW,
                         int ph, int pw) {
  const S1Plan p = make_plan(R, S, batch, KC, MC, IH, IW, OH, OW, ph, pw);
  return p.ok && p.splits == 1;
}

// A 32-pixel accumulator block must hold whole 2x2 windows: rows of 8 or 16 pixels (tile rows
// come in powers of two and start at even image rows), even image sizes, and one pass over the
// reduction channels (the partial sums of a split have no maximum yet).
bool conv_s1_fuses_pool(int R, int S, int batch, int KC, int MC, int IH, int IW, int OH, int OW,
                        int ph, int pw) {
  const S1Plan p = make_plan(R, S, batch, KC, MC, IH, IW, OH, OW, ph, pw);
  return p.ok && p.splits == 1 && p.tc <= 16 && p.args.TR >= 2 && OH % 2 == 0 && OW % 2 == 0 &&
         static_cast<long>(MC) * OH * OW < (1L << 31);
}

size_t conv_s1_workspace_bytes(int R, int S, int batch, int C, int Kc, int flip, int IH, int IW,
                               int OH, int OW, int ph, int pw) {
  const int KC = flip ? Kc : C, MC = flip ? C : Kc;
  const S1Plan p = make_plan(R, S, batch, KC, MC, IH, IW, OH, OW, ph, pw);
  if (!p.ok) return 0;
  size_t total = ws_align(sizeof(float) * static_cast<size_t>(R) * S * C * Kc);  // repacked filter
  if (p.splits > 1) total += ws_align(sizeof(float) * p.splits * p.args.part_stride);
  return total;
}

// wp = the filter in the kernel's layout [tap][kc][m] (R*S*C*Kc floats); flip as in conv_s1_run
int conv_s1_repack(int R, int S, int C, int Kc, int flip, const float *w, const uint8_t *tbl_dev,
                   float *wp) {
  ProfScope prof("conv_repack_weights", 8.0 * R * S * C * Kc, WORK_BYTE);
  TDH_LAUNCH(repack_weights_kernel, dim3(ceil_div(R * S * C * Kc, 256)), dim3(256), 0,
                     ctx().stream, w, tbl_dev, wp, C, Kc, R * S, flip);
  TDH_LAUNCH_CHECK();
  return TDH_OK;
}

// Runs out = conv(in, repack(w)) (+ bias) (* act'(y)); the caller has checked applicability
// and reserved conv_s1_workspace_bytes of scratch. flip = 0: forward, 1: dX. prepacked: the
// result of conv_s1_repack for this filter, when the caller already has it (w is not read).
int conv_s1_run(int R, int S, int batch, int C, int Kc, int flip, const float *in, const float *w,
                const uint8_t *tbl_dev, const float *bias, float *out, int IH, int IW, int OH,
                int OW, int ph, int pw, ActGrad ag, const char *tag, const float *prepacked,
                float *act_out, int act_kind, const PoolFuse *pool) {
  const int KC = flip ? Kc : C, MC = flip ? C : Kc;
  S1Plan p = make_plan(R, S, batch, KC, MC, IH, IW, OH, OW, ph, pw);
  if (!p.ok) return set_error(TDH_ERR_INVALID, "conv_s1_run: shape not supported");
  if (pool && (flip || !pool->out || !pool->argmax ||
               (pool->act_out && pool->act_kind != TDH_ACT_RELU) ||
               !conv_s1_fuses_pool(R, S, batch, KC, MC, IH, IW, OH, OW, ph, pw)))
    return set_error(TDH_ERR_INVALID, "conv_s1_run: this shape does not compute the pool layer behind it");
  if (!out && !pool && !(act_out && p.splits == 1))
    return set_error(TDH_ERR_INVALID, "conv_s1_run: no output tensor");
  const void *wp = prepacked;
  if (!prepacked) {
    void *fresh = nullptr;
    TDH_TRY(ws_take(sizeof(float) * static_cast<size_t>(R) * S * C * Kc, &fresh));
    TDH_TRY(conv_s1_repack(R, S, C, Kc, flip, w, tbl_dev, static_cast<float *>(fresh)));
    wp = fresh;
  }
  p.args.in = in; p.args.wp = static_cast<const float *>(wp); p.args.bias = bias;
  p.args.out = out; p.args.ag = ag;
  p.args.act_out = act_out; p.args.act_kind = act_kind;
  p.args.pool_out     = pool ? pool->out : nullptr;
  p.args.pool_argmax  = pool ? pool->argmax : nullptr;
  p.args.pool_act_out = pool ? pool->act_out : nullptr;
  if (p.splits > 1) {
    void *part = nullptr;
    TDH_TRY(ws_take(sizeof(float) * p.splits * p.args.part_stride, &part));
    p.args.part = static_cast<float *>(part);
  }
  {
    ProfScope prof(pool ? "conv_fwd_s1_pool" : tag, MC, batch * OH * OW, KC * R * S);
    const bool vec = IW % 4 == 0 && MC % 4 == 0 && aligned16(in) && aligned16(wp);
    if (vec) TDH_TRY(R == 3 ? s1_launch_3x3_vec(p) : s1_launch_5x5_vec(p));
    else TDH_TRY(R == 3 ? s1_launch_3x3_scalar(p) : s1_launch_5x5_scalar(p));
  }
  if (p.splits > 1) {
    SplitSum sum;
    sum.part = p.args.part; sum.splits = p.splits; sum.stride = p.args.part_stride;
    sum.bias = bias; sum.MC = MC; sum.div_plane = FastDiv(OH * OW); sum.ag = ag; sum.out = out;
    if (ctx().leave_split_sum && !act_out) {
      // the kernel that reads `out` next adds the partials up (and writes `out`)
      left_split_sum()     = sum;
      ctx().split_sum_left = true;
      return TDH_OK;
    }
    TDH_TRY(launch_split_reduce(sum, OH * OW, act_out, act_kind));
  }
  return TDH_OK;
}

SplitSum &left_split_sum() {
  static SplitSum sum;
  return sum;
}

int finish_split_sum() {
  if (!ctx().split_sum_left) return TDH_OK;
  ctx().split_sum_left = false;
  const SplitSum &sum = left_split_sum();
  return launch_split_reduce(sum, static_cast<int>(sum.div_plane.d), nullptr, TDH_ACT_NONE);
}

}  // namespace tdh
