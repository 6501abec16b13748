// fc.hip — fully-connected forward and backward as three fp32 MFMA GEMMs over tiny-dnn's
// [in][out] row-major weight matrix:
//   forward  Y[s][o]  = sum_c X[s][c] * W[c][o] + b[o]        M=batch N=out K=in
//   dX       dX[s][c] = sum_o dY[s][o] * W[c][o]              M=batch N=in  K=out
//   dW       dW[c][o] = sum_s X[s][c] * dY[s][o]              M=in    N=out K=batch
// dW is reduced over the batch inside the GEMM (K spans the samples) instead of being stored
// per sample and merged afterwards (fully_connected_op_internal.h:54-60, node.h:89-103).
#include <cfloat>

#include "gemm_mfma.h"

namespace tdh {

namespace {

// Products of a small network's fully-connected layers (a few million MACs, K <= 512): the
// tiled MFMA kernel pays one exposed memory latency per 16-deep K tile with only a handful of
// workgroups to hide it behind, 7-16 us for microseconds of arithmetic. Here a workgroup
// stages 128-deep panels of both operands with every load in flight at once (40 per thread;
// a panel costs one exposed memory latency, so the fewer the better: 64-deep panels made the
// backward kernels of the CIFAR net's two layers 10.6 us, 128-deep ones 8.6 us),
// and the four waves multiply out of LDS on the vector ALUs: wave w owns rows 4w..4w+3 of a
// 16 x 64 tile, so its A values are wave-uniform LDS broadcasts and its B values one
// conflict-free read per k. k ascends, one FMA per term: the summation order is fixed.
constexpr int SFC_TM = 16, SFC_TN = 64, SFC_KC = 128, SFC_NT = 256;
constexpr int SFC_NA = SFC_TM * SFC_KC / SFC_NT, SFC_NB = SFC_TN * SFC_KC / SFC_NT;

struct SfcSmem {
  __attribute__((aligned(16))) float As[SFC_KC][SFC_TM + 4];
  float Bs[SFC_KC][SFC_TN + 1];
};

// One 16 x 64 tile (bx, by) of C = A * B: acc[i] is row 4*(tid/64) + i, column tid%64 of the
// tile. The next panel's loads are issued before the current panel is multiplied. The last
// panel stays in LDS (rows past K hold zeros).
__device__ __forceinline__ void small_fc_accumulate(const StridedOperand &a, const StridedOperand &b,
                                                    const int M, const int N, const int K,
                                                    const int bx, const int by, SfcSmem &sm,
                                                    float (&acc)[4]) {
  const int tid = threadIdx.x, tn = tid & 63, tmg = tid >> 6;
  const int m0 = by * SFC_TM, n0 = bx * SFC_TN;
  // staging coordinates: consecutive threads walk the operand's contiguous direction
  const bool a_k_fast = a.s_k == 1, b_k_fast = b.s_k == 1;
  acc[0] = acc[1] = acc[2] = acc[3] = 0.0f;
  float ra[SFC_NA], rb[SFC_NB];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int i = 0; i < SFC_NA; ++i) {
      const int e = tid + SFC_NT * i;
      const int m = a_k_fast ? e / SFC_KC : e % SFC_TM, k = a_k_fast ? e % SFC_KC : e / SFC_TM;
      ra[i] = (m0 + m < M && k0 + k < K) ? a.p[(m0 + m) * a.s_mn + (k0 + k) * a.s_k] : 0.0f;
    }
#pragma unroll
    for (int i = 0; i < SFC_NB; ++i) {
      const int e = tid + SFC_NT * i;
      const int n = b_k_fast ? e / SFC_KC : e % SFC_TN, k = b_k_fast ? e % SFC_KC : e / SFC_TN;
      rb[i] = (n0 + n < N && k0 + k < K) ? b.p[(n0 + n) * b.s_mn + (k0 + k) * b.s_k] : 0.0f;
    }
  };
  fetch(0);
  for (int k0 = 0; k0 < K; k0 += SFC_KC) {
    if (k0 > 0) __syncthreads();  // the previous panel has been consumed
#pragma unroll
    for (int i = 0; i < SFC_NA; ++i) {
      const int e = tid + SFC_NT * i;
      sm.As[a_k_fast ? e % SFC_KC : e / SFC_TM][a_k_fast ? e / SFC_KC : e % SFC_TM] = ra[i];
    }
#pragma unroll
    for (int i = 0; i < SFC_NB; ++i) {
      const int e = tid + SFC_NT * i;
      sm.Bs[b_k_fast ? e % SFC_KC : e / SFC_TN][b_k_fast ? e / SFC_KC : e % SFC_TN] = rb[i];
    }
    __syncthreads();
    if (k0 + SFC_KC < K) fetch(k0 + SFC_KC);
    // the rows of the panel past K hold zeros: a short product leaves them out, eight at a time
    const int kend = min(SFC_KC, (K - k0 + 7) & ~7);
#pragma unroll 8
    for (int k = 0; k < kend; ++k) {
      const float4 av = *reinterpret_cast<const float4 *>(&sm.As[k][4 * tmg]);
      const float bv  = sm.Bs[k][tn];
      acc[0] += av.x * bv;
      acc[1] += av.y * bv;
      acc[2] += av.z * bv;
      acc[3] += av.w * bv;
    }
  }
}

// The tile with the epilogue applied.
template <class Epi>
__device__ __forceinline__ void small_fc_tile(const StridedOperand &a, const StridedOperand &b,
                                              const Epi &epi, const int M, const int N, const int K,
                                              const int bx, const int by, SfcSmem &sm) {
  const int tn = threadIdx.x & 63, tmg = threadIdx.x >> 6;
  const int m0 = by * SFC_TM, n0 = bx * SFC_TN;
  // what the epilogue reads from memory (the column's bias, the values a store adds to) is
  // asked for together with the panels: behind the product each would be a trip to memory
  // with nothing to hide it
  const int n = n0 + tn;
  typename Epi::Col c = epi.col(n < N ? n : 0);
  float before[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + 4 * tmg + i;
    before[i]   = (n < N && m < M) ? epi.prior(m, c) : 0.0f;
  }
  float acc[4];
  small_fc_accumulate(a, b, M, N, K, bx, by, sm, acc);
  if (n < N) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = m0 + 4 * tmg + i;
      if (m < M) epi.store(m, c, acc[i], before[i]);
    }
  }
}

template <class Epi>
__global__ void __launch_bounds__(SFC_NT)
small_fc_gemm_kernel(const StridedOperand a, const StridedOperand b, const Epi epi, const int M,
                     const int N, const int K) {
  __shared__ SfcSmem sm;
  small_fc_tile(a, b, epi, M, N, K, blockIdx.x, blockIdx.y, sm);
}

// dX of a fully-connected layer whose input is the output of a 2x2 / stride-2 max-pool (behind
// an activation whose gradient `row.ag` folds in): the value is stored as EpiRowMajor stores
// it, and also routed through the pool: to the input position its argmax record names, zeros
// to the other three positions of the window (maxpool_grad_op_internal,
// maxpool_op_internal.h:42-57, for windows that tile the input).
struct EpiRowMajorPool {
  EpiRowMajor row;
  PoolScatter pool;  // argmax == nullptr: no pool, plain EpiRowMajor
  FastDiv div_ow, div_oh;
  int sample_in;     // C*H*W
  struct Col {
    EpiRowMajor::Col c;
    int base;  // flat input index of the window's top-left corner
  };
  __device__ __forceinline__ Col col(int n) const {
    Col r{row.col(n), 0};
    if (pool.argmax) {
      uint32_t rest, ox, plane, oy;
      div_ow.divmod(static_cast<uint32_t>(n), rest, ox);
      div_oh.divmod(rest, plane, oy);
      r.base = static_cast<int>((plane * 2 * pool.OH + 2 * oy) * pool.W + 2 * ox);
    }
    return r;
  }
  __device__ __forceinline__ float prior(int m, const Col &c) const { return row.prior(m, c.c); }
  __device__ __forceinline__ void store(int m, const Col &c, float v, float before) const {
    const int idx = m * row.ld + c.c.n;
    row.store(m, c.c, v, before);
    if (!pool.argmax) return;
    // the value as stored (the same steps as EpiRowMajor::store)
    v += c.c.bias;
    if (row.ag.kind != TDH_ACT_NONE) v *= act_grad_factor(row.ag.kind, row.ag.y[idx]);
    v += before;
    const int a = pool.argmax[idx];
    float *p    = pool.dx + static_cast<size_t>(m) * sample_in + c.base;
    *reinterpret_cast<float2 *>(p) = make_float2(a == c.base ? v : 0.0f, a == c.base + 1 ? v : 0.0f);
    *reinterpret_cast<float2 *>(p + pool.W) =
      make_float2(a == c.base + pool.W ? v : 0.0f, a == c.base + pool.W + 1 ? v : 0.0f);
  }
};

// The whole backward pass of a small fully-connected layer in one launch: the first nx
// workgroups take the tiles of dX, the next nw those of dW, the rest 32 columns each of the bias
// gradient (rows g, g+8, ... per 32-lane group, group sums added in order, as the stand-alone
// column sum does). The three products only share their inputs, and none of them fills the chip.
struct FcBwdFused {
  StridedOperand xa, xb, wa, wb;
  EpiRowMajorPool xepi;
  EpiRowMajor wepi;
  int xM, xN, xK, x_tiles_n, nx;
  int wM, wN, wK, w_tiles_n, nw;
  const float *dy;
  float *db;
  int batch, out, db_accumulate;
};

__global__ void __launch_bounds__(SFC_NT) fc_bwd_fused_kernel(const FcBwdFused f) {
  __shared__ SfcSmem sm;
  const int b = blockIdx.x;
  if (b < f.nx) {
    small_fc_tile(f.xa, f.xb, f.xepi, f.xM, f.xN, f.xK, b % f.x_tiles_n, b / f.x_tiles_n, sm);
  } else if (b < f.nx + f.nw) {
    const int t = b - f.nx;
    small_fc_tile(f.wa, f.wb, f.wepi, f.wM, f.wN, f.wK, t % f.w_tiles_n, t / f.w_tiles_n, sm);
  } else {
    float(*part)[32] = reinterpret_cast<float(*)[32]>(&sm.Bs[0][0]);
    const int cl = threadIdx.x & 31, g = threadIdx.x >> 5;
    const int c  = (b - f.nx - f.nw) * 32 + cl;
    float s = 0.0f;
    if (c < f.out)
      for (int r = g; r < f.batch; r += 8) s += f.dy[static_cast<size_t>(r) * f.out + c];
    part[g][cl] = s;
    __syncthreads();
    if (g == 0 && c < f.out) {
      float t = part[0][cl];
#pragma unroll
      for (int i = 1; i < 8; ++i) t += part[i][cl];
      f.db[c] = f.db_accumulate ? f.db[c] + t : t;
    }
  }
}

// The last fully-connected layer of a net that ends in softmax and is trained with
// cross_entropy_multiclass (or ends in this layer and is trained with mse: then dz is
// 2/outputs * (y - t) and there is no softmax), from its input to the gradient of its input in
// one launch: every
// step of that chain stays inside a sample row (only the weight and bias gradients add over
// the batch; they are another launch, off the chain the next layer waits for). A workgroup
// takes 16 rows. The product is small_fc_accumulate's, the softmax and the loss gradient are
// softmax_fwd_xent_kernel's butterflies (a row's outputs sit in the lanes of one wave), the
// input gradient is the dX product of fc_bwd with the filters still in LDS: same terms, same
// order, same results as the three launches.
struct FcTail {
  StridedOperand a, b;  // X[s][k], W[k][n]
  const float *bias;    // or null
  float *out, *soft;    // the layer's output and the softmax layer's (null: the loss is mse)
  const float *t;
  float *dz;
  float mse_factor;     // 2 / outputs (mse::df, loss_function.h:28-36)
  EpiRowMajor xepi;     // dX (with the activation gradient of the layer in front folded in)
  int M, N, K;          // batch, out, in
};

__device__ __forceinline__ float sfc_wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}
__device__ __forceinline__ float sfc_wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}

__global__ void __launch_bounds__(SFC_NT) fc_softmax_xent_kernel(const FcTail f) {
  __shared__ SfcSmem sm;
  const int tn = threadIdx.x & 63, tmg = threadIdx.x >> 6;
  const int m0 = blockIdx.x * SFC_TM;
  // Everything the later phases read from memory is asked for now, with the panels: each of
  // these loads would otherwise be a trip to memory of its own in a chain that has nothing to
  // hide it behind. prev[] is the output of the activation in front (for its gradient factor)
  // at this thread's first 64 dX columns.
  const bool col   = tn < f.N;
  const float bias = (col && f.bias) ? f.bias[tn] : 0.0f;
  const int ag     = f.xepi.ag.kind;
  float tv[4], prev[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + 4 * tmg + i;
    tv[i]       = (col && m < f.M) ? f.t[m * f.N + tn] : 0.0f;
    prev[i]     = (ag != TDH_ACT_NONE && tn < f.K && m < f.M) ? f.xepi.ag.y[m * f.K + tn] : 0.0f;
  }
  float acc[4];
  small_fc_accumulate(f.a, f.b, f.M, f.N, f.K, 0, blockIdx.x, sm, acc);
  // every lane takes part in the butterflies; the lanes past the row's end hold neutral values
  float dzv[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m     = m0 + 4 * tmg + i;
    const bool live = col && m < f.M;
    const int idx   = m * f.N + tn;
    const float v   = (acc[i] + bias) + 0.0f;
    if (!f.soft) {  // mse on the layer's own output (the same for every lane)
      dzv[i] = live ? f.mse_factor * (v - tv[i]) : 0.0f;
      if (live) {
        f.out[idx] = v;
        f.dz[idx]  = dzv[i];
      }
      continue;
    }
    const float mx  = sfc_wave_max(col ? fmaxf(-FLT_MAX, v) : -FLT_MAX);
    const float e   = col ? expf(v - mx) : 0.0f;
    const float se  = sfc_wave_sum(e);
    const float st  = sfc_wave_sum(tv[i]);
    const float y   = e / se;
    dzv[i]          = live ? fmaf(y, st, -tv[i]) : 0.0f;
    if (live) {
      f.out[idx]  = v;
      f.soft[idx] = y;
      f.dz[idx]   = dzv[i];
    }
  }
  // dX[m][c] = sum_o dz[m][o] * W[c][o]: the tile of dz takes the place of the panel of X
  __syncthreads();
  float *dzs = &sm.As[0][0];  // [SFC_TM][SFC_TN]
#pragma unroll
  for (int i = 0; i < 4; ++i) dzs[(4 * tmg + i) * SFC_TN + tn] = dzv[i];
  __syncthreads();
  for (int c0 = 0; c0 < f.K; c0 += 64) {
    const int c = c0 + tn;
    if (c0 > 0) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int m = m0 + 4 * tmg + i;
        prev[i]     = (ag != TDH_ACT_NONE && c < f.K && m < f.M) ? f.xepi.ag.y[m * f.K + c] : 0.0f;
      }
    }
    float g[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int o = 0; o < f.N; ++o) {
      const float bv = sm.Bs[c][o];
#pragma unroll
      for (int i = 0; i < 4; ++i) g[i] += dzs[(4 * tmg + i) * SFC_TN + o] * bv;
    }
    if (c < f.K) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int m = m0 + 4 * tmg + i;
        if (m < f.M) {
          // the steps of EpiRowMajor::store without a bias, not accumulating
          float v = g[i] + 0.0f;
          if (ag != TDH_ACT_NONE) v *= act_grad_factor(ag, prev[i]);
          f.xepi.out[m * f.K + c] = v + 0.0f;
        }
      }
    }
  }
}

bool small_fc_applies(int M, int N, int K) {
  return K <= 4 * SFC_KC && static_cast<long>(M) * N <= (1L << 18) &&
         static_cast<long>(M) * N * K <= (1L << 24);
}

template <class Epi>
int launch_small_fc(const StridedOperand &a, const StridedOperand &b, const Epi &epi, int M, int N,
                    int K, const char *tag) {
  ProfScope prof(tag, M, N, K);
  TDH_LAUNCH((small_fc_gemm_kernel<Epi>), dim3(ceil_div(N, SFC_TN), ceil_div(M, SFC_TM)),
                     dim3(SFC_NT), 0, ctx().stream, a, b, epi, M, N, K);
  TDH_LAUNCH_CHECK();
  return TDH_OK;
}

}  // namespace

// dX, dW and db of this layer leave one launch (when all three are asked for)
bool fc_bwd_fuses(int in, int out, int batch) {
  return small_fc_applies(batch, in, out) && small_fc_applies(in, out, batch);
}
bool fc_bwd_scatters_pool(int in, int out, int batch) { return fc_bwd_fuses(in, out, batch); }

// forward, softmax, cross-entropy gradient and dX of this layer can leave one launch
bool fc_softmax_xent_applies(int in, int out, int batch) {
  return in <= SFC_KC && out <= SFC_TN && small_fc_applies(batch, out, in) && small_fc_applies(batch, in, out);
}

// soft == nullptr: the net ends in this layer and the loss is mse
int fc_softmax_xent(int in, int out, int has_bias, int batch, const float *x, const float *w,
                    const float *b, float *y, float *soft, const float *t, float *dz, float *dx,
                    ActGrad dx_act) {
  if (!fc_softmax_xent_applies(in, out, batch))
    return set_error(TDH_ERR_INVALID, "fc_softmax_xent: layer too large for the one-launch kernel");
  FcTail f;
  f.a    = StridedOperand{x, in, 1, batch};
  f.b    = StridedOperand{w, 1, out, out};
  f.bias = has_bias ? b : nullptr;
  f.out = y; f.soft = soft; f.t = t; f.dz = dz;
  f.mse_factor = 2.0f / static_cast<float>(out);
  f.xepi = EpiRowMajor{dx, in, nullptr, dx_act, 0};
  f.M = batch; f.N = out; f.K = in;
  ProfScope prof(soft ? "fc_fwd_softmax_xent_dx" : "fc_fwd_mse_dx", 4.0 * batch * in * out, WORK_FLOP);
  TDH_LAUNCH(fc_softmax_xent_kernel, dim3(ceil_div(batch, SFC_TM)), dim3(SFC_NT), 0, ctx().stream, f);
  TDH_LAUNCH_CHECK();
  return TDH_OK;
}

size_t fc_workspace_bytes(int in, int out, int batch) {
  return gemm_workspace_bytes(batch, out, in, true) + gemm_workspace_bytes(batch, in, out, true) +
         gemm_workspace_bytes(in, out, batch, true);
}

int fc_fwd(int in, int out, int has_bias, int batch, const float *x, const float *w,
           const float *b, float *y, float *act_out, int act_kind) {
  StridedOperand A{x, in, 1, batch};   // X[s][k], k contiguous
  StridedOperand B{w, 1, out, out};    // W[k][n], n contiguous
  if (act_out) {  // the pointwise activation layer that follows leaves the same kernel
    EpiRowMajorAct epi{y, out, has_bias ? b : nullptr, act_out, act_kind};
    if (small_fc_applies(batch, out, in)) return launch_small_fc(A, B, epi, batch, out, in, "fc_fwd_small");
    return launch_gemm<true, false, false, true>(A, B, epi, batch, out, in, true, "fc_fwd_gemm",
                                                "fc_fwd_splitk_reduce");
  }
  EpiRowMajor epi{y, out, has_bias ? b : nullptr, ActGrad(), 0};
  if (small_fc_applies(batch, out, in)) return launch_small_fc(A, B, epi, batch, out, in, "fc_fwd_small");
  return launch_gemm<true, false, false, true>(A, B, epi, batch, out, in, true, "fc_fwd_gemm",
                                              "fc_fwd_splitk_reduce");
}

int fc_bwd(int in, int out, int has_bias, int batch, const float *x, const float *w,
           const float *dy, float *dx, float *dw, float *db, int accumulate, ActGrad dx_act,
           const PoolScatter *pool) {
  const bool bias_grad = db && has_bias;
  if (pool && !(dx && dw && fc_bwd_fuses(in, out, batch) && pool->OH * pool->OW > 0 && in % (pool->OH * pool->OW) == 0))
    return set_error(TDH_ERR_INVALID, "fc_bwd: the pool scatter needs the one-launch kernel");
  if (dw && (dx || bias_grad) && fc_bwd_fuses(in, out, batch)) {
    FcBwdFused f;
    f.xa = StridedOperand{dy, out, 1, batch};
    f.xb = StridedOperand{w, out, 1, in};
    f.xepi.row = EpiRowMajor{dx, in, nullptr, dx_act, 0};
    if (pool) {
      f.xepi.pool      = *pool;
      f.xepi.div_ow    = FastDiv(pool->OW);
      f.xepi.div_oh    = FastDiv(pool->OH);
      f.xepi.sample_in = 4 * in;
    }
    f.xM = batch; f.xN = in; f.xK = out;
    f.x_tiles_n = ceil_div(in, SFC_TN);
    f.nx = dx ? f.x_tiles_n * ceil_div(batch, SFC_TM) : 0;  // no dX: its workgroups are left out
    f.wa = StridedOperand{x, 1, in, in};
    f.wb = StridedOperand{dy, 1, out, out};
    f.wepi = EpiRowMajor{dw, out, nullptr, ActGrad(), accumulate};
    f.wM = in; f.wN = out; f.wK = batch;
    f.w_tiles_n = ceil_div(out, SFC_TN);
    f.nw = f.w_tiles_n * ceil_div(in, SFC_TM);
    const bool bias = bias_grad;
    f.dy = dy; f.db = db; f.batch = batch; f.out = out; f.db_accumulate = accumulate;
    ProfScope prof(pool ? "fc_bwd_small_pool" : dx ? "fc_bwd_small" : "fc_dw_db_small", (dx ? 4.0 : 2.0) * batch * in * out, WORK_FLOP);
    TDH_LAUNCH(fc_bwd_fused_kernel, dim3(f.nx + f.nw + (bias ? ceil_div(out, 32) : 0)),
                       dim3(SFC_NT), 0, ctx().stream, f);
    TDH_LAUNCH_CHECK();
    return TDH_OK;
  }
  if (dx) {
    StridedOperand A{dy, out, 1, batch};  // dY[s][k]
    StridedOperand B{w, out, 1, in};      // W[n][k], k contiguous
    EpiRowMajor epi{dx, in, nullptr, dx_act, 0};
    if (small_fc_applies(batch, in, out))
      TDH_TRY(launch_small_fc(A, B, epi, batch, in, out, "fc_dx_small"));
    else
      TDH_TRY((launch_gemm<true, true, false, false>(A, B, epi, batch, in, out, true, "fc_dx_gemm",
                                                 "fc_dx_splitk_reduce")));
  }
  if (dw) {
    StridedOperand A{x, 1, in, in};      // X[k][m], m contiguous
    StridedOperand B{dy, 1, out, out};   // dY[k][n], n contiguous
    EpiRowMajor epi{dw, out, nullptr, ActGrad(), accumulate};
    if (small_fc_applies(in, out, batch))
      TDH_TRY(launch_small_fc(A, B, epi, in, out, batch, "fc_dw_small"));
    else
      TDH_TRY((launch_gemm<false, false, true, true>(A, B, epi, in, out, batch, true, "fc_dw_gemm",
                                                   "fc_dw_splitk_reduce")));
  }
  if (db && has_bias) TDH_TRY(launch_colsum(dy, batch, out, db, accumulate));
  return TDH_OK;
}

}  // namespace tdh
