// fc.hip — fully-connected forward and backward as three fp32 MFMA GEMMs over tiny-dnn's
// [in][out] row-major weight matrix:
//   forward  Y[s][o]  = sum_c X[s][c] * W[c][o] + b[o]        M=batch N=out K=in
//   dX       dX[s][c] = sum_o dY[s][o] * W[c][o]              M=batch N=in  K=out
//   dW       dW[c][o] = sum_s X[s][c] * dY[s][o]              M=in    N=out K=batch
// dW is reduced over the batch inside the GEMM (K spans the samples) instead of being stored
// per sample and merged afterwards (fully_connected_op_internal.h:54-60, node.h:89-103).
#include <cfloat>
#include <cstdlib>
#include <type_traits>

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
  int batch, out, db_accumulate, ndb;
  // the weight and bias gradients of another small layer of the same batch, whose workgroups
  // follow (n2 == 0: none)
  StridedOperand w2a, w2b;
  EpiRowMajor w2epi;
  int w2M, w2N, w2K, w2_tiles_n, nw2;
  const float *dy2;
  float *db2;
  int out2;
};

// 32 columns (block cb) of the column sums of dy[batch][out]
__device__ __forceinline__ void fc_bias_grad_block(const float *dy, float *db, int batch, int out, int accumulate,
                                                   int cb, SfcSmem &sm) {
  float(*part)[32] = reinterpret_cast<float(*)[32]>(&sm.Bs[0][0]);
  const int cl = threadIdx.x & 31, g = threadIdx.x >> 5;
  const int c  = cb * 32 + cl;
  float s = 0.0f;
  if (c < out)
    for (int r = g; r < batch; r += 8) s += dy[static_cast<size_t>(r) * out + c];
  part[g][cl] = s;
  __syncthreads();
  if (g == 0 && c < out) {
    float t = part[0][cl];
#pragma unroll
    for (int i = 1; i < 8; ++i) t += part[i][cl];
    db[c] = accumulate ? db[c] + t : t;
  }
}

__global__ void __launch_bounds__(SFC_NT) fc_bwd_fused_kernel(const FcBwdFused f) {
  __shared__ SfcSmem sm;
  int b = blockIdx.x;
  if (b < f.nx) {
    small_fc_tile(f.xa, f.xb, f.xepi, f.xM, f.xN, f.xK, b % f.x_tiles_n, b / f.x_tiles_n, sm);
    return;
  }
  b -= f.nx;
  if (b < f.nw) {
    small_fc_tile(f.wa, f.wb, f.wepi, f.wM, f.wN, f.wK, b % f.w_tiles_n, b / f.w_tiles_n, sm);
    return;
  }
  b -= f.nw;
  if (b < f.ndb) {
    fc_bias_grad_block(f.dy, f.db, f.batch, f.out, f.db_accumulate, b, sm);
    return;
  }
  b -= f.ndb;
  if (b < f.nw2) {
    small_fc_tile(f.w2a, f.w2b, f.w2epi, f.w2M, f.w2N, f.w2K, b % f.w2_tiles_n, b / f.w2_tiles_n, sm);
    return;
  }
  fc_bias_grad_block(f.dy2, f.db2, f.batch, f.out2, f.db_accumulate, b - f.nw2, sm);
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

// The closing classifier of a net, two fully-connected layers deep, in one launch:
//
//   fc A (K1 -> H) -> pointwise activation -> fc B (H -> O) [-> softmax] -> loss gradient
//     -> dX of fc B with the activation's gradient applied (= the gradient of fc A's output)
//
// Everything on that way stays inside a sample row. As separate kernels the chain is three
// launches of 4-10 us each with well under a microsecond of arithmetic in each: what they take is
// launch gaps, start-up, trips to memory one after the other, and instruction fetch: these
// kernels run once a step on a few compute units whose instruction caches hold other kernels'
// code by then, and cold straight-line code was measured to run at about a microsecond a
// kilobyte. So the kernel is written for few instructions and few taken branches: guards are
// clamped addresses and selects, per-kind arithmetic is folded into coefficients.
// (The gradients that add over the batch, and dX of fc A with its 2 K1 H flop a row, stay
// launches of their own: dX in this kernel had a 16-row block's share run on one compute
// unit, 11 us, as long as fc_bwd's launch that also computes dW and db beside it.)
//
// All products run on v_mfma_f32_16x16x4_f32 with both operands read in the fragment layout
// straight from memory (or from a 16-row tile in LDS), four consecutive floats a lane:
// lane (r = lane % 16, q = lane / 16) holds, of a 16-deep slice of the reduction, the four
// indices 4 q .. 4 q + 3, and the instruction that consumes component `comp` adds the terms
// k = 4 q + comp over q. Where the operand's four floats run along the output columns instead
// (fc A's filters, [k][h]), component cc feeds a product of its own, whose 16 column slots stand
// for columns 4 r + cc.
//
// Workgroup (split s, row block b), eight waves: wave w multiplies 16 rows by the 16-deep
// slice 128 s + 16 w of fc A, the eight partial tiles are added through LDS, stored, and the
// workgroup draws a ticket of row block b. The workgroup that draws the last one goes on alone,
// the others are done (nobody waits for anybody): it adds the splits in order, applies bias and
// activation, multiplies by fc B, applies softmax and loss gradient as fc_softmax_xent_kernel
// does, and takes the gradient back through fc B and the activation.
struct FcTail2 {
  const float *x, *w1, *bias1;      // X[s][k], W_A[k][h]
  const float *w2, *bias2;          // W_B[h][o]
  float *out1, *act1;               // fc A's output and the activation layer's
  int act1_kind;
  float *out2, *soft;               // fc B's output and the softmax layer's (null: the loss is mse)
  const float *t;
  float *dz;                        // loss gradient with respect to fc B's output
  float *dh;                        // gradient with respect to fc A's output (activation gradient applied)
  float mse_factor;
  float *partials;                  // [row block][split][16][64]
  unsigned int *tickets;            // [row block], zero between launches
  int M, K1, H, O, splits;
};

typedef float tail_f4 __attribute__((ext_vector_type(4)));
constexpr int TL_NT = 512, TL_WAVES = TL_NT / 64, TL_TM = 16, TL_KC = 16 * TL_WAVES, TL_LD = 68;

struct TailSmem {
  __attribute__((aligned(16))) float part[TL_WAVES][TL_TM][TL_LD];  // fc A: a partial tile a wave
  __attribute__((aligned(16))) float hs[TL_TM][TL_LD];              // act(fc A)
  __attribute__((aligned(16))) float zs[TL_TM][TL_LD];              // fc B
  __attribute__((aligned(16))) float dzs[TL_TM][TL_LD];             // loss gradient
  __attribute__((aligned(16))) float w2[64][TL_LD];                 // fc B's filters, zeros past H x O
};

// These kernels run once a step on a few compute units with cold instruction caches: what they
// cost is the instructions a wave executes and the branches it takes. Guards are therefore
// clamped addresses and selects, not branches around loads.
__device__ __forceinline__ float4 tail_ld4(const float *p) { return *reinterpret_cast<const float4 *>(p); }
__device__ __forceinline__ float4 tail_keep(const float4 &v, bool ok) {
  return make_float4(ok ? v.x : 0.0f, ok ? v.y : 0.0f, ok ? v.z : 0.0f, ok ? v.w : 0.0f);
}
// act_grad_factor for the pointwise activations (and none) as arithmetic on coefficients that
// are computed once: a select on the kind, which is uniform, becomes a branch tree per value.
// factor = yp * (yp * c2 + c1) + c0 + (y > 0 ? c3 : 0), yp = min(y, cap): the same operations and
// roundings as 1 - y * y (tanh), y * (1 - y) (sigmoid), y > 0 ? 1 : 0 (relu, cap = 0 keeps the
// polynomial at zero), 1 (none).
struct TailGrad {
  float c2, c1, c0, c3, cap;
};
__device__ __forceinline__ TailGrad tail_grad_coef(int kind) {
  TailGrad g{0.0f, 0.0f, 1.0f, 0.0f, FLT_MAX};
  if (kind == TDH_ACT_TANH) g = TailGrad{-1.0f, 0.0f, 1.0f, 0.0f, FLT_MAX};
  if (kind == TDH_ACT_SIGMOID) g = TailGrad{-1.0f, 1.0f, 0.0f, 0.0f, FLT_MAX};
  if (kind == TDH_ACT_RELU) g = TailGrad{0.0f, 0.0f, 0.0f, 1.0f, 0.0f};
  return g;
}
__device__ __forceinline__ float tail_grad_factor(const TailGrad &g, float y) {
  const float yp = fminf(y, g.cap);
  return fmaf(yp, fmaf(yp, g.c2, g.c1), g.c0) + (y > 0.0f ? g.c3 : 0.0f);
}
// all-reduce over each group of 16 lanes on the data-parallel-primitive path (no LDS round trips):
// neighbours, pairs, mirrored halves of 8, mirrored 16
template <bool MAX, int CTRL>
__device__ __forceinline__ float tail_dpp_step(float v) {
  const float o = __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), CTRL, 0xf, 0xf, true));
  return MAX ? fmaxf(v, o) : v + o;
}
template <bool MAX>
__device__ __forceinline__ float tail_reduce16(float v) {
  v = tail_dpp_step<MAX, 0xb1>(v);   // quad_perm [1, 0, 3, 2]
  v = tail_dpp_step<MAX, 0x4e>(v);   // quad_perm [2, 3, 0, 1]
  v = tail_dpp_step<MAX, 0x141>(v);  // row_half_mirror
  v = tail_dpp_step<MAX, 0x140>(v);  // row_mirror
  return v;
}
// ... and over the wave when the row is wider than 16 columns
template <bool MAX>
__device__ __forceinline__ float tail_reduce(float v, bool wide) {
  v = tail_reduce16<MAX>(v);
  if (wide) {
    float o = __shfl_xor(v, 16, 64);
    v = MAX ? fmaxf(v, o) : v + o;
    o = __shfl_xor(v, 32, 64);
    v = MAX ? fmaxf(v, o) : v + o;
  }
  return v;
}

__global__ void __launch_bounds__(TL_NT) fc_two_layer_tail_kernel(const FcTail2 f) {
  __shared__ TailSmem sm;
  __shared__ unsigned int drawn;
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int r = lane & 15, q = lane >> 4;
  const int sp = blockIdx.x, rb = blockIdx.y;
  const int m0 = rb * TL_TM;
  // ---- this wave's slice of fc A: rows m0 .. m0 + 15, k = kb .. kb + 3 a lane, all columns.
  //      Rows past the batch and columns past H hold finite values nobody uses.
  {
    const int kb = sp * TL_KC + 16 * w + 4 * q;
    const int mr = min(m0 + r, f.M - 1), kc = min(kb, f.K1 - 4), hc = 4 * r < f.H ? 4 * r : 0;
    const float4 a = tail_keep(tail_ld4(f.x + static_cast<size_t>(mr) * f.K1 + kc), kb < f.K1);
    const float *wrow = f.w1 + static_cast<size_t>(kc) * f.H + hc;
    float4 b[4];
#pragma unroll
    for (int comp = 0; comp < 4; ++comp) b[comp] = tail_ld4(wrow + comp * f.H);
    tail_f4 acc[4] = {{0.0f, 0.0f, 0.0f, 0.0f}, {0.0f, 0.0f, 0.0f, 0.0f}, {0.0f, 0.0f, 0.0f, 0.0f}, {0.0f, 0.0f, 0.0f, 0.0f}};
    const float av[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
    for (int comp = 0; comp < 4; ++comp) {
      acc[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[comp], b[comp].x, acc[0], 0, 0, 0);
      acc[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[comp], b[comp].y, acc[1], 0, 0, 0);
      acc[2] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[comp], b[comp].z, acc[2], 0, 0, 0);
      acc[3] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[comp], b[comp].w, acc[3], 0, 0, 0);
    }
    // acc[cc][i]: row 4 q + i, column 4 r + cc
#pragma unroll
    for (int i = 0; i < 4; ++i)
      *reinterpret_cast<float4 *>(&sm.part[w][4 * q + i][4 * r]) = make_float4(acc[0][i], acc[1][i], acc[2][i], acc[3][i]);
  }
  __syncthreads();
  // every thread owns two consecutive columns of a row from here to the activation
  const int orow = tid >> 5, ocol = 2 * (tid & 31);
  float2 sum = make_float2(0.0f, 0.0f);
#pragma unroll
  for (int v = 0; v < TL_WAVES; ++v) {
    const float2 p = *reinterpret_cast<const float2 *>(&sm.part[v][orow][ocol]);
    sum.x += p.x; sum.y += p.y;
  }
  if (f.splits > 1) {
    float2 *mine = reinterpret_cast<float2 *>(f.partials + (static_cast<size_t>(rb) * f.splits + sp) * (TL_TM * 64));
    mine[tid] = sum;
    // Every wave waits until its stores have reached the L2 cache (the vector L1 writes through);
    // behind the barrier one thread draws the ticket. Its release writes this L2's dirty lines
    // back for the whole workgroup, its acquire drops what this L2 and this compute unit's L1
    // hold of other L2s' lines: one device-wide fence a workgroup, not one a wave.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0) drawn = __hip_atomic_fetch_add(&f.tickets[rb], 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (drawn != static_cast<unsigned int>(f.splits - 1)) return;
    if (tid == 0) __hip_atomic_store(&f.tickets[rb], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  // ---- asked for now, used later: everything the rest reads from memory that does not depend
  //      on what is computed here, so that the trips to memory overlap
  float w2r[8];  // fc B's filters, on their way to LDS
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int e = tid + TL_NT * i, k = e >> 6, n = e & 63;
    const bool ok = k < f.H && n < f.O;
    const float v = f.w2[ok ? k * f.O + n : 0];
    w2r[i]        = ok ? v : 0.0f;
  }
  float tv[2];  // targets: wave w owns rows 2 w, 2 w + 1 in the softmax, a column a lane
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int m   = m0 + 2 * w + i;
    const bool ok = lane < f.O && m < f.M;
    const float v = f.t[ok ? m * f.O + lane : 0];
    tv[i]         = ok ? v : 0.0f;
  }
  float bias2 = 0.0f;
  if (f.bias2) bias2 = f.bias2[lane < f.O ? lane : 0];
  // ---- the splits in order, bias, activation
  {
    const bool on = ocol < f.H && m0 + orow < f.M;
    float2 bias = make_float2(0.0f, 0.0f);
    if (f.bias1) bias = *reinterpret_cast<const float2 *>(f.bias1 + (ocol < f.H ? ocol : 0));
    if (f.splits > 1) {
      const float2 *all = reinterpret_cast<const float2 *>(f.partials + static_cast<size_t>(rb) * f.splits * (TL_TM * 64));
      sum = make_float2(0.0f, 0.0f);
#pragma unroll 8
      for (int s = 0; s < f.splits; ++s) {
        const float2 p = all[s * TL_NT + tid];
        sum.x += p.x; sum.y += p.y;
      }
    }
    const float2 v = make_float2(sum.x + bias.x, sum.y + bias.y);
    float2 h;
    switch (f.act1_kind) {  // act_apply, one branch for the two
      case TDH_ACT_TANH: h = make_float2(tanhf(v.x), tanhf(v.y)); break;
      case TDH_ACT_RELU: h = make_float2(v.x > 0.0f ? v.x : 0.0f, v.y > 0.0f ? v.y : 0.0f); break;
      case TDH_ACT_SIGMOID: h = make_float2(1.0f / (1.0f + expf(-v.x)), 1.0f / (1.0f + expf(-v.y))); break;
      default: h = v; break;
    }
    if (on) {
      *reinterpret_cast<float2 *>(f.out1 + static_cast<size_t>(m0 + orow) * f.H + ocol) = v;
      *reinterpret_cast<float2 *>(f.act1 + static_cast<size_t>(m0 + orow) * f.H + ocol) = h;
    }
    *reinterpret_cast<float2 *>(&sm.hs[orow][ocol]) = make_float2(on ? h.x : 0.0f, on ? h.y : 0.0f);
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int e = tid + TL_NT * i;
    sm.w2[e >> 6][e & 63] = w2r[i];
  }
  __syncthreads();
  // ---- fc B: wave w the output columns 16 w .. 16 w + 15
  const int nob = (f.O + 15) >> 4;
  if (w < nob) {
    tail_f4 z = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      const float4 a   = *reinterpret_cast<const float4 *>(&sm.hs[r][16 * kk + 4 * q]);
      const float *wk  = &sm.w2[16 * kk + 4 * q][16 * w + r];
      z = __builtin_amdgcn_mfma_f32_16x16x4f32(a.x, wk[0], z, 0, 0, 0);
      z = __builtin_amdgcn_mfma_f32_16x16x4f32(a.y, wk[TL_LD], z, 0, 0, 0);
      z = __builtin_amdgcn_mfma_f32_16x16x4f32(a.z, wk[2 * TL_LD], z, 0, 0, 0);
      z = __builtin_amdgcn_mfma_f32_16x16x4f32(a.w, wk[3 * TL_LD], z, 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) sm.zs[4 * q + i][16 * w + r] = z[i];
  }
  __syncthreads();
  // ---- softmax and the loss gradient (fc_softmax_xent_kernel's steps): a row a wave at a time
  {
    const bool col = lane < f.O, wide = f.O > 16;
    float v[2], dzv[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) v[i] = col ? (sm.zs[2 * w + i][lane] + bias2) + 0.0f : 0.0f;
    if (f.soft) {
      float y[2], st[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const float mx = tail_reduce<true>(col ? fmaxf(-FLT_MAX, v[i]) : -FLT_MAX, wide);
        const float e  = col ? expf(v[i] - mx) : 0.0f;
        const float se = tail_reduce<false>(e, wide);
        st[i]          = tail_reduce<false>(tv[i], wide);
        y[i]           = e / se;
      }
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int m     = m0 + 2 * w + i;
        const bool live = col && m < f.M;
        dzv[i]          = live ? fmaf(y[i], st[i], -tv[i]) : 0.0f;
        if (live) {
          f.out2[m * f.O + lane] = v[i];
          f.soft[m * f.O + lane] = y[i];
          f.dz[m * f.O + lane]   = dzv[i];
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int m     = m0 + 2 * w + i;
        const bool live = col && m < f.M;
        dzv[i]          = live ? f.mse_factor * (v[i] - tv[i]) : 0.0f;
        if (live) {
          f.out2[m * f.O + lane] = v[i];
          f.dz[m * f.O + lane]   = dzv[i];
        }
      }
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) sm.dzs[2 * w + i][lane] = dzv[i];
  }
  __syncthreads();
  // ---- dX of fc B: dh[m][c] = (sum_o dz[m][o] * W_B[c][o]) * act'(h[m][c]); wave w the columns
  //      16 w .. 16 w + 15 of fc A's output (zeros past H: the filters in LDS are zero there)
  if (w < 4) {
    const TailGrad g1 = tail_grad_coef(f.act1_kind);
    tail_f4 g = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int kk = 0; kk < nob; ++kk) {
      const float4 a = *reinterpret_cast<const float4 *>(&sm.dzs[r][16 * kk + 4 * q]);
      const float4 b = *reinterpret_cast<const float4 *>(&sm.w2[16 * w + r][16 * kk + 4 * q]);
      g = __builtin_amdgcn_mfma_f32_16x16x4f32(a.x, b.x, g, 0, 0, 0);
      g = __builtin_amdgcn_mfma_f32_16x16x4f32(a.y, b.y, g, 0, 0, 0);
      g = __builtin_amdgcn_mfma_f32_16x16x4f32(a.z, b.z, g, 0, 0, 0);
      g = __builtin_amdgcn_mfma_f32_16x16x4f32(a.w, b.w, g, 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = 4 * q + i, m = m0 + row, c = 16 * w + r;
      const bool on = c < f.H && m < f.M;
      float v       = g[i] + 0.0f;
      v *= tail_grad_factor(g1, sm.hs[row][c]);
      v = on ? v + 0.0f : 0.0f;
      if (on) f.dh[m * f.H + c] = v;
    }
  }
}

// The backward pass of a small fully-connected layer on the matrix cores, one launch: dX, dW, db
// and, where asked for, dW and db of another small layer of the same batch (the closing layer of
// a classifier, whose dX left with the loss gradient). Same shape of work as
// fc_bwd_fused_kernel (a role per workgroup), but every product runs on
// v_mfma_f32_16x16x4_f32 with its operands read from memory in the fragment layout (see
// fc_two_layer_tail_kernel), so a wave executes a few dozen instructions instead of a 128-step
// loop out of LDS: 10.9 -> about 6 us for the CIFAR net's two layers.
//   dX[m][j]  = sum_c dY[m][c] W[j][c]: a wave a 16 x 16 block, both operands 16 bytes a lane along c
//   dW[k][o]  = sum_m X[m][k] dY[m][o]: a workgroup a strip of 16 rows k x 64 columns o, its four
//               waves every fourth 16-deep slice of the batch, added through LDS in wave order;
//               dY 16 bytes a lane along o (component cc: columns 4 r + cc), X a float a lane
//   the other layer's dW: 16 x 16 blocks, both operands a float a lane (its width need not be a
//               multiple of four)
struct FcBwdMfma {
  const float *x, *w, *dy;  // X[batch][in], W[in][out], dY[batch][out]; out a multiple of 4
  EpiRowMajorPool xepi;     // dX (row.out null: not asked for)
  float *dw, *db;
  int batch, in, out, accumulate;
  int nx, xcb;   // dX workgroups (four blocks each), column blocks ceil(in / 16)
  int nw, wcg;   // dW workgroups, column groups ceil(out / 64)
  int ndb;       // workgroups of 32 bias columns
  const float *x2, *dy2;    // the other layer: X2[batch][in2], dY2[batch][out2]
  float *dw2, *db2;
  int in2, out2, nw2, w2cb, ndb2;
};

__global__ void __launch_bounds__(256) fc_bwd_mfma_kernel(const FcBwdMfma f) {
  __shared__ __attribute__((aligned(16))) float red[4][16][TL_LD];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15, q = lane >> 4;
  int b = blockIdx.x;
  if (b < f.nx) {
    // ---- dX: block (rb, jb) of 16 rows and 16 columns
    const int blk = 4 * b + wave;
    const int rb = blk / f.xcb, jb = blk - rb * f.xcb;
    const int m0 = 16 * rb, j0 = 16 * jb;
    if (m0 >= f.batch) return;
    const int agk     = f.xepi.row.ag.kind;
    const bool pooled = f.xepi.pool.argmax != nullptr;
    // what the epilogue reads, asked for first: rows and columns past the end read the last ones
    const int j = j0 + r, jc = min(j, f.in - 1);
    float py[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    int am[4] = {0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int idx = min(m0 + 4 * q + i, f.batch - 1) * f.in + jc;
      if (agk != TDH_ACT_NONE) py[i] = f.xepi.row.ag.y[idx];
      if (pooled) am[i] = f.xepi.pool.argmax[idx];
    }
    const float *arow = f.dy + static_cast<size_t>(min(m0 + r, f.batch - 1)) * f.out;
    const float *brow = f.w + static_cast<size_t>(jc) * f.out;
    tail_f4 d = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int k0 = 0; k0 < f.out; k0 += 64) {
      float4 av[4], bv[4];
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) {
        const int kc  = k0 + 16 * kk + 4 * q;
        const bool ok = kc < f.out;
        av[kk] = tail_keep(tail_ld4(arow + (ok ? kc : 0)), ok);
        bv[kk] = tail_ld4(brow + (ok ? kc : 0));
      }
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) {
        d = __builtin_amdgcn_mfma_f32_16x16x4f32(av[kk].x, bv[kk].x, d, 0, 0, 0);
        d = __builtin_amdgcn_mfma_f32_16x16x4f32(av[kk].y, bv[kk].y, d, 0, 0, 0);
        d = __builtin_amdgcn_mfma_f32_16x16x4f32(av[kk].z, bv[kk].z, d, 0, 0, 0);
        d = __builtin_amdgcn_mfma_f32_16x16x4f32(av[kk].w, bv[kk].w, d, 0, 0, 0);
      }
    }
    if (j >= f.in) return;
    const TailGrad gx = tail_grad_coef(agk);
    const int cbase   = f.xepi.col(j).base;
    const int W       = f.xepi.pool.W;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = m0 + 4 * q + i;
      if (m >= f.batch) continue;
      // the steps of EpiRowMajorPool::store without a bias, not accumulating
      const float v = ((d[i] + 0.0f) * tail_grad_factor(gx, py[i])) + 0.0f;
      f.xepi.row.out[m * f.in + j] = v;
      if (pooled) {
        const int a = am[i] - cbase;
        float *p    = f.xepi.pool.dx + static_cast<size_t>(m) * f.xepi.sample_in + cbase;
        *reinterpret_cast<float2 *>(p)     = make_float2(a == 0 ? v : 0.0f, a == 1 ? v : 0.0f);
        *reinterpret_cast<float2 *>(p + W) = make_float2(a == W ? v : 0.0f, a == W + 1 ? v : 0.0f);
      }
    }
    return;
  }
  b -= f.nx;
  if (b < f.nw) {
    // ---- dW: rows k0 .. k0 + 15, columns o0 .. o0 + 63
    const int strip = b / f.wcg, cg = b - strip * f.wcg;
    const int k0 = 16 * strip, o0 = 64 * cg;
    const float *xcol = f.x + min(k0 + r, f.in - 1);
    const float *dcol = f.dy + (o0 + 4 * r < f.out ? o0 + 4 * r : 0);
    tail_f4 acc[4] = {{0.0f, 0.0f, 0.0f, 0.0f}, {0.0f, 0.0f, 0.0f, 0.0f}, {0.0f, 0.0f, 0.0f, 0.0f}, {0.0f, 0.0f, 0.0f, 0.0f}};
#pragma unroll 2
    for (int m16 = 16 * wave; m16 < f.batch; m16 += 64) {
      float a[4];
      float4 bv[4];
#pragma unroll
      for (int comp = 0; comp < 4; ++comp) {
        const int m   = m16 + 4 * q + comp;
        const bool ok = m < f.batch;
        const int mc  = ok ? m : f.batch - 1;
        const float v = xcol[static_cast<size_t>(mc) * f.in];
        a[comp]       = ok ? v : 0.0f;
        bv[comp]      = tail_ld4(dcol + static_cast<size_t>(mc) * f.out);
      }
#pragma unroll
      for (int comp = 0; comp < 4; ++comp) {
        acc[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[comp], bv[comp].x, acc[0], 0, 0, 0);
        acc[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[comp], bv[comp].y, acc[1], 0, 0, 0);
        acc[2] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[comp], bv[comp].z, acc[2], 0, 0, 0);
        acc[3] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[comp], bv[comp].w, acc[3], 0, 0, 0);
      }
    }
    // acc[cc][i]: row 4 q + i, column 4 r + cc
#pragma unroll
    for (int i = 0; i < 4; ++i)
      *reinterpret_cast<float4 *>(&red[wave][4 * q + i][4 * r]) = make_float4(acc[0][i], acc[1][i], acc[2][i], acc[3][i]);
    __syncthreads();
    const int row = tid >> 4, c4 = 4 * (tid & 15);
    float4 s = *reinterpret_cast<const float4 *>(&red[0][row][c4]);
#pragma unroll
    for (int v = 1; v < 4; ++v) {
      const float4 p = *reinterpret_cast<const float4 *>(&red[v][row][c4]);
      s.x += p.x; s.y += p.y; s.z += p.z; s.w += p.w;
    }
    if (k0 + row < f.in && o0 + c4 < f.out) {
      float4 *dst = reinterpret_cast<float4 *>(f.dw + static_cast<size_t>(k0 + row) * f.out + o0 + c4);
      if (f.accumulate) {
        const float4 old = *dst;
        s.x += old.x; s.y += old.y; s.z += old.z; s.w += old.w;
      }
      *dst = s;
    }
    return;
  }
  b -= f.nw;
  float(*part)[32] = reinterpret_cast<float(*)[32]>(&red[0][0][0]);
  auto bias_block = [&](const float *dy, float *db, const int out, const int cb) {
    // 32 columns of the column sums of dy[batch][out]: rows g, g + 8, ... per 32-lane group, the
    // group sums in order (as the stand-alone column sum does)
    const int cl = tid & 31, g = tid >> 5;
    const int c  = cb * 32 + cl;
    float s = 0.0f;
    if (c < out)
      for (int rr = g; rr < f.batch; rr += 8) s += dy[static_cast<size_t>(rr) * out + c];
    part[g][cl] = s;
    __syncthreads();
    if (g == 0 && c < out) {
      float t = part[0][cl];
#pragma unroll
      for (int i = 1; i < 8; ++i) t += part[i][cl];
      db[c] = f.accumulate ? db[c] + t : t;
    }
  };
  if (b < f.ndb) {
    bias_block(f.dy, f.db, f.out, b);
    return;
  }
  b -= f.ndb;
  if (b < f.nw2) {
    // ---- the other layer's dW: rows h0 .. h0 + 15, columns o0 .. o0 + 15
    const int rbk = b / f.w2cb, cbk = b - rbk * f.w2cb;
    const int h0 = 16 * rbk, o0 = 16 * cbk;
    const float *xcol = f.x2 + min(h0 + r, f.in2 - 1);
    const float *dcol = f.dy2 + min(o0 + r, f.out2 - 1);
    tail_f4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll 2
    for (int m16 = 16 * wave; m16 < f.batch; m16 += 64) {
      float a[4], bs[4];
#pragma unroll
      for (int comp = 0; comp < 4; ++comp) {
        const int m   = m16 + 4 * q + comp;
        const bool ok = m < f.batch;
        const int mc  = ok ? m : f.batch - 1;
        const float v = xcol[static_cast<size_t>(mc) * f.in2];
        a[comp]       = ok ? v : 0.0f;
        bs[comp]      = dcol[static_cast<size_t>(mc) * f.out2];
      }
#pragma unroll
      for (int comp = 0; comp < 4; ++comp) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[comp], bs[comp], acc, 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) red[wave][4 * q + i][r] = acc[i];
    __syncthreads();
    const int row = tid >> 4, col = tid & 15;
    float s = red[0][row][col];
#pragma unroll
    for (int v = 1; v < 4; ++v) s += red[v][row][col];
    if (h0 + row < f.in2 && o0 + col < f.out2) {
      float *dst = f.dw2 + static_cast<size_t>(h0 + row) * f.out2 + o0 + col;
      *dst = f.accumulate ? *dst + s : s;
    }
    return;
  }
  bias_block(f.dy2, f.db2, f.out2, b - f.nw2);
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

// the two closing fully-connected layers (in -> hidden -> out, a pointwise activation between
// them) can leave one launch with the loss gradient and both input gradients
bool fc_two_layer_tail_applies(int in, int hidden, int out, int batch) {
  return hidden <= 64 && hidden % 4 == 0 && out <= 64 && in >= 4 && in % 4 == 0 && in <= 64 * TL_KC && batch >= 1 &&
         static_cast<long>(batch) * in < (1L << 24);
}
// floats of partial sums and number of tickets the launch needs (the caller owns both; the
// tickets are zero before the first launch and the kernel leaves them zero)
size_t fc_two_layer_tail_partials(int in, int batch) {
  const int splits = ceil_div(in, TL_KC);
  return splits > 1 ? static_cast<size_t>(ceil_div(batch, TL_TM)) * splits * TL_TM * 64 : 0;
}
size_t fc_two_layer_tail_tickets(int batch) { return static_cast<size_t>(ceil_div(batch, TL_TM)); }

// soft == nullptr: the net ends in the second layer and the loss is mse.
int fc_two_layer_tail(int in, int hidden, int out, int has_bias1, int has_bias2, int batch, const float *x,
                      const float *w1, const float *b1, float *y1, float *a1, int act_kind, const float *w2,
                      const float *b2, float *y2, float *soft, const float *t, float *dz, float *dh,
                      float *partials, unsigned int *tickets) {
  if (!fc_two_layer_tail_applies(in, hidden, out, batch))
    return set_error(TDH_ERR_INVALID, "fc_two_layer_tail: layers too large for the one-launch kernel");
  FcTail2 f;
  f.x = x; f.w1 = w1; f.bias1 = has_bias1 ? b1 : nullptr;
  f.w2 = w2; f.bias2 = has_bias2 ? b2 : nullptr;
  f.out1 = y1; f.act1 = a1; f.act1_kind = act_kind;
  f.out2 = y2; f.soft = soft; f.t = t; f.dz = dz; f.dh = dh;
  f.mse_factor = 2.0f / static_cast<float>(out);
  f.partials = partials; f.tickets = tickets;
  f.M = batch; f.K1 = in; f.H = hidden; f.O = out;
  f.splits = ceil_div(in, TL_KC);
  if (f.splits > 1 && !(partials && tickets))
    return set_error(TDH_ERR_INVALID, "fc_two_layer_tail: no room for the partial sums");
  ProfScope prof("fc_two_layer_tail",
                 2.0 * batch * (static_cast<double>(in) * hidden + 2.0 * hidden * out), WORK_FLOP);
  TDH_LAUNCH(fc_two_layer_tail_kernel, dim3(f.splits, ceil_div(batch, TL_TM)), dim3(TL_NT), 0, ctx().stream, f);
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

// ---- dW of a large fully-connected layer, operands straight from memory
//
//   dW[i][o] (+)= sum_b X[b][i] * dY[b][o]        (fully_connected_op_internal.h:57-64)
//
// Both operands have the reduction index (the sample) as their slow one, so the fragment of a
// v_mfma_f32_32x32x2_f32 (lane = (column l%32, sample l/32)) is a coalesced read of a row: no
// LDS, no barrier. A lane reads four consecutive inputs and two consecutive outputs of its
// sample; component c of the first feeds the accumulator blocks whose 32 rows stand for the
// inputs 4 r + c, component d of the second those whose columns stand for the outputs 2 n + d.
// A wave so owns 128 inputs x 64 outputs (eight blocks, 128 accumulator registers) with six
// loaded registers per eight MFMAs; four sample pairs are loaded as a group while the group
// before is multiplied. The reduction is as short as the batch, so a tile is prologue,
// products and a 32 KB store, and the chip holds every workgroup of a 4096 x 4096 layer at
// once (two waves per SIMD).
constexpr int FDW_WM = 2, FDW_WN = 2;     // waves of a workgroup along the two
constexpr int FDW_DEPTH = 4;              // sample pairs per group of loads

struct FcDwDirect {
  const float *x, *dy;
  float *dw;
  int batch, in, out, accumulate;
};

typedef float fdw_x16 __attribute__((ext_vector_type(16)));

// CA, CB: consecutive inputs and outputs a lane reads. Measured on 4096 x 4096 x 256: 4 x 2
// (two waves per SIMD) 80 us, 4 x 4 (one wave per SIMD) 80 us, 2 x 2 (four waves) 93 us.
template <int CA, int CB>
__global__ void __launch_bounds__(64 * FDW_WM * FDW_WN) __attribute__((amdgpu_waves_per_eu(CA * CB > 8 ? 1 : CA * CB > 4 ? 2 : 4, 8)))
fc_dw_direct_kernel(const FcDwDirect f) {
  constexpr int FDW_TM = 32 * CA, FDW_TN = 32 * CB;
  typedef float avec __attribute__((ext_vector_type(CA)));
  typedef float bvec __attribute__((ext_vector_type(CB)));
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int m = lane & 31, h = lane >> 5;
  // Workgroups go to the eight XCDs (each with its own L2) round-robin in launch order. Each
  // XCD gets a compact block of the tile grid (a quarter of the rows x half of the columns
  // where the grid divides so, else a run of consecutive tiles), so that the panels its
  // workgroups read together fit its L2.
  int bx, by;
  {
    const int gx = gridDim.x, gy = gridDim.y;
    const int id = blockIdx.x + gx * blockIdx.y, total = gx * gy;
    const int xcd = id & 7, seq = id >> 3;
    if (gx % 2 == 0 && gy % 4 == 0) {
      const int hx = gx >> 1, qy = gy >> 2;
      bx = (xcd & 1) * hx + seq % hx;
      by = (xcd >> 1) * qy + seq / hx;
    } else {
      const int per = total >> 3;
      const int at  = id < (per << 3) ? xcd * per + seq : id;
      bx = at % gx;
      by = at / gx;
    }
  }
  const int i0 = (by * FDW_WM + (wave % FDW_WM)) * FDW_TM;
  const int o0 = (bx * FDW_WN + (wave / FDW_WM)) * FDW_TN;
  // (in is a multiple of four and out of two: a lane's inputs and outputs exist all or not at
  // all; what does not exist is read from column 0 and never stored)
  // (offsets in 32 bits on top of the tensors' uniform base pointers)
  const bool a_ok = i0 + CA * m < f.in, b_ok = o0 + CB * m < f.out;
  const unsigned acol = a_ok ? i0 + CA * m : 0, bcol = b_ok ? o0 + CB * m : 0;

  fdw_x16 acc[CA][CB];
#pragma unroll
  for (int c = 0; c < CA; ++c)
#pragma unroll
    for (int d = 0; d < CB; ++d)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[c][d][r] = 0.0f;

  avec ra[2][FDW_DEPTH];
  bvec rb[2][FDW_DEPTH];
  auto load = [&](int k0, auto to) {
    constexpr int T = decltype(to)::value;
#pragma unroll
    for (int j = 0; j < FDW_DEPTH; ++j) {
      const int kk = min(k0 + 2 * j + h, f.batch - 1);
      ra[T][j] = *reinterpret_cast<const avec *>(f.x + (static_cast<unsigned>(kk) * f.in + acol));
      rb[T][j] = *reinterpret_cast<const bvec *>(f.dy + (static_cast<unsigned>(kk) * f.out + bcol));
    }
  };
  // (the zeros of samples past the batch go in here, not where the loads are issued: a select
  // there would wait for the load it follows; a zero on one side is enough)
  auto products = [&](int k0, auto from) {
    constexpr int T = decltype(from)::value;
#pragma unroll
    for (int j = 0; j < FDW_DEPTH; ++j) {
      const bool on    = k0 + 2 * j + h < f.batch;
      float a[CA];
#pragma unroll
      for (int c = 0; c < CA; ++c) a[c] = on ? ra[T][j][c] : 0.0f;
      float b[CB];
#pragma unroll
      for (int d = 0; d < CB; ++d) b[d] = rb[T][j][d];
#pragma unroll
      for (int c = 0; c < CA; ++c)
#pragma unroll
        for (int d = 0; d < CB; ++d)
          acc[c][d] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[c], b[d], acc[c][d], 0, 0, 0);
    }
  };
  using Buf0 = std::integral_constant<int, 0>;
  using Buf1 = std::integral_constant<int, 1>;
  constexpr int GROUP = 2 * FDW_DEPTH;  // samples per group
  // (a group past the batch is clamped reads and products with zeros; the scheduling
  // barriers keep a group's loads in front of the products they run beside: left alone, the
  // compiler sinks each load to its first use)
  load(0, Buf0());
#pragma unroll 1
  for (int k0 = 0; k0 < f.batch; k0 += 2 * GROUP) {
    load(k0 + GROUP, Buf1());
    __builtin_amdgcn_sched_barrier(0);
    products(k0, Buf0());
    __builtin_amdgcn_sched_barrier(0);
    load(k0 + 2 * GROUP, Buf0());
    __builtin_amdgcn_sched_barrier(0);
    products(k0 + GROUP, Buf1());
    __builtin_amdgcn_sched_barrier(0);
  }

  // reg r of lane l of block (c, d): input i0 + CA*(8*(r/4) + 4*(l/32) + r%4) + c, output
  // o0 + 2*(l%32) + d; the two blocks d leave as one 8-byte store
  if (!b_ok) return;
  float *out = f.dw + o0 + CB * m;
  // (rows past the layer's inputs are read and written at row i0, with what row i0 holds:
  // loads and stores without conditions, sixteen loads in flight when the sums are added to
  // what the gradient held)
#pragma unroll
  for (int c = 0; c < CA; ++c) {
    bvec old[16];
    if (f.accumulate) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int i = i0 + CA * (8 * (r >> 2) + 4 * h + (r & 3)) + c;
        old[r] = *reinterpret_cast<const bvec *>(out + static_cast<size_t>(min(i, f.in - 1)) * f.out);
      }
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int i = i0 + CA * (8 * (r >> 2) + 4 * h + (r & 3)) + c;
      if (i >= f.in) continue;
      bvec v;
#pragma unroll
      for (int d = 0; d < CB; ++d) v[d] = f.accumulate ? old[r][d] + acc[c][d][r] : acc[c][d][r];
      *reinterpret_cast<bvec *>(out + static_cast<size_t>(i) * f.out) = v;
    }
  }
}

// the layer is large enough for every compute unit to get a workgroup of that kernel, and its
// rows allow the 16- and 8-byte reads
static bool fc_dw_direct_applies(int in, int out, int batch, const float *x, const float *dy, const float *dw) {
  const long wgs = static_cast<long>(ceil_div(in, 128 * FDW_WM)) * ceil_div(out, 64 * FDW_WN);
  return in % 4 == 0 && out % 2 == 0 && batch >= 2 && wgs >= 256 && ceil_div(in, 128 * FDW_WM) <= 65535 &&
         ceil_div(out, 64 * FDW_WN) <= 65535 &&
         static_cast<long>(batch) * std::max(in, out) < (1L << 30) &&
         !(reinterpret_cast<uintptr_t>(x) & 15) && !(reinterpret_cast<uintptr_t>(dy) & 7) &&
         !(reinterpret_cast<uintptr_t>(dw) & 7);
}

// ---- dX of a large fully-connected layer
//
//   dX[b][i] = sum_o dY[b][o] * W[i][o]        (fully_connected_op_internal.h:42-54)
//
// Both operands have the reduction index (the output) as their fast one, so a tile of either is
// staged with 16-byte reads along its rows and 16-byte LDS writes, untransposed: [row][128
// outputs], rows padded by four floats. A lane of a v_mfma_f32_32x32x2_f32 stands for (row l%32,
// reduction element l/32) on both sides, so one 16-byte LDS read, the row's outputs
// k + 4*(l/32) .. + 3, feeds four MFMAs: component j pairs output k + j (lanes 0-31) with
// k + 4 + j (lanes 32-63), the same pairing on both sides. No split of the reduction over
// workgroups and no second launch: a workgroup owns 64 samples x 64 inputs (one workgroup per
// compute unit for 256 x 4096), eight waves = 2 x 2 blocks of 32 x 32 times the two halves of
// every staged chunk, so a SIMD holds two waves that fill each other's waits; the halves meet in
// LDS at the end and add up in a fixed order. (Fragments read straight from memory, a lane's
// 16-byte word of its own row, touch 32 cache lines per load: 124 us against 96 for the general
// kernel and its split reduction.)
constexpr int FDX_BK = 128;            // outputs per staged chunk
constexpr int FDX_LD = FDX_BK + 4;     // floats of a staged row

struct FcDxTile {
  const float *dy, *w;
  float *dx;
  ActGrad ag;
  int batch, in, out, tiles_m, tiles_n, n_per_xcd;
};

__global__ void __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2)))
fc_dx_tile_kernel(const FcDxTile f) {
  __shared__ __attribute__((aligned(16))) float tile[2][128][FDX_LD];   // rows 0-63: dY, 64-127: W
  // (behind the last chunk the same memory carries the upper half's blocks, [block][register][lane])
  float (*halves)[16][64] = reinterpret_cast<float (*)[16][64]>(&tile[0][0][0]);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int m = lane & 31, h = lane >> 5;
  const int wm = wave & 1, wn = (wave >> 1) & 1, kh = wave >> 2;
  // Workgroups go to the eight XCDs round-robin in launch order. An XCD gets a run of column
  // tiles with all their row tiles, so that the rows of W it reads are read by nobody else and
  // its row tiles share them in its L2.
  const int xcd = blockIdx.x & 7, seq = blockIdx.x >> 3;
  const int tm = seq % f.tiles_m, tn = xcd * f.n_per_xcd + seq / f.tiles_m;
  if (tn >= f.tiles_n) return;
  const int b0 = tm * 64, i0 = tn * 64;

  // staging: thread t moves the 16-byte word t % W4 of the rows t / W4 + ROWS*i
  // (rows past the batch or the layer's inputs are read at the last row and never stored)
  constexpr int W4 = FDX_BK / 4, ROWS = 512 / W4, PASSES = 128 / ROWS;
  const int s_row = tid / W4, s_c4 = tid % W4;
  unsigned s_off[PASSES];
#pragma unroll
  for (int i = 0; i < PASSES; ++i) {
    const int row = s_row + ROWS * i;
    s_off[i] = i < PASSES / 2 ? static_cast<unsigned>(min(b0 + row, f.batch - 1)) * f.out
                              : static_cast<unsigned>(min(i0 + row - 64, f.in - 1)) * f.out;
  }
  // two chunks are on their way from memory while a third is multiplied: W streams in from
  // memory, and one chunk's products are shorter than that trip
  float4 stg[2][PASSES];
  auto fetch = [&](int k0, auto to) {
    constexpr int T = decltype(to)::value;
    const int k = min(k0 + 4 * s_c4, f.out - 4);
#pragma unroll
    for (int i = 0; i < PASSES; ++i)
      stg[T][i] = *reinterpret_cast<const float4 *>((i < PASSES / 2 ? f.dy : f.w) + (s_off[i] + static_cast<unsigned>(k)));
  };
  // (a word past the layer's outputs was read somewhere valid and is stored as zeros)
  auto stage = [&](int k0, int buf, auto from) {
    constexpr int T = decltype(from)::value;
    const bool on = k0 + 4 * s_c4 < f.out;
#pragma unroll
    for (int i = 0; i < PASSES; ++i)
      *reinterpret_cast<float4 *>(&tile[buf][s_row + ROWS * i][4 * s_c4]) = on ? stg[T][i] : make_float4(0.f, 0.f, 0.f, 0.f);
  };

  floatx16 acc0, acc1;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc0[r] = acc1[r] = 0.0f;
  const int a_row = wm * 32 + m, b_row = 64 + wn * 32 + m, k_lane = kh * (FDX_BK / 2) + 4 * h;
  auto products = [&](int buf) {
#pragma unroll
    for (int s = 0; s < FDX_BK / 16; ++s) {
      const float4 a = *reinterpret_cast<const float4 *>(&tile[buf][a_row][k_lane + 8 * s]);
      const float4 b = *reinterpret_cast<const float4 *>(&tile[buf][b_row][k_lane + 8 * s]);
      acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a.x, b.x, acc0, 0, 0, 0);
      acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a.y, b.y, acc1, 0, 0, 0);
      acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a.z, b.z, acc0, 0, 0, 0);
      acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a.w, b.w, acc1, 0, 0, 0);
    }
  };
  using Set0 = std::integral_constant<int, 0>;
  using Set1 = std::integral_constant<int, 1>;

  // chunk c sits in tile[c % 2]; chunk c + 1 waits in registers (set (c + 1) % 2), chunk c + 2
  // is asked for (fetches past the end read the last words again and are dropped)
  fetch(0, Set0());
  fetch(FDX_BK, Set1());
  stage(0, 0, Set0());
  __syncthreads();
#pragma unroll 1
  for (int k0 = 0; k0 < f.out; k0 += 2 * FDX_BK) {
    fetch(k0 + 2 * FDX_BK, Set0());
    products(0);
    stage(k0 + FDX_BK, 1, Set1());
    __syncthreads();
    if (k0 + FDX_BK >= f.out) break;
    fetch(k0 + 3 * FDX_BK, Set1());
    products(1);
    stage(k0 + 2 * FDX_BK, 0, Set0());
    __syncthreads();
  }

  const int blk = wm + 2 * wn;
  if (kh) {
#pragma unroll
    for (int r = 0; r < 16; ++r) halves[blk][r][lane] = acc0[r] + acc1[r];
  }
  __syncthreads();
  if (kh) return;
  // register r of lane l: sample b0 + 32*wm + 8*(r/4) + 4*(l/32) + r%4, input i0 + 32*wn + l%32
  const int i = i0 + wn * 32 + m;
  if (i >= f.in) return;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int b = b0 + wm * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
    if (b >= f.batch) continue;
    const size_t idx = static_cast<size_t>(b) * f.in + i;
    float v = (acc0[r] + acc1[r]) + halves[blk][r][lane];
    if (f.ag.kind != TDH_ACT_NONE) v *= act_grad_factor(f.ag.kind, f.ag.y[idx]);
    f.dx[idx] = v;
  }
}

// the layer is large enough to give (nearly) every compute unit a workgroup of that kernel, its
// reduction long enough for the kernel's two-chunk prologue to be a small part of it (the VGG
// classifier, 131072 -> 256, has two chunks in all and stays with the general kernel), and its
// rows allow the 16-byte reads
static bool fc_dx_tile_applies(int in, int out, int batch, const float *dy, const float *w) {
  const long wgs = static_cast<long>(ceil_div(batch, 64)) * ceil_div(in, 64);
  return out % 4 == 0 && out >= 8 * FDX_BK && wgs >= 192 && wgs <= 4096 &&
         static_cast<long>(std::max(batch, in)) * out < (1L << 30) &&
         !(reinterpret_cast<uintptr_t>(dy) & 15) && !(reinterpret_cast<uintptr_t>(w) & 15);
}

int fc_bwd(int in, int out, int has_bias, int batch, const float *x, const float *w,
           const float *dy, float *dx, float *dw, float *db, int accumulate, ActGrad dx_act,
           const PoolScatter *pool, const FcGrads *also) {
  const bool bias_grad = db && has_bias;
  if (also && !(dw && (dx || bias_grad) && fc_bwd_fuses(in, out, batch) && fc_bwd_fuses(also->in, also->out, batch)))
    return set_error(TDH_ERR_INVALID, "fc_bwd: another layer's gradients need the one-launch kernel");
  if (pool && !(dx && dw && fc_bwd_fuses(in, out, batch) && pool->OH * pool->OW > 0 && in % (pool->OH * pool->OW) == 0))
    return set_error(TDH_ERR_INVALID, "fc_bwd: the pool scatter needs the one-launch kernel");
  if (dw && (dx || bias_grad) && fc_bwd_fuses(in, out, batch) && out % 4 == 0 &&
      !(reinterpret_cast<uintptr_t>(dy) & 15) && !(reinterpret_cast<uintptr_t>(w) & 15) &&
      !(reinterpret_cast<uintptr_t>(dw) & 15) && static_cast<long>(batch) * in < (1L << 30)) {
    FcBwdMfma f;
    f.x = x; f.w = w; f.dy = dy;
    f.xepi.row = EpiRowMajor{dx, in, nullptr, dx_act, 0};
    if (pool) {
      f.xepi.pool      = *pool;
      f.xepi.div_ow    = FastDiv(pool->OW);
      f.xepi.div_oh    = FastDiv(pool->OH);
      f.xepi.sample_in = 4 * in;
    }
    f.dw = dw; f.db = bias_grad ? db : nullptr;
    f.batch = batch; f.in = in; f.out = out; f.accumulate = accumulate;
    f.xcb = ceil_div(in, 16);
    f.nx  = dx ? ceil_div(ceil_div(batch, 16) * f.xcb, 4) : 0;
    f.wcg = ceil_div(out, 64);
    f.nw  = ceil_div(in, 16) * f.wcg;
    f.ndb = bias_grad ? ceil_div(out, 32) : 0;
    f.x2 = f.dy2 = nullptr; f.dw2 = f.db2 = nullptr;
    f.in2 = f.out2 = 1; f.nw2 = f.w2cb = f.ndb2 = 0;
    double flop = (dx ? 4.0 : 2.0) * batch * in * out;
    if (also) {
      f.x2 = also->x; f.dy2 = also->dy; f.dw2 = also->dw; f.db2 = also->db;
      f.in2 = also->in; f.out2 = also->out;
      f.w2cb = ceil_div(also->out, 16);
      f.nw2  = ceil_div(also->in, 16) * f.w2cb;
      f.ndb2 = also->db ? ceil_div(also->out, 32) : 0;
      flop += 2.0 * batch * also->in * also->out;
    }
    ProfScope prof(also ? (pool ? "fc_bwd_small_pool_two" : "fc_bwd_small_two")
                        : pool ? "fc_bwd_small_pool" : dx ? "fc_bwd_small" : "fc_dw_db_small", flop, WORK_FLOP);
    TDH_LAUNCH(fc_bwd_mfma_kernel, dim3(f.nx + f.nw + f.ndb + f.nw2 + f.ndb2), dim3(256), 0, ctx().stream, f);
    TDH_LAUNCH_CHECK();
    return TDH_OK;
  }
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
    f.dy = dy; f.db = db; f.batch = batch; f.out = out; f.db_accumulate = accumulate;
    f.ndb = bias_grad ? ceil_div(out, 32) : 0;
    f.nw2 = 0;
    int ndb2 = 0;
    double flop = (dx ? 4.0 : 2.0) * batch * in * out;
    if (also) {
      f.w2a = StridedOperand{also->x, 1, also->in, also->in};
      f.w2b = StridedOperand{also->dy, 1, also->out, also->out};
      f.w2epi = EpiRowMajor{also->dw, also->out, nullptr, ActGrad(), accumulate};
      f.w2M = also->in; f.w2N = also->out; f.w2K = batch;
      f.w2_tiles_n = ceil_div(also->out, SFC_TN);
      f.nw2 = f.w2_tiles_n * ceil_div(also->in, SFC_TM);
      f.dy2 = also->dy; f.db2 = also->db; f.out2 = also->out;
      ndb2 = also->db ? ceil_div(also->out, 32) : 0;
      flop += 2.0 * batch * also->in * also->out;
    }
    ProfScope prof(also ? (pool ? "fc_bwd_small_pool_two" : "fc_bwd_small_two")
                        : pool ? "fc_bwd_small_pool" : dx ? "fc_bwd_small" : "fc_dw_db_small", flop, WORK_FLOP);
    TDH_LAUNCH(fc_bwd_fused_kernel, dim3(f.nx + f.nw + f.ndb + f.nw2 + ndb2), dim3(SFC_NT), 0, ctx().stream, f);
    TDH_LAUNCH_CHECK();
    return TDH_OK;
  }
  if (dx) {
    StridedOperand A{dy, out, 1, batch};  // dY[s][k]
    StridedOperand B{w, out, 1, in};      // W[n][k], k contiguous
    EpiRowMajor epi{dx, in, nullptr, dx_act, 0};
    if (small_fc_applies(batch, in, out)) {
      TDH_TRY(launch_small_fc(A, B, epi, batch, in, out, "fc_dx_small"));
    } else if (fc_dx_tile_applies(in, out, batch, dy, w)) {
      ProfScope prof("fc_dx_tile", batch, in, out);
      FcDxTile f{dy, w, dx, dx_act, batch, in, out, ceil_div(batch, 64), ceil_div(in, 64), 0};
      f.n_per_xcd = ceil_div(f.tiles_n, 8);
      TDH_LAUNCH(fc_dx_tile_kernel, dim3(8 * f.n_per_xcd * f.tiles_m), dim3(512), 0, ctx().stream, f);
      TDH_LAUNCH_CHECK();
    } else
      TDH_TRY((launch_gemm<true, true, false, false>(A, B, epi, batch, in, out, true, "fc_dx_gemm",
                                                 "fc_dx_splitk_reduce")));
  }
  if (dw) {
    StridedOperand A{x, 1, in, in};      // X[k][m], m contiguous
    StridedOperand B{dy, 1, out, out};   // dY[k][n], n contiguous
    EpiRowMajor epi{dw, out, nullptr, ActGrad(), accumulate};
    if (small_fc_applies(in, out, batch)) {
      TDH_TRY(launch_small_fc(A, B, epi, in, out, batch, "fc_dw_small"));
    } else if (fc_dw_direct_applies(in, out, batch, x, dy, dw)) {
      ProfScope prof("fc_dw_direct", in, out, batch);
      const FcDwDirect f{x, dy, dw, batch, in, out, accumulate};
      TDH_LAUNCH((fc_dw_direct_kernel<4, 2>), dim3(ceil_div(out, 64 * FDW_WN), ceil_div(in, 128 * FDW_WM)),
                 dim3(64 * FDW_WM * FDW_WN), 0, ctx().stream, f);
      TDH_LAUNCH_CHECK();
    } else
      TDH_TRY((launch_gemm<false, false, true, true>(A, B, epi, in, out, batch, true, "fc_dw_gemm",
                                                   "fc_dw_splitk_reduce")));
  }
  if (db && has_bias) TDH_TRY(launch_colsum(dy, batch, out, db, accumulate));
  return TDH_OK;
}

}  // namespace tdh
