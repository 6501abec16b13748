// conv_fwd_small.hip — forward convolution with few input channels (Cin*KH*KW <= 96: the first
// layer of an image net), any stride and dilation, optionally with the layers behind it:
// a pointwise activation, a 2x2/stride-2 max-pool and the activation behind that pool.
//
//   y[img][co][oy][ox] = b[co] + sum_{ci,ky,kx} W[co][ci][ky][kx] * x[img][ci][oy*sh+ky*dh-ph][ox*sw+kx*dw-pw]
//
// As a product: M = Cout, N = output pixels, K = Cin*KH*KW (75 for 3 channels and 5x5). K is so
// short that a lane keeps its whole column of the filter matrix in registers. A workgroup owns
// a band of output rows of one image and 32 output channels; it stages the input patch under
// the band in LDS (zero-filled where the window leaves the image) and the filter slice, and a
// wave then computes tiles of 2 rows x 32 columns x 32 channels, one accumulator block per row:
// per k-step and row one LDS read at patch[pixel] + offset(k) and one v_mfma_f32_32x32x2_f32
// (A lane = (co, k), B lane = (pixel, k)). A lane so holds both rows of its column, and the 2x2
// pooling window of an even lane is completed by its right neighbour: the max-pool (with its
// argmax record and the activation behind it) costs a lane swap in the epilogue and needs no
// kernel or pass over y of its own. Stores of y are whole rows of 32 floats per channel.
//
// Reference: conv2d_op_internal.h:13-74 (forward), maxpool_op_internal.h:17-47 (window scan:
// row by row, strict '>', start value lowest()).
#include <algorithm>
#include <cfloat>

#include "gemm_mfma.h"

namespace tdh {

namespace {

typedef float floatx4 __attribute__((ext_vector_type(4)));

struct FwdSmallArgs {
  const float *x, *w, *bias;
  float *out;
  float *act_out;          // act(out), or null
  float *pool_out;         // 2x2 max of (act_out ? act(out) : out), or null
  int32_t *pool_argmax;    // flat CHW index inside the sample of the pool's input
  float *pool_act_out;     // act2(pool_out), or null
  int act_kind, pool_act_kind;
  int C, Kc, H, W, OH, OW;
  int R, S, sh, sw, dh, dw, ph, pw;
  int band, bands, col_tiles;
  int rows_in, pitch, plane;
  int crs, x_floats;
  FastDiv div_pitch, div_rows_in, div_col_tiles;
};

// the value of lane l ^ 1 (a swap inside lane pairs, done by the DPP path of a move)
__device__ __forceinline__ float lane_xor1(const float v) {
  return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0xB1, 0xF, 0xF, true));
}

// act_apply on the 16 values of an accumulator block; the choice is made once, not per value
__device__ __forceinline__ void act_apply16(const int kind, float (&v)[16]) {
  switch (kind) {
    case TDH_ACT_RELU:
#pragma unroll
      for (int i = 0; i < 16; ++i) v[i] = act_apply(TDH_ACT_RELU, v[i]);
      break;
    case TDH_ACT_TANH:
#pragma unroll
      for (int i = 0; i < 16; ++i) v[i] = act_apply(TDH_ACT_TANH, v[i]);
      break;
    case TDH_ACT_SIGMOID:
#pragma unroll
      for (int i = 0; i < 16; ++i) v[i] = act_apply(TDH_ACT_SIGMOID, v[i]);
      break;
    default: break;
  }
}

// Stages the input patch under the band (zero-filled where the window leaves the image), the
// filter slice, the bias and the patch offset of every k into LDS: all loads of a thread are
// issued before its first store.
template <int NS>
__device__ __forceinline__ void fwd_small_stage(const FwdSmallArgs &a, float *xs, float *ws, float *bs, int *offs,
                                                const int img, const int co0, const int oy0, const int tid,
                                                const int nthr) {
  {
    const int iy0     = oy0 * a.sh - a.ph;
    const int x_total = a.C * a.rows_in * a.pitch;
    constexpr int DEPTH = 8;
    // the filter slice as 16-byte words, issued in front of the patch and stored behind it: one
    // trip to memory covers both (a thread's eight words hold 32 rows of up to 128 taps)
    const int w_total = 32 * a.crs;
    const int w_valid = min(32, a.Kc - co0) * a.crs;
    const float *wsrc = a.w + static_cast<size_t>(co0) * a.crs;
    const bool wvec   = (reinterpret_cast<uintptr_t>(wsrc) & 15u) == 0 && (w_valid & 3) == 0 &&
                      w_total <= 4 * DEPTH * nthr;
    floatx4 wq[DEPTH];
    if (wvec) {
#pragma unroll
      for (int k = 0; k < DEPTH; ++k)  // (every load is issued: a word past the slice repeats its last one)
        wq[k] = *reinterpret_cast<const floatx4 *>(wsrc + min(4 * (tid + k * nthr), w_valid - 4));
    }
    for (int e0 = tid; e0 < x_total; e0 += DEPTH * nthr) {
      float xv[DEPTH];
      int xo[DEPTH];
#pragma unroll
      for (int k = 0; k < DEPTH; ++k) {
        const int e = e0 + k * nthr;
        xv[k] = 0.0f;
        xo[k] = -1;
        if (e < x_total) {
          const int rr = a.div_pitch.div(e), cx = e - rr * a.pitch;
          const int ci = a.div_rows_in.div(rr), r = rr - ci * a.rows_in;
          const int iy = iy0 + r, ix = cx - a.pw;
          xo[k] = ci * a.plane + r * a.pitch + cx;
          if (iy >= 0 && iy < a.H && ix >= 0 && ix < a.W)
            xv[k] = a.x[(static_cast<size_t>(img * a.C + ci) * a.H + iy) * a.W + ix];
        }
      }
#pragma unroll
      for (int k = 0; k < DEPTH; ++k)
        if (xo[k] >= 0) xs[xo[k]] = xv[k];
    }
    if (wvec) {
#pragma unroll
      for (int k = 0; k < DEPTH; ++k) {
        const int e = 4 * (tid + k * nthr);
        const floatx4 zero4 = {0.0f, 0.0f, 0.0f, 0.0f};
        if (e < w_total) *reinterpret_cast<floatx4 *>(ws + e) = e < w_valid ? wq[k] : zero4;
      }
    }
    for (int e0 = wvec ? w_total : tid; e0 < w_total; e0 += DEPTH * nthr) {
      float wv[DEPTH];
#pragma unroll
      for (int k = 0; k < DEPTH; ++k) {
        const int e = e0 + k * nthr;
        wv[k] = e < w_valid ? wsrc[e] : 0.0f;
      }
#pragma unroll
      for (int k = 0; k < DEPTH; ++k) {
        const int e = e0 + k * nthr;
        if (e < w_total) ws[e] = wv[k];
      }
    }
    if (tid < 32) {
      const int m = co0 + tid;
      bs[tid]     = (a.bias && m < a.Kc) ? a.bias[m] : 0.0f;
    }
    if (tid < 2 * NS) {
      int o = -1;
      if (tid < a.crs) {
        const int rs = a.R * a.S;
        const int ci = tid / rs, tap = tid - ci * rs;
        const int ky = tap / a.S, kx = tap - ky * a.S;
        o = ci * a.plane + ky * a.dh * a.pitch + kx * a.dw;
      }
      offs[tid] = max(o, 0);
    }
  }
}

template <int NS>
__global__ void __launch_bounds__(256, 2) conv_fwd_small_kernel(const FwdSmallArgs a) {
  extern __shared__ __align__(16) float lds[];
  float *xs = lds;
  float *ws = lds + a.x_floats;  // [32][crs], rows past Cout are zero
  float *bs = ws + 32 * a.crs;   // [32] bias, zero past Cout or without bias
  int *offs = reinterpret_cast<int *>(bs + 32);  // [2*NS] patch offset of k (0 past K)
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // (an image's bands share rows: they go to one XCD)
  const int wg = xcd_compact_id(blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z),
                                gridDim.x * gridDim.y * gridDim.z);
  const int bandi = wg % gridDim.x, img = (wg / gridDim.x) % gridDim.y, co0 = (wg / (gridDim.x * gridDim.y)) * 32;
  const int oy0 = bandi * a.band;
  const int nthr = blockDim.x;  // one wave per tile of the band, two to four waves

  fwd_small_stage<NS>(a, xs, ws, bs, offs, img, co0, oy0, tid, nthr);
  __syncthreads();

  // ---- per-lane constants: the lane's column of the filter matrix
  // (k = 2*s + half), the bias of its 16 output channels
  const int nl = lane & 31, half = lane >> 5;
  float areg[NS];
#pragma unroll
  for (int s = 0; s < NS; ++s) {
    const int k = 2 * s + half;
    areg[s]     = k < a.crs ? ws[nl * a.crs + k] : 0.0f;
  }
  const int *offh = offs + half;  // the offsets stay in LDS: one broadcast read per k-step
  float bias_r[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    bias_r[i] = bs[(i >> 2) * 8 + half * 4 + (i & 3)];
  }

  const int ohw = a.OH * a.OW;
  const int POH = a.OH >> 1, POW = a.OW >> 1;
  const int tiles = (a.band >> 1) * a.col_tiles;
#pragma unroll 1
  for (int tile = wave; tile < tiles; tile += (nthr >> 6)) {
    const int rp = a.div_col_tiles.div(tile), ct = tile - rp * a.col_tiles;
    const int r = 2 * rp, c = 32 * ct + nl;  // band-relative upper row, column
    const float *xb0 = xs + r * a.sh * a.pitch + c * a.sw;
    const float *xb1 = xb0 + a.sh * a.pitch;
    floatx16 acc0, acc1;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc0[i] = acc1[i] = 0.0f;
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      const int o = offh[2 * s];
      acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(areg[s], xb0[o], acc0, 0, 0, 0);
      acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(areg[s], xb1[o], acc1, 0, 0, 0);
    }

    // ---- epilogue: reg i of lane l holds channel 8*(i/4) + 4*(l/32) + i%4 at column l%32
    const int oy = oy0 + r, ox = c;
    const bool ok0 = oy < a.OH && ox < a.OW, ok1 = oy + 1 < a.OH && ox < a.OW;
    const size_t pbase = static_cast<size_t>(img) * a.Kc * ohw + oy * a.OW + ox;
    const int mlo = co0 + half * 4;  // channel of reg i: mlo + 8*(i/4) + i%4
    float v0[16], v1[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      v0[i] = acc0[i] + bias_r[i];
      v1[i] = acc1[i] + bias_r[i];
    }
    if (a.out) {  // (null: the layers behind leave this kernel too and nobody reads the convolution's own output)
      float *o = a.out + pbase;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int m = mlo + (i >> 2) * 8 + (i & 3);
        if (ok0 && m < a.Kc) o[m * ohw] = v0[i];
        if (ok1 && m < a.Kc) o[m * ohw + a.OW] = v1[i];
      }
    }
    if (a.act_out) {
      act_apply16(a.act_kind, v0);
      act_apply16(a.act_kind, v1);
      float *o = a.act_out + pbase;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int m = mlo + (i >> 2) * 8 + (i & 3);
        if (ok0 && m < a.Kc) o[m * ohw] = v0[i];
        if (ok1 && m < a.Kc) o[m * ohw + a.OW] = v1[i];
      }
    }
    if (a.pool_out) {
      // the window of an even lane in scan order: its own value, its right neighbour's, and the
      // same two of the row below; every lane runs the exchange, even lanes keep the result
      int sel[16];
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float w4[4] = {v0[i], lane_xor1(v0[i]), v1[i], lane_xor1(v1[i])};
        float best = -FLT_MAX;
        sel[i]     = -1;
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (w4[j] > best) {
            best   = w4[j];
            sel[i] = j;
          }
        v0[i] = best;
      }
      const bool anchor = ok0 && !(nl & 1);
      const size_t pobase = static_cast<size_t>(img) * a.Kc * (POH * POW) + (oy >> 1) * POW + (ox >> 1);
      if (anchor) {
        float *o   = a.pool_out + pobase;
        int32_t *g = a.pool_argmax + pobase;
        const int pix = oy * a.OW + ox;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int m = mlo + (i >> 2) * 8 + (i & 3);
          if (m < a.Kc) {
            o[m * (POH * POW)] = v0[i];
            g[m * (POH * POW)] = sel[i] < 0 ? 0 : m * ohw + pix + (sel[i] >> 1) * a.OW + (sel[i] & 1);
          }
        }
      }
      if (a.pool_act_out) {
        act_apply16(a.pool_act_kind, v0);
        if (anchor) {
          float *o = a.pool_act_out + pobase;
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const int m = mlo + (i >> 2) * 8 + (i & 3);
            if (m < a.Kc) o[m * (POH * POW)] = v0[i];
          }
        }
      }
    }
  }
}

// The same tiles for a layer where nothing needs a guard or a choice per value: every band has
// whole row pairs, the width is a multiple of 32 columns, the channels a multiple of 32, there is
// no activation between convolution and pool, and the activation behind the pool is relu or
// none. These tiles are bound by the vector instructions around the MFMAs (about 25 per MFMA
// in the kernel above, guards, 64-bit addresses and saved exec masks most of them), so here
// everything that depends on the tile is kept in scalar registers (the wave index is read from
// the first lane for that), a lane adds one offset of its own that is computed once, and no
// store has a condition.
template <int NS>
__global__ void __launch_bounds__(256, 2) conv_fwd_small_full_kernel(const FwdSmallArgs a) {
  extern __shared__ __align__(16) float lds[];
  float *xs = lds;
  float *ws = lds + a.x_floats;
  float *bs = ws + 32 * a.crs;
  int *offs = reinterpret_cast<int *>(bs + 32);
  const int tid = threadIdx.x, lane = tid & 63;
  // (an image's bands share rows: they go to one XCD)
  const int wg = xcd_compact_id(blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z),
                                gridDim.x * gridDim.y * gridDim.z);
  const int bandi = wg % gridDim.x, img = (wg / gridDim.x) % gridDim.y, co0 = (wg / (gridDim.x * gridDim.y)) * 32;
  const int oy0 = bandi * a.band;
  const int nthr = blockDim.x;
  fwd_small_stage<NS>(a, xs, ws, bs, offs, img, co0, oy0, tid, nthr);
  __syncthreads();

  const int nl = lane & 31, half = lane >> 5;
  float areg[NS];
#pragma unroll
  for (int s = 0; s < NS; ++s) {
    const int k = 2 * s + half;
    areg[s]     = k < a.crs ? ws[nl * a.crs + k] : 0.0f;
  }
  // the patch offset of every k-step: the same for all tiles of the wave
  int o[NS];
#pragma unroll
  for (int s = 0; s < NS; ++s) o[s] = offs[2 * s + half];
  float bias_r[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) bias_r[i] = bs[(i >> 2) * 8 + half * 4 + (i & 3)];

  const uint32_t ohw = a.OH * a.OW, OW = a.OW, POW = a.OW >> 1, pohw = (a.OH >> 1) * POW;
  const uint32_t tiles = (a.band >> 1) * a.col_tiles;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6), nwaves = __builtin_amdgcn_readfirstlane(nthr >> 6);
  // the lane's own part of every address: its channel group and its column
  const uint32_t lane_out = half * 4 * ohw + nl, lane_pool = half * 4 * pohw + (nl >> 1);
  const bool even  = !(nl & 1);
  const bool pool  = a.pool_out != nullptr;
  const float floor_v = a.pool_act_kind == TDH_ACT_RELU ? 0.0f : -INFINITY;  // relu as a max
  float *out_img        = a.out + (static_cast<size_t>(img) * a.Kc + co0) * ohw;
  float *pool_img       = a.pool_out + (static_cast<size_t>(img) * a.Kc + co0) * pohw;
  float *pool_act_img   = a.pool_act_out + (static_cast<size_t>(img) * a.Kc + co0) * pohw;
  int32_t *argmax_img   = a.pool_argmax + (static_cast<size_t>(img) * a.Kc + co0) * pohw;
#pragma unroll 1
  for (uint32_t tile = wave; tile < tiles; tile += nwaves) {
    const uint32_t rp = a.div_col_tiles.div(tile), ct = tile - rp * a.col_tiles;
    const uint32_t r = 2 * rp, c0 = 32 * ct;
    const float *xb0 = xs + r * a.sh * a.pitch + (c0 + nl) * a.sw;
    const float *xb1 = xb0 + a.sh * a.pitch;
    floatx16 acc0, acc1;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc0[i] = acc1[i] = 0.0f;
    // The patch values of eight k-steps are read while the products of the eight before them
    // run: read and product one after the other would wait for LDS in every step.
    constexpr int G = 8;
    static_assert(NS % G == 0, "k-steps come in groups");
    float b0[2][G], b1[2][G];
    auto read_patch = [&](int g, int to) {
#pragma unroll
      for (int j = 0; j < G; ++j) {
        b0[to][j] = xb0[o[g * G + j]];
        b1[to][j] = xb1[o[g * G + j]];
      }
    };
    read_patch(0, 0);
#pragma unroll
    for (int g = 0; g < NS / G; ++g) {
      const int cur = g & 1;
      if (g + 1 < NS / G) read_patch(g + 1, cur ^ 1);
#pragma unroll
      for (int j = 0; j < G; ++j) {
        acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(areg[g * G + j], b0[cur][j], acc0, 0, 0, 0);
        acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(areg[g * G + j], b1[cur][j], acc1, 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);  // (the reads stay in front of the group they were written for)
    }
    // reg i of lane l holds channel 8*(i/4) + 4*(l/32) + i%4 at column l%32
    const uint32_t oy = oy0 + r;
    const uint32_t first = oy * OW + c0;  // of the tile inside a channel plane
    float v0[16], v1[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      v0[i] = acc0[i] + bias_r[i];
      v1[i] = acc1[i] + bias_r[i];
    }
    if (a.out) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        float *o = out_img + (((i >> 2) * 8 + (i & 3)) * ohw + first);  // scalar
        o[lane_out]        = v0[i];
        (o + OW)[lane_out] = v1[i];
      }
    }
    if (pool) {
      // as above: the window of an even lane in scan order, strict '>', start value lowest();
      // where: the winner's distance from the window's first element (0, 1, OW, OW + 1), -1 when
      // no value beat the start value
      const uint32_t pfirst = (oy >> 1) * POW + (c0 >> 1);
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float w4[4] = {v0[i], lane_xor1(v0[i]), v1[i], lane_xor1(v1[i])};
        const int at[4]   = {0, 1, static_cast<int>(OW), static_cast<int>(OW) + 1};
        float best = -FLT_MAX;
        int where  = -1;
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (w4[j] > best) {
            best  = w4[j];
            where = at[j];
          }
        const uint32_t ch     = (i >> 2) * 8 + (i & 3);
        const uint32_t chfirst = (co0 + ch) * ohw + first;  // scalar: flat CHW index of the tile's first element
        if (even) {
          (pool_img + (ch * pohw + pfirst))[lane_pool]   = best;
          (argmax_img + (ch * pohw + pfirst))[lane_pool] = where < 0 ? 0 : static_cast<int>(chfirst + lane_out) + where;
          if (a.pool_act_out) (pool_act_img + (ch * pohw + pfirst))[lane_pool] = best > floor_v ? best : floor_v;
        }
      }
    }
  }
}

struct FwdSmallPlan {
  FwdSmallArgs a;
  int ns;  // k-steps, rounded up to the next instantiated count
  size_t lds_bytes;
  dim3 grid;
  bool ok;
};

FwdSmallPlan make_fwd_small_plan(int batch, int C, int Kc, int H, int W, int OH, int OW, int R, int S,
                                 int sh, int sw, int dh, int dw, int ph, int pw) {
  FwdSmallPlan p;
  p.ok = false;
  FwdSmallArgs &a = p.a;
  a.x = a.w = a.bias = nullptr;
  a.out = a.act_out = a.pool_out = a.pool_act_out = nullptr;
  a.pool_argmax = nullptr;
  a.act_kind = a.pool_act_kind = TDH_ACT_NONE;
  a.C = C; a.Kc = Kc; a.H = H; a.W = W; a.OH = OH; a.OW = OW;
  a.R = R; a.S = S; a.sh = sh; a.sw = sw; a.dh = dh; a.dw = dw; a.ph = ph; a.pw = pw;
  a.crs = C * R * S;
  if (a.crs > 96 || batch < 1 || batch > 65535 || OH < 1 || OW < 1) return p;
  p.ns = ((a.crs + 1) / 2 + 7) / 8 * 8;
  a.col_tiles = ceil_div(OW, 32);
  a.pitch     = (a.col_tiles * 32 - 1) * sw + (S - 1) * dw + 1;
  a.pitch |= 1;
  const int co_tiles = ceil_div(Kc, 32);
  if (co_tiles > 65535) return p;
  const int cus  = ctx().compute_units > 0 ? ctx().compute_units : 256;
  const int OH2  = (OH + 1) & ~1;
  auto lds_floats = [&](int band) {
    const int rows_in = (band - 1) * sh + (R - 1) * dh + 1;
    const size_t x_fl = (static_cast<size_t>(C) * (rows_in * a.pitch + 1) + 3) & ~static_cast<size_t>(3);
    return x_fl + 32u * a.crs + 32u + 96u;
  };
  // an even band: the largest that fits and still gives two workgroups per compute unit; never
  // fewer than four tiles (one per wave) for that
  int best = 0;
  for (int band = OH2; band >= 2; band -= 2) {
    if (lds_floats(band) * sizeof(float) > 64 * 1024) continue;
    best = band;
    if (static_cast<long long>(batch) * ceil_div(OH, band) * co_tiles >= 4LL * cus ||
        (band / 2) * a.col_tiles <= 4)
      break;
  }
  if (best == 0) return p;
  // (the same number of bands, the rows spread evenly over them)
  best      = std::min(best, (ceil_div(OH2, ceil_div(OH2, best)) + 1) & ~1);
  a.band    = best;
  a.bands   = ceil_div(OH, best);
  a.rows_in = (best - 1) * sh + (R - 1) * dh + 1;
  a.plane   = a.rows_in * a.pitch + 1;
  a.x_floats = static_cast<int>((static_cast<size_t>(C) * a.plane + 3) & ~static_cast<size_t>(3));
  a.div_pitch     = FastDiv(a.pitch);
  a.div_rows_in   = FastDiv(a.rows_in);
  a.div_col_tiles = FastDiv(a.col_tiles);
  p.lds_bytes = lds_floats(best) * sizeof(float);
  p.grid      = dim3(a.bands, batch, co_tiles);
  p.ok        = true;
  return p;
}

template <int NS>
int launch_fwd_small(const FwdSmallPlan &p) {
  const int tiles = (p.a.band / 2) * p.a.col_tiles;
  const FwdSmallArgs &a = p.a;
  const bool full = a.OH % a.band == 0 && a.band % 2 == 0 && a.OW % 32 == 0 && a.Kc % 32 == 0 && !a.act_out &&
                    (a.pool_act_kind == TDH_ACT_RELU || a.pool_act_kind == TDH_ACT_NONE || !a.pool_act_out) &&
                    static_cast<long long>(a.Kc) * a.OH * a.OW < (1LL << 30);
  if (full) {
    TDH_LAUNCH((conv_fwd_small_full_kernel<NS>), p.grid, dim3(64 * std::min(4, std::max(2, tiles))), p.lds_bytes,
               ctx().stream, p.a);
    TDH_LAUNCH_CHECK();
    return TDH_OK;
  }
  TDH_LAUNCH((conv_fwd_small_kernel<NS>), p.grid, dim3(64 * std::min(4, std::max(2, tiles))), p.lds_bytes,
             ctx().stream, p.a);
  TDH_LAUNCH_CHECK();
  return TDH_OK;
}

}  // namespace

bool conv_fwd_small_applicable(int batch, int C, int Kc, int H, int W, int OH, int OW, int R, int S,
                               int sh, int sw, int dh, int dw, int ph, int pw) {
  return make_fwd_small_plan(batch, C, Kc, H, W, OH, OW, R, S, sh, sw, dh, dw, ph, pw).ok;
}

int conv_fwd_small_run(int batch, int C, int Kc, const float *x, const float *w, const float *bias,
                       float *out, int H, int W, int OH, int OW, int R, int S, int sh, int sw, int dh,
                       int dw, int ph, int pw, float *act_out, int act_kind, const PoolFuse *pool) {
  FwdSmallPlan p = make_fwd_small_plan(batch, C, Kc, H, W, OH, OW, R, S, sh, sw, dh, dw, ph, pw);
  if (!p.ok) return set_error(TDH_ERR_INVALID, "conv_fwd_small_run: shape not supported");
  if (pool && ((OH | OW) & 1))
    return set_error(TDH_ERR_INVALID, "conv_fwd_small_run: a fused 2x2 pool needs even output sizes");
  if (!out && !pool && !act_out) return set_error(TDH_ERR_INVALID, "conv_fwd_small_run: no output");
  p.a.x = x; p.a.w = w; p.a.bias = bias; p.a.out = out;
  p.a.act_out  = act_out;
  p.a.act_kind = act_kind;
  if (pool) {
    p.a.pool_out      = pool->out;
    p.a.pool_argmax   = pool->argmax;
    p.a.pool_act_out  = pool->act_out;
    p.a.pool_act_kind = pool->act_kind;
  }
  ProfScope prof(pool ? "conv_fwd_small_pool" : "conv_fwd_small", Kc, batch * OH * OW, p.a.crs);
  switch (p.ns) {
    case 8: return launch_fwd_small<8>(p);
    case 16: return launch_fwd_small<16>(p);
    case 24: return launch_fwd_small<24>(p);
    case 32: return launch_fwd_small<32>(p);
    case 40: return launch_fwd_small<40>(p);
    default: return launch_fwd_small<48>(p);
  }
}

}  // namespace tdh
