// conv.hip — 2-D convolution forward and backward as implicit GEMMs (no im2col / col2im
// buffer is ever materialised and padding::same costs no copies):
//
//   forward  Y[img][co][p]      M = Cout        N = batch*OH*OW   K = Cin*KH*KW
//            A = W (OIHW rows), B = input gathered at (p, tap)
//   dW       dW[co][ci,ky,kx]   M = Cout        N = Cin*KH*KW     K = batch*OH*OW
//            A = dY, B = input gathered at (p, tap); K spans the whole batch, so the
//            gradient leaves the kernel already reduced over samples
//   dX       dX[img][ci][q]     M = Cin         N = batch*H*W     K = Cout*KH*KW
//            A = W regrouped by input channel, B = dY gathered at the output positions
//            whose window covers q (the gather form of the reference's scatter)
//   db       row sums of dY per output channel, fixed two-stage order
//
// Reference: conv2d_op_internal.h:13-74 (forward), :78-181 (backward).
#include <algorithm>
#include <vector>

#include "gemm_mfma.h"

namespace tdh {

namespace {

struct ConvGeom {
  int C, H, W, Kc, R, S, OH, OW;
  int pad_h, pad_w, sh, sw, dh, dw;
  FastDiv div_ohw, div_ow, div_rs, div_s, div_hw, div_w, div_sh, div_sw;
};

ConvGeom make_geom(const tdh_conv_desc *d) {
  ConvGeom g;
  g.C = d->in_c; g.H = d->in_h; g.W = d->in_w;
  g.Kc = d->out_c; g.R = d->k_h; g.S = d->k_w;
  g.OW = conv_out_length(d->in_w, d->k_w, d->w_stride, d->w_dilation, d->pad_same);
  g.OH = conv_out_length(d->in_h, d->k_h, d->h_stride, d->h_dilation, d->pad_same);
  // padding::same puts k/2 zeros before the data (conv_params.h:119-120)
  g.pad_h = d->pad_same ? d->k_h / 2 : 0;
  g.pad_w = d->pad_same ? d->k_w / 2 : 0;
  g.sh = d->h_stride; g.sw = d->w_stride; g.dh = d->h_dilation; g.dw = d->w_dilation;
  g.div_ohw = FastDiv(g.OH * g.OW); g.div_ow = FastDiv(g.OW);
  g.div_rs = FastDiv(g.R * g.S); g.div_s = FastDiv(g.S);
  g.div_hw = FastDiv(g.H * g.W); g.div_w = FastDiv(g.W);
  g.div_sh = FastDiv(g.sh); g.div_sw = FastDiv(g.sw);
  return g;
}

// forward B operand: n = (img, oy, ox), k = (ci, ky, kx) -> x[img][ci][oy*sh + ky*dh - pad][..]
struct FwdInputOperand {
  const float *x;
  ConvGeom g;
  int n_extent;
  struct Fix {
    int base, iy0, ix0;
    bool valid;
  };
  struct KDec {
    int coff, dy, dx;
  };
  __device__ __forceinline__ Fix fix(int n) const {
    uint32_t img, p, oy, ox;
    g.div_ohw.divmod(n, img, p);
    g.div_ow.divmod(p, oy, ox);
    return {static_cast<int>(img) * g.C * g.H * g.W, static_cast<int>(oy) * g.sh - g.pad_h,
            static_cast<int>(ox) * g.sw - g.pad_w, n < n_extent};
  }
  __device__ __forceinline__ KDec kdec(int k) const {
    uint32_t ci, t, ky, kx;
    g.div_rs.divmod(k, ci, t);
    g.div_s.divmod(t, ky, kx);
    return {static_cast<int>(ci) * g.H * g.W, static_cast<int>(ky) * g.dh,
            static_cast<int>(kx) * g.dw};
  }
  __device__ __forceinline__ float load(const Fix &f, const KDec &k) const {
    const int iy = f.iy0 + k.dy, ix = f.ix0 + k.dx;
    const bool ok = f.valid && static_cast<unsigned>(iy) < static_cast<unsigned>(g.H) &&
                    static_cast<unsigned>(ix) < static_cast<unsigned>(g.W);
    return ok ? x[f.base + k.coff + iy * g.W + ix] : 0.0f;
  }
};

// dW A operand: m = co, k = (img, p) -> dy[img][co][p]
struct DwDyOperand {
  const float *dy;
  int Kc, ohw;
  FastDiv div_ohw;
  struct Fix {
    int off;
    bool valid;
  };
  struct KDec {
    int off;
  };
  __device__ __forceinline__ Fix fix(int m) const { return {m * ohw, m < Kc}; }
  __device__ __forceinline__ KDec kdec(int k) const {
    uint32_t img, p;
    div_ohw.divmod(k, img, p);
    return {static_cast<int>(img) * Kc * ohw + static_cast<int>(p)};
  }
  __device__ __forceinline__ float load(const Fix &f, const KDec &k) const {
    return f.valid ? dy[f.off + k.off] : 0.0f;
  }
};

// dW B operand: n = (ci, ky, kx), k = (img, oy, ox) -> x[img][ci][oy*sh + ky - pad][..]
struct DwInputOperand {
  const float *x;
  ConvGeom g;
  int n_extent;
  struct Fix {
    int coff, dy, dx;
    bool valid;
  };
  struct KDec {
    int base, iy0, ix0;
  };
  __device__ __forceinline__ Fix fix(int n) const {
    uint32_t ci, t, ky, kx;
    g.div_rs.divmod(n, ci, t);
    g.div_s.divmod(t, ky, kx);
    return {static_cast<int>(ci) * g.H * g.W, static_cast<int>(ky) - g.pad_h,
            static_cast<int>(kx) - g.pad_w, n < n_extent};
  }
  __device__ __forceinline__ KDec kdec(int k) const {
    uint32_t img, p, oy, ox;
    g.div_ohw.divmod(k, img, p);
    g.div_ow.divmod(p, oy, ox);
    return {static_cast<int>(img) * g.C * g.H * g.W, static_cast<int>(oy) * g.sh,
            static_cast<int>(ox) * g.sw};
  }
  __device__ __forceinline__ float load(const Fix &f, const KDec &k) const {
    const int iy = k.iy0 + f.dy, ix = k.ix0 + f.dx;
    const bool ok = f.valid && static_cast<unsigned>(iy) < static_cast<unsigned>(g.H) &&
                    static_cast<unsigned>(ix) < static_cast<unsigned>(g.W);
    return ok ? x[k.base + f.coff + iy * g.W + ix] : 0.0f;
  }
};

// dX A operand: m = ci, k = (co, ky, kx) -> w[co][ci][ky][kx]
struct DxWeightOperand {
  const float *w;
  int C, rs;
  FastDiv div_rs;
  struct Fix {
    int off;
    bool valid;
  };
  struct KDec {
    int off;
  };
  __device__ __forceinline__ Fix fix(int m) const { return {m * rs, m < C}; }
  __device__ __forceinline__ KDec kdec(int k) const {
    uint32_t co, t;
    div_rs.divmod(k, co, t);
    return {static_cast<int>(co) * C * rs + static_cast<int>(t)};
  }
  __device__ __forceinline__ float load(const Fix &f, const KDec &k) const {
    return f.valid ? w[f.off + k.off] : 0.0f;
  }
};

// dX B operand: n = (img, iy, ix), k = (co, ky, kx) -> dy[img][co][oy][ox] where
// oy*sh + ky = iy + pad (and likewise in x); zero when no such output exists
struct DxDyOperand {
  const float *dy;
  ConvGeom g;
  int n_extent;
  struct Fix {
    int base, ty, tx;
    bool valid;
  };
  struct KDec {
    int coff, ky, kx;
  };
  __device__ __forceinline__ Fix fix(int n) const {
    uint32_t img, q, iy, ix;
    g.div_hw.divmod(n, img, q);
    g.div_w.divmod(q, iy, ix);
    return {static_cast<int>(img) * g.Kc * g.OH * g.OW, static_cast<int>(iy) + g.pad_h,
            static_cast<int>(ix) + g.pad_w, n < n_extent};
  }
  __device__ __forceinline__ KDec kdec(int k) const {
    uint32_t co, t, ky, kx;
    g.div_rs.divmod(k, co, t);
    g.div_s.divmod(t, ky, kx);
    return {static_cast<int>(co) * g.OH * g.OW, static_cast<int>(ky), static_cast<int>(kx)};
  }
  __device__ __forceinline__ float load(const Fix &f, const KDec &k) const {
    const int uy = f.ty - k.ky, ux = f.tx - k.kx;
    if (!f.valid || uy < 0 || ux < 0) return 0.0f;
    uint32_t oy = uy, ox = ux;
    if (g.sh != 1 || g.sw != 1) {
      uint32_t ry, rx;
      g.div_sh.divmod(uy, oy, ry);
      g.div_sw.divmod(ux, ox, rx);
      if (ry != 0 || rx != 0) return 0.0f;
    }
    if (oy >= static_cast<uint32_t>(g.OH) || ox >= static_cast<uint32_t>(g.OW)) return 0.0f;
    return dy[f.base + k.coff + static_cast<int>(oy) * g.OW + static_cast<int>(ox)];
  }
};

// connection_table support: w_masked[i] = w[i] * tbl[ci][co]; dw (+)= tmp * tbl
__global__ void __launch_bounds__(256)
mask_weights_kernel(const float *__restrict__ src, const uint8_t *__restrict__ tbl,
                    float *__restrict__ dst, const int n, const int C, const int Kc, const int rs,
                    const int accumulate) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const int pair = i / rs;  // co*C + ci
  const int co = pair / C, ci = pair - co * C;
  const float v = tbl[ci * Kc + co] ? src[i] : 0.0f;
  dst[i]        = accumulate ? dst[i] + v : v;
}

// dX for convolutions with very few input channels (the first layer of an image network:
// M = Cin = 1..4 would leave 7/8 of every 32-row MFMA block empty). Direct form on the vector
// ALUs, stride 1. A workgroup of four waves owns a band of input rows of one image: lane l of
// EVERY wave owns the same DXS_PX adjacent pixels of the band, and the waves split the output
// channels between them (the pixels alone would not fill the chip), so the four partial sums
// are added through LDS at the end, always in wave order. dY rows that can reach the band are
// staged in LDS (zero halo) DXS_CO_CHUNK channels at a time, the next chunk travelling in
// registers while the current one is used; a lane reads its 4+S-1 tile values of a filter row
// as 16-byte words and reuses them for all S taps and Cin channels.
constexpr int DXS_MAX_CIN  = 4;
constexpr int DXS_WAVES    = 4;
constexpr int DXS_CPW      = 2;                      // output channels per wave in a chunk
constexpr int DXS_CO_CHUNK = DXS_WAVES * DXS_CPW;
constexpr int DXS_PX       = 4;                      // adjacent pixels per lane
constexpr int DXS_NT       = 64 * DXS_WAVES;
constexpr int DXS_MAX_STAGE = 20;                    // staged tile elements per thread and chunk
constexpr int DXS_MAX_PSTAGE = 8;                    // POOLED: staged pool windows per thread and chunk

struct DxsPlan {
  int tile_rows, bands, gw, trows, tcols;  // gw: pixel groups per row; tile = [trows][tcols]
  FastDiv div_gw, div_tcols, div_tile;
  size_t lds_bytes;
  // POOLED: the 2x2 pool windows that can touch a tile, [pnr][pnc] per channel
  int pnr, pnc;
  FastDiv div_pnc, div_ptile;
  bool pooled_ok;
};

// KR, KS: compile-time window (0 = use the run-time g.R, g.S); CIN: input channels computed.
// POOLED: dY is not in memory but given through the 2x2 / stride-2 max-pool behind the layer.
// A thread stages pool windows instead of tile elements: one gradient and one argmax record per
// window, and writes the window's four elements into the tile (the gradient where the record
// names the element, else zero; windows outside the image give the zero halo).
template <int KR, int KS, int CIN, bool POOLED>
__global__ void __launch_bounds__(DXS_NT)
conv_dx_small_cin_kernel(const float *__restrict__ dy, const float *__restrict__ w,
                         float *__restrict__ dx, const ConvGeom g, const DxsPlan p,
                         const ActGrad ag, const PoolGather pooled) {
  extern __shared__ __align__(16) float smem[];
  const int R = KR ? KR : g.R, S = KS ? KS : g.S;
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int wg  = xcd_compact_id(blockIdx.x, gridDim.x);  // (an image's bands share rows: one XCD)
  const int img = wg / p.bands;
  const int y0  = (wg - img * p.bands) * p.tile_rows;
  const int tsz = p.trows * p.tcols, rs = R * S;
  const int oy0 = y0 + g.pad_h - (R - 1), ox0 = g.pad_w - (S - 1);
  const int ohw = g.OH * g.OW;
  const int pow_ = g.OW >> 1, pohw = (g.OH >> 1) * pow_;
  const float *dy_img = POOLED ? pooled.g + static_cast<size_t>(img) * g.Kc * pohw
                               : dy + static_cast<size_t>(img) * g.Kc * ohw;
  const int32_t *rec_img = POOLED ? pooled.argmax + static_cast<size_t>(img) * g.Kc * pohw : nullptr;
  float *tile = smem;                                                  // [DXS_CO_CHUNK][tsz]
  float4 *wl  = reinterpret_cast<float4 *>(smem + DXS_CO_CHUNK * tsz);  // [DXS_CO_CHUNK][rs]

  // this lane's pixels: row prow of the band, columns 4*grp .. 4*grp+3
  uint32_t prow, grp;
  p.div_gw.divmod(lane, prow, grp);
  const bool lane_live = static_cast<int>(prow) < p.tile_rows;
  const int toff       = lane_live ? prow * p.tcols + 4 * grp : 0;

  float acc[CIN][DXS_PX];
#pragma unroll
  for (int c = 0; c < CIN; ++c)
#pragma unroll
    for (int i = 0; i < DXS_PX; ++i) acc[c][i] = 0.0f;

  // staging plan, the same for every chunk: element e = tid + DXS_NT*j of the chunk tile ->
  // channel inside the chunk and offset inside that channel's plane (-1: outside the image)
  constexpr int NS = POOLED ? 1 : DXS_MAX_STAGE, NP = POOLED ? DXS_MAX_PSTAGE : 1;
  float stage[NS];
  int soff[NS], sch[NS];
  if (!POOLED) {
#pragma unroll
    for (int j = 0; j < NS; ++j) {
      const uint32_t e = tid + DXS_NT * j;
      uint32_t c, rem, r, q;
      p.div_tile.divmod(e, c, rem);
      p.div_tcols.divmod(rem, r, q);
      const int oy = oy0 + static_cast<int>(r), ox = ox0 + static_cast<int>(q);
      const bool in = static_cast<unsigned>(oy) < static_cast<unsigned>(g.OH) &&
                      static_cast<unsigned>(ox) < static_cast<unsigned>(g.OW);
      sch[j]  = static_cast<int>(c);
      soff[j] = in ? static_cast<int>(c) * ohw + oy * g.OW + ox : -1;
    }
  }
  // POOLED: window e = tid + DXS_NT*j of the chunk -> offset in the pooled planes (-1: outside
  // the image), flat index of its top left element inside the channel, its channel, and where
  // its four elements lie in LDS (those outside the tile: a word behind the weights that
  // nobody reads, so that the stores need no branches)
  float pgrad[NP];
  int poff[NP], pflat[NP], pch[NP], prec[NP], pat[NP][4];
  const int nowhere = DXS_CO_CHUNK * tsz + 4 * DXS_CO_CHUNK * rs;
  if (POOLED) {
    const int pr0 = oy0 >> 1, pc0 = ox0 >> 1;  // (floor: the tile may start outside the image)
#pragma unroll
    for (int j = 0; j < NP; ++j) {
      const uint32_t e = tid + DXS_NT * j;
      uint32_t c, rem, i, k;
      p.div_ptile.divmod(e, c, rem);
      p.div_pnc.divmod(rem, i, k);
      const int pr = pr0 + static_cast<int>(i), pc = pc0 + static_cast<int>(k);
      const bool live = c < static_cast<uint32_t>(DXS_CO_CHUNK);
      const bool in = live && static_cast<unsigned>(pr) < static_cast<unsigned>(g.OH >> 1) &&
                      static_cast<unsigned>(pc) < static_cast<unsigned>(pow_);
      const int r0 = 2 * pr - oy0, q0 = 2 * pc - ox0;  // tile position of the top left element
      const bool ra = static_cast<unsigned>(r0) < static_cast<unsigned>(p.trows),
                 rb = static_cast<unsigned>(r0 + 1) < static_cast<unsigned>(p.trows),
                 qa = static_cast<unsigned>(q0) < static_cast<unsigned>(p.tcols),
                 qb = static_cast<unsigned>(q0 + 1) < static_cast<unsigned>(p.tcols);
      poff[j]  = in ? static_cast<int>(c) * pohw + pr * pow_ + pc : -1;
      pflat[j] = static_cast<int>(c) * ohw + 2 * pr * g.OW + 2 * pc;
      pch[j]   = static_cast<int>(c);
      const int at = static_cast<int>(c) * tsz + r0 * p.tcols + q0;
      pat[j][0] = live && ra && qa ? at : nowhere;
      pat[j][1] = live && ra && qb ? at + 1 : nowhere;
      pat[j][2] = live && rb && qa ? at + p.tcols : nowhere;
      pat[j][3] = live && rb && qb ? at + p.tcols + 1 : nowhere;
    }
  }
  // The chunk's weights as [c][tap] -> (w[ci=0..3]), taps flipped so that the inner loops walk
  // the tile forwards. The first two per thread travel with the tile (512 cover 8 channels of
  // up to 8x8 taps); loaded behind the barrier they would cost a trip to memory per chunk.
  float4 wreg[2];
  auto load_w = [&](int co0, int e) {
    const int c = e / rs, t = e - c * rs;
    const float *wc = w + (static_cast<size_t>(co0 + c) * g.C) * rs + (rs - 1 - t);
    float4 v;
    v.x = wc[0];
    v.y = g.C > 1 ? wc[rs] : 0.0f;
    v.z = g.C > 2 ? wc[2 * rs] : 0.0f;
    v.w = g.C > 3 ? wc[3 * rs] : 0.0f;
    return v;
  };
  auto fetch = [&](int co0) {
    const int nco     = min(DXS_CO_CHUNK, g.Kc - co0);
    const float *base = dy_img + co0 * (POOLED ? pohw : ohw);
    if (POOLED) {
#pragma unroll
      for (int j = 0; j < NP; ++j) {
        const bool live = poff[j] >= 0 && pch[j] < nco;
        pgrad[j] = live ? base[poff[j]] : 0.0f;
        // the record minus the flat index of the window's top left element: 0, 1, OW or OW+1
        prec[j] = live ? rec_img[co0 * pohw + poff[j]] - (co0 * ohw + pflat[j]) : -1;
      }
    } else {
#pragma unroll
      for (int j = 0; j < NS; ++j)
        stage[j] = (soff[j] >= 0 && sch[j] < nco) ? base[soff[j]] : 0.0f;
    }
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const int e = tid + DXS_NT * k;
      wreg[k]     = e < nco * rs ? load_w(co0, e) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
  };

  fetch(0);
  for (int co0 = 0; co0 < g.Kc; co0 += DXS_CO_CHUNK) {
    const int nco = min(DXS_CO_CHUNK, g.Kc - co0);
    __syncthreads();  // the previous chunk has been consumed
    if (POOLED) {
#pragma unroll
      for (int j = 0; j < NP; ++j) {
        smem[pat[j][0]] = prec[j] == 0 ? pgrad[j] : 0.0f;
        smem[pat[j][1]] = prec[j] == 1 ? pgrad[j] : 0.0f;
        smem[pat[j][2]] = prec[j] == g.OW ? pgrad[j] : 0.0f;
        smem[pat[j][3]] = prec[j] == g.OW + 1 ? pgrad[j] : 0.0f;
      }
    } else {
#pragma unroll
      for (int j = 0; j < NS; ++j) {
        const int e = tid + DXS_NT * j;
        if (e < DXS_CO_CHUNK * tsz) tile[e] = stage[j];
      }
    }
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const int e = tid + DXS_NT * k;
      if (e < nco * rs) wl[e] = wreg[k];
    }
    for (int e = tid + 2 * DXS_NT; e < nco * rs; e += DXS_NT) wl[e] = load_w(co0, e);  // larger windows
    __syncthreads();
    if (co0 + DXS_CO_CHUNK < g.Kc) fetch(co0 + DXS_CO_CHUNK);  // in flight during the math

#pragma unroll
    for (int cc = 0; cc < DXS_CPW; ++cc) {
      const int c = wv * DXS_CPW + cc;
      if (c >= nco) break;
      const float *t   = tile + c * tsz + toff;
      const float4 *wc = wl + c * rs;
      if (KR != 0) {
        constexpr int NV = (DXS_PX + (KS ? KS : 1) - 1 + 3) / 4;  // 16-byte words per filter row
#pragma unroll
        for (int fy = 0; fy < KR; ++fy) {
          float v[4 * NV];
#pragma unroll
          for (int q = 0; q < NV; ++q) {
            const float4 f = *reinterpret_cast<const float4 *>(t + fy * p.tcols + 4 * q);
            v[4 * q] = f.x; v[4 * q + 1] = f.y; v[4 * q + 2] = f.z; v[4 * q + 3] = f.w;
          }
#pragma unroll
          for (int fx = 0; fx < KS; ++fx) {
            const float4 wq  = wc[fy * KS + fx];
            const float wa[4] = {wq.x, wq.y, wq.z, wq.w};
#pragma unroll
            for (int ci = 0; ci < CIN; ++ci)
#pragma unroll
              for (int i = 0; i < DXS_PX; ++i) acc[ci][i] += wa[ci] * v[i + fx];
          }
        }
      } else {
        for (int fy = 0; fy < R; ++fy)
          for (int fx = 0; fx < S; ++fx) {
            const float4 wq  = wc[fy * S + fx];
            const float wa[4] = {wq.x, wq.y, wq.z, wq.w};
#pragma unroll
            for (int i = 0; i < DXS_PX; ++i) {
              const float v = t[fy * p.tcols + fx + i];
#pragma unroll
              for (int ci = 0; ci < CIN; ++ci) acc[ci][i] += wa[ci] * v;
            }
          }
      }
    }
  }

  // partial sums of the four waves -> red[wave][ci][lane*4 + i], then one fixed-order add
  __syncthreads();
  float *red = smem;
#pragma unroll
  for (int ci = 0; ci < CIN; ++ci)
    *reinterpret_cast<float4 *>(red + (wv * CIN + ci) * (64 * DXS_PX) + lane * DXS_PX) =
      make_float4(acc[ci][0], acc[ci][1], acc[ci][2], acc[ci][3]);
  __syncthreads();
  {
    uint32_t orow, ogrp;
    p.div_gw.divmod(tid >> 2, orow, ogrp);  // tid = lane*4 + i of the pixel it finishes
    const int y = y0 + static_cast<int>(orow), x = 4 * static_cast<int>(ogrp) + (tid & 3);
    if (static_cast<int>(orow) < p.tile_rows && y < g.H && x < g.W) {
      const size_t img_off = static_cast<size_t>(img) * g.C * g.H * g.W;
#pragma unroll
      for (int ci = 0; ci < CIN; ++ci) {
        if (ci >= g.C) break;
        float v = red[ci * (64 * DXS_PX) + tid];
#pragma unroll
        for (int k = 1; k < DXS_WAVES; ++k) v += red[(k * CIN + ci) * (64 * DXS_PX) + tid];
        const size_t idx = img_off + (static_cast<size_t>(ci) * g.H + y) * g.W + x;
        if (ag.kind != TDH_ACT_NONE) v *= act_grad_factor(ag.kind, ag.y[idx]);
        dx[idx] = v;
      }
    }
  }
}

// dX of a first convolution (stride 1, 3x3 or 5x5, Cin*S <= 16, rows of 16, 32 or 64 outputs)
// on the matrix cores, in two steps. For an input row y,
//   D[c][(ci,fx)] = sum over (co, fy) of dY[co][y + pad - (R-1) + fy][c] * wflip[co][ci][fy][fx]
// is a product with the dY columns c as rows (blocks of 16), Cin*S <= 16 columns and the output
// channels x filter rows as the reduction (v_mfma_f32_16x16x4_f32: the A operand is one LDS
// read of the staged rows of dY, which need no halo columns, the B operand one LDS read per
// step and eight channels), and
//   dX[ci][y][x] = sum over fx of D[x + fx + pad - (S-1)][(ci,fx)]
// is gathered out of LDS at the end, added in filter-column order. A workgroup owns a band of
// rows of one image and stages 32 output channels of it at once; its four waves split the rows,
// so nothing is added across waves. Every thread stages one position (a pool window, or four
// adjacent elements) of up to 16 channels with all loads in flight together.
//
// The geometry is a template argument (NMB blocks of 16 columns in a row, so 16/NMB rows a
// band): every LDS offset of the product loop is then an immediate of its instruction. With
// run-time offsets the loop took 7 us instead of 2: forty address additions per eight
// channels, branches around reads that a condition guarded, and accumulators moved between
// register files. Nothing that is loaded stands under a condition either: a load under a
// condition becomes a branch with a wait behind it (sixteen trips to memory one after the
// other, 6.5 us); what must not be used is read from a valid place and dropped when stored.
constexpr int DXM_NT    = 256;
constexpr int DXM_WAVES = 4;
constexpr int DXM_MCH   = 32;  // output channels staged at a time
constexpr int DXM_MAXCH = 16;  // channels a thread stages (of DXM_MCH)
constexpr int DXM_WREG  = 13;  // filter values a thread stages per chunk (32 channels x 4 x 25 / 256)

// The weight (and bias) gradient of the same layer out of the same launch (DWNT > 0: the
// number of 32-column blocks of its product, Cin*KH*KW + 1 columns, the last one the bias):
//   dW[co][(ci,ky,kx)] = sum over the band's output positions of dY[co][p] * X[ci][p + (ky,kx)]
// reads the staged rows of dY a second time, as the A operand of v_mfma_f32_32x32x2_f32 (lane =
// (output channel, one of two positions)), and the input patch under the band, staged next to
// them, as B (one LDS read at patch[position] + offset(column), the offset a per-lane
// constant). The four waves split the band's positions, their sums meet in LDS and the
// workgroup writes one slice [band][co][column] that a split reduction adds to the others.
// Reference: conv2d_op_internal.h:127-180.
struct FirstDwArgs {
  const float *x;
  float *partial_dw, *partial_db;  // [bands of the batch][Kc][crs], [..][Kc] (or null)
  int pitch, plane, rows_in;       // the staged patch: floats per row (odd) and channel, rows
  int x_total;                     // its elements
  FastDiv div_pitch, div_rows_in;
};

template <int KR, int NMB, bool POOLED>
struct DxmGeom {
  static constexpr int OW        = 16 * NMB;
  static constexpr int RPW       = 4 / NMB;            // rows of the band a wave owns
  static constexpr int TILE_ROWS = DXM_WAVES * RPW;
  static constexpr int TROWS     = TILE_ROWS + KR - 1;
  // floats per staged channel: the rows, a spare word for stores that fall outside the tile,
  // padded to 16 (mod 32) so that four channels' rows lie in different banks
  static constexpr int PLANE   = ((TROWS * OW + 1 + 15) / 32) * 32 + 16;
  static constexpr int PER_ROW = POOLED ? OW / 2 : OW / 4;  // staging positions per row of them
  static constexpr int NPOS    = (POOLED ? TROWS / 2 + 1 : TROWS) * PER_ROW;
  static constexpr int GROUPS  = DXM_NT / NPOS;
  static constexpr int CPT     = (DXM_MCH + GROUPS - 1) / GROUPS;  // channels per thread
  static constexpr int WROW    = 4 * KR * KR;          // staged filter floats per output channel
  static constexpr int WL      = DXM_MCH * WROW;
  static constexpr int GATHER  = DXM_WAVES * RPW * OW * 17;
  static constexpr int STAGE   = DXM_MCH * PLANE + WL;
  static constexpr int LDS_FLOATS = STAGE > GATHER ? STAGE : GATHER;
  static constexpr bool FITS = GROUPS >= 1 && CPT <= DXM_MAXCH && LDS_FLOATS * 4 <= 64 * 1024;
};

template <int KR, int KS, int NMB, bool POOLED, int DWNT = 0>
__global__ void __launch_bounds__(DXM_NT, DWNT > 0 ? 2 : 1)
conv_dx_first_mfma_kernel(const float *__restrict__ dy, const float *__restrict__ w, float *__restrict__ dx,
                          const ConvGeom g, const ActGrad ag, const PoolGather pooled, const FirstDwArgs dwa) {
  using G = DxmGeom<KR, NMB, POOLED>;
  extern __shared__ __align__(16) float smem[];
  typedef float f4 __attribute__((ext_vector_type(4)));
  typedef float f16 __attribute__((ext_vector_type(16)));
  constexpr int RS = KR * KS, NJ = 2 * KR;  // step j: filter row j/2, channels 4*(j%2) + (0..3) of eight
  constexpr int OW = G::OW, PLANE = G::PLANE;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int mr = lane & 15, mq = lane >> 4;
  const int bands = (g.H + G::TILE_ROWS - 1) / G::TILE_ROWS;
  const int wg  = xcd_compact_id(blockIdx.x, gridDim.x);  // (an image's bands share rows: one XCD)
  const int img = wg / bands;
  const int y0  = (wg - img * bands) * G::TILE_ROWS;
  const int oy0 = y0 + g.pad_h - (KR - 1), ox0 = g.pad_w - (KS - 1);
  const int ohw = g.OH * OW, pohw = (g.OH >> 1) * (OW / 2);
  float *wl = smem + DXM_MCH * PLANE;  // the chunk's filters [co][ci (4)][tap]

  // ---- this thread's staging position: the same for every channel it stages
  const int grp = tid / G::NPOS, pos = tid - grp * G::NPOS;
  const int pi = pos / G::PER_ROW, pk = pos - pi * G::PER_ROW;
  const bool stager = grp < G::GROUPS;
  int src = -1;   // offset inside a channel's plane in memory, or -1
  int flat = 0;   // POOLED: flat index of the window's top left element
  int at[4] = {PLANE - 1, PLANE - 1, PLANE - 1, PLANE - 1};  // offsets inside a staged plane
  if (POOLED) {
    const int pr = (oy0 >> 1) + pi;  // (floor: the band's tile may start above the image)
    if (stager && static_cast<unsigned>(pr) < static_cast<unsigned>(g.OH >> 1)) src = pr * (OW / 2) + pk;
    flat = 2 * pr * OW + 2 * pk;
    const int r0 = 2 * pr - oy0;
    if (static_cast<unsigned>(r0) < static_cast<unsigned>(G::TROWS)) {
      at[0] = r0 * OW + 2 * pk;
      at[1] = at[0] + 1;
    }
    if (static_cast<unsigned>(r0 + 1) < static_cast<unsigned>(G::TROWS)) {
      at[2] = (r0 + 1) * OW + 2 * pk;
      at[3] = at[2] + 1;
    }
  } else {
    const int oy = oy0 + pi;
    if (stager && static_cast<unsigned>(oy) < static_cast<unsigned>(g.OH)) src = oy * OW + 4 * pk;
    at[0] = pi * OW + 4 * pk;
  }
  const float *dy_img = POOLED ? pooled.g + static_cast<size_t>(img) * g.Kc * pohw
                               : dy + static_cast<size_t>(img) * g.Kc * ohw;
  const int32_t *rec_img = POOLED ? pooled.argmax + static_cast<size_t>(img) * g.Kc * pohw : nullptr;
  const int chan = POOLED ? pohw : ohw;  // floats per channel in memory

  // ---- block b of this wave: row wv*RPW + b/NMB of the band, columns 16*(b%NMB)..+15
  f4 dacc[4];
#pragma unroll
  for (int b = 0; b < 4; ++b) dacc[b] = f4{0.0f, 0.0f, 0.0f, 0.0f};
  // B column of this lane: (ci, fx) = (mr / S, mr % S); the filter is staged as it lies in
  // memory and read flipped. A lane whose column stands for no input channel reads something
  // valid: its column of D is never gathered, and columns do not mix.
  const int ci_n = min(mr / KS, 3), fx_n = mr % KS;
  const float *bbase = wl + (mq * 4 + ci_n) * RS + (RS - 1 - fx_n);
  const float *abase = smem + mq * PLANE + wv * (G::RPW * OW) + mr;
  const int crs      = g.C * RS;

  // ---- the weight gradient's side: column n of block t belongs to lane n % 32
  constexpr int NT_ = DWNT > 0 ? DWNT : 1;
  constexpr int XDEPTH = 8;
  f16 wacc[NT_];
  int woff[NT_];
  bool wone[NT_];
  float *xs = smem + G::STAGE;  // the input patch [ci][rows_in][pitch]
  if constexpr (DWNT > 0) {
#pragma unroll
    for (int t = 0; t < DWNT; ++t) {
      const int n  = t * 32 + (lane & 31);
      const int ci = n / RS, tap = n - ci * RS;
      wone[t] = n == crs;
      woff[t] = n < crs ? ci * dwa.plane + (tap / KS) * dwa.pitch + tap % KS : 0;
    }
  }

  for (int co0 = 0; co0 < g.Kc; co0 += DXM_MCH) {
    // ---- everything this chunk needs from memory, asked for together
    float sv[POOLED ? DXM_MAXCH : 1];
    int srec[POOLED ? DXM_MAXCH : 1];
    f4 sq[POOLED ? 1 : DXM_MAXCH];
#pragma unroll
    for (int jj = 0; jj < G::CPT; ++jj) {
      const int c = grp + G::GROUPS * jj;
      const bool live = src >= 0 && c < DXM_MCH && co0 + c < g.Kc;
      const int off = live ? (co0 + c) * chan + src : 0;
      if (POOLED) {
        sv[jj]   = dy_img[off];
        srec[jj] = rec_img[off];
      } else {
        sq[jj] = *reinterpret_cast<const f4 *>(dy_img + off);
      }
    }
    float wreg[DXM_WREG];
    const int nw = min(DXM_MCH, g.Kc - co0) * crs;
#pragma unroll
    for (int k = 0; k < DXM_WREG; ++k) wreg[k] = w[static_cast<size_t>(co0) * crs + min(tid + DXM_NT * k, nw - 1)];
    // the input patch under the band (zero where the window leaves the image): the first
    // XDEPTH elements of a thread travel with the loads above
    float xv[XDEPTH];
    int xo[XDEPTH];
    auto load_x = [&](int e0) {
#pragma unroll
      for (int k = 0; k < XDEPTH; ++k) {
        const int e = e0 + k * DXM_NT;
        xv[k] = 0.0f;
        xo[k] = -1;
        if (e < dwa.x_total) {
          const int rr = dwa.div_pitch.div(e), cx = e - rr * dwa.pitch;
          const int ci = dwa.div_rows_in.div(rr), r = rr - ci * dwa.rows_in;
          const int iy = y0 - g.pad_h + r, ix = cx - g.pad_w;
          xo[k] = ci * dwa.plane + r * dwa.pitch + cx;
          if (iy >= 0 && iy < g.H && ix >= 0 && ix < g.W)
            xv[k] = dwa.x[(static_cast<size_t>(img * g.C + ci) * g.H + iy) * g.W + ix];
        }
      }
    };
    auto store_x = [&]() {
#pragma unroll
      for (int k = 0; k < XDEPTH; ++k)
        if (xo[k] >= 0) xs[xo[k]] = xv[k];
    };
    if constexpr (DWNT > 0) load_x(tid);
    if (co0 > 0) __syncthreads();  // the previous chunk has been consumed
    // filters: element e = (co, ci, tap) of memory goes to [co][ci][tap] with four ci slots
#pragma unroll
    for (int k = 0; k < DXM_WREG; ++k) {
      const int e = tid + DXM_NT * k;
      if (e < DXM_MCH * crs) {
        const int co = e / crs, rest = e - co * crs;
        const int ci = rest / RS, tap = rest - ci * RS;
        wl[(co * 4 + ci) * RS + tap] = e < nw ? wreg[k] : 0.0f;
      }
    }
    if (stager) {
#pragma unroll
      for (int jj = 0; jj < G::CPT; ++jj) {
        const int c = grp + G::GROUPS * jj;
        if (c >= DXM_MCH) break;
        float *plane = smem + c * PLANE;
        const bool live = src >= 0 && co0 + c < g.Kc;
        if (POOLED) {
          // the record minus the flat index of the window's top left element: 0, 1, OW or OW+1
          const int where = live ? srec[jj] - ((co0 + c) * ohw + flat) : -1;
          plane[at[0]] = where == 0 ? sv[jj] : 0.0f;
          plane[at[1]] = where == 1 ? sv[jj] : 0.0f;
          plane[at[2]] = where == OW ? sv[jj] : 0.0f;
          plane[at[3]] = where == OW + 1 ? sv[jj] : 0.0f;
        } else {
          *reinterpret_cast<f4 *>(plane + at[0]) = live ? sq[jj] : f4{0.0f, 0.0f, 0.0f, 0.0f};
        }
      }
    }
    if constexpr (DWNT > 0) {
      store_x();
      for (int e0 = tid + XDEPTH * DXM_NT; e0 < dwa.x_total; e0 += XDEPTH * DXM_NT) {
        load_x(e0);
        store_x();
      }
    }
    __syncthreads();
    // ---- products: eight staged channels per pass, the four blocks of the wave side by side
#pragma unroll
    for (int sub = 0; sub < DXM_MCH / 8; ++sub) {
      if (co0 + 8 * sub >= g.Kc) break;
      float breg[NJ];
#pragma unroll
      for (int j = 0; j < NJ; ++j) breg[j] = bbase[(8 * sub + 4 * (j & 1)) * G::WROW - (j >> 1) * KS];
#pragma unroll
      for (int j = 0; j < NJ; ++j)
#pragma unroll
        for (int b = 0; b < 4; ++b)
          dacc[b] = __builtin_amdgcn_mfma_f32_16x16x4f32(
            abase[(8 * sub + 4 * (j & 1)) * PLANE + ((b / NMB) + (j >> 1)) * OW + 16 * (b % NMB)], breg[j], dacc[b], 0,
            0, 0);
    }
    if constexpr (DWNT > 0) {
      // ---- the weight gradient's products: output rows y0 .. of the band, which the staged
      //      rows hold from row KR-1-pad on; a half wave takes four consecutive positions a trip
      // (one chunk of output channels: the sums start here, behind everything the staging held)
#pragma unroll
      for (int t = 0; t < DWNT; ++t)
#pragma unroll
        for (int i = 0; i < 16; ++i) wacc[t][i] = 0.0f;
      const int half  = lane >> 5;
      const int units = max(min(G::TILE_ROWS, g.OH - y0), 0) * (OW / 4);
      const float *arow = smem + (lane & 31) * PLANE + (KR - 1 - g.pad_h) * OW;
      for (int it = 0; it < (units + 7) / 8; ++it) {
        const int u   = it * 8 + wv * 2 + half;
        const bool ok = u < units;
        const int pos = ok ? 4 * u : 0;
        f4 av         = *reinterpret_cast<const f4 *>(arow + pos);
        if (!ok) av = f4{0.0f, 0.0f, 0.0f, 0.0f};
        const float *xb = xs + (pos / OW) * dwa.pitch + pos % OW;
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int t = 0; t < DWNT; ++t) {
            float b = xb[j + woff[t]];
            b       = wone[t] ? 1.0f : b;
            wacc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[j], b, wacc[t], 0, 0, 0);
          }
      }
    }
  }

  if constexpr (DWNT > 0) {
    // ---- the four waves' sums meet in LDS (over the staged rows, which are done with) and
    //      leave as one slice, added in wave order
    constexpr int TILE = 32 * 32 * DWNT;
    __syncthreads();
    float *red = smem + wv * TILE;
#pragma unroll
    for (int t = 0; t < DWNT; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i)
        red[((i >> 2) * 8 + (lane >> 5) * 4 + (i & 3)) * (32 * DWNT) + t * 32 + (lane & 31)] = wacc[t][i];
    __syncthreads();
    float sums[TILE / DXM_NT];
#pragma unroll
    for (int i = 0; i < TILE / DXM_NT; ++i) {
      const int e = tid + DXM_NT * i;
      sums[i]     = (smem[e] + smem[TILE + e]) + (smem[2 * TILE + e] + smem[3 * TILE + e]);
    }
    // (a slice per band of OUTPUT rows: without padding the last bands of input rows have none)
    const int wbands = (g.OH + G::TILE_ROWS - 1) / G::TILE_ROWS, band = wg - img * bands;
    const size_t slice = static_cast<size_t>(img) * wbands + band;
#pragma unroll
    for (int i = 0; i < TILE / DXM_NT; ++i) {
      const int e = tid + DXM_NT * i;
      const int m = e / (32 * DWNT), n = e - m * (32 * DWNT);
      if (band >= wbands || m >= g.Kc || n > crs) continue;
      if (n < crs) dwa.partial_dw[(slice * g.Kc + m) * crs + n] = sums[i];
      else if (dwa.partial_db) dwa.partial_db[slice * g.Kc + m] = sums[i];
    }
  }

  // ---- D -> T[row of the wave][dY column][17] (reg i of lane l: column 4*(l/16) + i of the
  //      block, entry l%16), then an output is S reads of it
  __syncthreads();
  float *T = smem + wv * (G::RPW * OW * 17);
#pragma unroll
  for (int b = 0; b < 4; ++b)
#pragma unroll
    for (int i = 0; i < 4; ++i) T[((b / NMB) * OW + 16 * (b % NMB) + 4 * mq + i) * 17 + mr] = dacc[b][i];
  __syncthreads();
  const size_t img_off = static_cast<size_t>(img) * g.C * g.H * g.W;
#pragma unroll
  for (int u = 0; u < G::RPW; ++u) {
    const int y = y0 + wv * G::RPW + u;
    if (y >= g.H) break;
    for (int e = lane; e < g.C * g.W; e += 64) {
      uint32_t ci, x;
      g.div_w.divmod(e, ci, x);
      float v = 0.0f;
#pragma unroll
      for (int fx = 0; fx < KS; ++fx) {
        const int d = static_cast<int>(x) + fx + ox0;  // dY column
        if (static_cast<unsigned>(d) < static_cast<unsigned>(OW)) v += T[(u * OW + d) * 17 + ci * KS + fx];
      }
      const size_t idx = img_off + (static_cast<size_t>(ci) * g.H + y) * g.W + x;
      if (ag.kind != TDH_ACT_NONE) v *= act_grad_factor(ag.kind, ag.y[idx]);
      dx[idx] = v;
    }
  }
}

// the launch of the instance for this geometry, or false when there is none
template <int KR, int NMB, bool POOLED>
static bool launch_first_dx_mfma_inst(const ConvGeom &g, int batch, const float *dy, const float *w, float *dx,
                                      ActGrad ag, PoolGather pooled, bool only_ask) {
  using G = DxmGeom<KR, NMB, POOLED>;
  if constexpr (!G::FITS) {
    return false;
  } else {
    if (g.H < G::TILE_ROWS) return false;
    if (only_ask) return true;
    const int bands = ceil_div(g.H, G::TILE_ROWS);
    TDH_LAUNCH((conv_dx_first_mfma_kernel<KR, KR, NMB, POOLED>), dim3(batch * bands), dim3(DXM_NT),
               sizeof(float) * G::LDS_FLOATS, ctx().stream, dy, w, dx, g, ag, pooled, FirstDwArgs());
    return true;
  }
}

// ... and of the instance that also computes the weight and bias gradient; dwa comes in without
// its patch geometry, which depends on the instance's band
template <int KR, int NMB, bool POOLED, int DWNT>
static bool launch_first_both_inst(const ConvGeom &g, int batch, const float *dy, const float *w, float *dx,
                                   ActGrad ag, PoolGather pooled, FirstDwArgs dwa, bool only_ask) {
  using G = DxmGeom<KR, NMB, POOLED>;
  if constexpr (!G::FITS) {
    return false;
  } else {
    const int bands = ceil_div(g.H, G::TILE_ROWS);
    // every output row lies in the staged rows of the band that starts at the same row
    if (g.H < G::TILE_ROWS || g.OH > bands * G::TILE_ROWS || g.pad_h > KR - 1) return false;
    dwa.pitch   = (g.OW + KR - 1) | 1;  // odd: the taps of one column fall into different LDS banks
    dwa.rows_in = G::TILE_ROWS + KR - 1;
    dwa.plane   = dwa.rows_in * dwa.pitch + 1;
    dwa.x_total = g.C * dwa.rows_in * dwa.pitch;
    dwa.div_pitch   = FastDiv(dwa.pitch);
    dwa.div_rows_in = FastDiv(dwa.rows_in);
    const size_t x_floats = (static_cast<size_t>(g.C) * dwa.plane + 3) & ~static_cast<size_t>(3);
    const size_t floats   = std::max<size_t>(G::STAGE + x_floats, std::max<size_t>(G::GATHER, 4u * 32 * 32 * DWNT));
    if (floats * sizeof(float) > 76 * 1024) return false;  // (two workgroups a compute unit)
    if (only_ask) return true;
    auto kernel = conv_dx_first_mfma_kernel<KR, KR, NMB, POOLED, DWNT>;
    static bool raised = false;
    if (!raised) {  // more than the 64 KB a kernel may use without asking
      if (hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                              76 * 1024) != hipSuccess)
        return false;
      raised = true;
    }
    TDH_LAUNCH(kernel, dim3(batch * bands), dim3(DXM_NT), sizeof(float) * floats, ctx().stream, dy, w, dx, g, ag,
               pooled, dwa);
    return true;
  }
}

// Launches the matrix-core kernel where it applies (only_ask: tells whether it would) and
// returns whether it does.
template <bool POOLED>
static bool first_dx_mfma(const ConvGeom &g, int batch, const float *dy, const float *w, float *dx, ActGrad ag,
                          PoolGather pooled, bool only_ask) {
  if (g.sh != 1 || g.sw != 1 || g.dh != 1 || g.dw != 1 || g.R != g.S || (g.R != 3 && g.R != 5)) return false;
  if (g.C * g.S > 16 || g.C > 4 || (POOLED && g.OH % 2 != 0)) return false;
  if (static_cast<long>(g.Kc) * g.OH * g.OW >= (1L << 30) || DXM_MCH * g.C * g.R * g.S > DXM_WREG * DXM_NT) return false;
  if (!only_ask && !POOLED && (reinterpret_cast<uintptr_t>(dy) & 15)) return false;
#define TDH_DXM(KR_, NMB_) launch_first_dx_mfma_inst<KR_, NMB_, POOLED>(g, batch, dy, w, dx, ag, pooled, only_ask)
  switch (g.OW) {
    case 16: return g.R == 3 ? TDH_DXM(3, 1) : TDH_DXM(5, 1);
    case 32: return g.R == 3 ? TDH_DXM(3, 2) : TDH_DXM(5, 2);
    case 64: return g.R == 3 ? TDH_DXM(3, 4) : TDH_DXM(5, 4);
    default: return false;
  }
#undef TDH_DXM
}

// dX, dW and db of a first convolution in one launch: where the matrix-core dX kernel applies,
// the layer has at most 32 output channels (one staged chunk) and an instance exists for its
// window and channel count, and every compute unit gets a workgroup. Returns whether it applies
// (only_ask) / has been launched; band_rows: the rows of a band (one slice per band and image).
template <bool POOLED>
static bool first_bwd_both(const ConvGeom &g, int batch, const float *dy, const float *w, float *dx, ActGrad ag,
                           PoolGather pooled, FirstDwArgs dwa, bool only_ask, int *band_rows) {
  if (g.Kc > DXM_MCH || g.R != g.S || batch > 65535) return false;
  if (!first_dx_mfma<POOLED>(g, batch, dy, w, dx, ag, pooled, true)) return false;
  if (!only_ask && !POOLED && (reinterpret_cast<uintptr_t>(dy) & 15)) return false;
  const int nt = ceil_div(g.C * g.R * g.S + 1, 32);
  const int nmb = g.OW / 16;
  const int cus = ctx().compute_units > 0 ? ctx().compute_units : 256;
#define TDH_BOTH(KR_, NMB_, NT_) \
  (*band_rows = DxmGeom<KR_, NMB_, POOLED>::TILE_ROWS, \
   static_cast<long>(batch) * ceil_div(g.H, *band_rows) >= cus && \
   launch_first_both_inst<KR_, NMB_, POOLED, NT_>(g, batch, dy, w, dx, ag, pooled, dwa, only_ask))
  if (g.R == 5 && nt == 3 && nmb == 2) return TDH_BOTH(5, 2, 3);
  if (g.R == 5 && nt == 3 && nmb == 1) return TDH_BOTH(5, 1, 3);
  if (g.R == 5 && nt == 1 && nmb == 2) return TDH_BOTH(5, 2, 1);
  if (g.R == 5 && nt == 1 && nmb == 1) return TDH_BOTH(5, 1, 1);
  if (g.R == 3 && nt == 1 && nmb == 2) return TDH_BOTH(3, 2, 1);
  if (g.R == 3 && nt == 1 && nmb == 1) return TDH_BOTH(3, 1, 1);
#undef TDH_BOTH
  return false;
}

// true when the direct kernel applies; fills the launch geometry
static bool small_cin_dx_plan(const ConvGeom &g, DxsPlan &p) {
  if (g.C > DXS_MAX_CIN || g.sh != 1 || g.sw != 1) return false;
  p.gw = ceil_div(g.W, DXS_PX);
  if (p.gw > 64) return false;
  p.tile_rows = std::min(64 / p.gw, g.H);
  p.bands     = ceil_div(g.H, p.tile_rows);
  p.trows     = p.tile_rows + g.R - 1;
  p.tcols     = (DXS_PX * p.gw + g.S - 1 + 3) & ~3;  // lanes read whole 16-byte words
  const int tsz = p.trows * p.tcols;
  if (DXS_CO_CHUNK * tsz > DXS_MAX_STAGE * DXS_NT) return false;
  p.div_gw    = FastDiv(p.gw);
  p.div_tcols = FastDiv(p.tcols);
  p.div_tile  = FastDiv(tsz);
  p.pnr       = p.trows / 2 + 1;
  p.pnc       = p.tcols / 2 + 1;
  p.div_pnc   = FastDiv(p.pnc);
  p.div_ptile = FastDiv(p.pnr * p.pnc);
  p.pooled_ok = DXS_CO_CHUNK * p.pnr * p.pnc <= DXS_MAX_PSTAGE * DXS_NT;
  // (one more word: where the POOLED kernels store what falls outside the tile)
  const size_t stage_floats = static_cast<size_t>(DXS_CO_CHUNK) * tsz + 4 * DXS_CO_CHUNK * g.R * g.S + 1;
  const size_t red_floats   = static_cast<size_t>(DXS_WAVES) * DXS_MAX_CIN * 64 * DXS_PX;
  p.lds_bytes = sizeof(float) * std::max(stage_floats, red_floats);
  return p.lds_bytes <= 64 * 1024;
}

template <int KR, int KS, bool POOLED>
static void launch_small_cin_dx(const ConvGeom &g, const DxsPlan &p, int batch, const float *dy,
                                const float *w, float *dx, ActGrad ag, PoolGather pooled) {
  const dim3 grid(batch * p.bands), block(DXS_NT);
  switch (KR ? g.C : DXS_MAX_CIN) {
    case 1: TDH_LAUNCH((conv_dx_small_cin_kernel<KR, KS, 1, POOLED>), grid, block, p.lds_bytes, ctx().stream, dy, w, dx, g, p, ag, pooled); break;
    case 2: TDH_LAUNCH((conv_dx_small_cin_kernel<KR, KS, 2, POOLED>), grid, block, p.lds_bytes, ctx().stream, dy, w, dx, g, p, ag, pooled); break;
    case 3: TDH_LAUNCH((conv_dx_small_cin_kernel<KR, KS, 3, POOLED>), grid, block, p.lds_bytes, ctx().stream, dy, w, dx, g, p, ag, pooled); break;
    default: TDH_LAUNCH((conv_dx_small_cin_kernel<KR, KS, 4, POOLED>), grid, block, p.lds_bytes, ctx().stream, dy, w, dx, g, p, ag, pooled); break;
  }
}

template <bool POOLED>
static void launch_small_cin_dx_window(const ConvGeom &g, const DxsPlan &p, int batch, const float *dy,
                                       const float *w, float *dx, ActGrad ag, PoolGather pooled) {
  if (g.R == 3 && g.S == 3)
    launch_small_cin_dx<3, 3, POOLED>(g, p, batch, dy, w, dx, ag, pooled);
  else if (g.R == 5 && g.S == 5)
    launch_small_cin_dx<5, 5, POOLED>(g, p, batch, dy, w, dx, ag, pooled);
  else
    launch_small_cin_dx<0, 0, POOLED>(g, p, batch, dy, w, dx, ag, pooled);
}


static bool fwd_small_applies(const ConvGeom &g, int batch) {
  return conv_fwd_small_applicable(batch, g.C, g.Kc, g.H, g.W, g.OH, g.OW, g.R, g.S, g.sh, g.sw, g.dh,
                                   g.dw, g.pad_h, g.pad_w);
}

}  // namespace

static size_t first_both_workspace_bytes(const tdh_conv_desc *d, const ConvGeom &g, int batch);

size_t conv2d_workspace_bytes(const tdh_conv_desc *d, int batch) {
  const ConvGeom g = make_geom(d);
  const int ohw = g.OH * g.OW, crs = g.C * g.R * g.S;
  size_t total = 0;
  total += gemm_workspace_bytes(g.Kc, batch * ohw, crs, true);        // forward
  total += gemm_workspace_bytes(g.Kc, crs, batch * ohw, true);        // dW
  total += gemm_workspace_bytes(g.C, batch * g.H * g.W, g.Kc * g.R * g.S, true);  // dX
  total += rowsum_workspace_bytes(batch, g.Kc, ohw);                  // db
  if (d->tbl) total += ws_align(static_cast<size_t>(g.C) * g.Kc) + 2 * ws_align(sizeof(float) * g.Kc * crs);
  total += conv_dw_small_workspace_bytes(batch, g.C, g.Kc, g.H, g.W, g.OH, g.OW, g.R, g.S, g.sh, g.sw,
                                         g.dh, g.dw, g.pad_h, g.pad_w);
  total += first_both_workspace_bytes(d, g, batch);
  if (g.sh == 1 && g.sw == 1)
    total += conv_dw_halo_workspace_bytes(g.R, g.S, batch, g.C, g.Kc, g.H, g.W, g.OH, g.OW, g.pad_h, g.pad_w);
  if (g.sh == 1 && g.sw == 1) {  // LDS-halo kernel: repacked filters and split partial sums
    total += conv_s1_workspace_bytes(g.R, g.S, batch, g.C, g.Kc, 0, g.H, g.W, g.OH, g.OW, g.pad_h, g.pad_w);
    total += conv_s1_workspace_bytes(g.R, g.S, batch, g.C, g.Kc, 1, g.OH, g.OW, g.H, g.W,
                                     g.R - 1 - g.pad_h, g.S - 1 - g.pad_w);
  }

  return total;
}

// Uploads the connection table (if any) and returns masked weights in scratch.
// `tbl_resident`: a device copy the caller keeps (a network does, so that a captured graph
// holds no host copies); otherwise the host table is uploaded into scratch here.
static int prepare_table(const tdh_conv_desc *d, const ConvGeom &g, const float *w,
                         const uint8_t *tbl_resident, const uint8_t **tbl_dev,
                         const float **w_eff) {
  *tbl_dev = nullptr;
  *w_eff   = w;
  if (!d->tbl) return TDH_OK;
  void *t = nullptr, *wm = nullptr;
  const int nw = g.Kc * g.C * g.R * g.S;
  TDH_TRY(ws_take(static_cast<size_t>(g.C) * g.Kc, &t));
  TDH_TRY(ws_take(sizeof(float) * nw, &wm));
  if (tbl_resident) {
    t = const_cast<uint8_t *>(tbl_resident);
  } else {
    // pageable source: the copy is staged before the call returns
    TDH_HIP(hipMemcpyAsync(t, d->tbl, static_cast<size_t>(g.C) * g.Kc, hipMemcpyHostToDevice,
                           ctx().stream));
    TDH_HIP(hipStreamSynchronize(ctx().stream));
  }
  ProfScope prof("conv_mask_weights", 8.0 * nw, WORK_BYTE);
  TDH_LAUNCH(mask_weights_kernel, dim3(ceil_div(nw, 256)), dim3(256), 0, ctx().stream, w,
                     static_cast<const uint8_t *>(t), static_cast<float *>(wm), nw, g.C, g.Kc,
                     g.R * g.S, 0);
  TDH_LAUNCH_CHECK();
  *tbl_dev = static_cast<const uint8_t *>(t);
  *w_eff   = static_cast<const float *>(wm);
  return TDH_OK;
}

// the forward kernel of this layer can write a following pointwise activation as well
// (prepacked: the caller passes the filters in the stride-1 kernel's layout)
__global__ void __launch_bounds__(256) splitk_reduce_multi_kernel(const ReduceJobs jobs) {
  __shared__ float sm[REDUCE_GROUPS][REDUCE_OUTPUTS];
  int j = 0;
  while (j + 1 < jobs.n && jobs.first_block[j + 1] <= static_cast<int>(blockIdx.x)) ++j;
  const ReduceJob &r = jobs.job[j];
  splitk_reduce_block(r.partial, r.splits, r.M, r.N, r.epi, static_cast<int>(blockIdx.x) - jobs.first_block[j], sm);
}

static std::vector<ReduceJob> &deferred_reduces() {
  static std::vector<ReduceJob> jobs;
  return jobs;
}

int flush_deferred_reduces(bool launch) {
  std::vector<ReduceJob> &all = deferred_reduces();
  if (!launch) all.clear();
  for (size_t at = 0; at < all.size(); at += REDUCE_MULTI_MAX) {
    ReduceJobs jobs;
    jobs.n = static_cast<int>(std::min<size_t>(REDUCE_MULTI_MAX, all.size() - at));
    int blocks = 0;
    double bytes = 0.0;
    for (int j = 0; j < jobs.n; ++j) {
      jobs.job[j]         = all[at + j];
      jobs.first_block[j] = blocks;
      blocks += ceil_div(jobs.job[j].M * jobs.job[j].N, REDUCE_OUTPUTS);
      bytes += 4.0 * jobs.job[j].M * jobs.job[j].N * (jobs.job[j].splits + 1);
    }
    jobs.first_block[jobs.n] = blocks;
    ProfScope prof("conv_dw_splitk_reduce_multi", bytes, WORK_BYTE);
    TDH_LAUNCH(splitk_reduce_multi_kernel, dim3(blocks), dim3(256), 0, ctx().stream, jobs);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
      all.clear();
      return set_error(TDH_ERR_HIP, "splitk_reduce_multi_kernel: %s", hipGetErrorString(e));
    }
  }
  all.clear();
  return TDH_OK;
}

bool peek_deferred_reduces(OptPending *out) {
  const std::vector<ReduceJob> &all = deferred_reduces();
  out->n = 0;
  if (all.empty() || all.size() > static_cast<size_t>(OPT_PENDING_MAX)) return false;
  for (const ReduceJob &r : all)  // plain accumulating sums into a dense tensor only
    if (!(r.epi.accumulate && r.epi.ld == r.N && !r.epi.bias_n && r.epi.ag.kind == TDH_ACT_NONE)) return false;
  for (const ReduceJob &r : all)
    out->sum[out->n++] = OptPendingSum{r.partial, r.epi.out, static_cast<uint32_t>(r.splits),
                                       static_cast<uint32_t>(r.M) * static_cast<uint32_t>(r.N)};
  return true;
}

bool defer_reduce(const float *partial, int splits, int M, int N, const EpiRowMajor &epi) {
  if (!ctx().defer_reduce) return false;
  deferred_reduces().push_back(ReduceJob{partial, splits, M, N, epi});
  return true;
}

static bool dw_small_applies(const tdh_conv_desc *d, const ConvGeom &g, int batch) {
  return !d->tbl && conv_dw_small_applicable(batch, g.C, g.Kc, g.H, g.W, g.OH, g.OW, g.R, g.S, g.sh, g.sw,
                                             g.dh, g.dw, g.pad_h, g.pad_w);
}

bool conv_bwd_reads_pooled(const tdh_conv_desc *d, const tdh_pool_desc *pool, int batch) {
  const ConvGeom g = make_geom(d);
  DxsPlan dxs;
  if (!dw_small_applies(d, g, batch) || !small_cin_dx_plan(g, dxs) ||
      !(dxs.pooled_ok || first_dx_mfma<true>(g, batch, nullptr, nullptr, nullptr, ActGrad(), PoolGather(), true)))
    return false;
  if (pool->pool_w != 2 || pool->pool_h != 2 || pool->stride_w != 2 || pool->stride_h != 2 ||
      pool->in_w != g.OW || pool->in_h != g.OH || pool->in_c != g.Kc || g.OW % 4 != 0 || g.OH % 2 != 0)
    return false;
  return conv_dw_small_reads_pooled(batch, g.C, g.Kc, g.H, g.W, g.OH, g.OW, g.R, g.S, g.sh, g.sw, g.dh,
                                    g.dw, g.pad_h, g.pad_w);
}

bool conv_dw_gives_db(const tdh_conv_desc *d, int batch) {
  const ConvGeom g = make_geom(d);
  if (dw_small_applies(d, g, batch)) return true;
  return !d->tbl && g.sh == 1 && g.sw == 1 &&
         conv_dw_halo_applicable(g.R, g.S, batch, g.C, g.Kc, g.H, g.W, g.OH, g.OW, g.pad_h, g.pad_w);
}

bool conv_fwd_applies_act(const tdh_conv_desc *d, int batch, bool prepacked) {
  // every forward kernel does: the packed stride-1 kernel, the first-layer kernel, the
  // stride-1 kernel that packs for itself and the GEMM (in its epilogue or its split reduction)
  return prepacked ? conv_uses_packed(d, batch, 0) : true;
}

// the stride-1 kernel runs this forward pass (with filters packed by the caller, or by itself)
static bool fwd_s1_applies(const tdh_conv_desc *d, const ConvGeom &g, int batch, bool prepacked) {
  if (prepacked) return conv_uses_packed(d, batch, 0);
  return !fwd_small_applies(g, batch) && g.sh == 1 && g.sw == 1 && g.dh == 1 && g.dw == 1 &&
         conv_s1_applicable(g.R, g.S, batch, g.C, g.Kc, g.H, g.W, g.OH, g.OW, g.pad_h, g.pad_w);
}

bool conv_fwd_fuses_pool(const tdh_conv_desc *d, const tdh_pool_desc *pool, int batch, bool prepacked) {
  const ConvGeom g = make_geom(d);
  if (!(pool->pool_w == 2 && pool->pool_h == 2 && pool->stride_w == 2 && pool->stride_h == 2 &&
        pool->in_w == g.OW && pool->in_h == g.OH && pool->in_c == g.Kc && g.OW % 2 == 0 && g.OH % 2 == 0))
    return false;
  if (!prepacked && fwd_small_applies(g, batch)) return true;
  return fwd_s1_applies(d, g, batch, prepacked) &&
         conv_s1_fuses_pool(g.R, g.S, batch, g.C, g.Kc, g.H, g.W, g.OH, g.OW, g.pad_h, g.pad_w);
}

bool conv_fwd_out_optional(const tdh_conv_desc *d, int batch, bool prepacked) {
  const ConvGeom g = make_geom(d);
  if (!prepacked && fwd_small_applies(g, batch)) return true;
  return fwd_s1_applies(d, g, batch, prepacked) &&
         conv_s1_single_pass(g.R, g.S, batch, g.C, g.Kc, g.H, g.W, g.OH, g.OW, g.pad_h, g.pad_w);
}

bool conv_fwd_pool_applies_act(const tdh_conv_desc *d, int batch, bool prepacked, int act_kind) {
  const ConvGeom g = make_geom(d);
  // the first-layer kernel applies any pointwise kind, the stride-1 kernel relu
  if (!prepacked && fwd_small_applies(g, batch)) return true;
  return act_kind == TDH_ACT_RELU;
}

bool conv_uses_packed(const tdh_conv_desc *d, int batch, int flip) {
  const ConvGeom g = make_geom(d);
  if (g.sh != 1 || g.sw != 1) return false;
  if (!flip)
    return g.dh == 1 && g.dw == 1 && !fwd_small_applies(g, batch) &&
           conv_s1_applicable(g.R, g.S, batch, g.C, g.Kc, g.H, g.W, g.OH, g.OW, g.pad_h, g.pad_w);
  DxsPlan dxs;
  if (small_cin_dx_plan(g, dxs)) return false;
  return conv_s1_applicable(g.R, g.S, batch, g.Kc, g.C, g.OH, g.OW, g.H, g.W, g.R - 1 - g.pad_h,
                            g.S - 1 - g.pad_w);
}

int conv_pack_filters(const tdh_conv_desc *d, int flip, const float *w, const uint8_t *tbl_resident,
                      float *wp) {
  return conv_s1_repack(d->k_h, d->k_w, d->in_c, d->out_c, flip, w, d->tbl ? tbl_resident : nullptr, wp);
}

int conv2d_fwd(const tdh_conv_desc *d, int batch, const float *x, const float *w, const float *b,
               float *y, const uint8_t *tbl_resident, const float *prepacked, float *act_out,
               int act_kind, const PoolFuse *pool) {
  const ConvGeom g = make_geom(d);
  if (pool) {
    tdh_pool_desc behind{};
    behind.in_w = g.OW; behind.in_h = g.OH; behind.in_c = g.Kc;
    behind.pool_w = behind.pool_h = behind.stride_w = behind.stride_h = 2;
    if (!conv_fwd_fuses_pool(d, &behind, batch, prepacked != nullptr) ||
        (pool->act_out && !conv_fwd_pool_applies_act(d, batch, prepacked != nullptr, pool->act_kind)))
      return set_error(TDH_ERR_INVALID, "conv2d_fwd: this kernel does not compute the pool layer behind it");
  }
  // (y null: only a kernel that also writes the activation or the pool behind the layer can leave it out)
  if (!y && !pool && !(act_out && conv_fwd_out_optional(d, batch, prepacked != nullptr)))
    return set_error(TDH_ERR_INVALID, "conv2d_fwd: no output tensor");
  if (prepacked)
    return conv_s1_run(g.R, g.S, batch, g.C, g.Kc, 0, x, w, nullptr, d->has_bias ? b : nullptr, y, g.H,
                       g.W, g.OH, g.OW, g.pad_h, g.pad_w, ActGrad(), "conv_fwd_s1", prepacked, act_out,
                       act_kind, pool);
  const int ohw = g.OH * g.OW, crs = g.C * g.R * g.S;
  const uint8_t *tbl_dev;
  const float *w_eff;
  TDH_TRY(prepare_table(d, g, w, tbl_resident, &tbl_dev, &w_eff));
  if (fwd_small_applies(g, batch))
    return conv_fwd_small_run(batch, g.C, g.Kc, x, w_eff, d->has_bias ? b : nullptr, y, g.H, g.W, g.OH, g.OW,
                              g.R, g.S, g.sh, g.sw, g.dh, g.dw, g.pad_h, g.pad_w, act_out, act_kind, pool);
  if (g.sh == 1 && g.sw == 1 && g.dh == 1 && g.dw == 1 &&
      conv_s1_applicable(g.R, g.S, batch, g.C, g.Kc, g.H, g.W, g.OH, g.OW, g.pad_h, g.pad_w))
    return conv_s1_run(g.R, g.S, batch, g.C, g.Kc, 0, x, w_eff, nullptr,
                       d->has_bias ? b : nullptr, y, g.H, g.W, g.OH, g.OW, g.pad_h, g.pad_w,
                       ActGrad(), "conv_fwd_s1", nullptr, act_out, act_kind, pool);
  StridedOperand A{w_eff, crs, 1, g.Kc};
  FwdInputOperand B{x, g, batch * ohw};
  if (act_out) {  // the pointwise activation layer that follows leaves the same kernel
    EpiImageRowsAct epi{y, g.Kc, ohw, g.div_ohw, d->has_bias ? b : nullptr, act_out, act_kind};
    return launch_gemm<true, false>(A, B, epi, g.Kc, batch * ohw, crs, true, "conv_fwd_gemm", "conv_fwd_splitk_reduce");
  }
  EpiImageRows epi{y, g.Kc, ohw, g.div_ohw, d->has_bias ? b : nullptr, ActGrad()};
  return launch_gemm<true, false>(A, B, epi, g.Kc, batch * ohw, crs, true, "conv_fwd_gemm", "conv_fwd_splitk_reduce");
}

// the rows of a band of the launch that computes dX, dW and db of this layer together, or 0
static int one_launch_band(const tdh_conv_desc *d, const ConvGeom &g, int batch, bool pooled) {
  if (d->tbl) return 0;
  int rows = 0;
  const bool ok =
      pooled ? first_bwd_both<true>(g, batch, nullptr, nullptr, nullptr, ActGrad(), PoolGather(), FirstDwArgs(), true, &rows)
             : first_bwd_both<false>(g, batch, nullptr, nullptr, nullptr, ActGrad(), PoolGather(), FirstDwArgs(), true, &rows);
  return ok ? rows : 0;
}
bool conv_bwd_one_launch(const tdh_conv_desc *d, int batch, bool pooled) {
  return one_launch_band(d, make_geom(d), batch, pooled) > 0;
}

// the slices of that launch: one per band and image
static size_t first_both_workspace_bytes(const tdh_conv_desc *d, const ConvGeom &g, int batch) {
  size_t most = 0;
  for (int pooled = 0; pooled < 2; ++pooled) {
    const int rows = one_launch_band(d, g, batch, pooled != 0);
    if (!rows) continue;
    const size_t blocks = static_cast<size_t>(batch) * ceil_div(g.OH, rows);
    most = std::max(most, ws_align(blocks * g.Kc * g.C * g.R * g.S * sizeof(float)) + ws_align(blocks * g.Kc * sizeof(float)));
  }
  return most;
}

// dX, dW and (optionally) db of a first convolution as one launch plus the split reduction of
// its slices; the caller has asked conv_bwd_one_launch
template <bool POOLED>
static int run_first_both(const ConvGeom &g, int batch, const float *x, const float *dy, const float *w, float *dx,
                          float *dw, float *db, int accumulate, ActGrad dx_act, PoolGather pooled) {
  const int crs = g.C * g.R * g.S;
  int rows = 0;
  if (!first_bwd_both<POOLED>(g, batch, dy, w, dx, dx_act, pooled, FirstDwArgs(), true, &rows))
    return set_error(TDH_ERR_INVALID, "conv2d_bwd: the one-launch kernel does not apply");
  const int blocks = batch * ceil_div(g.OH, rows);
  void *pw_ws = nullptr, *pb_ws = nullptr;
  TDH_TRY(ws_take(static_cast<size_t>(blocks) * g.Kc * crs * sizeof(float), &pw_ws));
  if (db) TDH_TRY(ws_take(static_cast<size_t>(blocks) * g.Kc * sizeof(float), &pb_ws));
  FirstDwArgs dwa{};
  dwa.x = x;
  dwa.partial_dw = static_cast<float *>(pw_ws);
  dwa.partial_db = static_cast<float *>(pb_ws);
  {
    ProfScope prof("conv_bwd_first_both", 2.0 * batch * (static_cast<double>(g.C) * g.H * g.W * g.Kc * g.R * g.S +
                                                         static_cast<double>(g.Kc) * (crs + (db ? 1 : 0)) * g.OH * g.OW),
                   WORK_FLOP);
    if (!first_bwd_both<POOLED>(g, batch, dy, w, dx, dx_act, pooled, dwa, false, &rows))
      return set_error(TDH_ERR_HIP, "conv2d_bwd: the one-launch kernel could not be launched");
    TDH_LAUNCH_CHECK();
  }
  EpiRowMajor epi_w{dw, crs, nullptr, ActGrad(), accumulate};
  EpiRowMajor epi_b{db, 1, nullptr, ActGrad(), accumulate};
  // the two reductions leave as one launch: collected by the train step, or here
  const bool collect_here = !ctx().defer_reduce;
  if (collect_here) flush_deferred_reduces(false);  // nothing may be left from a failed call
  ctx().defer_reduce = true;
  defer_reduce(dwa.partial_dw, blocks, g.Kc, crs, epi_w);
  if (db) defer_reduce(dwa.partial_db, blocks, g.Kc, 1, epi_b);
  if (!collect_here) return TDH_OK;
  ctx().defer_reduce = false;
  return flush_deferred_reduces();
}

int conv2d_bwd(const tdh_conv_desc *d, int batch, const float *x, const float *w, const float *dy,
               float *dx, float *dw, float *db, int accumulate, ActGrad dx_act,
               const uint8_t *tbl_resident, const float *prepacked_dx, const PoolGather *dy_pool) {
  const ConvGeom g = make_geom(d);
  const int ohw = g.OH * g.OW, crs = g.C * g.R * g.S;
  if (dy_pool) {
    // only the two first-layer kernels read the gradient this way, and they leave nothing over
    tdh_pool_desc over{};
    over.in_w = g.OW; over.in_h = g.OH; over.in_c = g.Kc;
    over.pool_w = over.pool_h = over.stride_w = over.stride_h = 2;
    if (!conv_bwd_reads_pooled(d, &over, batch) || !dy_pool->g || !dy_pool->argmax ||
        (reinterpret_cast<uintptr_t>(dy_pool->g) & 7) || (reinterpret_cast<uintptr_t>(dy_pool->argmax) & 7) ||
        (db && !dw))
      return set_error(TDH_ERR_INVALID, "conv2d_bwd: the pooled gradient cannot be read for this layer");
    if (dx && dw && conv_bwd_one_launch(d, batch, true))
      return run_first_both<true>(g, batch, x, nullptr, w, dx, dw, db, accumulate, dx_act, *dy_pool);
    DxsPlan dxs;
    small_cin_dx_plan(g, dxs);
    if (dx) {
      if (first_dx_mfma<true>(g, batch, nullptr, w, dx, dx_act, *dy_pool, true)) {
        ProfScope prof("conv_dx_first_mfma", g.C, batch * g.H * g.W, g.Kc * g.R * g.S);
        first_dx_mfma<true>(g, batch, nullptr, w, dx, dx_act, *dy_pool, false);
      } else {
        ProfScope prof("conv_dx_small_cin", g.C, batch * g.H * g.W, g.Kc * g.R * g.S);
        launch_small_cin_dx_window<true>(g, dxs, batch, nullptr, w, dx, dx_act, *dy_pool);
      }
      TDH_LAUNCH_CHECK();
    }
    if (dw)
      // (with the bands of the launch that would also compute dX: the same sums either way)
      TDH_TRY(conv_dw_small_run(batch, g.C, g.Kc, x, nullptr, dw, db, g.H, g.W, g.OH, g.OW, g.R, g.S, g.sh,
                                g.sw, g.dh, g.dw, g.pad_h, g.pad_w, accumulate, dy_pool,
                                one_launch_band(d, g, batch, true)));
    return TDH_OK;
  }
  if (dx && prepacked_dx) {
    TDH_TRY(conv_s1_run(g.R, g.S, batch, g.C, g.Kc, 1, dy, w, nullptr, nullptr, dx, g.OH, g.OW, g.H,
                        g.W, g.R - 1 - g.pad_h, g.S - 1 - g.pad_w, dx_act, "conv_dx_s1", prepacked_dx));
    dx = nullptr;
    if (!dw && !db) return TDH_OK;
  }
  if (dx && dw && !prepacked_dx && !(reinterpret_cast<uintptr_t>(dy) & 15) && conv_bwd_one_launch(d, batch, false))
    return run_first_both<false>(g, batch, x, dy, w, dx, dw, db, accumulate, dx_act, PoolGather());
  const uint8_t *tbl_dev;
  const float *w_eff;
  TDH_TRY(prepare_table(d, g, w, tbl_resident, &tbl_dev, &w_eff));
  DxsPlan dxs;
  if (dx && small_cin_dx_plan(g, dxs) && !(reinterpret_cast<uintptr_t>(dy) & 15) &&
      first_dx_mfma<false>(g, batch, dy, w_eff, dx, dx_act, PoolGather(), true)) {
    ProfScope prof("conv_dx_first_mfma", g.C, batch * g.H * g.W, g.Kc * g.R * g.S);
    first_dx_mfma<false>(g, batch, dy, w_eff, dx, dx_act, PoolGather(), false);
    TDH_LAUNCH_CHECK();
  } else if (dx && small_cin_dx_plan(g, dxs)) {
    ProfScope prof("conv_dx_small_cin", g.C, batch * g.H * g.W, g.Kc * g.R * g.S);
    launch_small_cin_dx_window<false>(g, dxs, batch, dy, w_eff, dx, dx_act, PoolGather());
    TDH_LAUNCH_CHECK();
  } else if (dx && g.sh == 1 && g.sw == 1 &&
             conv_s1_applicable(g.R, g.S, batch, g.Kc, g.C, g.OH, g.OW, g.H, g.W,
                                g.R - 1 - g.pad_h, g.S - 1 - g.pad_w)) {
    TDH_TRY(conv_s1_run(g.R, g.S, batch, g.C, g.Kc, 1, dy, w_eff, nullptr, nullptr, dx, g.OH,
                        g.OW, g.H, g.W, g.R - 1 - g.pad_h, g.S - 1 - g.pad_w, dx_act,
                        "conv_dx_s1"));
  } else if (dx) {
    DxWeightOperand A{w_eff, g.C, g.R * g.S, g.div_rs};
    DxDyOperand B{dy, g, batch * g.H * g.W};
    EpiImageRows epi{dx, g.C, g.H * g.W, g.div_hw, nullptr, dx_act};
    TDH_TRY((launch_gemm<true, false>(A, B, epi, g.C, batch * g.H * g.W, g.Kc * g.R * g.S, true, "conv_dx_gemm", "conv_dx_splitk_reduce")));
  }
  if (dw && dw_small_applies(d, g, batch) && !(reinterpret_cast<uintptr_t>(dy) & 15)) {
    TDH_TRY(conv_dw_small_run(batch, g.C, g.Kc, x, dy, dw, db, g.H, g.W, g.OH, g.OW, g.R, g.S, g.sh, g.sw,
                              g.dh, g.dw, g.pad_h, g.pad_w, accumulate, nullptr, one_launch_band(d, g, batch, false)));
    return TDH_OK;
  }
  if (dw) {
    DwDyOperand A{dy, g.Kc, ohw, g.div_ohw};
    DwInputOperand B{x, g, crs};
    const bool halo = g.sh == 1 && g.sw == 1 &&
                      conv_dw_halo_applicable(g.R, g.S, batch, g.C, g.Kc, g.H, g.W, g.OH, g.OW,
                                              g.pad_h, g.pad_w);
    if (tbl_dev) {
      // the masking kernel below reads the reduced gradient: its reduction cannot wait
      struct NoDefer {
        bool was = ctx().defer_reduce;
        NoDefer() { ctx().defer_reduce = false; }
        ~NoDefer() { ctx().defer_reduce = was; }
      } no_defer;
      void *tmp = nullptr;
      TDH_TRY(ws_take(sizeof(float) * g.Kc * crs, &tmp));
      EpiRowMajor epi{static_cast<float *>(tmp), crs, nullptr, ActGrad(), 0};
      if (halo)
        TDH_TRY(conv_dw_halo_run(g.R, g.S, batch, g.C, g.Kc, x, dy, static_cast<float *>(tmp), g.H,
                                 g.W, g.OH, g.OW, g.pad_h, g.pad_w, 0));
      else
        TDH_TRY((launch_gemm<true, true>(A, B, epi, g.Kc, crs, batch * ohw, true, "conv_dw_gemm", "conv_dw_splitk_reduce")));
      ProfScope prof("conv_mask_weights", 8.0 * g.Kc * crs, WORK_BYTE);
      TDH_LAUNCH(mask_weights_kernel, dim3(ceil_div(g.Kc * crs, 256)), dim3(256), 0,
                         ctx().stream, static_cast<const float *>(tmp), tbl_dev, dw, g.Kc * crs,
                         g.C, g.Kc, g.R * g.S, accumulate);
      TDH_LAUNCH_CHECK();
    } else if (halo) {
      // the kernel adds up the dY words it stages: the bias gradient needs no pass of its own
      TDH_TRY(conv_dw_halo_run(g.R, g.S, batch, g.C, g.Kc, x, dy, dw, g.H, g.W, g.OH, g.OW, g.pad_h,
                               g.pad_w, accumulate, db));
      db = nullptr;
    } else {
      EpiRowMajor epi{dw, crs, nullptr, ActGrad(), accumulate};
      TDH_TRY((launch_gemm<true, true>(A, B, epi, g.Kc, crs, batch * ohw, true, "conv_dw_gemm",
                                       "conv_dw_splitk_reduce")));
    }
  }
  if (db) TDH_TRY(launch_rowsum(dy, batch, g.Kc, ohw, db, accumulate));
  return TDH_OK;
}

}  // namespace tdh
