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
// ALUs, stride 1: a workgroup owns a band of input rows of one image, stages the dY rows that
// can reach it (with zero halo) in LDS eight output channels at a time, and every thread
// accumulates its pixels for all Cin channels. Filter taps are wave-uniform reads.
constexpr int DXS_MAX_CIN  = 4;
constexpr int DXS_CO_CHUNK = 8;
constexpr int DXS_PX       = 4;  // pixels per thread

// KR, KS: compile-time window (0 = use the run-time g.R, g.S)
template <int KR, int KS>
__global__ void __launch_bounds__(256)
conv_dx_small_cin_kernel(const float *__restrict__ dy, const float *__restrict__ w,
                         float *__restrict__ dx, const ConvGeom g, const int tile_rows,
                         const int bands, const ActGrad ag) {
  extern __shared__ float smem[];  // dY tile [DXS_CO_CHUNK][trows][tcols], then weights
  const int R = KR ? KR : g.R, S = KS ? KS : g.S;
  const int img   = blockIdx.x / bands;
  const int y0    = (blockIdx.x - img * bands) * tile_rows;
  const int rows  = min(tile_rows, g.H - y0);
  const int trows = tile_rows + R - 1, tcols = g.W + S - 1;
  const int oy0 = y0 + g.pad_h - (R - 1), ox0 = g.pad_w - (S - 1);
  const int ohw = g.OH * g.OW, rs = R * S;
  const float *dy_img = dy + static_cast<size_t>(img) * g.Kc * ohw;
  float *tile = smem;
  float4 *wl  = reinterpret_cast<float4 *>(smem + ((DXS_CO_CHUNK * trows * tcols + 3) & ~3));

  float acc[DXS_MAX_CIN][DXS_PX];
#pragma unroll
  for (int c = 0; c < DXS_MAX_CIN; ++c)
#pragma unroll
    for (int i = 0; i < DXS_PX; ++i) acc[c][i] = 0.0f;

  // pixel i of this thread: p = tid + 256*i -> (py, px); its tile offset for tap (R-1, S-1)
  int toff[DXS_PX];
  bool live[DXS_PX];
#pragma unroll
  for (int i = 0; i < DXS_PX; ++i) {
    const int p  = threadIdx.x + 256 * i;
    const int py = p / g.W, px = p - py * g.W;
    live[i] = py < rows;
    toff[i] = live[i] ? py * tcols + px : 0;
  }

  for (int co0 = 0; co0 < g.Kc; co0 += DXS_CO_CHUNK) {
    const int nco = min(DXS_CO_CHUNK, g.Kc - co0);
    __syncthreads();
    for (int e = threadIdx.x; e < nco * trows * tcols; e += 256) {
      const int c = e / (trows * tcols);
      const int r = (e - c * trows * tcols) / tcols;
      const int q = e - c * trows * tcols - r * tcols;
      const int oy = oy0 + r, ox = ox0 + q;
      float v = 0.0f;
      if (static_cast<unsigned>(oy) < static_cast<unsigned>(g.OH) &&
          static_cast<unsigned>(ox) < static_cast<unsigned>(g.OW))
        v = dy_img[(co0 + c) * ohw + oy * g.OW + ox];
      tile[e] = v;
    }
    // weights of the chunk as [c][tap] -> (w[ci=0..3]); tap stored flipped so that the
    // inner loops walk the tile forwards
    for (int e = threadIdx.x; e < nco * rs; e += 256) {
      const int c = e / rs, t = e - c * rs;
      const float *wc = w + (static_cast<size_t>(co0 + c) * g.C) * rs + (rs - 1 - t);
      float4 v;
      v.x = wc[0];
      v.y = g.C > 1 ? wc[rs] : 0.0f;
      v.z = g.C > 2 ? wc[2 * rs] : 0.0f;
      v.w = g.C > 3 ? wc[3 * rs] : 0.0f;
      wl[e] = v;
    }
    __syncthreads();
    for (int c = 0; c < nco; ++c) {
      const float *t = tile + c * trows * tcols;
#pragma unroll
      for (int fy = 0; fy < (KR ? KR : 1); ++fy)
        for (int fyy = fy; fyy < R; fyy += (KR ? R : 1)) {
#pragma unroll
          for (int fx = 0; fx < (KS ? KS : 1); ++fx)
            for (int fxx = fx; fxx < S; fxx += (KS ? S : 1)) {
              // flipped tap (fyy, fxx) reads tile[(py + fyy)][px + fxx]
              const float4 wv = wl[c * rs + fyy * S + fxx];
#pragma unroll
              for (int i = 0; i < DXS_PX; ++i) {
                const float v = t[toff[i] + fyy * tcols + fxx];
                acc[0][i] += wv.x * v;
                acc[1][i] += wv.y * v;
                acc[2][i] += wv.z * v;
                acc[3][i] += wv.w * v;
              }
            }
        }
    }
  }
  float *dx_img = dx + static_cast<size_t>(img) * g.C * g.H * g.W;
#pragma unroll
  for (int i = 0; i < DXS_PX; ++i) {
    if (!live[i]) continue;
    const int p  = threadIdx.x + 256 * i;
    const int py = p / g.W, px = p - py * g.W;
#pragma unroll
    for (int ci = 0; ci < DXS_MAX_CIN; ++ci) {
      if (ci >= g.C) break;
      const size_t idx = (static_cast<size_t>(ci) * g.H + y0 + py) * g.W + px;
      float v = acc[ci][i];
      if (ag.kind != TDH_ACT_NONE)
        v *= act_grad_factor(ag.kind, ag.y[static_cast<size_t>(img) * g.C * g.H * g.W + idx]);
      dx_img[idx] = v;
    }
  }
}

// true when the direct kernel applies; fills the launch geometry
static bool small_cin_dx_plan(const ConvGeom &g, int &tile_rows, int &bands, size_t &lds_bytes) {
  if (g.C > DXS_MAX_CIN || g.sh != 1 || g.sw != 1 || g.W > 256 * DXS_PX) return false;
  tile_rows = (256 * DXS_PX) / g.W;
  if (tile_rows > g.H) tile_rows = g.H;
  // keep at least ~2 workgroups per image so that small batches still fill the chip
  if (tile_rows > 8 && tile_rows * 2 > g.H) tile_rows = (g.H + 1) / 2;
  bands     = ceil_div(g.H, tile_rows);
  lds_bytes = sizeof(float) * (((DXS_CO_CHUNK * (tile_rows + g.R - 1) * (g.W + g.S - 1) + 3) & ~3) +
                               4 * DXS_CO_CHUNK * g.R * g.S);
  return lds_bytes <= 64 * 1024;
}

}  // namespace

size_t conv2d_workspace_bytes(const tdh_conv_desc *d, int batch) {
  const ConvGeom g = make_geom(d);
  const int ohw = g.OH * g.OW, crs = g.C * g.R * g.S;
  size_t total = 0;
  total += gemm_workspace_bytes(g.Kc, batch * ohw, crs, true);        // forward
  total += gemm_workspace_bytes(g.Kc, crs, batch * ohw, true);        // dW
  total += gemm_workspace_bytes(g.C, batch * g.H * g.W, g.Kc * g.R * g.S, true);  // dX
  total += rowsum_workspace_bytes(batch, g.Kc, ohw);                  // db
  if (d->tbl) total += ws_align(static_cast<size_t>(g.C) * g.Kc) + 2 * ws_align(sizeof(float) * g.Kc * crs);
  total += 2 * conv_s1_workspace_bytes(g.R, g.S, g.C, g.Kc);          // repacked filters

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
  hipLaunchKernelGGL(mask_weights_kernel, dim3(ceil_div(nw, 256)), dim3(256), 0, ctx().stream, w,
                     static_cast<const uint8_t *>(t), static_cast<float *>(wm), nw, g.C, g.Kc,
                     g.R * g.S, 0);
  TDH_LAUNCH_CHECK();
  *tbl_dev = static_cast<const uint8_t *>(t);
  *w_eff   = static_cast<const float *>(wm);
  return TDH_OK;
}

int conv2d_fwd(const tdh_conv_desc *d, int batch, const float *x, const float *w, const float *b,
               float *y, const uint8_t *tbl_resident) {
  const ConvGeom g = make_geom(d);
  const int ohw = g.OH * g.OW, crs = g.C * g.R * g.S;
  const uint8_t *tbl_dev;
  const float *w_eff;
  TDH_TRY(prepare_table(d, g, w, tbl_resident, &tbl_dev, &w_eff));
  if (g.sh == 1 && g.sw == 1 && g.dh == 1 && g.dw == 1 &&
      conv_s1_applicable(g.R, g.S, batch, g.C, g.Kc, g.H, g.W, g.OH, g.OW, g.pad_h, g.pad_w))
    return conv_s1_run(g.R, g.S, batch, g.C, g.Kc, 0, x, w_eff, nullptr,
                       d->has_bias ? b : nullptr, y, g.H, g.W, g.OH, g.OW, g.pad_h, g.pad_w,
                       ActGrad(), "conv_fwd_s1");
  StridedOperand A{w_eff, crs, 1, g.Kc};
  FwdInputOperand B{x, g, batch * ohw};
  EpiImageRows epi{y, g.Kc, ohw, g.div_ohw, d->has_bias ? b : nullptr, ActGrad()};
  return launch_gemm<true, false>(A, B, epi, g.Kc, batch * ohw, crs, true, "conv_fwd_gemm", "conv_fwd_splitk_reduce");
}

int conv2d_bwd(const tdh_conv_desc *d, int batch, const float *x, const float *w, const float *dy,
               float *dx, float *dw, float *db, int accumulate, ActGrad dx_act,
               const uint8_t *tbl_resident) {
  const ConvGeom g = make_geom(d);
  const int ohw = g.OH * g.OW, crs = g.C * g.R * g.S;
  const uint8_t *tbl_dev;
  const float *w_eff;
  TDH_TRY(prepare_table(d, g, w, tbl_resident, &tbl_dev, &w_eff));
  int tile_rows = 0, bands = 0;
  size_t lds_bytes = 0;
  if (dx && small_cin_dx_plan(g, tile_rows, bands, lds_bytes)) {
    ProfScope prof("conv_dx_small_cin", g.C, batch * g.H * g.W, g.Kc * g.R * g.S);
    if (g.R == 3 && g.S == 3)
      hipLaunchKernelGGL((conv_dx_small_cin_kernel<3, 3>), dim3(batch * bands), dim3(256),
                         lds_bytes, ctx().stream, dy, w_eff, dx, g, tile_rows, bands, dx_act);
    else if (g.R == 5 && g.S == 5)
      hipLaunchKernelGGL((conv_dx_small_cin_kernel<5, 5>), dim3(batch * bands), dim3(256),
                         lds_bytes, ctx().stream, dy, w_eff, dx, g, tile_rows, bands, dx_act);
    else
      hipLaunchKernelGGL((conv_dx_small_cin_kernel<0, 0>), dim3(batch * bands), dim3(256),
                         lds_bytes, ctx().stream, dy, w_eff, dx, g, tile_rows, bands, dx_act);
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
  if (dw) {
    DwDyOperand A{dy, g.Kc, ohw, g.div_ohw};
    DwInputOperand B{x, g, crs};
    if (tbl_dev) {
      void *tmp = nullptr;
      TDH_TRY(ws_take(sizeof(float) * g.Kc * crs, &tmp));
      EpiRowMajor epi{static_cast<float *>(tmp), crs, nullptr, ActGrad(), 0};
      TDH_TRY((launch_gemm<true, true>(A, B, epi, g.Kc, crs, batch * ohw, true, "conv_dw_gemm", "conv_dw_splitk_reduce")));
      ProfScope prof("conv_mask_weights", 8.0 * g.Kc * crs, WORK_BYTE);
      hipLaunchKernelGGL(mask_weights_kernel, dim3(ceil_div(g.Kc * crs, 256)), dim3(256), 0,
                         ctx().stream, static_cast<const float *>(tmp), tbl_dev, dw, g.Kc * crs,
                         g.C, g.Kc, g.R * g.S, accumulate);
      TDH_LAUNCH_CHECK();
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
