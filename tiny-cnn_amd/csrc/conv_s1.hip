// conv_s1.hip — stride-1 convolution forward and dX as one LDS-halo MFMA kernel.
//
// Both products have the form
//   out[img][m][oy][ox] = sum_{kc,fy,fx} wp[(fy,fx)][kc][m] * in[img][kc][oy+fy-ph][ox+fx-pw]
// (zero outside the input):
//   forward  in = x,  m = out channel, kc = in channel,  wp[t][ci][co] = W[co][ci][t]
//   dX       in = dY, m = in channel,  kc = out channel, wp[t][co][ci] = W[co][ci][RS-1-t],
//            ph = R-1-pad_h, pw = S-1-pad_w   (correlation with the flipped filter)
//
// A workgroup (four wave64) owns BM = 32*TM channels x PIX = 128*TN output pixels, the pixels
// being TI images x TR rows x TC columns. Per chunk of KCH reduction channels it stages the
// input patch WITH its halo once in LDS ([kc][ti][TR+R-1][TC+S-1]) together with the filter
// slice ([tap][kc][m]); every filter tap then reads the same patch at a compile-time offset,
// so each input element is fetched from global memory once per workgroup instead of once per
// tap, and the inner loop is ds_read + v_mfma_f32_32x32x2_f32 only. The next chunk's global
// loads are issued before the current chunk's MFMAs and parked in registers.
//
// MFMA operand mapping: A = filter slice (lane: m = l%32, k = l/32 selects channel 2p or 2p+1),
// B = input patch (lane: pixel = l%32 of a 32-pixel block, k likewise), D = 32 channels x 32
// pixels. Stores are contiguous along pixels.
#include "common.h"

namespace tdh {

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int S1_NI_MAX = 24;  // input-patch elements a thread stages per chunk (at most)

struct ConvS1Args {
  const float *in, *wp, *bias;
  float *out;
  ActGrad ag;
  int batch, KC, MC, IH, IW, OH, OW, ph, pw;
  int TR, TI;                  // tile rows, images per tile (TI*TR*TC = PIX), powers of two
  int log_tr, log_ti;
  int tiles_x, tiles_y;        // tiles per image row / column direction
  FastDiv div_rows, div_pitch; // by (TR+R-1)*(TC+S-1) and by (TC+S-1)
  // split over the reduction channels: workgroup z sums channels [z*kc_split, (z+1)*kc_split)
  // into part[z][...] (laid out like out); part == nullptr: one pass, written to out
  int kc_split;
  float *part;
  size_t part_stride;
};

template <int R, int S, int TC, int KCH, int TM, int TN>
__global__ void __launch_bounds__(256, 2) conv_s1_kernel(const ConvS1Args a) {
  constexpr int RS    = R * S;
  constexpr int BM    = 32 * TM;
  constexpr int PIX   = 128 * TN;
  constexpr int PITCH = TC + S - 1;
  constexpr int TPC   = 256 / KCH;               // threads staging one channel plane
  constexpr int NWT   = RS * KCH * BM;           // filter elements per chunk
  constexpr int NW    = (NWT + 255) / 256;       // ... per thread
  constexpr int LOG_TC = TC == 64 ? 6 : TC == 32 ? 5 : TC == 16 ? 4 : 3;
  static_assert(PIX % TC == 0, "tile width must divide the pixel tile");

  extern __shared__ float smem[];
  const int TRH   = a.TR + R - 1;
  const int plane = a.TI * TRH * PITCH;          // one channel of the staged patch
  float *in_l     = smem;                        // [KCH][plane]
  float *w_l      = smem + KCH * plane;          // [RS][KCH][BM]

  const int tid = threadIdx.x, lane = tid & 63, wn = tid >> 6;
  // tile coordinates
  int bt          = blockIdx.x;
  const int tx    = bt % a.tiles_x;
  bt /= a.tiles_x;
  const int ty    = bt % a.tiles_y;
  const int tb    = bt / a.tiles_y;
  const int img0  = tb << a.log_ti;
  const int y0    = ty << a.log_tr;
  const int x0    = tx * TC;
  const int m0    = blockIdx.y * BM;
  const int ihw   = a.IH * a.IW;
  const int kc_lo = blockIdx.z * a.kc_split;
  const int kc_hi = min(a.KC, kc_lo + a.kc_split);

  // ---- staging plan of the input patch: thread -> channel kcl, elements tl + TPC*i of a plane
  const int kcl = tid / TPC, tl = tid % TPC;
  const int ni  = (plane + TPC - 1) / TPC;
  int goff[S1_NI_MAX];
  unsigned vmask = 0;
  {
#pragma unroll
    for (int i = 0; i < S1_NI_MAX; ++i) {
      goff[i] = 0;
      const int pe = tl + TPC * i;
      if (i < ni && pe < plane) {
        uint32_t ti, rem, r, c;
        a.div_rows.divmod(pe, ti, rem);
        a.div_pitch.divmod(rem, r, c);
        const int img = img0 + ti, iy = y0 - a.ph + static_cast<int>(r),
                  ix = x0 - a.pw + static_cast<int>(c);
        if (img < a.batch && static_cast<unsigned>(iy) < static_cast<unsigned>(a.IH) &&
            static_cast<unsigned>(ix) < static_cast<unsigned>(a.IW)) {
          vmask |= 1u << i;
          goff[i] = img * a.KC * ihw + iy * a.IW + ix;
        }
      }
    }
  }

  // ---- MFMA operand offsets
  int boff[TN];
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int q  = (wn * TN + j) * 32 + (lane & 31);
    const int ti = q >> (a.log_tr + LOG_TC);
    const int r  = (q >> LOG_TC) & (a.TR - 1);
    const int c  = q & (TC - 1);
    boff[j]      = (ti * TRH + r) * PITCH + c + (lane >> 5) * plane;
  }
  const int aoff = (lane >> 5) * BM + (lane & 31);

  floatx16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  float rin[S1_NI_MAX], rw[NW];

  auto fetch = [&](int kc0) {
    const bool ch_ok  = kc0 + kcl < kc_hi;
    const float *base = a.in + static_cast<size_t>(kc0 + kcl) * ihw;
#pragma unroll
    for (int i = 0; i < S1_NI_MAX; ++i)
      rin[i] = (i < ni && ch_ok && ((vmask >> i) & 1u)) ? base[goff[i]] : 0.0f;
#pragma unroll
    for (int i = 0; i < NW; ++i) {
      const int e = tid + 256 * i;
      const int m = e % BM, kcw = (e / BM) % KCH, t = e / (BM * KCH);
      const bool ok = (e < NWT) && (kc0 + kcw < kc_hi) && (m0 + m < a.MC);
      rw[i] = ok ? a.wp[(static_cast<size_t>(t) * a.KC + kc0 + kcw) * a.MC + m0 + m] : 0.0f;
    }
  };
  auto stage = [&]() {
#pragma unroll
    for (int i = 0; i < S1_NI_MAX; ++i) {
      const int pe = tl + TPC * i;
      if (i < ni && pe < plane) in_l[kcl * plane + pe] = rin[i];
    }
#pragma unroll
    for (int i = 0; i < NW; ++i)
      if (tid + 256 * i < NWT) w_l[tid + 256 * i] = rw[i];
  };

  fetch(kc_lo);
  for (int kc0 = kc_lo; kc0 < kc_hi; kc0 += KCH) {
    if (kc0 > kc_lo) __syncthreads();  // everyone is done reading the previous chunk
    stage();
    __syncthreads();
    if (kc0 + KCH < kc_hi) fetch(kc0 + KCH);
#pragma unroll
    for (int p = 0; p < KCH / 2; ++p) {
      const float *inp = in_l + 2 * p * plane;
      const float *wlp = w_l + 2 * p * BM + aoff;
#pragma unroll
      for (int t = 0; t < RS; ++t) {
        const int fy = t / S, fx = t % S;
        float af[TM], bf[TN];
#pragma unroll
        for (int i = 0; i < TM; ++i) af[i] = wlp[t * KCH * BM + i * 32];
#pragma unroll
        for (int j = 0; j < TN; ++j) bf[j] = inp[boff[j] + fy * PITCH + fx];
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i], bf[j], acc[i][j], 0, 0, 0);
      }
    }
  }

  // ---- epilogue: reg r of lane l holds channel 8*(r/4) + 4*(l/32) + r%4, pixel l%32
  const int ohw = a.OH * a.OW;
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int q   = (wn * TN + j) * 32 + (lane & 31);
    const int ti  = q >> (a.log_tr + LOG_TC);
    const int r   = (q >> LOG_TC) & (a.TR - 1);
    const int c   = q & (TC - 1);
    const int img = img0 + ti, oy = y0 + r, ox = x0 + c;
    if (img >= a.batch || oy >= a.OH || ox >= a.OW) continue;
    const size_t pbase = static_cast<size_t>(img) * a.MC * ohw + oy * a.OW + ox;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int rr = 0; rr < 16; ++rr) {
        const int m = m0 + 32 * i + 8 * (rr >> 2) + 4 * (lane >> 5) + (rr & 3);
        if (m >= a.MC) continue;
        const size_t idx = pbase + static_cast<size_t>(m) * ohw;
        float v = acc[i][j][rr];
        if (a.part) {
          a.part[blockIdx.z * a.part_stride + idx] = v;
          continue;
        }
        if (a.bias) v += a.bias[m];
        if (a.ag.kind != TDH_ACT_NONE) v *= act_grad_factor(a.ag.kind, a.ag.y[idx]);
        a.out[idx] = v;
      }
  }
}

// out = part[0] + part[1] + ... (in this order) (+ bias[m]) (* act'(y)); four elements per
// thread when a channel plane is a multiple of four
template <int VEC>
__global__ void __launch_bounds__(256)
s1_split_reduce_kernel(const float *__restrict__ part, const int splits, const size_t stride,
                       float *__restrict__ out, const float *__restrict__ bias, const ActGrad ag,
                       const int MC, const FastDiv div_plane, const size_t total) {
  const size_t i = (static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x) * VEC;
  if (i >= total) return;
  float v[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) v[e] = 0.0f;
  for (int z = 0; z < splits; ++z) {
    if (VEC == 4) {
      const float4 f = *reinterpret_cast<const float4 *>(part + z * stride + i);
      v[0] += f.x; v[1] += f.y; v[2] += f.z; v[VEC - 1] += f.w;
    } else {
      v[0] += part[z * stride + i];
    }
  }
  const int m = div_plane.div(static_cast<uint32_t>(i)) % MC;  // the plane of all VEC elements
  const float b = bias ? bias[m] : 0.0f;
#pragma unroll
  for (int e = 0; e < VEC; ++e) {
    v[e] += b;
    if (ag.kind != TDH_ACT_NONE) v[e] *= act_grad_factor(ag.kind, ag.y[i + e]);
  }
  if (VEC == 4)
    *reinterpret_cast<float4 *>(out + i) = make_float4(v[0], v[1], v[2], v[VEC - 1]);
  else
    out[i] = v[0];
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

struct S1Plan {
  bool ok;
  int tc, kch, tm, tn;
  ConvS1Args args;
  size_t lds_bytes;
  dim3 grid;
  int splits;
};

// Splits the reduction channels over grid.z when the tiles alone leave most of the chip idle.
void choose_split(S1Plan &p, long blocks) {
  const int nchunks = ceil_div(p.args.KC, p.kch);
  int splits = 1;
  if (blocks < 384 && nchunks >= 4) {
    splits = static_cast<int>(std::min<long>(8, (512 + blocks - 1) / blocks));
    splits = std::min(splits, nchunks / 2);
  }
  const int per      = ceil_div(nchunks, splits) * p.kch;
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
  if (MC < 16 || OW < 4 || OH < 1) return best;
  static const int cand_wide[3][2]   = {{2, 2}, {2, 1}, {1, 1}};  // MC > 32
  static const int cand_narrow[3][2] = {{1, 4}, {1, 2}, {1, 1}};  // MC <= 32
  long best_blocks = 0;
  for (int ci = 0; ci < 3; ++ci) {
    S1Plan p;
    p.ok = false;
    p.tc = OW >= 48 ? 64 : OW >= 24 ? 32 : OW >= 12 ? 16 : 8;
    p.tm = MC > 32 ? cand_wide[ci][0] : cand_narrow[ci][0];
    p.tn = MC > 32 ? cand_wide[ci][1] : cand_narrow[ci][1];
    p.kch = (R == 5 || KC <= 4) ? 4 : 8;
    const int pix = 128 * p.tn;
    if (pix < p.tc) continue;
    int tr = pix / p.tc;
    if (tr > pow2_ceil(OH)) tr = pow2_ceil(OH);
    const int ti = pix / (tr * p.tc);
    ConvS1Args &a = p.args;
    a.batch = batch; a.KC = KC; a.MC = MC; a.IH = IH; a.IW = IW; a.OH = OH; a.OW = OW;
    a.ph = ph; a.pw = pw;
    a.TR = tr; a.TI = ti; a.log_tr = ilog2(tr); a.log_ti = ilog2(ti);
    a.tiles_x = ceil_div(OW, p.tc);
    a.tiles_y = ceil_div(OH, tr);
    const int plane = ti * (tr + R - 1) * (p.tc + S - 1);
    const int tpc   = 256 / p.kch;
    a.div_rows  = FastDiv((tr + R - 1) * (p.tc + S - 1));
    a.div_pitch = FastDiv(p.tc + S - 1);
    if (ceil_div(plane, tpc) > S1_NI_MAX) continue;
    p.lds_bytes = sizeof(float) * (static_cast<size_t>(p.kch) * plane + R * S * p.kch * 32 * p.tm);
    if (p.lds_bytes > 64 * 1024) continue;
    const long tiles  = static_cast<long>(a.tiles_x) * a.tiles_y * ceil_div(batch, ti);
    const long blocks = tiles * ceil_div(MC, 32 * p.tm);
    if (tiles > 2000000000L) continue;
    p.grid = dim3(static_cast<unsigned>(tiles), ceil_div(MC, 32 * p.tm), 1);
    p.ok   = true;
    choose_split(p, blocks);
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

template <int R, int S, int TC>
int launch_s1_tc(const S1Plan &p) {
  const ConvS1Args &a = p.args;
#define TDH_S1(KCH, TM, TN)                                                                     \
  hipLaunchKernelGGL((conv_s1_kernel<R, S, TC, KCH, TM, TN>), p.grid, dim3(256), p.lds_bytes,   \
                     ctx().stream, a)
  const int shape = p.tm * 10 + p.tn;
  if (p.kch == 8) {
    switch (shape) {
      case 22: TDH_S1(8, 2, 2); break;
      case 21: TDH_S1(8, 2, 1); break;
      case 14: TDH_S1(8, 1, 4); break;
      case 12: TDH_S1(8, 1, 2); break;
      default: TDH_S1(8, 1, 1); break;
    }
  } else {
    switch (shape) {
      case 22: TDH_S1(4, 2, 2); break;
      case 21: TDH_S1(4, 2, 1); break;
      case 14: TDH_S1(4, 1, 4); break;
      case 12: TDH_S1(4, 1, 2); break;
      default: TDH_S1(4, 1, 1); break;
    }
  }
#undef TDH_S1
  TDH_LAUNCH_CHECK();
  return TDH_OK;
}

template <int R, int S>
int launch_s1_rs(const S1Plan &p) {
  switch (p.tc) {
    case 64: return launch_s1_tc<R, S, 64>(p);
    case 32: return launch_s1_tc<R, S, 32>(p);
    case 16: return launch_s1_tc<R, S, 16>(p);
    default: return launch_s1_tc<R, S, 8>(p);
  }
}

}  // namespace

bool conv_s1_applicable(int R, int S, int batch, int KC, int MC, int IH, int IW, int OH, int OW,
                        int ph, int pw) {
  return make_plan(R, S, batch, KC, MC, IH, IW, OH, OW, ph, pw).ok;
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
  hipLaunchKernelGGL(repack_weights_kernel, dim3(ceil_div(R * S * C * Kc, 256)), dim3(256), 0,
                     ctx().stream, w, tbl_dev, wp, C, Kc, R * S, flip);
  TDH_LAUNCH_CHECK();
  return TDH_OK;
}

// Runs out = conv(in, repack(w)) (+ bias) (* act'(y)); the caller has checked applicability
// and reserved conv_s1_workspace_bytes of scratch. flip = 0: forward, 1: dX. prepacked: the
// result of conv_s1_repack for this filter, when the caller already has it (w is not read).
int conv_s1_run(int R, int S, int batch, int C, int Kc, int flip, const float *in, const float *w,
                const uint8_t *tbl_dev, const float *bias, float *out, int IH, int IW, int OH,
                int OW, int ph, int pw, ActGrad ag, const char *tag, const float *prepacked) {
  const int KC = flip ? Kc : C, MC = flip ? C : Kc;
  S1Plan p = make_plan(R, S, batch, KC, MC, IH, IW, OH, OW, ph, pw);
  if (!p.ok) return set_error(TDH_ERR_INVALID, "conv_s1_run: shape not supported");
  const void *wp = prepacked;
  if (!prepacked) {
    void *fresh = nullptr;
    TDH_TRY(ws_take(sizeof(float) * static_cast<size_t>(R) * S * C * Kc, &fresh));
    TDH_TRY(conv_s1_repack(R, S, C, Kc, flip, w, tbl_dev, static_cast<float *>(fresh)));
    wp = fresh;
  }
  p.args.in = in; p.args.wp = static_cast<const float *>(wp); p.args.bias = bias;
  p.args.out = out; p.args.ag = ag;
  if (p.splits > 1) {
    void *part = nullptr;
    TDH_TRY(ws_take(sizeof(float) * p.splits * p.args.part_stride, &part));
    p.args.part = static_cast<float *>(part);
  }
  {
    ProfScope prof(tag, MC, batch * OH * OW, KC * R * S);
    TDH_TRY(R == 3 ? (launch_s1_rs<3, 3>(p)) : (launch_s1_rs<5, 5>(p)));
  }
  if (p.splits > 1) {
    const size_t total = p.args.part_stride;
    const int plane    = OH * OW;
    ProfScope prof("conv_s1_split_reduce", 4.0 * total * (p.splits + 1 + (ag.kind != TDH_ACT_NONE)),
                   WORK_BYTE);
    if (plane % 4 == 0)
      hipLaunchKernelGGL((s1_split_reduce_kernel<4>), dim3(static_cast<unsigned>(ceil_div_sz(total / 4, 256))), dim3(256), 0,
                         ctx().stream, p.args.part, p.splits, total, out, bias, ag, MC,
                         FastDiv(plane), total);
    else
      hipLaunchKernelGGL((s1_split_reduce_kernel<1>), dim3(static_cast<unsigned>(ceil_div_sz(total, 256))), dim3(256), 0,
                         ctx().stream, p.args.part, p.splits, total, out, bias, ag, MC,
                         FastDiv(plane), total);
    TDH_LAUNCH_CHECK();
  }
  return TDH_OK;
}

}  // namespace tdh
