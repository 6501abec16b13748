// conv_dw_small.hip — weight and bias gradient of a convolution with few input channels
// (Cin*KH*KW + 1 <= 96: the first layer of an image net), any stride and dilation.
//
//   dW[co][ci,ky,kx] = sum over (img, oy, ox) of dY[img][co][oy][ox] * X[img][ci][iy][ix]
//   db[co]           = sum over (img, oy, ox) of dY[img][co][oy][ox]
//
// As a product the shape is M = Cout, N = Cin*KH*KW (75 for 3 channels and 5x5), K = batch*OH*OW:
// a tile of a general GEMM kernel is mostly padding in N, and its B operand is gathered from
// global memory element by element. Here a workgroup owns a band of output rows of one image.
// It stages the input patch under the band (zero-filled where the window leaves the image) once
// and the band of dY chunk by chunk into LDS, a thread's loads all in flight together and the
// next chunk's issued before the current chunk is multiplied, and then every MFMA
// (v_mfma_f32_32x32x2_f32: A lane = (co, k), B lane = (n, k)) takes its B value with one LDS read
// at patch[pos(k)] + offset(n); offset(n) is a per-lane constant. Column N of the product has
// B = 1: it is the bias gradient, which so costs no pass over dY of its own. The four waves of
// a workgroup split the band's positions; their accumulators are added through LDS and the
// workgroup writes one partial dW (and db) which a split reduction adds in a fixed order.
//
// Reference: conv2d_op_internal.h:127-180 (dW accumulation and db).
#include <algorithm>

#include "gemm_mfma.h"

namespace tdh {

namespace {

typedef float floatx4 __attribute__((ext_vector_type(4)));

struct DwSmallArgs {
  const float *x, *dy;
  float *partial_dw, *partial_db;  // [blocks][Kc][crs], [blocks][Kc] (db may be null)
  int C, Kc, H, W, OH, OW;
  int R, S, sh, sw, dh, dw, ph, pw;
  int band, bands;      // output rows per workgroup, workgroups per image
  int chunk;            // output rows staged and multiplied at a time (chunk*OW <= 256)
  int rows_in, pitch;   // staged patch: rows per channel, floats per row
  int plane;            // floats per channel in LDS
  int dy_pitch;         // floats per output channel of a staged dY chunk
  int crs;
  int x_floats;         // LDS floats in front of the two dY buffers
  int dy_floats;        // LDS floats of one dY buffer
  FastDiv div_pitch, div_rows_in, div_quads, div_ow;
  // dY given through a 2x2 max-pool (POOLED kernels): pooled gradient and argmax records
  const float *pool_g;
  const int32_t *pool_argmax;
  FastDiv div_units, div_ow4;  // units of two pooled elements per channel and chunk; per pooled row
};

// A workgroup walks its band in chunks of rows. The dY rows of the next chunk are loaded into
// registers while the MFMAs of the current one run, and go to the other of two LDS buffers.
// POOLED: dY is not in memory; a thread loads two adjacent elements of the pooled gradient with
// their argmax records (half the bytes of the 2x4 block of dY that they stand for) and routes
// them into that block on the way to LDS. Bands and chunks hold an even number of rows then.
template <int NT, bool POOLED>
__global__ void __launch_bounds__(256, 2) conv_dw_small_kernel(const DwSmallArgs a) {
  extern __shared__ __align__(16) float lds[];
  float *xs  = lds;
  float *dys = lds + a.x_floats;  // two chunk buffers; later the accumulators of the four waves
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // (an image's bands share rows: they go to one XCD)
  const int wg = xcd_compact_id(blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z),
                                gridDim.x * gridDim.y * gridDim.z);
  const int bandi = wg % gridDim.x, img = (wg / gridDim.x) % gridDim.y, co0 = (wg / (gridDim.x * gridDim.y)) * 32;
  const int oy0   = bandi * a.band;
  const int rows_here = min(a.band, a.OH - oy0);
  const int nchunks   = (rows_here + a.chunk - 1) / a.chunk;

  // ---- staging. A thread issues all its loads of a stage before it stores any of them, so
  // that their latencies overlap; zero where the window leaves the image, for output channels
  // past Cout and for rows past the band.
  const int iy0     = oy0 * a.sh - a.ph;
  const int x_total = a.C * a.rows_in * a.pitch;
  const int quads   = a.chunk * a.OW / 4;  // per output channel and chunk
  constexpr int DEPTH = 8;
  float xv[DEPTH];
  int xo[DEPTH];
  floatx4 dv[DEPTH];
  auto load_x = [&](int e0) {
#pragma unroll
    for (int k = 0; k < DEPTH; ++k) {
      const int e = e0 + k * 256;
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
  };
  auto store_x = [&]() {
#pragma unroll
    for (int k = 0; k < DEPTH; ++k)
      if (xo[k] >= 0) xs[xo[k]] = xv[k];
  };
  // chunk c of the band: 32 output channels x quads 16-byte pieces, at most DEPTH per thread
  const int units = quads / 2;  // POOLED: 2x4 blocks of dY per output channel and chunk
  auto load_dy = [&](int c) {
    const int row0     = c * a.chunk;
    const int quads_ok = min(a.chunk, rows_here - row0) * a.OW / 4;
    if (POOLED) {
      const int poh = a.OH >> 1, pow_ = a.OW >> 1;
#pragma unroll
      for (int k = 0; k < DEPTH / 2; ++k) {
        const int u = tid + k * 256;
        dv[k] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
        if (u < 32 * units) {
          const int m = a.div_units.div(u), r = u - m * units;
          if (co0 + m < a.Kc && 2 * r < quads_ok) {
            const int pr = a.div_ow4.div(r), pc = r - pr * (a.OW >> 2);
            const size_t o = (static_cast<size_t>(img * a.Kc + co0 + m) * poh + ((oy0 + row0) >> 1) + pr) * pow_ + 2 * pc;
            const float2 g2 = *reinterpret_cast<const float2 *>(a.pool_g + o);
            const int2 a2   = *reinterpret_cast<const int2 *>(a.pool_argmax + o);
            dv[k] = floatx4{g2.x, g2.y, __int_as_float(a2.x), __int_as_float(a2.y)};
          }
        }
      }
      return;
    }
#pragma unroll
    for (int k = 0; k < DEPTH; ++k) {
      const int q = tid + k * 256;
      dv[k] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
      if (q < 32 * quads) {
        const int m = a.div_quads.div(q), c4 = q - m * quads;
        if (co0 + m < a.Kc && c4 < quads_ok)
          dv[k] = *reinterpret_cast<const floatx4 *>(
              a.dy + (static_cast<size_t>(img * a.Kc + co0 + m) * a.OH + oy0 + row0) * a.OW + c4 * 4);
      }
    }
  };
  auto store_dy = [&](float *buf, int c) {
    if (POOLED) {
      const int row0 = c * a.chunk;
#pragma unroll
      for (int k = 0; k < DEPTH / 2; ++k) {
        const int u = tid + k * 256;
        if (u < 32 * units) {
          const int m = a.div_units.div(u), r = u - m * units;
          const int pr = a.div_ow4.div(r), pc = r - pr * (a.OW >> 2);
          // flat index of the block's top left element inside the sample, as the records hold it
          const int at = ((co0 + m) * a.OH + oy0 + row0 + 2 * pr) * a.OW + 4 * pc;
          const float gx = dv[k][0], gy = dv[k][1];
          const int ax = __float_as_int(dv[k][2]) - at, ay = __float_as_int(dv[k][3]) - at;
          float *dst = buf + m * a.dy_pitch + 2 * pr * a.OW + 4 * pc;
          *reinterpret_cast<floatx4 *>(dst) =
            floatx4{ax == 0 ? gx : 0.0f, ax == 1 ? gx : 0.0f, ay == 2 ? gy : 0.0f, ay == 3 ? gy : 0.0f};
          *reinterpret_cast<floatx4 *>(dst + a.OW) =
            floatx4{ax == a.OW ? gx : 0.0f, ax == a.OW + 1 ? gx : 0.0f, ay == a.OW + 2 ? gy : 0.0f,
                    ay == a.OW + 3 ? gy : 0.0f};
        }
      }
      return;
    }
#pragma unroll
    for (int k = 0; k < DEPTH; ++k) {
      const int q = tid + k * 256;
      if (q < 32 * quads) {
        const int m = a.div_quads.div(q), c4 = q - m * quads;
        *reinterpret_cast<floatx4 *>(buf + m * a.dy_pitch + c4 * 4) = dv[k];
      }
    }
  };
  load_dy(0);
  load_x(tid);
  // ---- per-lane constants of the B gather (worked out while the first loads are on their way)
  const int nl = lane & 31, half = lane >> 5;
  int off[NT];
  bool ones[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int n = t * 32 + nl;
    ones[t]     = n == a.crs;
    int o       = 0;
    if (n < a.crs) {
      const int rs = a.R * a.S;
      const int ci = n / rs, tap = n - ci * rs;
      const int ky = tap / a.S, kx = tap - ky * a.S;
      o = ci * a.plane + ky * a.dh * a.pitch + kx * a.dw;
    }
    off[t] = o;
  }
  store_dy(dys, 0);
  store_x();
  for (int e0 = tid + DEPTH * 256; e0 < x_total; e0 += DEPTH * 256) {
    load_x(e0);
    store_x();
  }
  floatx16 acc[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[t][i] = 0.0f;
  __syncthreads();

  // ---- products: a half wave takes four consecutive positions of one output row per trip
  for (int c = 0; c < nchunks; ++c) {
    const bool more = c + 1 < nchunks;
    if (more) load_dy(c + 1);
    const float *arow = dys + (c & 1) * a.dy_floats + nl * a.dy_pitch;
    const int row0    = c * a.chunk;
    const int units   = min(a.chunk, rows_here - row0) * a.OW / 4;
    const int trips   = (units + 7) / 8;
    for (int it = 0; it < trips; ++it) {
      const int u   = it * 8 + wave * 2 + half;
      const bool ok = u < units;
      const int pos = ok ? u * 4 : 0;
      const int oy  = a.div_ow.div(pos), ox = pos - oy * a.OW;
      floatx4 av    = *reinterpret_cast<const floatx4 *>(arow + pos);
      if (!ok) av = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
      const float *xb = xs + (row0 + oy) * a.sh * a.pitch + ox * a.sw;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
#pragma unroll
        for (int t = 0; t < NT; ++t) {
          float b = xb[j * a.sw + off[t]];
          b       = ones[t] ? 1.0f : b;
          acc[t]  = __builtin_amdgcn_mfma_f32_32x32x2f32(av[j], b, acc[t], 0, 0, 0);
        }
      }
    }
    if (more) store_dy(dys + ((c + 1) & 1) * a.dy_floats, c + 1);
    __syncthreads();  // the next chunk is in place; every wave is done with this one
  }

  // ---- add the four waves' accumulators and write this workgroup's partial
  constexpr int TILE = 32 * 32 * NT;
  float *red = dys + wave * TILE;
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int m = (i >> 2) * 8 + half * 4 + (i & 3);
      red[m * (32 * NT) + t * 32 + nl] = acc[t][i];
    }
  __syncthreads();
  const int blk = img * a.bands + bandi;
  // (all LDS reads of a thread first: read, add and store one output at a time is twelve trips
  // to LDS one after the other)
  float sums[TILE / 256];
#pragma unroll
  for (int i = 0; i < TILE / 256; ++i) {
    const int e = tid + 256 * i;
    sums[i]     = (dys[e] + dys[TILE + e]) + (dys[2 * TILE + e] + dys[3 * TILE + e]);
  }
#pragma unroll
  for (int i = 0; i < TILE / 256; ++i) {
    const int e = tid + 256 * i;
    const int m = e / (32 * NT), n = e - m * (32 * NT);
    if (co0 + m >= a.Kc || n > a.crs) continue;
    if (n < a.crs)
      a.partial_dw[(static_cast<size_t>(blk) * a.Kc + co0 + m) * a.crs + n] = sums[i];
    else if (a.partial_db)
      a.partial_db[static_cast<size_t>(blk) * a.Kc + co0 + m] = sums[i];
  }
}

struct DwSmallPlan {
  DwSmallArgs a;
  int nt;
  size_t lds_bytes;
  dim3 grid;
  bool ok;
};

// even_rows: bands and chunks of an even number of rows (what the POOLED kernels need);
// force_band > 0: bands of that many rows (the bands of the kernel that computes this gradient
// together with the layer's dX, so that the same sums come out with and without the dX)
DwSmallPlan make_dw_small_plan(int batch, int C, int Kc, int H, int W, int OH, int OW, int R, int S,
                               int sh, int sw, int dh, int dw, int ph, int pw, bool even_rows = false,
                               int force_band = 0) {
  DwSmallPlan p;
  p.ok = false;
  DwSmallArgs &a = p.a;
  a.x = a.dy = nullptr;
  a.partial_dw = a.partial_db = nullptr;
  a.C = C; a.Kc = Kc; a.H = H; a.W = W; a.OH = OH; a.OW = OW;
  a.R = R; a.S = S; a.sh = sh; a.sw = sw; a.dh = dh; a.dw = dw; a.ph = ph; a.pw = pw;
  a.crs = C * R * S;
  p.nt  = ceil_div(a.crs + 1, 32);
  if (p.nt > 3 || OW % 4 != 0 || OH < 1 || batch < 1 || batch > 65535) return p;
  if (even_rows && (OH % 2 != 0 || OW > 128)) return p;
  a.pitch = (OW - 1) * sw + (S - 1) * dw + 1;
  a.pitch |= 1;  // odd: the taps of one column fall into different LDS banks
  const int co_tiles = ceil_div(Kc, 32);
  if (co_tiles > 65535) return p;
  const int cus = ctx().compute_units > 0 ? ctx().compute_units : 256;
  // rows per chunk: at most 256 positions (eight 16-byte loads per thread); two chunks per band
  // where the band allows, so that loading overlaps the products
  const size_t reduce_fl = 4u * 32 * 32 * p.nt;
  int chunk_cap = std::max(1, 256 / OW);  // rows per chunk at most
  auto chunk_of = [&](int band) {
    int c = std::max(1, std::min(band, chunk_cap));
    if (c == band && band > 1) c = (band + 1) / 2;
    if (even_rows) c = std::max(2, c & ~1);
    return c;
  };
  auto lds_floats = [&](int band) {
    const int rows_in = (band - 1) * sh + (R - 1) * dh + 1;
    const size_t x_fl = (static_cast<size_t>(C) * (rows_in * a.pitch + 1) + 3) & ~static_cast<size_t>(3);
    const size_t dy_fl = 2u * 32 * (static_cast<size_t>(chunk_of(band)) * OW + 4);
    return x_fl + std::max(dy_fl, reduce_fl);
  };
  if (OW > 256) return p;
  // the largest band whose LDS fits twice per compute unit and that gives two workgroups per
  // compute unit; a band is not made shorter than 256 positions for that
  auto best_band = [&]() {
    int best = 0;
    for (int band = OH; band >= 1; --band) {
      if (even_rows && band % 2 != 0) continue;
      if (lds_floats(band) * sizeof(float) > 72 * 1024) continue;
      best = band;
      if (static_cast<long long>(batch) * ceil_div(OH, band) * co_tiles >= 2LL * cus || band * OW <= 256)
        break;
    }
    return best;
  };
  // Wide rows: two chunk buffers of 256 positions leave LDS for a patch of two or three rows,
  // and every workgroup then pays its prologue, its reduction over the waves and a partial
  // slice for 256 positions (128-column images at batch 64: 8192 slices, 29 MB). Shorter
  // chunks buy a longer band: taken where that at least doubles the band.
  int best = best_band();
  for (int cap = chunk_cap / 2; cap >= (even_rows ? 2 : 1); cap /= 2) {
    const int keep = chunk_cap;
    chunk_cap      = cap;
    const int b    = best_band();
    if (b >= 2 * best && b > 0) best = b;
    else chunk_cap = keep;
  }
  if (best == 0) return p;
  {
    // a few bands more where that fills the last round of workgroups (two per compute unit run
    // at a time): 768 workgroups are two rounds just as 1024 are
    const long long slots = 2LL * cus;
    auto fill = [&](int nb) {
      const long long wgs = static_cast<long long>(batch) * nb * co_tiles;
      return static_cast<double>(wgs) / static_cast<double>((wgs + slots - 1) / slots * slots);
    };
    int nb = ceil_div(OH, best), pick = nb;
    for (int more = nb + 1; more <= std::min(OH, nb + nb / 2 + 1) && fill(pick) < 0.9; ++more)
      if (fill(more) > fill(pick) + 0.05) pick = more;
    if (pick != nb) {
      int band = ceil_div(OH, pick);
      if (even_rows && band % 2 != 0) ++band;
      best = std::min(best, band);
    }
  }
  {
    // the same number of bands, the rows spread evenly: 32 rows in bands of 10 are 10 + 10 +
    // 10 + 2, and the workgroups of the last band idle while the others multiply
    int even = ceil_div(OH, ceil_div(OH, best));
    if (even_rows && even % 2 != 0) ++even;
    best = std::min(best, even);
  }
  if (force_band > 0) {
    chunk_cap = std::max(1, 256 / OW);
    if ((even_rows && force_band % 2 != 0) || lds_floats(force_band) * sizeof(float) > 72 * 1024) return p;
    best = force_band;
  }
  a.band    = best;
  a.bands   = ceil_div(OH, best);
  a.chunk   = chunk_of(best);
  a.rows_in = (best - 1) * sh + (R - 1) * dh + 1;
  a.plane   = a.rows_in * a.pitch + 1;
  a.x_floats  = static_cast<int>((static_cast<size_t>(C) * a.plane + 3) & ~static_cast<size_t>(3));
  a.dy_pitch  = a.chunk * OW + 4;
  a.dy_floats = 32 * a.dy_pitch;
  a.div_pitch   = FastDiv(a.pitch);
  a.div_rows_in = FastDiv(a.rows_in);
  a.div_quads   = FastDiv(a.chunk * OW / 4);
  a.div_ow      = FastDiv(OW);
  a.pool_g      = nullptr;
  a.pool_argmax = nullptr;
  a.div_units   = FastDiv(std::max(1, a.chunk * OW / 8));
  a.div_ow4     = FastDiv(OW / 4);
  p.lds_bytes = lds_floats(best) * sizeof(float);
  p.grid      = dim3(a.bands, batch, co_tiles);
  if (static_cast<long long>(batch) * a.bands > (1 << 20)) return p;
  p.ok = true;
  return p;
}

template <int NT, bool POOLED>
int launch_dw_small(const DwSmallPlan &p) {
  static bool raised = false;
  if (!raised) {  // more than the 64 KB a kernel may use without asking
    TDH_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&conv_dw_small_kernel<NT, POOLED>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, 72 * 1024));
    raised = true;
  }
  TDH_LAUNCH((conv_dw_small_kernel<NT, POOLED>), p.grid, dim3(256), p.lds_bytes, ctx().stream, p.a);
  TDH_LAUNCH_CHECK();
  return TDH_OK;
}

}  // namespace

bool conv_dw_small_applicable(int batch, int C, int Kc, int H, int W, int OH, int OW, int R, int S,
                              int sh, int sw, int dh, int dw, int ph, int pw) {
  return make_dw_small_plan(batch, C, Kc, H, W, OH, OW, R, S, sh, sw, dh, dw, ph, pw).ok;
}

size_t conv_dw_small_workspace_bytes(int batch, int C, int Kc, int H, int W, int OH, int OW, int R,
                                     int S, int sh, int sw, int dh, int dw, int ph, int pw) {
  size_t most = 0;
  for (int even = 0; even < 2; ++even) {  // (a layer may run either kernel)
    const DwSmallPlan p = make_dw_small_plan(batch, C, Kc, H, W, OH, OW, R, S, sh, sw, dh, dw, ph, pw, even != 0);
    if (!p.ok) continue;
    const size_t blocks = static_cast<size_t>(batch) * p.a.bands;
    most = std::max(most, ws_align(blocks * Kc * p.a.crs * sizeof(float)) + ws_align(blocks * Kc * sizeof(float)));
  }
  return most;
}

// the kernel can read dY through a 2x2 / stride-2 max-pool over the layer's output: whole 2x4
// blocks per band and chunk, records that fit an int
bool conv_dw_small_reads_pooled(int batch, int C, int Kc, int H, int W, int OH, int OW, int R, int S,
                                int sh, int sw, int dh, int dw, int ph, int pw) {
  const DwSmallPlan p = make_dw_small_plan(batch, C, Kc, H, W, OH, OW, R, S, sh, sw, dh, dw, ph, pw, true);
  return p.ok && p.a.band % 2 == 0 && p.a.chunk % 2 == 0 && static_cast<long long>(Kc) * OH * OW < (1LL << 30);
}

// dw (required) and db (optional) of one layer; both follow `accumulate`.
int conv_dw_small_run(int batch, int C, int Kc, const float *x, const float *dy, float *dw_out,
                      float *db_out, int H, int W, int OH, int OW, int R, int S, int sh, int sw, int dh,
                      int dw, int ph, int pw, int accumulate, const PoolGather *dy_pool, int force_band) {
  DwSmallPlan p = make_dw_small_plan(batch, C, Kc, H, W, OH, OW, R, S, sh, sw, dh, dw, ph, pw, dy_pool != nullptr);
  if (force_band > 0) {  // (the hint is dropped where the kernel cannot follow it)
    const DwSmallPlan forced =
        make_dw_small_plan(batch, C, Kc, H, W, OH, OW, R, S, sh, sw, dh, dw, ph, pw, dy_pool != nullptr, force_band);
    if (forced.ok && forced.a.chunk * OW % 32 == 0) p = forced;
  }
  if (dy_pool) {
    if (!conv_dw_small_reads_pooled(batch, C, Kc, H, W, OH, OW, R, S, sh, sw, dh, dw, ph, pw) || p.a.band % 2 != 0 ||
        p.a.chunk % 2 != 0 ||
        !dy_pool->g || !dy_pool->argmax || (reinterpret_cast<uintptr_t>(dy_pool->g) & 7) ||
        (reinterpret_cast<uintptr_t>(dy_pool->argmax) & 7))
      return set_error(TDH_ERR_INVALID, "conv_dw_small_run: the pooled gradient cannot be read for this shape");
    p.a.pool_g      = dy_pool->g;
    p.a.pool_argmax = dy_pool->argmax;
  } else if (!p.ok || (reinterpret_cast<uintptr_t>(dy) & 15)) {
    return set_error(TDH_ERR_INVALID, "conv_dw_small_run: shape or alignment not supported");
  }
  const int blocks = batch * p.a.bands;
  void *pw_ws = nullptr, *pb_ws = nullptr;
  TDH_TRY(ws_take(static_cast<size_t>(blocks) * Kc * p.a.crs * sizeof(float), &pw_ws));
  if (db_out) TDH_TRY(ws_take(static_cast<size_t>(blocks) * Kc * sizeof(float), &pb_ws));
  p.a.x = x;
  p.a.dy = dy;
  p.a.partial_dw = static_cast<float *>(pw_ws);
  p.a.partial_db = static_cast<float *>(pb_ws);
  {
    ProfScope prof("conv_dw_small", Kc, p.a.crs + (db_out ? 1 : 0), batch * OH * OW);
    if (dy_pool) {
      switch (p.nt) {
        case 1: TDH_TRY((launch_dw_small<1, true>(p))); break;
        case 2: TDH_TRY((launch_dw_small<2, true>(p))); break;
        default: TDH_TRY((launch_dw_small<3, true>(p))); break;
      }
    } else {
      switch (p.nt) {
        case 1: TDH_TRY((launch_dw_small<1, false>(p))); break;
        case 2: TDH_TRY((launch_dw_small<2, false>(p))); break;
        default: TDH_TRY((launch_dw_small<3, false>(p))); break;
      }
    }
  }
  EpiRowMajor epi_w{dw_out, p.a.crs, nullptr, ActGrad(), accumulate};
  EpiRowMajor epi_b{db_out, 1, nullptr, ActGrad(), accumulate};
  // the two reductions leave as one launch: collected by the train step, or here
  const bool collect_here = !ctx().defer_reduce;
  if (collect_here) flush_deferred_reduces(false);  // nothing may be left from a failed call
  ctx().defer_reduce = true;
  defer_reduce(p.a.partial_dw, blocks, Kc, p.a.crs, epi_w);
  if (db_out) defer_reduce(p.a.partial_db, blocks, Kc, 1, epi_b);
  if (!collect_here) return TDH_OK;
  ctx().defer_reduce = false;
  return flush_deferred_reduces();
}

}  // namespace tdh
