// conv_dw.hip — weight gradient of a stride-1 3x3 convolution from LDS-staged tiles.
//
//   dW[co][ci][fy][fx] = sum_{img,oy,ox} dY[img][co][oy][ox] * X[img][ci][oy+fy-ph][ox+fx-pw]
//
// MFMA mapping (v_mfma_f32_32x32x2_f32): M = 32 output channels (A lane: co = l%32), N = 32
// input channels (B lane: ci = l%32), K = output pixels, two per instruction (k = l/32). Every
// filter tap is its own 32x32 accumulator: one dY fragment feeds all taps, and the X fragment
// of tap (fy,fx) is the same staged patch read (fy rows, fx columns) further on.
//
// The two pixels of an instruction are NOT neighbours: within a tile row of TC pixels, k = 0
// lanes walk the left half and k = 1 lanes the right half. A lane therefore needs consecutive
// pixels in consecutive instructions, so both fragments come out of LDS as 16-byte words in the
// tensors' own (pixel-fastest) layout: per four pixels and filter row one dY word and two X
// words serve 4*S instructions. Channel planes are padded to 4 (mod 32) floats, which spreads
// eight lanes' words over all banks.
//
// A workgroup owns 32*WCO output channels x 32 input channels x all taps for a range of pixel
// chunks (one image, TRw*WK output rows x TC columns). Waves: WCO channel blocks x WK row
// groups of the chunk x WFY filter-row groups; a wave keeps (R/WFY)*S accumulators, up to 144
// registers, so the kernel runs one workgroup per CU with the full register file. The next
// chunk's global loads are issued before the current chunk's MFMAs and parked in registers.
// At the end the WK row-group sums are added in wave order through LDS and the workgroup
// writes one slice [slice][co][ci][tap]; splitk_reduce_kernel adds the slices in order.
#include "gemm_mfma.h"

namespace tdh {

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int DWH_NX_MAX  = 36;  // X elements a thread stages per chunk (at most)
constexpr int DWH_NDY_MAX = 8;   // dY 16-byte words a thread stages per chunk (at most)

struct DwHaloArgs {
  const float *x, *dy;
  float *partial;  // [slices][Kc][C*R*S]
  int batch, C, Kc, H, W, OH, OW, ph, pw;
  int TRw;         // output rows one wave row-group takes per chunk
  int tiles_x, chunks_total, chunks_per_slice;
  int plane, plane_p, dyp;  // staged X plane (rows*PITCH), its padded stride, dY channel stride
  int nx, ndy;              // staging trips per thread
  int dy_vec;               // dY rows allow aligned 16-byte loads
  FastDiv div_pitch, div_rowchunks, div_dyq;  // by PITCH, chunks per image, words per dY channel
};

template <int R, int S, int TC, int WCO, int WK, int WFY>
__global__ void __launch_bounds__(64 * WCO * WK * WFY, 1) conv_dw_halo_kernel(const DwHaloArgs a) {
  constexpr int NT    = 64 * WCO * WK * WFY;
  constexpr int RPW   = R / WFY;  // filter rows per wave
  constexpr int NACC  = RPW * S;
  constexpr int BCO   = 32 * WCO;
  constexpr int PITCH = (TC + S - 1 + 3) & ~3;
  constexpr int NG    = TC / 8;   // 4-pixel groups per row and half
  constexpr int TPC   = NT / 32;  // threads staging one X channel plane
  constexpr int LOG_TC = TC == 64 ? 6 : TC == 32 ? 5 : TC == 16 ? 4 : 3;
  static_assert(R % WFY == 0, "filter rows must divide among the waves");
  static_assert(S <= 5, "two 16-byte words per filter row hold 4+S-1 <= 8 pixels");

  extern __shared__ __align__(16) float smem[];
  float *dy_l = smem;                // [BCO][dyp]
  float *x_l  = smem + BCO * a.dyp;  // [32][plane_p]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wco = wave % WCO, wk = (wave / WCO) % WK, wfy = wave / (WCO * WK);
  const int tx = blockIdx.x % a.tiles_x, slice = blockIdx.x / a.tiles_x;
  const int x0 = tx * TC, co0 = blockIdx.y * BCO, ci0 = blockIdx.z * 32;
  const int TR = a.TRw * WK;
  const int hw = a.H * a.W, ohw = a.OH * a.OW;

  // ---- X staging plan: thread -> channel xc, elements xl + TPC*i of the plane [rows][PITCH]
  const int xc = tid / TPC, xl = tid % TPC;
  const bool xch_ok = ci0 + xc < a.C;
  int xrel[DWH_NX_MAX];
  unsigned long long xcol = 0;  // element i lies in a column inside the image
#pragma unroll
  for (int i = 0; i < DWH_NX_MAX; ++i) {
    xrel[i] = 0;
    const int pe = xl + TPC * i;
    if (i < a.nx && pe < a.plane) {
      uint32_t r, c;
      a.div_pitch.divmod(pe, r, c);
      const int ix = x0 - a.pw + static_cast<int>(c);
      xrel[i]      = static_cast<int>(r) * a.W + ix;
      if (static_cast<int>(c) < TC + S - 1 && static_cast<unsigned>(ix) < static_cast<unsigned>(a.W))
        xcol |= 1ull << i;
    }
  }
  const float *x_chan = a.x + static_cast<size_t>(ci0 + xc) * hw;

  // ---- dY staging plan: word e4 = tid + NT*i -> channel co, row r, columns c..c+3
  int dyoff[DWH_NDY_MAX], dyrow[DWH_NDY_MAX], dylds[DWH_NDY_MAX], dycol[DWH_NDY_MAX];
#pragma unroll
  for (int i = 0; i < DWH_NDY_MAX; ++i) {
    dyoff[i] = 0; dylds[i] = 0; dycol[i] = 0;
    dyrow[i] = 1 << 20;  // never inside the image
    const int e4 = tid + NT * i;
    if (i < a.ndy && e4 < BCO * (TR << LOG_TC) / 4) {
      uint32_t co, q;
      a.div_dyq.divmod(e4, co, q);
      const int r = static_cast<int>(4 * q) >> LOG_TC, c = static_cast<int>(4 * q) & (TC - 1);
      dylds[i] = co * a.dyp + 4 * q;
      if (co0 + static_cast<int>(co) < a.Kc && x0 + c < a.OW) {
        dyrow[i] = r;
        dycol[i] = x0 + c;
        dyoff[i] = (co0 + co) * ohw + r * a.OW + x0 + c;
      }
    }
  }

  floatx16 acc[NACC];
#pragma unroll
  for (int t = 0; t < NACC; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[t][r] = 0.0f;

  float rx[DWH_NX_MAX];
  float4 rdy[DWH_NDY_MAX];

  auto fetch = [&](int chunk) {
    uint32_t img, rc;
    a.div_rowchunks.divmod(chunk, img, rc);
    const int y0    = rc * TR;
    const float *xb = x_chan + static_cast<size_t>(img) * a.C * hw;
    const int ybase = (y0 - a.ph) * a.W;
#pragma unroll
    for (int i = 0; i < DWH_NX_MAX; ++i) {
      const int rel = xrel[i] + ybase;
      const bool ok = i < a.nx && xch_ok && ((xcol >> i) & 1ull) &&
                      static_cast<unsigned>(rel) < static_cast<unsigned>(hw);
      rx[i] = ok ? xb[rel] : 0.0f;
    }
    const float *dyb = a.dy + static_cast<size_t>(img) * a.Kc * ohw + y0 * a.OW;
#pragma unroll
    for (int i = 0; i < DWH_NDY_MAX; ++i) {
      float4 v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
      if (i < a.ndy && y0 + dyrow[i] < a.OH) {
        const float *p = dyb + dyoff[i];
        if (a.dy_vec) {
          v = *reinterpret_cast<const float4 *>(p);
        } else {
          v.x = p[0];
          if (dycol[i] + 1 < a.OW) v.y = p[1];
          if (dycol[i] + 2 < a.OW) v.z = p[2];
          if (dycol[i] + 3 < a.OW) v.w = p[3];
        }
      }
      rdy[i] = v;
    }
  };
  auto stage = [&]() {
#pragma unroll
    for (int i = 0; i < DWH_NX_MAX; ++i) {
      const int pe = xl + TPC * i;
      if (i < a.nx && pe < a.plane) x_l[xc * a.plane_p + pe] = rx[i];
    }
#pragma unroll
    for (int i = 0; i < DWH_NDY_MAX; ++i)
      if (i < a.ndy && tid + NT * i < BCO * (TR << LOG_TC) / 4)
        *reinterpret_cast<float4 *>(dy_l + dylds[i]) = rdy[i];
  };

  // fragment bases of this lane: half k = lane/32 starts TC/2 pixels into the row
  const float *ap = dy_l + (wco * 32 + (lane & 31)) * a.dyp + ((wk * a.TRw) << LOG_TC) + (lane >> 5) * (TC / 2);
  const float *bp = x_l + (lane & 31) * a.plane_p + (wk * a.TRw + wfy * RPW) * PITCH + (lane >> 5) * (TC / 2);

  const int c_begin = slice * a.chunks_per_slice;
  const int c_end   = min(a.chunks_total, c_begin + a.chunks_per_slice);
  if (c_begin < c_end) fetch(c_begin);
  for (int chunk = c_begin; chunk < c_end; ++chunk) {
    if (chunk > c_begin) __syncthreads();  // everyone is done reading the previous chunk
    stage();
    __syncthreads();
    if (chunk + 1 < c_end) fetch(chunk + 1);
    for (int r = 0; r < a.TRw; ++r) {
#pragma unroll
      for (int g = 0; g < NG; ++g) {
        const float4 av4 = *reinterpret_cast<const float4 *>(ap + (r << LOG_TC) + 4 * g);
        const float av[4] = {av4.x, av4.y, av4.z, av4.w};
        float bv[RPW][8];
#pragma unroll
        for (int fy = 0; fy < RPW; ++fy) {
          const float4 b0 = *reinterpret_cast<const float4 *>(bp + (r + fy) * PITCH + 4 * g);
          const float4 b1 = *reinterpret_cast<const float4 *>(bp + (r + fy) * PITCH + 4 * g + 4);
          bv[fy][0] = b0.x; bv[fy][1] = b0.y; bv[fy][2] = b0.z; bv[fy][3] = b0.w;
          bv[fy][4] = b1.x; bv[fy][5] = b1.y; bv[fy][6] = b1.z; bv[fy][7] = b1.w;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int fy = 0; fy < RPW; ++fy)
#pragma unroll
            for (int fx = 0; fx < S; ++fx)
              acc[fy * S + fx] =
                __builtin_amdgcn_mfma_f32_32x32x2f32(av[j], bv[fy][j + fx], acc[fy * S + fx], 0, 0, 0);
      }
    }
  }

  // ---- add the WK row-group sums in wave order, then write the slice
  if (WK > 1) {
    float *red = smem;  // [WCO*WFY][NACC*16][64]
    for (int s = 1; s < WK; ++s) {
      __syncthreads();
      if (wk == s) {
        float *dst = red + static_cast<size_t>(wco + WCO * wfy) * (NACC * 16 * 64) + lane;
#pragma unroll
        for (int t = 0; t < NACC; ++t)
#pragma unroll
          for (int r = 0; r < 16; ++r) dst[(t * 16 + r) * 64] = acc[t][r];
      }
      __syncthreads();
      if (wk == 0) {
        const float *src = red + static_cast<size_t>(wco + WCO * wfy) * (NACC * 16 * 64) + lane;
#pragma unroll
        for (int t = 0; t < NACC; ++t)
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[t][r] += src[(t * 16 + r) * 64];
      }
    }
  }
  if (wk == 0) {
    // reg r of lane l: row (co) 8*(r/4) + 4*(l/32) + r%4, column (ci) l%32
    const int ci = ci0 + (lane & 31);
    const int crs = a.C * R * S;
    if (ci < a.C) {
      float *dst = a.partial + static_cast<size_t>(blockIdx.x) * a.Kc * crs + ci * (R * S) + wfy * RPW * S;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int co = co0 + wco * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        if (co >= a.Kc) continue;
#pragma unroll
        for (int t = 0; t < NACC; ++t) dst[static_cast<size_t>(co) * crs + t] = acc[t][r];
      }
    }
  }
}

struct DwHaloPlan {
  bool ok;
  int tc, wco, wk, wfy, nt;
  DwHaloArgs args;
  size_t lds_bytes;
  dim3 grid;
  int slices;
};

int pad_to_4_mod_32(int v) {
  while ((v & 31) != 4) ++v;
  return v;
}

DwHaloPlan make_dw_plan(int R, int S, int batch, int C, int Kc, int H, int W, int OH, int OW, int ph,
                        int pw) {
  DwHaloPlan p;
  p.ok = false;
  // 3x3 windows only: with 25 taps the accumulators of a channel block no longer fit one wave,
  // and splitting the filter rows over five waves measured slower than the generic GEMM on
  // the small images such layers see here
  if (!(R == 3 && S == 3)) return p;
  if (C < 16 || Kc < 16 || OW < 8 || OH < 2) return p;
  p.tc = OW >= 48 ? 64 : OW >= 24 ? 32 : OW >= 12 ? 16 : 8;
  p.wfy = 1;
  p.wco = Kc > 32 ? 2 : 1;
  p.wk  = 4 / p.wco;
  p.nt = 64 * p.wco * p.wk * p.wfy;
  DwHaloArgs &a = p.args;
  a.batch = batch; a.C = C; a.Kc = Kc; a.H = H; a.W = W; a.OH = OH; a.OW = OW; a.ph = ph; a.pw = pw;
  a.TRw = std::max(1, 64 / p.tc);
  const int tr    = a.TRw * p.wk;
  const int pitch = (p.tc + S - 1 + 3) & ~3;
  a.plane   = (tr + R - 1) * pitch;
  a.plane_p = pad_to_4_mod_32(a.plane);
  a.dyp     = pad_to_4_mod_32(tr * p.tc);
  a.nx      = ceil_div(a.plane, p.nt / 32);
  a.ndy     = ceil_div(32 * p.wco * tr * p.tc / 4, p.nt);
  if (a.nx > DWH_NX_MAX || a.ndy > DWH_NDY_MAX) return p;
  a.dy_vec        = (OW % 4 == 0) ? 1 : 0;
  a.tiles_x       = ceil_div(OW, p.tc);
  const int row_chunks = ceil_div(OH, tr);
  a.chunks_total  = batch * row_chunks;
  a.div_pitch     = FastDiv(pitch);
  a.div_rowchunks = FastDiv(row_chunks);
  a.div_dyq       = FastDiv(tr * p.tc / 4);
  const int co_blocks = ceil_div(Kc, 32 * p.wco), ci_blocks = ceil_div(C, 32);
  const long base = static_cast<long>(a.tiles_x) * co_blocks * ci_blocks;
  // one workgroup per CU; a slice should still cover a few chunks so that its prologue and
  // its partial tile are paid for
  long slices = std::max<long>(1, 256 / base);
  slices = std::min<long>(slices, std::max(1, a.chunks_total / 2));
  a.chunks_per_slice = ceil_div(a.chunks_total, static_cast<int>(slices));
  p.slices           = ceil_div(a.chunks_total, a.chunks_per_slice);
  const size_t stage_floats = static_cast<size_t>(32 * p.wco) * a.dyp + 32 * static_cast<size_t>(a.plane_p);
  const size_t red_floats   = p.wk > 1 ? static_cast<size_t>(p.wco * p.wfy) * (R / p.wfy) * S * 16 * 64 : 0;
  p.lds_bytes = sizeof(float) * std::max(stage_floats, red_floats);
  if (p.lds_bytes > 150 * 1024) return p;
  if (static_cast<long>(a.tiles_x) * p.slices > 65535L * 16) return p;
  p.grid = dim3(a.tiles_x * p.slices, co_blocks, ci_blocks);
  p.ok   = true;
  return p;
}

template <int R, int S, int TC, int WCO, int WK, int WFY>
int launch_dw_inst(const DwHaloPlan &p) {
  auto kernel = conv_dw_halo_kernel<R, S, TC, WCO, WK, WFY>;
  if (p.lds_bytes > 64 * 1024) {
    // raised once per kernel instance and size: the default dynamic LDS limit is 64 KiB
    static size_t raised = 0;
    if (p.lds_bytes > raised) {
      TDH_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                  hipFuncAttributeMaxDynamicSharedMemorySize,
                                  static_cast<int>(p.lds_bytes)));
      raised = p.lds_bytes;
    }
  }
  hipLaunchKernelGGL(kernel, p.grid, dim3(p.nt), p.lds_bytes, ctx().stream, p.args);
  TDH_LAUNCH_CHECK();
  return TDH_OK;
}

template <int TC>
int launch_dw_tc(const DwHaloPlan &p) {
  if (p.wco == 2) return launch_dw_inst<3, 3, TC, 2, 2, 1>(p);
  return launch_dw_inst<3, 3, TC, 1, 4, 1>(p);
}

}  // namespace

bool conv_dw_halo_applicable(int R, int S, int batch, int C, int Kc, int H, int W, int OH, int OW,
                             int ph, int pw) {
  return make_dw_plan(R, S, batch, C, Kc, H, W, OH, OW, ph, pw).ok;
}

size_t conv_dw_halo_workspace_bytes(int R, int S, int batch, int C, int Kc, int H, int W, int OH,
                                    int OW, int ph, int pw) {
  const DwHaloPlan p = make_dw_plan(R, S, batch, C, Kc, H, W, OH, OW, ph, pw);
  if (!p.ok) return 0;
  return ws_align(sizeof(float) * static_cast<size_t>(p.grid.x) * Kc * C * R * S);
}

// dw (+)= sum over the batch; the caller has checked applicability and reserved the workspace
int conv_dw_halo_run(int R, int S, int batch, int C, int Kc, const float *x, const float *dy,
                     float *dw, int H, int W, int OH, int OW, int ph, int pw, int accumulate) {
  DwHaloPlan p = make_dw_plan(R, S, batch, C, Kc, H, W, OH, OW, ph, pw);
  if (!p.ok) return set_error(TDH_ERR_INVALID, "conv_dw_halo_run: shape not supported");
  const int crs = C * R * S;
  void *part = nullptr;
  TDH_TRY(ws_take(sizeof(float) * static_cast<size_t>(p.grid.x) * Kc * crs, &part));
  p.args.x = x; p.args.dy = dy; p.args.partial = static_cast<float *>(part);
  {
    ProfScope prof("conv_dw_halo", Kc, crs, batch * OH * OW);
    switch (p.tc) {
      case 64: TDH_TRY(launch_dw_tc<64>(p)); break;
      case 32: TDH_TRY(launch_dw_tc<32>(p)); break;
      case 16: TDH_TRY(launch_dw_tc<16>(p)); break;
      default: TDH_TRY(launch_dw_tc<8>(p)); break;
    }
  }
  const int slices = static_cast<int>(p.grid.x);
  ProfScope prof("conv_dw_splitk_reduce", 4.0 * Kc * crs * (slices + 1), WORK_BYTE);
  EpiRowMajor epi{dw, crs, nullptr, ActGrad(), accumulate};
  hipLaunchKernelGGL((splitk_reduce_kernel<EpiRowMajor>), dim3(ceil_div(Kc * crs, REDUCE_OUTPUTS)),
                     dim3(256), 0, ctx().stream, p.args.partial, slices, Kc, crs, epi);
  TDH_LAUNCH_CHECK();
  return TDH_OK;
}

}  // namespace tdh
