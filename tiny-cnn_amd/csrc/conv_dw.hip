// conv_dw.hip — weight gradient of a stride-1 3x3 or 5x5 convolution from LDS-staged tiles.
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
// pixels in consecutive instructions: per four pixels and filter row one 16-byte dY word and
// 4+S-1 X floats serve 4*S instructions. dY channel planes are padded to 4 (mod 32) floats (eight
// lanes' 16-byte words cover all banks), X channel planes to an odd stride (32 lanes' floats
// cover all banks).
//
// Staging is by aligned 16-byte words of the tensors' own rows: the staged X patch starts at
// the image column x0 - pwa, pwa the padding rounded up to 4, so that every word is either
// wholly inside a row or wholly outside; the fragment reads start pwa - pw floats in. A thread
// keeps one relative offset per word; whether the word exists for a given chunk (row inside the
// image, image inside the batch) is ONE unsigned compare of offset + chunk base against a
// limit, and words that do not exist are read from a zero word instead, which keeps the loads
// free of branches. Tensors whose rows are not multiples of four floats take the same words as
// four scalar loads.
//
// A workgroup owns 32*WCO output channels x 32 input channels x its taps for a range of pixel
// chunks (WK row groups of 64/TC output rows x TC columns). Waves: WCO channel blocks x WK row groups of the
// chunk x WFY filter-row groups; a wave keeps (R/WFY)*S accumulators, up to 144 registers, so
// the kernel runs one workgroup per CU with the full register file. The next chunk's global
// loads are issued before the current chunk's MFMAs and parked in registers. At the end the
// WK row-group sums are added pairwise through LDS and the workgroup writes one slice
// [slice][co][ci][tap]; splitk_reduce_kernel adds the slices in order.
//
// 5x5 windows: 25 accumulators do not fit one wave, so the filter rows go to different
// WORKGROUPS (grid z = channel block x filter row) and the kernel runs as a 1x5 window whose
// input rows are shifted by the filter row. Such a window needs no halo rows, so on small
// images a chunk holds TI whole images stacked as rows.
#include "gemm_mfma.h"

namespace tdh {

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int DWH_NDY = 8;   // dY words a thread stages per chunk
constexpr int DWH_NEVER = -(1 << 30);  // relative offset of a word that never exists

// a word that does not exist is loaded from here (not const: the loads must stay in the global
// address space, like those of the tensors)
__device__ __align__(16) float dwh_zero_word[4] = {0.0f, 0.0f, 0.0f, 0.0f};

struct DwHaloArgs {
  const float *x, *dy;
  float *partial;  // [slices][Kc][C*RF*S]
  // Bias gradient on the way (or null): the workgroups of input-channel block 0 / filter row 0
  // add up the dY words they stage anyway; [slices][Kc], reduced like the dW slices.
  float *partial_db;
  int batch, C, Kc, H, W, OH, OW, ph, pw;
  int TI;          // whole images stacked in a chunk (1: a chunk is WK*64/TC rows of one image)
  int tiles_x, chunks_total, chunks_per_slice;
  int plane_p;     // channel stride of the staged X planes (odd)
  int dyp;         // channel stride of the staged dY planes (4 mod 32)
  int pwa;         // staged X column 0 is image column x0 - pwa
  FastDiv div_rowchunks, div_oh;
  FastDiv div_gy, div_gz, div_tiles_x;  // grid y and z, tiles per row: the workgroup's place
};

// R: filter rows one workgroup covers, RF: filter rows of the window (RF/R workgroups share a
// channel block), VEC: the rows of X and dY allow aligned 16-byte loads
template <int R, int S, int TC, int WCO, int WK, int WFY, int RF, bool VEC>
__global__ void __launch_bounds__(64 * WCO * WK * WFY, 1) conv_dw_halo_kernel(const DwHaloArgs a) {
  constexpr int NT    = 64 * WCO * WK * WFY;
  constexpr int FYB   = RF / R;
  constexpr int RPW   = R / WFY;  // filter rows per wave
  constexpr int NACC  = RPW * S;
  constexpr int BCO   = 32 * WCO;
  constexpr int NQ    = (3 + TC + S - 1 + 3) / 4;  // words per staged X row
  constexpr int PITCH = 4 * NQ;
  constexpr int TPC   = NT / 32;  // threads staging one X channel plane
  constexpr int NG    = TC / 8;   // 4-pixel groups per row and half
  constexpr int TRW   = 64 / TC;  // output rows one wave row-group takes per chunk
  constexpr int STEPS = TRW * NG; // (row, group) steps of a chunk's MFMA loop: always 8
  constexpr int TR    = TRW * WK;
  constexpr int PRQ   = (TR + R - 1) * NQ;        // words of a staged X plane
  constexpr int NXI   = (PRQ + TPC - 1) / TPC;    // X words a thread stages per chunk
  static_assert(NXI <= 16, "the keep bits of the scalar loads cover 16 words");
  constexpr int LOG_TC = TC == 64 ? 6 : TC == 32 ? 5 : TC == 16 ? 4 : 3;
  constexpr int DQ    = 16 * WK;  // words per staged dY channel: 64 pixels per row group
  constexpr int DCO   = NT / DQ;  // dY channels one staging trip covers
  static_assert(R % WFY == 0, "filter rows must divide among the waves");
  static_assert(RF % R == 0, "filter rows must divide among the workgroups");
  static_assert(BCO * DQ == NT * DWH_NDY, "dY staging trips");
  static_assert(WFY == 1 || WK == 1, "row groups and filter-row groups are not combined");

  extern __shared__ __align__(16) float smem[];
  float *dy_l = smem;                // [BCO][dyp]
  float *x_l  = smem + BCO * a.dyp;  // [32][plane_p]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wco = wave % WCO, wk = (wave / WCO) % WK, wfy = wave / (WCO * WK);
  // Workgroups are handed to the eight XCDs (each with its own L2) round-robin in launch
  // order. Renumber them so that the workgroups that read the same tiles (the filter rows of a
  // channel block share dY and X, the input-channel blocks share dY, the output-channel blocks
  // share X) are neighbours on one XCD.
  int bx, by, bz;
  {
    const int gy = gridDim.y, gz = gridDim.z;
    const int total = gridDim.x * gy * gz, per = total >> 3;
    int id = blockIdx.x + gridDim.x * (blockIdx.y + gy * blockIdx.z);
    if (id < (per << 3)) id = (id & 7) * per + (id >> 3);
    uint32_t rest, q, m;  // filter row fastest, then input-channel block
    a.div_gz.divmod(static_cast<uint32_t>(id), rest, m);
    bz = static_cast<int>(m);
    a.div_gy.divmod(rest, q, m);
    by = static_cast<int>(m);
    bx = static_cast<int>(q);
  }
  uint32_t slice_u, tx_u;
  a.div_tiles_x.divmod(static_cast<uint32_t>(bx), slice_u, tx_u);
  const int tx = static_cast<int>(tx_u), slice = static_cast<int>(slice_u);
  const int x0 = tx * TC, co0 = by * BCO;
  const int ci0 = (bz / FYB) * 32, fy0 = (bz % FYB) * R;
  const int hw = a.H * a.W, ohw = a.OH * a.OW;
  const int chw = a.C * hw, kohw = a.Kc * ohw;

  // ---- X staging plan: thread -> channel xc, words xl + TPC*i of the plane [rows][NQ]
  const int xc = tid / TPC, xl = tid % TPC;
  int xrel[NXI];            // offset of word i from the chunk's base, or DWH_NEVER
  unsigned long long xkeep = 0; // scalar loads: 4 bits per word, float k lies inside the row
  // (written without branches: the plan runs once, cold, in front of the first load)
  const bool stacked = a.TI > 1;
#pragma unroll
  for (int i = 0; i < NXI; ++i) {
    const int pe = xl + TPC * i;
    const int r = pe / NQ, q = pe - r * NQ;
    const int ix = x0 - a.pwa + 4 * q;
    unsigned keep = 0;
    if (VEC) {
      keep = (ix >= 0 && ix + 3 < a.W) ? 15u : 0u;
    } else {
#pragma unroll
      for (int k = 0; k < 4; ++k) keep |= (static_cast<unsigned>(ix + k) < static_cast<unsigned>(a.W) ? 1u : 0u) << k;
    }
    // stacked whole images: the row inside its image is fixed, the chunk only picks images
    uint32_t il, rr;
    a.div_oh.divmod(static_cast<uint32_t>(r), il, rr);
    const int rs   = static_cast<int>(rr) + fy0 - a.ph;
    const bool in  = !stacked || (static_cast<int>(il) < a.TI && static_cast<unsigned>(rs) < static_cast<unsigned>(a.H));
    const bool ok  = (pe < PRQ) & (ci0 + xc < a.C) & (VEC ? keep == 15u : keep != 0u) & in;
    const int base = stacked ? static_cast<int>(il) * chw : 0;
    xrel[i] = ok ? base + (stacked ? rs : r) * a.W + ix : DWH_NEVER;
    if (!VEC) xkeep |= static_cast<unsigned long long>(ok ? keep : 0u) << (4 * i);
  }
  const float *x_chan = a.x + static_cast<size_t>(ci0 + xc) * hw;

  // ---- dY staging plan: word tid + NT*i -> channel dco + DCO*i, the same row and column for
  //      every i
  const int dq = tid % DQ, dco = tid / DQ;
  const int dcol = x0 + ((4 * dq) & (TC - 1));
  int dyrel = DWH_NEVER;
  {
    int r = (4 * dq) >> LOG_TC, base = 0;
    bool ok = VEC ? dcol + 3 < a.OW : dcol < a.OW;
    if (a.TI > 1) {
      uint32_t il, rr;
      a.div_oh.divmod(static_cast<uint32_t>(r), il, rr);
      ok   = ok && static_cast<int>(il) < a.TI;
      base = static_cast<int>(il) * kohw;
      r    = static_cast<int>(rr);
    }
    if (ok) dyrel = base + r * a.OW + dcol;
  }
  const float *dy_chan = a.dy + static_cast<size_t>(co0 + dco) * ohw;
  const float *zero = dwh_zero_word;

  floatx4 rx[NXI];
  floatx4 rdy[DWH_NDY];
  const bool sums_dy = a.partial_db != nullptr && bz == 0;
  float dbs[DWH_NDY];  // this thread's share of the bias gradient of channels dco + DCO*i
#pragma unroll
  for (int i = 0; i < DWH_NDY; ++i) dbs[i] = 0.0f;

  // The loads of a chunk are issued in STEPS parts, one per step of the MFMA loop of the chunk
  // before: every workgroup of the grid fetches at the same time, and a chunk's words issued
  // in one go wait for HBM while the matrix cores idle.
  const float *xb = nullptr, *dyb = nullptr;  // the chunk's image, this thread's channel
  int xbase = 0, dybase = 0;                  // added to the words' relative offsets
  unsigned xlimit = 0, dylimit = 0;
  auto fetch_begin = [&](int chunk) {
    uint32_t img, rc;
    a.div_rowchunks.divmod(chunk, img, rc);
    img *= a.TI;
    const int y0   = a.TI > 1 ? 0 : rc * TR;
    const int nimg = min(a.TI, a.batch - static_cast<int>(img));
    xb      = x_chan + static_cast<size_t>(img) * chw;
    xbase   = a.TI > 1 ? 0 : (y0 - a.ph + fy0) * a.W;
    xlimit  = a.TI > 1 ? nimg * chw : hw;
    dyb     = dy_chan + static_cast<size_t>(img) * kohw;
    dybase  = y0 * a.OW;
    dylimit = a.TI > 1 ? nimg * kohw : ohw;
  };
  // (in the first half of the steps: a load issued in the last steps has no MFMAs left to hide
  // behind, and the next stage() would wait a whole trip to memory for it)
  constexpr int LOAD_STEPS = STEPS / 2;
  auto fetch_part = [&](int part) {
#pragma unroll
    for (int i = 0; i < NXI; ++i) {
      if (i % LOAD_STEPS != part) continue;
      const int rel = xrel[i] + xbase;
      const bool ok = static_cast<unsigned>(rel) < xlimit;
      if (VEC) {
        rx[i] = *reinterpret_cast<const floatx4 *>(ok ? xb + rel : zero);
      } else {
        const unsigned keep = ok ? static_cast<unsigned>(xkeep >> (4 * (i & 15))) & 15u : 0u;
        rx[i].x = *((keep & 1u) ? xb + rel : zero);
        rx[i].y = *((keep & 2u) ? xb + rel + 1 : zero);
        rx[i].z = *((keep & 4u) ? xb + rel + 2 : zero);
        rx[i].w = *((keep & 8u) ? xb + rel + 3 : zero);
      }
    }
#pragma unroll
    for (int i = 0; i < DWH_NDY; ++i) {
      if (i % LOAD_STEPS != part) continue;
      const int rel  = dyrel + dybase;
      const bool oki = static_cast<unsigned>(rel) < dylimit && co0 + dco + DCO * i < a.Kc;
      const float *p = dyb + static_cast<size_t>(DCO * i) * ohw + rel;
      if (VEC) {
        rdy[i] = *reinterpret_cast<const floatx4 *>(oki ? p : zero);
      } else {
        rdy[i].x = *(oki ? p : zero);
        rdy[i].y = *((oki && dcol + 1 < a.OW) ? p + 1 : zero);
        rdy[i].z = *((oki && dcol + 2 < a.OW) ? p + 2 : zero);
        rdy[i].w = *((oki && dcol + 3 < a.OW) ? p + 3 : zero);
      }
    }
  };
  auto stage = [&]() {
    float *xd = x_l + xc * a.plane_p + 4 * xl;
#pragma unroll
    for (int i = 0; i < NXI; ++i) {
      if (xl + TPC * i < PRQ) {
        float *d = xd + 4 * TPC * i;
        d[0] = rx[i].x; d[1] = rx[i].y; d[2] = rx[i].z; d[3] = rx[i].w;
      }
    }
    float *dd = dy_l + dco * a.dyp + 4 * dq;
#pragma unroll
    for (int i = 0; i < DWH_NDY; ++i) *reinterpret_cast<floatx4 *>(dd + DCO * i * a.dyp) = rdy[i];
    if (sums_dy) {
#pragma unroll
      for (int i = 0; i < DWH_NDY; ++i) dbs[i] += (rdy[i].x + rdy[i].y) + (rdy[i].z + rdy[i].w);
    }
  };

  const int c_begin = slice * a.chunks_per_slice;
  const int c_end   = min(a.chunks_total, c_begin + a.chunks_per_slice);
  if (c_begin < c_end) {
    fetch_begin(c_begin);
#pragma unroll
    for (int s = 0; s < STEPS; ++s) fetch_part(s);
  }

  floatx16 acc[NACC];
#pragma unroll
  for (int t = 0; t < NACC; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[t][r] = 0.0f;

  // fragment bases of this lane: half k = lane/32 starts TC/2 pixels into the row
  const float *ap = dy_l + (wco * 32 + (lane & 31)) * a.dyp + ((wk * TRW) << LOG_TC) + (lane >> 5) * (TC / 2);
  const float *bp = x_l + (lane & 31) * a.plane_p + (wk * TRW + wfy * RPW) * PITCH + (a.pwa - a.pw) +
                    (lane >> 5) * (TC / 2);

  for (int chunk = c_begin; chunk < c_end; ++chunk) {
    if (chunk > c_begin) __syncthreads();  // everyone is done reading the previous chunk
    stage();
    __syncthreads();
    // (behind the last chunk the same loads run against empty limits and fetch the zero word:
    // a step without branches is one block that the compiler can interleave)
    const bool more = chunk + 1 < c_end;
    fetch_begin(more ? chunk + 1 : chunk);
    if (!more) xlimit = dylimit = 0;
    // The fragments of step s+1 are read from LDS before the products of step s are issued,
    // and the next chunk's global loads between them: with one wave per SIMD nothing else
    // would cover their latencies.
    floatx4 av4[2];
    float bv[2][RPW][4 + S - 1];
    auto read_fragments = [&](int s, int to) {
      const int r = s / NG, g = s % NG;
      av4[to] = *reinterpret_cast<const floatx4 *>(ap + (r << LOG_TC) + 4 * g);
#pragma unroll
      for (int fy = 0; fy < RPW; ++fy)
#pragma unroll
        for (int k = 0; k < 4 + S - 1; ++k) bv[to][fy][k] = bp[(r + fy) * PITCH + 4 * g + k];
    };
    read_fragments(0, 0);
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      const int cur = s & 1;
      if (s + 1 < STEPS) read_fragments(s + 1, cur ^ 1);
      const float av[4] = {av4[cur].x, av4[cur].y, av4[cur].z, av4[cur].w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
#pragma unroll
        for (int fy = 0; fy < RPW; ++fy)
#pragma unroll
          for (int fx = 0; fx < S; ++fx)
            acc[fy * S + fx] =
              __builtin_amdgcn_mfma_f32_32x32x2f32(av[j], bv[cur][fy][j + fx], acc[fy * S + fx], 0, 0, 0);
        if (j == 0) fetch_part(s);
      }
      __builtin_amdgcn_sched_barrier(0);  // (the loads stay in the step they were written for)
    }
  }

  // ---- add the WK row-group sums pairwise (upper half of the groups onto the lower half)
  if (WK > 1) {
    float *red = smem;  // [WK/2][WCO][NACC*16][64]
    for (int h = WK / 2; h >= 1; h >>= 1) {
      __syncthreads();
      if (wk >= h && wk < 2 * h) {
        float *dst = red + static_cast<size_t>((wk - h) * WCO + wco) * (NACC * 16 * 64) + lane;
#pragma unroll
        for (int t = 0; t < NACC; ++t)
#pragma unroll
          for (int r = 0; r < 16; ++r) dst[(t * 16 + r) * 64] = acc[t][r];
      }
      __syncthreads();
      if (wk < h) {
        const float *src = red + static_cast<size_t>(wk * WCO + wco) * (NACC * 16 * 64) + lane;
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
    const int crs = a.C * RF * S;
    if (ci < a.C) {
      float *dst = a.partial + static_cast<size_t>(bx) * a.Kc * crs + ci * (RF * S) +
                   (fy0 + wfy * RPW) * S;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int co = co0 + wco * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        if (co >= a.Kc) continue;
#pragma unroll
        for (int t = 0; t < NACC; ++t) dst[static_cast<size_t>(co) * crs + t] = acc[t][r];
      }
    }
  }
  if (sums_dy) {
    // channel c = dco + DCO*i was summed by the DQ threads dco*DQ .. dco*DQ + DQ-1: add their
    // shares in thread order
    float *sh = smem;  // [DWH_NDY][NT]
    __syncthreads();
#pragma unroll
    for (int i = 0; i < DWH_NDY; ++i) sh[i * NT + tid] = dbs[i];
    __syncthreads();
    if (tid < BCO && co0 + tid < a.Kc) {
      const float *src = sh + (tid / DCO) * NT + (tid % DCO) * DQ;
      float s = 0.0f;
      for (int q = 0; q < DQ; ++q) s += src[q];
      a.partial_db[static_cast<size_t>(bx) * a.Kc + co0 + tid] = s;
    }
  }
}


// ---- 5x5 windows (padding 2, stride 1) on 8x8 images: every filter row in one workgroup
//
// The kernel above gives such a layer workgroups of (one filter row) x (two chunks of images):
// 1280 wave-sized pieces of 160 MFMAs for 1024 SIMDs, so some SIMD runs two whatever the split,
// five workgroups stage the same tiles, and a wave's slice leaves as 80 scattered 4-byte stores.
// Here a workgroup owns 32 output channels x 32 input channels x one of FOUR GROUPS OF TAPS
// (7 + 6 + 6 + 6 of the 25, each group lies in two filter rows) for a run of chunks of four
// images; its four waves take one image each, so a wave's piece is 224 (or 192) MFMAs and a
// 32 -> 64-channel layer at batch 128 is 256 workgroups of one chunk: every SIMD gets one wave.
// An image is staged whole with its zero frame (12 x 12 per channel), so the X fragment of
// output row oy and filter row fy is two 16-byte reads, eight floats, that serve all five taps
// of the row; a dY fragment (one 16-byte read per output row) serves all taps of the group.
// The pixel pairing is the one of the kernel above: k = 0 lanes take the left half of a row,
// k = 1 lanes the right half. The four waves' sums meet in LDS (pairwise, image order), and the
// whole workgroup stores the slice. The bias gradient comes from the workgroups of tap group 0
// and input-channel block 0, out of the dY they stage anyway.
//
// 16x16 images (IS = 16) run the same way with ONE image a chunk: a wave takes four of its rows,
// 64 pixels again, as eight groups of eight; with more than one chunk a workgroup the next
// chunk's words travel while the current one is multiplied.
constexpr int I8_NT  = 256;
constexpr int I8_DYP = 4 * 64 + 4;    // floats per staged dY channel: 256 pixels (4 mod 64)
// geometry of a chunk for images of IS x IS pixels
template <int IS> struct I8Geom {
  static constexpr int IPC   = IS == 8 ? 4 : 1;              // images a chunk
  static constexpr int FP    = IS + 4;                       // framed row
  static constexpr int XP    = IPC * FP * FP + 4;            // floats per staged X channel (4 mod 32 / 20 mod 32)
  static constexpr int WAVEX = IS == 8 ? FP * FP : 4 * FP;   // a wave's first framed row: its image / its four rows
  static constexpr int LDS_FLOATS = 32 * I8_DYP + 32 * XP;
};

struct DwImg8Args {
  const float *x, *dy;
  float *partial;      // [slices][Kc][C*25]
  float *partial_db;   // [slices][Kc], or null
  int batch, C, Kc;
  int chunks_total, chunks_per_slice;   // chunks of four images
  int co_blocks, ci_blocks;
};

// tap group G: taps T0 .. T0+N-1 of the 25 (tap = 5*fy + fx)
template <int G> struct I8Taps {
  static constexpr int T0 = G == 0 ? 0 : G == 1 ? 7 : G == 2 ? 13 : 19;
  static constexpr int N  = G == 0 ? 7 : 6;
  static constexpr int FY0 = T0 / 5, FY1 = (T0 + N - 1) / 5;
};

// the products of the wave's 64 pixels (eight groups of eight: an image's rows, or halves of four
// rows) for tap group G: acc[t - T0] += dY x X shifted by tap t
template <int G, int IS>
__device__ __forceinline__ void img8_products(const float *ap, const float *bp, floatx16 (&acc)[7]) {
  using TG = I8Taps<G>;
  constexpr int FP = I8Geom<IS>::FP;
#pragma unroll
  for (int u = 0; u < 8; ++u) {
    const int oy = IS == 8 ? u : u >> 1, ox = IS == 8 ? 0 : 8 * (u & 1);
    const floatx4 a4 = *reinterpret_cast<const floatx4 *>(ap + u * 8);
    const float av[4] = {a4.x, a4.y, a4.z, a4.w};
#pragma unroll
    for (int fy = TG::FY0; fy <= TG::FY1; ++fy) {
      const floatx4 b0 = *reinterpret_cast<const floatx4 *>(bp + (oy + fy) * FP + ox);
      const floatx4 b1 = *reinterpret_cast<const floatx4 *>(bp + (oy + fy) * FP + ox + 4);
      const float bv[8] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
#pragma unroll
      for (int fx = 0; fx < 5; ++fx) {
        const int t = 5 * fy + fx - TG::T0;
        if (t < 0 || t >= TG::N) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[j], bv[j + fx], acc[t], 0, 0, 0);
      }
    }
  }
}

template <int IS>
__global__ void __launch_bounds__(I8_NT, 1) conv_dw_img8_kernel(const DwImg8Args a) {
  using GE = I8Geom<IS>;
  constexpr int I8_XP = GE::XP, IPC = GE::IPC, FP = GE::FP, PIX = IS * IS;
  extern __shared__ __align__(16) float smem[];
  float *dy_l = smem;                 // [32][I8_DYP]
  float *x_l  = smem + 32 * I8_DYP;   // [32][I8_XP], frames of zeros around the images
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // workgroups that read the same tiles (the four tap groups and the output-channel blocks of a
  // slice) are neighbours after the renumbering, and so share an XCD's L2
  int id = xcd_compact_id(static_cast<int>(blockIdx.x), static_cast<int>(gridDim.x));
  const int grp = id & 3;
  id >>= 2;
  const int cob = id % a.co_blocks;
  id /= a.co_blocks;
  const int cib = id % a.ci_blocks, slice = id / a.ci_blocks;
  const int co0 = cob * 32, ci0 = cib * 32;
  const int kohw = a.Kc * PIX, chw = a.C * PIX;

  floatx16 acc[7];
#pragma unroll
  for (int t = 0; t < 7; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[t][r] = 0.0f;
  const bool sums_dy = a.partial_db != nullptr && grp == 0 && cib == 0;
  float dbs = 0.0f;   // this thread's share of the bias gradient of channel tid / 8

  // fragment bases: A lane = (output channel l%32, half l/32), B lane = (input channel l%32, half)
  const float *ap = dy_l + (lane & 31) * I8_DYP + wave * 64 + 4 * (lane >> 5);
  const float *bp = x_l + (lane & 31) * I8_XP + wave * GE::WAVEX + 4 * (lane >> 5);

  const int c_begin = slice * a.chunks_per_slice;
  const int c_end   = min(a.chunks_total, c_begin + a.chunks_per_slice);
  // ---- staging: a thread moves eight 16-byte words of dY and eight of X per chunk, all loads
  //      asked for before the first store (an image past the batch reads image 0 and is stored
  //      as zeros). Word e: IS = 8: image e / 512 of the chunk's four, channel (e / 16) % 32,
  //      word e % 16 of its 64 pixels; IS = 16: channel e / 64, word e % 64 of the image.
  floatx4 rdy[8], rx[8];
  auto fetch = [&](int chunk) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int e = tid + I8_NT * i;
      const int im = IS == 8 ? e >> 9 : 0, c = IS == 8 ? (e >> 4) & 31 : e >> 6, q = IS == 8 ? e & 15 : e & 63;
      const int img = chunk * IPC + im;
      const size_t ig = img < a.batch ? img : 0;
      rdy[i] = *reinterpret_cast<const floatx4 *>(a.dy + ig * kohw + static_cast<size_t>(co0 + c) * PIX + 4 * q);
      rx[i]  = *reinterpret_cast<const floatx4 *>(a.x + ig * chw + static_cast<size_t>(ci0 + c) * PIX + 4 * q);
    }
  };
  fetch(c_begin);
  for (int chunk = c_begin; chunk < c_end; ++chunk) {
    if (chunk == c_begin) {   // the frames of zeros, written while the first loads are on their way
      for (int i = tid; i < 32 * I8_XP / 4; i += I8_NT) reinterpret_cast<floatx4 *>(x_l)[i] = floatx4{0.f, 0.f, 0.f, 0.f};
    }
    __syncthreads();   // (the previous chunk's fragments have been read; the first time: the zeros are in place)
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int e = tid + I8_NT * i;
      const int im = IS == 8 ? e >> 9 : 0, c = IS == 8 ? (e >> 4) & 31 : e >> 6, q = IS == 8 ? e & 15 : e & 63;
      const bool on = chunk * IPC + im < a.batch;
      const floatx4 z = floatx4{0.f, 0.f, 0.f, 0.f};
      *reinterpret_cast<floatx4 *>(dy_l + c * I8_DYP + im * 64 + 4 * q) = on ? rdy[i] : z;
      // X row, word of the row -> framed row + 2, columns 2 + 4 * word .. + 3 (8-byte aligned)
      constexpr int WPR = IS / 4;   // words per image row
      const floatx4 v = on ? rx[i] : z;
      float *d = x_l + c * I8_XP + im * (FP * FP) + ((q / WPR) + 2) * FP + 2 + 4 * (q % WPR);
      *reinterpret_cast<float2 *>(d)     = make_float2(v.x, v.y);
      *reinterpret_cast<float2 *>(d + 2) = make_float2(v.z, v.w);
    }
    __syncthreads();
    if (chunk + 1 < c_end) fetch(chunk + 1);   // (travels while this chunk is multiplied)
    if (sums_dy) {   // channel tid/8, floats (tid%8)*32 .. +31 of its 256 pixels
      const floatx4 *row = reinterpret_cast<const floatx4 *>(dy_l + (tid >> 3) * I8_DYP + (tid & 7) * 32);
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        const floatx4 v = row[k];
        dbs += (v.x + v.y) + (v.z + v.w);
      }
    }
    switch (grp) {
      case 0: img8_products<0, IS>(ap, bp, acc); break;
      case 1: img8_products<1, IS>(ap, bp, acc); break;
      case 2: img8_products<2, IS>(ap, bp, acc); break;
      default: img8_products<3, IS>(ap, bp, acc); break;
    }
  }

  // ---- the four images' sums, pairwise in image order: (0 + 2) + (1 + 3). Waves 2 and 3 park
  //      their sums, waves 0 and 1 add them to their own and park the two results transposed,
  //      [output channel][input channel][tap] (rows of nine floats: no two lanes of a store share
  //      a bank), and the whole workgroup adds those two and stores: a lane's neighbours then
  //      write neighbouring taps and input channels, seven cache lines a store instead of 64.
  float *red = smem;   // [2][7*16][64], then [2][32*32][9]
  const int ntaps = grp == 0 ? 7 : 6, t0 = grp == 0 ? 0 : 1 + 6 * grp;
  __syncthreads();
  if (wave >= 2) {
    float *dst = red + (wave - 2) * (7 * 16 * 64) + lane;
#pragma unroll
    for (int t = 0; t < 7; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) dst[(t * 16 + r) * 64] = acc[t][r];
  }
  __syncthreads();
  if (wave < 2) {
    const float *src = red + wave * (7 * 16 * 64) + lane;
#pragma unroll
    for (int t = 0; t < 7; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[t][r] += src[(t * 16 + r) * 64];
  }
  __syncthreads();
  if (wave < 2) {
    // reg r of lane l: output channel 8*(r/4) + 4*(l/32) + r%4, input channel l%32
    float *dst = red + wave * (32 * 32 * 9) + (4 * (lane >> 5) * 32 + (lane & 31)) * 9;
#pragma unroll
    for (int r = 0; r < 16; ++r)
#pragma unroll
      for (int t = 0; t < 7; ++t) dst[(8 * (r >> 2) + (r & 3)) * (32 * 9) + t] = acc[t][r];
  }
  __syncthreads();
  const int crs = a.C * 25;
  float *out = a.partial + (static_cast<size_t>(slice) * a.Kc + co0) * crs + ci0 * 25 + t0;
  for (int e = tid; e < 32 * 32 * 8; e += I8_NT) {
    const int t = e & 7, pair = e >> 3;   // pair = output channel * 32 + input channel
    if (t < ntaps)
      out[static_cast<size_t>(pair >> 5) * crs + (pair & 31) * 25 + t] = red[pair * 9 + t] + red[32 * 32 * 9 + pair * 9 + t];
  }
  if (sums_dy) {
    // the eight shares of a channel sit in neighbouring lanes: added with a fixed butterfly
    dbs += __shfl_xor(dbs, 1, 64);
    dbs += __shfl_xor(dbs, 2, 64);
    dbs += __shfl_xor(dbs, 4, 64);
    if ((tid & 7) == 0) a.partial_db[static_cast<size_t>(slice) * a.Kc + co0 + (tid >> 3)] = dbs;
  }
}

struct DwHaloPlan {
  bool ok;
  bool img8;            // the image-sized kernel runs this shape
  int img_size;         // ... on images of 8x8 or 16x16 pixels
  DwImg8Args i8;
  int tc, wco, wk, wfy, nt;
  int rows_block;  // filter rows one workgroup covers
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
                        int pw, bool allow_img8 = true) {
  DwHaloPlan p;
  p.ok = false;
  const bool five = R == 5 && S == 5;
  if (!(R == 3 && S == 3) && !five) return p;
  if (C < 16 || Kc < 16 || OW < 8 || OH < 2 || pw > 4) return p;
  p.img8 = false;
  // (16x16 images: from the batch on where the chunks give every compute unit a workgroup; the
  // kernel below has fewer, longer workgroups, which is what a step that runs it beside its
  // main chain wants)
  const int is = H == 8 ? 8 : 16;
  if (allow_img8 && five && H == is && W == is && OH == is && OW == is && ph == 2 && pw == 2 && C % 32 == 0 &&
      Kc % 32 == 0 && batch >= (is == 8 ? 4 : 96) && static_cast<long>(batch) * std::max(C, Kc) * is * is < (1L << 30)) {
    DwImg8Args &i = p.i8;
    p.img_size = is;
    i.batch = batch; i.C = C; i.Kc = Kc;
    i.co_blocks = Kc / 32; i.ci_blocks = C / 32;
    i.chunks_total = is == 8 ? ceil_div(batch, 4) : batch;
    // one workgroup per compute unit where the batch allows it
    const int base = 4 * i.co_blocks * i.ci_blocks;
    int slices = std::max(1, 256 / base);
    slices = std::min(slices, i.chunks_total);
    i.chunks_per_slice = ceil_div(i.chunks_total, slices);
    p.slices = ceil_div(i.chunks_total, i.chunks_per_slice);
    p.grid   = dim3(static_cast<unsigned>(p.slices));   // (grid.x counts the slices, as below; the launch multiplies)
    p.lds_bytes = sizeof(float) * (is == 8 ? I8Geom<8>::LDS_FLOATS : I8Geom<16>::LDS_FLOATS);
    p.img8 = true;
    p.ok   = true;
    return p;
  }
  p.tc = OW >= 48 ? 64 : OW >= 24 ? 32 : OW >= 12 ? 16 : 8;
  p.wfy = 1;
  // more than 32 output channels: two channel blocks share a workgroup's staged X patch (half
  // the row groups each), which also keeps the 5x5 kernel's LDS footprint small enough for a
  // convolution workgroup of the main chain to share the compute unit
  p.wco = Kc > 32 ? 2 : 1;
  p.wk  = 4 / p.wco;
  p.nt = 64 * p.wco * p.wk * p.wfy;
  p.rows_block = five ? 1 : R;
  DwHaloArgs &a = p.args;
  a.batch = batch; a.C = C; a.Kc = Kc; a.H = H; a.W = W; a.OH = OH; a.OW = OW; a.ph = ph; a.pw = pw;
  const int tr = (64 / p.tc) * p.wk;
  const int nq = (3 + p.tc + S - 1 + 3) / 4;
  a.pwa = (pw + 3) & ~3;
  a.TI = 1;
  // whole images stacked as rows; rows past the last whole image stay empty
  if (five && tr > OH) a.TI = tr / OH;
  const int prq = (tr + p.rows_block - 1) * nq;
  a.plane_p = (4 * prq) | 1;
  a.dyp     = pad_to_4_mod_32(tr * p.tc);
  // the keep bits of the scalar loads cover 16 words a thread
  if (ceil_div(prq, p.nt / 32) > 16) return p;
  // offsets inside a chunk are 32-bit and must stay clear of the never-exists marker
  if (static_cast<long>(a.TI) * std::max<long>(static_cast<long>(C) * H * W, static_cast<long>(Kc) * OH * OW) >=
      (1L << 29))
    return p;
  a.tiles_x = ceil_div(OW, p.tc);
  const int row_chunks = a.TI > 1 ? 1 : ceil_div(OH, tr);
  a.chunks_total  = a.TI > 1 ? ceil_div(batch, a.TI) : batch * row_chunks;
  a.div_rowchunks = FastDiv(row_chunks);
  a.div_oh        = FastDiv(OH);
  const int co_blocks = ceil_div(Kc, 32 * p.wco), ci_blocks = ceil_div(C, 32) * (R / p.rows_block);
  const long base = static_cast<long>(a.tiles_x) * co_blocks * ci_blocks;
  // one workgroup per CU; a slice should still cover a few chunks so that its prologue and
  // its partial tile are paid for
  long slices = std::max<long>(1, 256 / base);
  slices = std::min<long>(slices, std::max(1, a.chunks_total / 2));
  a.chunks_per_slice = ceil_div(a.chunks_total, static_cast<int>(slices));
  p.slices           = ceil_div(a.chunks_total, a.chunks_per_slice);
  const int nacc = (p.rows_block / p.wfy) * S;
  const size_t stage_floats = static_cast<size_t>(32 * p.wco) * a.dyp + 32 * static_cast<size_t>(a.plane_p);
  const size_t red_floats   = static_cast<size_t>(p.wk / 2) * p.wco * nacc * 16 * 64;
  p.lds_bytes = sizeof(float) * std::max(stage_floats, red_floats);
  if (p.lds_bytes > 150 * 1024) return p;
  if (static_cast<long>(a.tiles_x) * p.slices > 65535L * 16) return p;
  p.grid = dim3(a.tiles_x * p.slices, co_blocks, ci_blocks);
  a.div_gy      = FastDiv(co_blocks);
  a.div_gz      = FastDiv(ci_blocks);
  a.div_tiles_x = FastDiv(a.tiles_x);
  p.ok   = true;
  return p;
}

template <int R, int S, int TC, int WCO, int WK, int WFY, int RF, bool VEC>
int launch_dw_inst(const DwHaloPlan &p) {
  auto kernel = conv_dw_halo_kernel<R, S, TC, WCO, WK, WFY, RF, VEC>;
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
  TDH_LAUNCH(kernel, p.grid, dim3(p.nt), p.lds_bytes, ctx().stream, p.args);
  TDH_LAUNCH_CHECK();
  return TDH_OK;
}

template <int TC, bool VEC>
int launch_dw_tc(const DwHaloPlan &p) {
  if (p.rows_block == 1)
    return p.wco == 2 ? launch_dw_inst<1, 5, TC, 2, 2, 1, 5, VEC>(p) : launch_dw_inst<1, 5, TC, 1, 4, 1, 5, VEC>(p);
  if (p.wco == 2) return launch_dw_inst<3, 3, TC, 2, 2, 1, 3, VEC>(p);
  // 8 columns x 4 row groups would stage 17 words a thread; the plan leaves that tile out
  if (TC == 8) return set_error(TDH_ERR_INVALID, "conv_dw_halo_run: tile not built");
  return launch_dw_inst<3, 3, (TC == 8 ? 16 : TC), 1, 4, 1, 3, VEC>(p);
}

template <bool VEC>
int launch_dw_vec(const DwHaloPlan &p) {
  switch (p.tc) {
    case 64: return launch_dw_tc<64, VEC>(p);
    case 32: return launch_dw_tc<32, VEC>(p);
    case 16: return launch_dw_tc<16, VEC>(p);
    default: return launch_dw_tc<8, VEC>(p);
  }
}

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace

bool conv_dw_halo_applicable(int R, int S, int batch, int C, int Kc, int H, int W, int OH, int OW,
                             int ph, int pw) {
  return make_dw_plan(R, S, batch, C, Kc, H, W, OH, OW, ph, pw).ok;
}

size_t conv_dw_halo_workspace_bytes(int R, int S, int batch, int C, int Kc, int H, int W, int OH,
                                    int OW, int ph, int pw) {
  const DwHaloPlan p = make_dw_plan(R, S, batch, C, Kc, H, W, OH, OW, ph, pw);
  if (!p.ok) return 0;
  // (tensors that are not 16-byte aligned take the general kernel's plan where the 8x8-image
  // kernel would run: room for whichever has more slices)
  const DwHaloPlan q = p.img8 ? make_dw_plan(R, S, batch, C, Kc, H, W, OH, OW, ph, pw, false) : p;
  const size_t slices = std::max(p.grid.x, q.ok ? q.grid.x : 0u);
  return ws_align(sizeof(float) * slices * Kc * C * R * S) + ws_align(sizeof(float) * slices * Kc);
}

// dw (+)= sum over the batch; the caller has checked applicability and reserved the workspace
int conv_dw_halo_run(int R, int S, int batch, int C, int Kc, const float *x, const float *dy,
                     float *dw, int H, int W, int OH, int OW, int ph, int pw, int accumulate,
                     float *db) {
  const bool vec = W % 4 == 0 && OW % 4 == 0 && aligned16(x) && aligned16(dy);
  DwHaloPlan p = make_dw_plan(R, S, batch, C, Kc, H, W, OH, OW, ph, pw, /*allow_img8=*/vec);
  if (!p.ok) return set_error(TDH_ERR_INVALID, "conv_dw_halo_run: shape not supported");
  const int crs = C * R * S;
  void *part = nullptr;
  TDH_TRY(ws_take(sizeof(float) * static_cast<size_t>(p.grid.x) * Kc * crs, &part));
  p.args.x = x; p.args.dy = dy; p.args.partial = static_cast<float *>(part);
  p.args.partial_db = nullptr;
  if (db) {
    void *part_db = nullptr;
    TDH_TRY(ws_take(sizeof(float) * static_cast<size_t>(p.grid.x) * Kc, &part_db));
    p.args.partial_db = static_cast<float *>(part_db);
  }
  {
    ProfScope prof(db ? "conv_dw_db_halo" : "conv_dw_halo", Kc, crs, batch * OH * OW);
    if (p.img8) {
      p.i8.x = x; p.i8.dy = dy; p.i8.partial = p.args.partial; p.i8.partial_db = p.args.partial_db;
      static bool raised[2] = {false, false};
      const int which = p.img_size == 8 ? 0 : 1;
      void (*kernel)(const DwImg8Args) = which ? conv_dw_img8_kernel<16> : conv_dw_img8_kernel<8>;
      if (!raised[which]) {
        TDH_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(p.lds_bytes)));
        raised[which] = true;
      }
      TDH_LAUNCH(kernel, dim3(p.slices * p.i8.ci_blocks * p.i8.co_blocks * 4), dim3(I8_NT), p.lds_bytes,
                 ctx().stream, p.i8);
      TDH_LAUNCH_CHECK();
    } else if (vec) {
      TDH_TRY(launch_dw_vec<true>(p));
    } else {
      TDH_TRY(launch_dw_vec<false>(p));
    }
  }
  const int slices = static_cast<int>(p.grid.x);
  EpiRowMajor epi{dw, crs, nullptr, ActGrad(), accumulate};
  EpiRowMajor epi_b{db, 1, nullptr, ActGrad(), accumulate};
  // the two reductions leave as one launch: collected by the train step, or here
  const bool collect_here = !ctx().defer_reduce;
  if (collect_here) flush_deferred_reduces(false);  // nothing may be left from a failed call
  ctx().defer_reduce = true;
  defer_reduce(p.args.partial, slices, Kc, crs, epi);
  if (db) defer_reduce(p.args.partial_db, slices, Kc, 1, epi_b);
  if (!collect_here) return TDH_OK;
  ctx().defer_reduce = false;
  return flush_deferred_reduces();
}

}  // namespace tdh
