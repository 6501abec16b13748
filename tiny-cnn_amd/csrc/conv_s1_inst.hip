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
// being TI images x TR rows x TC columns. Per chunk of 8 or 16 reduction channels it stages the
// input patch WITH its halo once in LDS ([kc][ti][TR+R-1][row words]) together with the filter
// slice ([tap][kc][m]); every filter tap then reads the same patch at a compile-time offset,
// so each input element is fetched from global memory once per workgroup instead of once per
// tap, and the inner loop is ds_read + v_mfma_f32_32x32x2_f32 only.
//
// Staging is by aligned 16-byte words: the staged patch starts at the image column x0 - pwa,
// pwa the padding rounded up to 4, so that every word of a row is wholly inside or outside the
// image and the fragment reads simply start pwa - pw floats in. Which words of a tile exist
// (image in the batch, row and column in the image) is fixed per thread, so a chunk's loads are
// an offset add and a select against a zero word; the filter slice is rows of BM consecutive
// floats. The next chunk's words are loaded into registers while the current chunk's MFMAs
// run, a few loads per MFMA step, so that the memory system sees a steady stream. Tensors
// whose rows are not multiples of four floats take the same words as four scalar loads.
//
// MFMA operand mapping: A = filter slice (lane: m = l%32, k = l/32 selects channel 2p or 2p+1),
// B = input patch (lane: pixel = l%32 of a 32-pixel block, k likewise), D = 32 channels x 32
// pixels. Stores are contiguous along pixels.
//
// This file holds the kernel and is compiled four times, -DTDH_S1_PART=0..3: 3x3 and 5x5 windows,
// each with 16-byte and with scalar loads.
#include "conv_s1.h"
#include <type_traits>

namespace tdh {

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

// a word that does not exist is loaded from here (not const: the loads must stay in the global
// address space, like those of the tensors)
__device__ __align__(16) float s1_zero_word[4] = {0.0f, 0.0f, 0.0f, 0.0f};

// the value of lane l ^ 1 (a swap inside lane pairs, done by the DPP path of a move)
__device__ __forceinline__ float s1_lane_xor1(const float v) {
  return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0xB1, 0xF, 0xF, true));
}
// the value of lane l ^ X, X = 8 or 16 (a swizzle inside groups of 32 lanes: and 0x1F, or 0, xor X)
template <int X>
__device__ __forceinline__ float s1_lane_xor(const float v) {
  return __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(v), (X << 10) | 0x1F));
}

template <int R, int S, int TC, int TM, int TN, bool VEC>
__global__ void __launch_bounds__(256, 2) conv_s1_kernel(const ConvS1Args a) {
  constexpr int KCH   = s1_kch(R * S, TM, TN);
  constexpr int S1_NIQ = s1_niq(R, S, TC, TM, TN);
  constexpr int RS    = R * S;
  constexpr int BM    = 32 * TM;
  constexpr int NQ    = (3 + TC + S - 1 + 3) / 4;  // words per staged row
  constexpr int PITCH = 4 * NQ;
  constexpr int TPC   = 256 / KCH;                 // threads staging one channel plane
  constexpr int WROW  = BM / 4 * KCH;              // filter words per tap: [kc][m/4]
  constexpr int NWQ   = (RS * WROW + 255) / 256;   // filter words per thread
  constexpr int WTAPS = 256 / WROW;                // taps one staging trip covers (2 or 1)
  // the MFMA loop of a chunk runs in groups of PU channel pairs; the first group also issues
  // the next chunk's loads, spread over its STEPS (channel pair, tap) steps
  constexpr int PU    = RS >= 25 ? 2 : KCH / 2;
  constexpr int STEPS = PU * RS;
  constexpr int NLOAD = S1_NIQ + NWQ;
  static_assert((KCH / 2) % PU == 0, "groups cover the chunk");
  constexpr int LOG_TC = TC == 64 ? 6 : TC == 32 ? 5 : TC == 16 ? 4 : 3;
  static_assert(256 % WROW == 0, "a staging trip covers whole taps");

  extern __shared__ __align__(16) float smem[];
  const int TRH    = a.TR + R - 1;
  const int planeq = a.TI * TRH * NQ;            // words of one channel of the staged patch
  const int plane  = 4 * planeq;
  float *in_l      = smem;                       // [KCH][plane]
  float *w_l       = smem + KCH * plane;         // [RS][KCH][BM]

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

  // ---- staging plan of the input patch: thread -> channel kcl, words tl + TPC*i of its plane
  const int kcl = tid / TPC, tl = tid % TPC;
  int goff[S1_NIQ];             // offset of word i inside a channel's images, -1: never exists
  unsigned long long gkeep = 0; // scalar loads: 4 bits per word, float k lies inside the row
#pragma unroll
  for (int i = 0; i < S1_NIQ; ++i) {
    goff[i] = -1;
    const int pe = tl + TPC * i;
    if (pe < planeq) {
      uint32_t ti, rem;
      a.div_rows.divmod(pe, ti, rem);
      const int r = rem / NQ, q = rem - r * NQ;
      const int img = img0 + ti, iy = y0 - a.ph + r, ix = x0 - a.pwa + 4 * q;
      unsigned keep = 0;
#pragma unroll
      for (int k = 0; k < 4; ++k)
        if (static_cast<unsigned>(ix + k) < static_cast<unsigned>(a.IW)) keep |= 1u << k;
      if (img < a.batch && static_cast<unsigned>(iy) < static_cast<unsigned>(a.IH) &&
          (VEC ? keep == 15u : keep != 0u)) {
        goff[i] = img * a.KC * ihw + iy * a.IW + ix;
        if (!VEC) gkeep |= static_cast<unsigned long long>(keep) << (4 * i);
      }
    }
  }

  // ---- staging plan of the filter slice: word tid + 256*i -> tap wt0 + WTAPS*i, the same
  //      channel and columns for every i
  const int wm4 = tid % (BM / 4), wkc = (tid / (BM / 4)) % KCH, wt0 = tid / WROW;
  unsigned wkeep = 0;
#pragma unroll
  for (int k = 0; k < 4; ++k)
    if (m0 + 4 * wm4 + k < a.MC) wkeep |= 1u << k;
  const bool w_ok = VEC ? wkeep == 15u : wkeep != 0u;
  const size_t wtap = static_cast<size_t>(a.KC) * a.MC;  // floats per tap of wp

  // ---- MFMA operand offsets
  int boff[TN];
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int q  = (wn * TN + j) * 32 + (lane & 31);
    const int ti = q >> (a.log_tr + LOG_TC);
    const int r  = (q >> LOG_TC) & (a.TR - 1);
    const int c  = q & (TC - 1);
    boff[j]      = (ti * TRH + r) * PITCH + c + (a.pwa - a.pw) + (lane >> 5) * plane;
  }
  const int aoff = (lane >> 5) * BM + (lane & 31);

  floatx16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  floatx4 rin[S1_NIQ], rw[NWQ];
  const float *zero = s1_zero_word;

  // loads of the chunk starting at channel kc0 that belong to step `part` of the MFMA loop
  // (part < 0: all of them)
  auto fetch_part = [&](int kc0, int part) {
    const bool ch_ok  = kc0 + kcl < kc_hi;
    const float *base = a.in + static_cast<size_t>(kc0 + kcl) * ihw;
#pragma unroll
    for (int i = 0; i < S1_NIQ; ++i) {
      if (part >= 0 && (i * STEPS) / NLOAD != part) continue;
      const bool ok = ch_ok && goff[i] >= 0;
      if (VEC) {
        rin[i] = *reinterpret_cast<const floatx4 *>(ok ? base + goff[i] : zero);
      } else {
        const unsigned keep = ok ? static_cast<unsigned>(gkeep >> (4 * i)) & 15u : 0u;
        rin[i].x = *((keep & 1u) ? base + goff[i] : zero);
        rin[i].y = *((keep & 2u) ? base + goff[i] + 1 : zero);
        rin[i].z = *((keep & 4u) ? base + goff[i] + 2 : zero);
        rin[i].w = *((keep & 8u) ? base + goff[i] + 3 : zero);
      }
    }
    const bool wch_ok = w_ok && kc0 + wkc < kc_hi;
    const float *wb   = a.wp + static_cast<size_t>(kc0 + wkc) * a.MC + m0 + 4 * wm4;
#pragma unroll
    for (int i = 0; i < NWQ; ++i) {
      if (part >= 0 && ((S1_NIQ + i) * STEPS) / NLOAD != part) continue;
      const int t    = wt0 + WTAPS * i;
      const bool ok  = wch_ok && t < RS;
      const float *p = wb + static_cast<size_t>(t) * wtap;
      if (VEC) {
        rw[i] = *reinterpret_cast<const floatx4 *>(ok ? p : zero);
      } else {
        const unsigned keep = ok ? wkeep : 0u;
        rw[i].x = *((keep & 1u) ? p : zero);
        rw[i].y = *((keep & 2u) ? p + 1 : zero);
        rw[i].z = *((keep & 4u) ? p + 2 : zero);
        rw[i].w = *((keep & 8u) ? p + 3 : zero);
      }
    }
  };
  auto stage = [&]() {
    float *id = in_l + kcl * plane + 4 * tl;
#pragma unroll
    for (int i = 0; i < S1_NIQ; ++i)
      if (tl + TPC * i < planeq) *reinterpret_cast<floatx4 *>(id + 4 * TPC * i) = rin[i];
#pragma unroll
    for (int i = 0; i < NWQ; ++i)
      if (wt0 + WTAPS * i < RS) *reinterpret_cast<floatx4 *>(w_l + 4 * (tid + 256 * i)) = rw[i];
  };

  // one group of PU channel pairs starting at pair p0; next_kc0 >= 0: also issue the loads of
  // that chunk. The choice is made at every step on purpose: the branch keeps the address
  // arithmetic of a load next to it, where a straight-line version computes the addresses of
  // all loads up front and runs out of registers.
  auto mfma_group = [&](int p0, int next_kc0, auto with_loads) {
    // the fragments of step u + 1 are read from LDS before the products of step u are issued:
    // TM + TN registers more, and a wave no longer waits out an LDS read at every step
    float af[2][TM], bf[2][TN];
    auto read_fragments = [&](int u, int to) {
      const int pp = u / RS, t = u % RS;
      const int fy = t / S, fx = t % S;
      const float *inp = in_l + 2 * (p0 + pp) * plane;
      const float *wlp = w_l + 2 * (p0 + pp) * BM + aoff;
#pragma unroll
      for (int i = 0; i < TM; ++i) af[to][i] = wlp[t * KCH * BM + i * 32];
#pragma unroll
      for (int j = 0; j < TN; ++j) bf[to][j] = inp[boff[j] + fy * PITCH + fx];
    };
    read_fragments(0, 0);
#pragma unroll
    for (int u = 0; u < PU * RS; ++u) {
      const int cur = u & 1;
      if (u + 1 < PU * RS) read_fragments(u + 1, cur ^ 1);
      if (decltype(with_loads)::value) fetch_part(next_kc0, u);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[cur][i], bf[cur][j], acc[i][j], 0, 0, 0);
      // (keeps the steps apart: left alone, the compiler moves the LDS reads ahead over many
      // steps, which costs more registers than two resident workgroups have)
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  fetch_part(kc_lo, -1);
  for (int kc0 = kc_lo; kc0 < kc_hi; kc0 += KCH) {
    if (kc0 > kc_lo) __syncthreads();  // everyone is done reading the previous chunk
    stage();
    __syncthreads();
    if (kc0 + KCH < kc_hi) mfma_group(0, kc0 + KCH, std::true_type());
    else mfma_group(0, 0, std::false_type());
#pragma unroll 1
    for (int p0 = PU; p0 < KCH / 2; p0 += PU) mfma_group(p0, 0, std::false_type());
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
    for (int i = 0; i < TM; ++i) {
      // the 16 values of this lane: channels mb + 8*(rr/4) + rr%4, all at pixel pbase
      const int mb = m0 + 32 * i + 4 * (lane >> 5);
      float *dst = a.part ? a.part + blockIdx.z * a.part_stride : a.out;
      float v[16];
#pragma unroll
      for (int rr = 0; rr < 16; ++rr) v[rr] = acc[i][j][rr];
      if (!a.part) {
        if (a.bias) {
#pragma unroll
          for (int rr = 0; rr < 16; ++rr) {
            const int m = mb + 8 * (rr >> 2) + (rr & 3);
            v[rr] += a.bias[min(m, a.MC - 1)];
          }
        }
        if (a.ag.kind != TDH_ACT_NONE) {
          // all loads of y first: one at a time they would each cost a trip to memory
          float yv[16];
#pragma unroll
          for (int rr = 0; rr < 16; ++rr) {
            const int m = mb + 8 * (rr >> 2) + (rr & 3);
            yv[rr] = a.ag.y[pbase + static_cast<size_t>(min(m, a.MC - 1)) * ohw];
          }
#pragma unroll
          for (int rr = 0; rr < 16; ++rr) v[rr] *= act_grad_factor(a.ag.kind, yv[rr]);
        }
      }
      if (dst) {  // (null: the pool behind leaves this kernel too and nobody reads the convolution's own output)
#pragma unroll
        for (int rr = 0; rr < 16; ++rr) {
          const int m = mb + 8 * (rr >> 2) + (rr & 3);
          if (m < a.MC) dst[pbase + static_cast<size_t>(m) * ohw] = v[rr];
        }
      }
      if (!a.part && a.act_out) {
#pragma unroll
        for (int rr = 0; rr < 16; ++rr) {
          const int m = mb + 8 * (rr >> 2) + (rr & 3);
          v[rr]       = act_apply(a.act_kind, v[rr]);
          if (m < a.MC) a.act_out[pbase + static_cast<size_t>(m) * ohw] = v[rr];
        }
      }
      if constexpr (TC <= 16) {
        if (!a.part && a.pool_out) {
          // A 32-pixel block is whole rows of TC pixels, the first one even: the window of the
          // lane with an even row and column is its own value, lane^1's, lane^TC's and
          // lane^(TC+1)'s, scanned in that order with strict '>' from lowest()
          // (maxpool_op_internal.h:17-47). Every lane runs the exchange, the anchors store.
          const bool anchor = !(lane & 1) && !(lane & TC);
          const int pw2 = a.OW >> 1, pohw = (a.OH >> 1) * pw2;
          const size_t pobase = static_cast<size_t>(img) * a.MC * pohw + (oy >> 1) * pw2 + (ox >> 1);
          const int pix = oy * a.OW + ox;
#pragma unroll
          for (int rr = 0; rr < 16; ++rr) {
            const int m = mb + 8 * (rr >> 2) + (rr & 3);
            const float right = s1_lane_xor1(v[rr]);
            const float w4[4] = {v[rr], right, s1_lane_xor<TC>(v[rr]), s1_lane_xor<TC>(right)};
            float best = -3.402823466e+38f;
            int sel    = -1;
#pragma unroll
            for (int k = 0; k < 4; ++k)
              if (w4[k] > best) {
                best = w4[k];
                sel  = k;
              }
            if (anchor && m < a.MC) {
              const size_t at = pobase + static_cast<size_t>(m) * pohw;
              a.pool_out[at]    = best;
              a.pool_argmax[at] = sel < 0 ? 0 : m * ohw + pix + (sel >> 1) * a.OW + (sel & 1);
              if (a.pool_act_out) a.pool_act_out[at] = best > 0.0f ? best : 0.0f;
            }
          }
        }
      }
    }
  }
}

template <int R, int S, int TC, int TM, int TN, bool VEC>
int launch_s1_inst(const S1Plan &p) {
  auto kernel = conv_s1_kernel<R, S, TC, TM, TN, VEC>;
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
  TDH_LAUNCH(kernel, p.grid, dim3(256), p.lds_bytes, ctx().stream, p.args);
  TDH_LAUNCH_CHECK();
  return TDH_OK;
}

template <int R, int S, int TC, bool VEC>
int launch_s1_tc(const S1Plan &p) {
  switch (p.tm * 10 + p.tn) {
    case 22: return launch_s1_inst<R, S, TC, 2, 2, VEC>(p);
    case 21: return launch_s1_inst<R, S, TC, 2, 1, VEC>(p);
    case 14: return launch_s1_inst<R, S, TC, 1, 4, VEC>(p);
    case 12: return launch_s1_inst<R, S, TC, 1, 2, VEC>(p);
    default: return launch_s1_inst<R, S, TC, 1, 1, VEC>(p);
  }
}

template <int R, int S, bool VEC>
int launch_s1_rs(const S1Plan &p) {
  switch (p.tc) {
    case 64: return launch_s1_tc<R, S, 64, VEC>(p);
    case 32: return launch_s1_tc<R, S, 32, VEC>(p);
    case 16: return launch_s1_tc<R, S, 16, VEC>(p);
    default: return launch_s1_tc<R, S, 8, VEC>(p);
  }
}

}  // namespace

#if TDH_S1_PART == 0
int s1_launch_3x3_vec(const S1Plan &p) { return launch_s1_rs<3, 3, true>(p); }
#elif TDH_S1_PART == 1
int s1_launch_3x3_scalar(const S1Plan &p) { return launch_s1_rs<3, 3, false>(p); }
#elif TDH_S1_PART == 2
int s1_launch_5x5_vec(const S1Plan &p) { return launch_s1_rs<5, 5, true>(p); }
#elif TDH_S1_PART == 3
int s1_launch_5x5_scalar(const S1Plan &p) { return launch_s1_rs<5, 5, false>(p); }
#else
#error "TDH_S1_PART must be 0..3"
#endif

}  // namespace tdh
