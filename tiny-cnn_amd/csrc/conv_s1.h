// conv_s1.h — what the host side of the stride-1 convolution kernel (conv_s1.hip) and the
// translation units that instantiate the kernel (conv_s1_inst.hip, compiled once per window and
// load width so that they build in parallel) share.
#pragma once
#include "common.h"

namespace tdh {

// Reduction channels per chunk. Tiles of four accumulator blocks a wave take 8 (4 with 25
// taps), tiles of two channel blocks with 25 taps 8: two workgroups share a CU's 512 registers, and
// beside that many accumulators the staged words of 16 channels no longer fit.
constexpr int s1_kch(int RS, int TM, int TN) {
  return TM * TN >= 4 ? (RS >= 25 ? 4 : 8) : (TM == 2 && TN == 1 && RS >= 25 ? 8 : 16);
}

// Input-patch words a thread stages per chunk at most: a tile of 128*TN pixels in rows of TC,
// cut into at most two images (two halos), 256/KCH threads to a channel plane.
constexpr int s1_niq(int R, int S, int TC, int TM, int TN) {
  const int nq  = (3 + TC + S - 1 + 3) / 4;
  const int tpc = 256 / s1_kch(R * S, TM, TN);
  const int n   = ((128 * TN / TC + 2 * (R - 1)) * nq + tpc - 1) / tpc;
  return n > 16 ? 16 : n;
}

struct ConvS1Args {
  const float *in, *wp, *bias;
  float *out;
  ActGrad ag;
  float *act_out;              // forward: act(out) of the pointwise activation layer that follows
  int act_kind;
  // forward: the 2x2 / stride-2 max-pool layer behind the convolution (or behind act_out) and
  // the relu behind that pool, all null when the pool runs as a kernel of its own. Only tiles
  // whose 32-pixel blocks hold whole pool windows (rows of 8 or 16 pixels, no split) take it.
  float *pool_out;
  int32_t *pool_argmax;        // flat CHW index inside the sample of the pool's input
  float *pool_act_out;         // max(pool_out, 0), or null
  int batch, KC, MC, IH, IW, OH, OW, ph, pw;
  int pwa;                     // staged column 0 is image column x0 - pwa
  int TR, TI;                  // tile rows, images per tile (TI*TR*TC = PIX), powers of two
  int log_tr, log_ti;
  int tiles_x, tiles_y;        // tiles per image row / column direction
  FastDiv div_rows;            // by the words of one image of the staged patch, (TR+R-1)*NQ
  // split over the reduction channels: workgroup z sums channels [z*kc_split, (z+1)*kc_split)
  // into part[z][...] (laid out like out); part == nullptr: one pass, written to out
  int kc_split;
  float *part;
  size_t part_stride;
};

struct S1Plan {
  bool ok;
  int tc, tm, tn;
  ConvS1Args args;
  size_t lds_bytes;
  dim3 grid;
  int splits;
};

// one launcher per translation unit of kernel instances
int s1_launch_3x3_vec(const S1Plan &p);
int s1_launch_3x3_scalar(const S1Plan &p);
int s1_launch_5x5_vec(const S1Plan &p);
int s1_launch_5x5_scalar(const S1Plan &p);

}  // namespace tdh
