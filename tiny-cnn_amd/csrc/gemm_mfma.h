// gemm_mfma.h — LDS-tiled fp32 MFMA GEMM for gfx950 with pluggable operand loaders.
//
// C[M][N] = sum_k A[m][k] * B[k][n], computed by 256-thread workgroups (four wave64)
// with v_mfma_f32_32x32x2_f32. Operands are not required to be matrices in memory:
// each side is a small functor that maps a GEMM coordinate to a global address, which
// is how convolution gradients (implicit im2col / col2im) and the three fully-connected
// products share one kernel. Out-of-range coordinates read as zero.
//
// Work decomposition
//   grid.x = N tiles, grid.y = M tiles, grid.z = K splits. With more than one split
//   every workgroup writes its partial tile to scratch[z][M][N] and a second kernel adds
//   the splits in index order 0..S-1, so the result does not depend on scheduling.
//   The number of splits is a function of the problem shape only.
//
// Operand loader concept (device side)
//   struct Op {
//     struct Fix;                              // per-thread state of its fixed m (or n)
//     struct KDec;                             // decomposed reduction index
//     __device__ Fix  fix(int mn) const;       // must tolerate mn >= extent (valid=false)
//     __device__ KDec kdec(int k) const;       // k < K guaranteed by the caller
//     __device__ float load(const Fix&, const KDec&) const;   // 0 when fix is invalid
//   };
//   LANE_K = true : consecutive lanes walk k (operand contiguous along k)
//   LANE_K = false: consecutive lanes walk m/n (operand contiguous along m/n); k is then
//                   wave-uniform and its decomposition runs on the scalar unit.
//
// Epilogue concept
//   struct Epi { struct Col; __device__ Col col(int n) const;
//                __device__ float prior(int m, const Col&) const;   // old value if the store adds
//                __device__ void store(int m, const Col&, float v, float prior) const;
//                __device__ void store(int m, const Col&, float v) const; };
#pragma once

#include "common.h"

namespace tdh {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int GEMM_BK      = 16;
constexpr int GEMM_LDS_PAD = 4;

// four floats with 4-byte alignment: lets the compiler emit one dwordx4 access where the
// address is only float-aligned (global memory tolerates it)
struct __attribute__((packed, aligned(4))) float4u {
  float x, y, z, w;
};

// ------------------------------------------------------------ plain matrices
// element(mn, k) = p[mn * s_mn + k * s_k]
struct StridedOperand {
  const float *p;
  int s_mn, s_k, extent;
  struct Fix {
    int off;
    bool valid;
  };
  struct KDec {
    int off;
  };
  __device__ __forceinline__ Fix fix(int mn) const { return {mn * s_mn, mn < extent}; }
  __device__ __forceinline__ KDec kdec(int k) const { return {k * s_k}; }
  __device__ __forceinline__ float load(const Fix &f, const KDec &k) const {
    return f.valid ? p[f.off + k.off] : 0.0f;
  }
  // four consecutive k (needs s_k == 1)
  __device__ __forceinline__ float4 load4k(const Fix &f, const KDec &k) const {
    if (!f.valid) return make_float4(0.f, 0.f, 0.f, 0.f);
    const float4u v = *reinterpret_cast<const float4u *>(p + f.off + k.off);
    return make_float4(v.x, v.y, v.z, v.w);
  }
  // four consecutive m/n starting at f (needs s_mn == 1); `count` of them are in range
  __device__ __forceinline__ float4 load4m(const Fix &f, const KDec &k, int mn) const {
    float4 r = make_float4(0.f, 0.f, 0.f, 0.f);
    if (mn + 3 < extent) {
      const float4u v = *reinterpret_cast<const float4u *>(p + f.off + k.off);
      r = make_float4(v.x, v.y, v.z, v.w);
    } else {
      if (mn < extent) r.x = p[f.off + k.off];
      if (mn + 1 < extent) r.y = p[f.off + k.off + 1];
      if (mn + 2 < extent) r.z = p[f.off + k.off + 2];
    }
    return r;
  }
};

// ------------------------------------------------------------------ epilogues
// out[m*ld + n] = (accumulate ? out : 0) + (v + bias_n[n]) * act'(y[m*ld + n])
struct EpiRowMajor {
  float *out;
  int ld;
  const float *bias_n;
  ActGrad ag;
  int accumulate;
  struct Col {
    int n;
    float bias;
  };
  __device__ __forceinline__ Col col(int n) const { return {n, bias_n ? bias_n[n] : 0.0f}; }
  // what the output holds before the store, when the store adds to it (else 0). A kernel that
  // stores several values a lane asks for all of them first: loads between its stores would
  // each wait for the store before (they may alias), one trip to memory per value.
  __device__ __forceinline__ float prior(int m, const Col &c) const {
    return accumulate ? out[m * ld + c.n] : 0.0f;
  }
  __device__ __forceinline__ void store(int m, const Col &c, float v, float before) const {
    const int idx = m * ld + c.n;
    v += c.bias;
    if (ag.kind != TDH_ACT_NONE) v *= act_grad_factor(ag.kind, ag.y[idx]);
    out[idx] = v + before;
  }
  __device__ __forceinline__ void store(int m, const Col &c, float v) const { store(m, c, v, prior(m, c)); }
};

// forward product followed by a pointwise activation layer:
// out[m*ld + n] = v + bias_n[n], act_out[m*ld + n] = act(out[m*ld + n])
struct EpiRowMajorAct {
  float *out;
  int ld;
  const float *bias_n;
  float *act_out;
  int act_kind;
  struct Col {
    int n;
    float bias;
  };
  __device__ __forceinline__ Col col(int n) const { return {n, bias_n ? bias_n[n] : 0.0f}; }
  __device__ __forceinline__ float prior(int, const Col &) const { return 0.0f; }
  __device__ __forceinline__ void store(int m, const Col &c, float v, float = 0.0f) const {
    const int idx = m * ld + c.n;
    v += c.bias;
    out[idx]     = v;
    act_out[idx] = act_apply(act_kind, v);
  }
};

// GEMM column n = (img, p) with p < pix; out[(img*rows + m)*pix + p] = (v + bias_m[m]) * act'
struct EpiImageRows {
  float *out;
  int rows, pix;
  FastDiv pix_div;
  const float *bias_m;
  ActGrad ag;
  struct Col {
    int base;  // img*rows*pix + p
  };
  __device__ __forceinline__ Col col(int n) const {
    uint32_t img, p;
    pix_div.divmod(static_cast<uint32_t>(n), img, p);
    return {static_cast<int>(img) * rows * pix + static_cast<int>(p)};
  }
  __device__ __forceinline__ float prior(int, const Col &) const { return 0.0f; }
  __device__ __forceinline__ void store(int m, const Col &c, float v, float = 0.0f) const {
    const int idx = c.base + m * pix;
    if (bias_m) v += bias_m[m];
    if (ag.kind != TDH_ACT_NONE) v *= act_grad_factor(ag.kind, ag.y[idx]);
    out[idx] = v;
  }
};

// forward convolution followed by a pointwise activation layer:
// out = v + bias_m[m], act_out = act(out), both laid out like EpiImageRows
struct EpiImageRowsAct {
  float *out;
  int rows, pix;
  FastDiv pix_div;
  const float *bias_m;
  float *act_out;
  int act_kind;
  struct Col {
    int base;
  };
  __device__ __forceinline__ Col col(int n) const {
    uint32_t img, p;
    pix_div.divmod(static_cast<uint32_t>(n), img, p);
    return {static_cast<int>(img) * rows * pix + static_cast<int>(p)};
  }
  __device__ __forceinline__ float prior(int, const Col &) const { return 0.0f; }
  __device__ __forceinline__ void store(int m, const Col &c, float v, float = 0.0f) const {
    const int idx = c.base + m * pix;
    if (bias_m) v += bias_m[m];
    out[idx]     = v;
    act_out[idx] = act_apply(act_kind, v);
  }
};

// --------------------------------------------------------------------- kernel
template <int BM, int BN, int WM, int WN, bool A_LANE_K, bool B_LANE_K, bool A_VEC, bool B_VEC,
          class AOp, class BOp, class Epi>
__global__ void __launch_bounds__(64 * WM * WN) __attribute__((amdgpu_waves_per_eu(3, 8)))
gemm_mfma_kernel(const AOp aop, const BOp bop, const Epi epi, const int M, const int N,
                 const int K, const int k_per_split, float *__restrict__ partial) {
  constexpr int BK  = GEMM_BK;
  constexpr int NT  = 64 * WM * WN;  // threads per workgroup
  constexpr int TM  = BM / WM / 32;  // 32x32 MFMA blocks per wave along M
  constexpr int TN  = BN / WN / 32;
  constexpr int CA  = BM * BK / NT;  // elements of A each thread stages per tile
  constexpr int CB  = BN * BK / NT;
  constexpr int LDA = BM + GEMM_LDS_PAD;
  constexpr int LDB = BN + GEMM_LDS_PAD;
  static_assert(TM >= 1 && TN >= 1, "wave tile must hold at least one 32x32 block");
  static_assert(TM * 32 * WM == BM && TN * 32 * WN == BN, "tile is not a whole number of blocks");
  static_assert((BM * BK) % NT == 0 && (BN * BK) % NT == 0, "tile/threads mismatch");
  // vectorised staging: a thread moves groups of four floats (four k of one row, or four rows
  // of one k). Groups per thread: CA/4, CB/4.
  static_assert(!A_VEC || (CA % 4 == 0 && (A_LANE_K || (4 * NT) % BM == 0)), "A vec4 shape");
  static_assert(!B_VEC || (CB % 4 == 0 && (B_LANE_K || (4 * NT) % BN == 0)), "B vec4 shape");

  __shared__ __attribute__((aligned(16))) float As[2][BK][LDA];
  __shared__ __attribute__((aligned(16))) float Bs[2][BK][LDB];

  const int tid  = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm   = wave % WM;
  const int wn   = wave / WM;
  // Workgroups are handed to the eight XCDs (each with its own L2) round-robin in launch
  // order. Renumber them so that workgroups that are neighbours in (n-tile, m-tile, split)
  // order, which read the same rows of A or columns of B, run on the same XCD.
  int bx, by, bz;
  {
    const int gx = gridDim.x, gy = gridDim.y;
    const int total = gx * gy * gridDim.z, per = total >> 3;
    int id = blockIdx.x + gx * (blockIdx.y + gy * blockIdx.z);
    if (id < (per << 3)) id = (id & 7) * per + (id >> 3);
    bx = id % gx;
    id /= gx;
    by = id % gy;
    bz = id / gy;
  }
  const int m0   = by * BM;
  const int n0   = bx * BN;
  const int kbeg = bz * k_per_split;
  const int kend = min(K, kbeg + k_per_split);

  // ---- per-thread staging assignment
  // LANE_K : k_local = tid % 16 (fixed), rows (tid/16) + (NT/16)*i
  // !LANE_K: element e = tid + NT*i of the tile, row = e % BM, k_local = e / BM; when the
  //          tile width is a multiple of NT the row is the same for every i
  constexpr bool A_ONE_ROW = (NT % BM) == 0;
  constexpr bool B_ONE_ROW = (NT % BN) == 0;
  typename AOp::Fix fa[(A_LANE_K || !A_ONE_ROW) ? CA : 1];
  typename BOp::Fix fb[(B_LANE_K || !B_ONE_ROW) ? CB : 1];
  if constexpr (A_VEC && A_LANE_K) {
    // k group = tid % 4, rows (tid/4) + (NT/4)*i
#pragma unroll
    for (int i = 0; i < CA / 4; ++i) fa[i] = aop.fix(m0 + (tid >> 2) + (NT / 4) * i);
  } else if constexpr (A_VEC) {
    // row group = tid % (BM/4) (rows 4g..4g+3), k_local = tid/(BM/4) + (4*NT/BM)*i
    fa[0] = aop.fix(m0 + 4 * (tid % (BM / 4)));
  } else if (A_LANE_K) {
#pragma unroll
    for (int i = 0; i < CA; ++i) fa[i] = aop.fix(m0 + (tid >> 4) + (NT / 16) * i);
  } else if (A_ONE_ROW) {
    fa[0] = aop.fix(m0 + tid % BM);
  } else {
#pragma unroll
    for (int i = 0; i < CA; ++i) fa[i] = aop.fix(m0 + (tid + NT * i) % BM);
  }
  if constexpr (B_VEC && B_LANE_K) {
#pragma unroll
    for (int i = 0; i < CB / 4; ++i) fb[i] = bop.fix(n0 + (tid >> 2) + (NT / 4) * i);
  } else if constexpr (B_VEC) {
    fb[0] = bop.fix(n0 + 4 * (tid % (BN / 4)));
  } else if (B_LANE_K) {
#pragma unroll
    for (int i = 0; i < CB; ++i) fb[i] = bop.fix(n0 + (tid >> 4) + (NT / 16) * i);
  } else if (B_ONE_ROW) {
    fb[0] = bop.fix(n0 + tid % BN);
  } else {
#pragma unroll
    for (int i = 0; i < CB; ++i) fb[i] = bop.fix(n0 + (tid + NT * i) % BN);
  }

  float ra[CA], rb[CB];

  auto fetch = [&](int kt) {
    if constexpr (A_VEC && A_LANE_K) {
      const int k = kt + 4 * (tid & 3);
#pragma unroll
      for (int i = 0; i < CA / 4; ++i) {
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (k + 3 < kend) {
          v = aop.load4k(fa[i], aop.kdec(k));
        } else {
          if (k < kend) v.x = aop.load(fa[i], aop.kdec(k));
          if (k + 1 < kend) v.y = aop.load(fa[i], aop.kdec(k + 1));
          if (k + 2 < kend) v.z = aop.load(fa[i], aop.kdec(k + 2));
        }
        ra[4 * i] = v.x; ra[4 * i + 1] = v.y; ra[4 * i + 2] = v.z; ra[4 * i + 3] = v.w;
      }
    } else if constexpr (A_VEC) {
#pragma unroll
      for (int i = 0; i < CA / 4; ++i) {
        int k = kt + tid / (BM / 4) + (4 * NT / BM) * i;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (k < kend) v = aop.load4m(fa[0], aop.kdec(k), m0 + 4 * (tid % (BM / 4)));
        ra[4 * i] = v.x; ra[4 * i + 1] = v.y; ra[4 * i + 2] = v.z; ra[4 * i + 3] = v.w;
      }
    } else if (A_LANE_K) {
      const int k = kt + (tid & 15);
      if (k < kend) {
        const typename AOp::KDec kd = aop.kdec(k);
#pragma unroll
        for (int i = 0; i < CA; ++i) ra[i] = aop.load(fa[i], kd);
      } else {
#pragma unroll
        for (int i = 0; i < CA; ++i) ra[i] = 0.0f;
      }
    } else {
#pragma unroll
      for (int i = 0; i < CA; ++i) {
        int k = kt + (tid + NT * i) / BM;
        if (BM % 64 == 0) k = __builtin_amdgcn_readfirstlane(k);
        ra[i] = (k < kend) ? aop.load(fa[A_ONE_ROW ? 0 : i], aop.kdec(k)) : 0.0f;
      }
    }
    if constexpr (B_VEC && B_LANE_K) {
      const int k = kt + 4 * (tid & 3);
#pragma unroll
      for (int i = 0; i < CB / 4; ++i) {
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (k + 3 < kend) {
          v = bop.load4k(fb[i], bop.kdec(k));
        } else {
          if (k < kend) v.x = bop.load(fb[i], bop.kdec(k));
          if (k + 1 < kend) v.y = bop.load(fb[i], bop.kdec(k + 1));
          if (k + 2 < kend) v.z = bop.load(fb[i], bop.kdec(k + 2));
        }
        rb[4 * i] = v.x; rb[4 * i + 1] = v.y; rb[4 * i + 2] = v.z; rb[4 * i + 3] = v.w;
      }
    } else if constexpr (B_VEC) {
#pragma unroll
      for (int i = 0; i < CB / 4; ++i) {
        int k = kt + tid / (BN / 4) + (4 * NT / BN) * i;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (k < kend) v = bop.load4m(fb[0], bop.kdec(k), n0 + 4 * (tid % (BN / 4)));
        rb[4 * i] = v.x; rb[4 * i + 1] = v.y; rb[4 * i + 2] = v.z; rb[4 * i + 3] = v.w;
      }
    } else if (B_LANE_K) {
      const int k = kt + (tid & 15);
      if (k < kend) {
        const typename BOp::KDec kd = bop.kdec(k);
#pragma unroll
        for (int i = 0; i < CB; ++i) rb[i] = bop.load(fb[i], kd);
      } else {
#pragma unroll
        for (int i = 0; i < CB; ++i) rb[i] = 0.0f;
      }
    } else {
#pragma unroll
      for (int i = 0; i < CB; ++i) {
        int k = kt + (tid + NT * i) / BN;
        if (BN % 64 == 0) k = __builtin_amdgcn_readfirstlane(k);
        rb[i] = (k < kend) ? bop.load(fb[B_ONE_ROW ? 0 : i], bop.kdec(k)) : 0.0f;
      }
    }
  };

  auto stage = [&](int buf) {
    if constexpr (A_VEC && A_LANE_K) {
#pragma unroll
      for (int i = 0; i < CA / 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          As[buf][4 * (tid & 3) + j][(tid >> 2) + (NT / 4) * i] = ra[4 * i + j];
    } else if constexpr (A_VEC) {
#pragma unroll
      for (int i = 0; i < CA / 4; ++i)
        *reinterpret_cast<float4 *>(&As[buf][tid / (BM / 4) + (4 * NT / BM) * i][4 * (tid % (BM / 4))]) =
          make_float4(ra[4 * i], ra[4 * i + 1], ra[4 * i + 2], ra[4 * i + 3]);
    } else if (A_LANE_K) {
#pragma unroll
      for (int i = 0; i < CA; ++i) As[buf][tid & 15][(tid >> 4) + (NT / 16) * i] = ra[i];
    } else {
#pragma unroll
      for (int i = 0; i < CA; ++i) As[buf][(tid + NT * i) / BM][(tid + NT * i) % BM] = ra[i];
    }
    if constexpr (B_VEC && B_LANE_K) {
#pragma unroll
      for (int i = 0; i < CB / 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          Bs[buf][4 * (tid & 3) + j][(tid >> 2) + (NT / 4) * i] = rb[4 * i + j];
    } else if constexpr (B_VEC) {
#pragma unroll
      for (int i = 0; i < CB / 4; ++i)
        *reinterpret_cast<float4 *>(&Bs[buf][tid / (BN / 4) + (4 * NT / BN) * i][4 * (tid % (BN / 4))]) =
          make_float4(rb[4 * i], rb[4 * i + 1], rb[4 * i + 2], rb[4 * i + 3]);
    } else if (B_LANE_K) {
#pragma unroll
      for (int i = 0; i < CB; ++i) Bs[buf][tid & 15][(tid >> 4) + (NT / 16) * i] = rb[i];
    } else {
#pragma unroll
      for (int i = 0; i < CB; ++i) Bs[buf][(tid + NT * i) / BN][(tid + NT * i) % BN] = rb[i];
    }
  };

  floatx16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  const int a_col = wm * (BM / WM) + (lane & 31);
  const int b_col = wn * (BN / WN) + (lane & 31);
  const int k_sub = lane >> 5;

  int cur = 0;
  if (kbeg < kend) {
    fetch(kbeg);
    stage(0);
  }
  __syncthreads();

  for (int kt = kbeg; kt < kend; kt += BK) {
    const bool has_next = kt + BK < kend;
    if (has_next) fetch(kt + BK);

#pragma unroll
    for (int kk = 0; kk < BK / 2; ++kk) {
      float af[TM], bf[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) af[i] = As[cur][2 * kk + k_sub][a_col + 32 * i];
#pragma unroll
      for (int j = 0; j < TN; ++j) bf[j] = Bs[cur][2 * kk + k_sub][b_col + 32 * j];
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i], bf[j], acc[i][j], 0, 0, 0);
    }

    if (has_next) stage(cur ^ 1);
    __syncthreads();
    cur ^= 1;
  }

  // ---- epilogue: D[i][j] of a 32x32 block lives in reg r of lane l at
  //      i = 8*(r/4) + 4*(l/32) + r%4, j = l%32
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int n = n0 + wn * (BN / WN) + 32 * j + (lane & 31);
    if (n >= N) continue;
    if (partial != nullptr) {
      float *dst = partial + static_cast<size_t>(bz) * M * N + n;
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int m = m0 + wm * (BM / WM) + 32 * i + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
          if (m < M) dst[static_cast<size_t>(m) * N] = acc[i][j][r];
        }
    } else {
      const typename Epi::Col c = epi.col(n);
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        float before[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int m = m0 + wm * (BM / WM) + 32 * i + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
          before[r]   = m < M ? epi.prior(m, c) : 0.0f;
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int m = m0 + wm * (BM / WM) + 32 * i + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
          if (m < M) epi.store(m, c, acc[i][j][r], before[r]);
        }
      }
    }
  }
}

// Adds the K-split partial tiles and applies the epilogue. A workgroup owns 32 consecutive
// outputs; its eight 32-lane groups each add every eighth slice (g, g+8, ...) and the eight
// group sums are then added in group order, so the summation tree depends on the split
// count only.
constexpr int REDUCE_OUTPUTS = 32;
constexpr int REDUCE_GROUPS  = 8;

template <class Epi>
__device__ __forceinline__ void splitk_reduce_block(const float *__restrict__ partial, const int splits,
                                                    const int M, const int N, const Epi &epi,
                                                    const int block, float (*sm)[REDUCE_OUTPUTS]) {
  const int o   = threadIdx.x & (REDUCE_OUTPUTS - 1);
  const int g   = threadIdx.x / REDUCE_OUTPUTS;
  const int idx = block * REDUCE_OUTPUTS + o;
  const size_t mn = static_cast<size_t>(M) * N;
  float s = 0.0f;
  if (idx < M * N) {
    // eight slices per trip: the loads are issued together, the adds keep slice order
    int z = g;
    for (; z + 7 * REDUCE_GROUPS < splits; z += 8 * REDUCE_GROUPS) {
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = partial[(z + u * REDUCE_GROUPS) * mn + idx];
#pragma unroll
      for (int u = 0; u < 8; ++u) s += v[u];
    }
    for (; z < splits; z += REDUCE_GROUPS) s += partial[z * mn + idx];
  }
  sm[g][o] = s;
  __syncthreads();
  if (g == 0 && idx < M * N) {
    float t = sm[0][o];
#pragma unroll
    for (int i = 1; i < REDUCE_GROUPS; ++i) t += sm[i][o];
    const int m = idx / N, n = idx - m * N;
    epi.store(m, epi.col(n), t);
  }
}

template <class Epi>
__global__ void __launch_bounds__(256)
splitk_reduce_kernel(const float *__restrict__ partial, const int splits, const int M, const int N,
                     const Epi epi) {
  __shared__ float sm[REDUCE_GROUPS][REDUCE_OUTPUTS];
  splitk_reduce_block(partial, splits, M, N, epi, blockIdx.x, sm);
}

// The same sums for a large result (N a multiple of four): a thread owns four neighbouring
// outputs and reads every slice as one 16-byte word, eight slices in flight. Slice z still
// goes to group z % 8 and the groups are added in order, so the result is the one of the
// kernel above bit for bit; that kernel gives a workgroup 32 outputs, which for a million
// outputs and eight slices is 32768 workgroups of one load a thread.
template <class Epi>
__global__ void __launch_bounds__(256)
splitk_reduce_wide_kernel(const float *__restrict__ partial, const int splits, const int M, const int N,
                          const Epi epi) {
  typedef float f4 __attribute__((ext_vector_type(4)));
  const size_t mn = static_cast<size_t>(M) * N;
  const size_t idx = (static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x) * 4;
  if (idx >= mn) return;
  f4 s[REDUCE_GROUPS];
#pragma unroll
  for (int g = 0; g < REDUCE_GROUPS; ++g) s[g] = f4{0.0f, 0.0f, 0.0f, 0.0f};
  for (int z0 = 0; z0 < splits; z0 += REDUCE_GROUPS) {
    f4 v[REDUCE_GROUPS];
#pragma unroll
    for (int g = 0; g < REDUCE_GROUPS; ++g)  // (every load is issued: a slice past the last repeats it and is dropped)
      v[g] = *reinterpret_cast<const f4 *>(partial + static_cast<size_t>(min(z0 + g, splits - 1)) * mn + idx);
#pragma unroll
    for (int g = 0; g < REDUCE_GROUPS; ++g)
      if (z0 + g < splits) s[g] += v[g];
  }
  f4 t = s[0];
#pragma unroll
  for (int g = 1; g < REDUCE_GROUPS; ++g) t += s[g];
  const int m = static_cast<int>(idx / N), n = static_cast<int>(idx - static_cast<size_t>(m) * N);
  typename Epi::Col c[4];
  float before[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    c[e]      = epi.col(n + e);
    before[e] = epi.prior(m, c[e]);
  }
#pragma unroll
  for (int e = 0; e < 4; ++e) epi.store(m, c[e], t[e], before[e]);
}
constexpr long REDUCE_WIDE_MIN = 1L << 18;  // outputs from which the wide kernel is launched

// Several reductions in one launch: the weight gradients of a train step's layers, whose
// partial tiles are all complete when the last dW kernel ends. Job j owns the workgroups
// [first_block[j], first_block[j+1]).
constexpr int REDUCE_MULTI_MAX = 8;
struct ReduceJob {
  const float *partial;
  int splits, M, N;
  EpiRowMajor epi;
};
struct ReduceJobs {
  ReduceJob job[REDUCE_MULTI_MAX];
  int first_block[REDUCE_MULTI_MAX + 1];
  int n;
};
__global__ void __launch_bounds__(256) splitk_reduce_multi_kernel(const ReduceJobs jobs);

// While ctx().defer_reduce is set, a split reduction with the row-major epilogue is recorded
// instead of launched; flush_deferred_reduces() (common.h) launches what was recorded.
bool defer_reduce(const float *partial, int splits, int M, int N, const EpiRowMajor &epi);
template <class Epi>
inline bool defer_reduce(const float *, int, int, int, const Epi &) { return false; }

// ------------------------------------------------------------------- launcher
struct GemmPlan {
  int cfg;          // index into the tile table below
  int bm, bn;       // tile
  int splits;       // K splits
  int k_per_split;  // multiple of GEMM_BK
};

// tile table: {BM, BN, waves along M, waves along N}
struct TileCfg {
  int bm, bn, wm, wn;
};
constexpr TileCfg kTiles[] = {
  {128, 128, 2, 2},  // 0
  {128, 64, 2, 2},   // 1
  {64, 128, 2, 2},   // 2
  {64, 64, 2, 2},    // 3
  {32, 128, 1, 4},   // 4
  {32, 256, 1, 4},   // 5
  {32, 64, 1, 2},    // 6
  {64, 32, 2, 1},    // 7
  {32, 32, 1, 1},    // 8
  {64, 96, 2, 1},    // 9
};
constexpr int kNumTiles = sizeof(kTiles) / sizeof(kTiles[0]);

// Optional override "cfg,splits[,M]" from the environment (tuning runs only; with M only
// products of that many rows).
bool gemm_plan_override(int *cfg, int *splits, int M);

// Shape-only heuristics (no device queries) so that results are reproducible anywhere.
inline GemmPlan plan_gemm(int M, int N, int K, bool allow_split) {
  // relative MFMA efficiency of a tile (operand fetches per MFMA, prologue share)
  static const double kEff[kNumTiles] = {1.00, 0.80, 0.80, 0.72, 0.62, 0.80, 0.50, 0.50, 0.36, 0.84};
  const double kSlots = 512.0;  // workgroups of 256 threads the chip runs at full rate
  int best = 0, best_splits = 1;
  double best_cost = 1e300;
  for (int c = 0; c < kNumTiles; ++c) {
    const TileCfg &t = kTiles[c];
    if (t.bm > 32 && t.bm >= 2 * M && M > 0 && t.bm / 2 >= 32) continue;  // half the rows empty
    if (t.bn > 32 && t.bn >= 2 * N && t.bn / 2 >= 32) continue;
    const double tiles = static_cast<double>(ceil_div(M, t.bm)) * ceil_div(N, t.bn);
    const double slots = kSlots * 256.0 / (64.0 * t.wm * t.wn);
    int splits = 1;
    if (allow_split && tiles < slots) {
      splits = static_cast<int>(slots / tiles);
      const int max_by_k = K / 16 > 0 ? K / 16 : 1;
      if (splits > max_by_k) splits = max_by_k;
      if (splits < 1) splits = 1;
    }
    const double work  = tiles * t.bm * t.bn * static_cast<double>(K);  // padded MACs
    const double waves = tiles * splits / slots;
    const double fill  = waves >= 1.0 ? waves / static_cast<double>(static_cast<long>(waves + 0.999)) : waves;
    // a workgroup's prologue and epilogue weigh like bm*bn/160 more steps of K: large tiles
    // lose on short reductions (4096 x 4096 x 256: 128x128 tiles 88 us, 64x64 tiles 91 us,
    // 128x64 and 64x128 tiles 101-103 us)
    // (unsplit products only: split ones keep every workgroup resident at once)
    const double eff = splits > 1 ? kEff[c] : kEff[c] * K / (K + t.bm * t.bn / 160.0);
    double cost = work / (eff * (fill > 1.0 ? 1.0 : fill));
    if (splits > 1) cost += 2.0 * tiles * t.bm * t.bn * splits * 64.0;  // partial tile traffic
    if (cost < best_cost) {
      best_cost = cost;
      best = c;
      best_splits = splits;
    }
  }
  int ocfg, osplits;
  if (gemm_plan_override(&ocfg, &osplits, M)) {
    best = ocfg;
    best_splits = allow_split ? osplits : 1;
    if (best_splits > K / GEMM_BK && K >= GEMM_BK) best_splits = K / GEMM_BK;
    if (best_splits < 1) best_splits = 1;
  }
  GemmPlan p;
  p.cfg = best;
  p.bm = kTiles[best].bm;
  p.bn = kTiles[best].bn;
  p.k_per_split = ceil_div(ceil_div(K, best_splits), GEMM_BK) * GEMM_BK;
  p.splits      = ceil_div(K, p.k_per_split);
  if (p.splits < 1) p.splits = 1;
  return p;
}

inline size_t gemm_workspace_bytes(int M, int N, int K, bool allow_split) {
  // the plan can be overridden at run time, so reserve for the largest split count any
  // plan may use for this shape
  const GemmPlan p = plan_gemm(M, N, K, allow_split);
  int ocfg, osplits;
  int splits = p.splits;
  if (gemm_plan_override(&ocfg, &osplits, M) && osplits > splits) splits = osplits;
  return splits > 1 ? ws_align(static_cast<size_t>(splits) * M * N * sizeof(float)) : 0;
}

template <int BM, int BN, int WM, int WN, bool A_LANE_K, bool B_LANE_K, bool A_VEC, bool B_VEC,
          class AOp, class BOp, class Epi>
int launch_gemm_tile(const AOp &a, const BOp &b, const Epi &epi, int M, int N, int K,
                     const GemmPlan &p, float *partial, const char *tag) {
  ProfScope prof(tag, M, N, K);
  dim3 grid(ceil_div(N, BN), ceil_div(M, BM), p.splits);
  TDH_LAUNCH((gemm_mfma_kernel<BM, BN, WM, WN, A_LANE_K, B_LANE_K, A_VEC, B_VEC, AOp, BOp,
                                       Epi>), grid,
                     dim3(64 * WM * WN), 0, ctx().stream, a, b, epi, M, N, K, p.k_per_split,
                     partial);
  TDH_LAUNCH_CHECK();
  return TDH_OK;
}

// A_VEC / B_VEC: the operand provides load4k (LANE_K) or load4m (otherwise) and its layout
// allows groups of four; used by the tiles wide enough for it (the rest stage scalars).
template <bool A_LANE_K, bool B_LANE_K, bool A_VEC = false, bool B_VEC = false, class AOp,
          class BOp, class Epi>
int launch_gemm(const AOp &a, const BOp &b, const Epi &epi, int M, int N, int K,
                bool allow_split, const char *tag, const char *reduce_tag) {
  if (M <= 0 || N <= 0) return TDH_OK;
  TDH_CHECK_ARG(static_cast<long>(M) * N < (1L << 31), "gemm: M*N=%ld too large",
                static_cast<long>(M) * N);
  const GemmPlan p = plan_gemm(M, N, K, allow_split);
  float *partial   = nullptr;
  if (p.splits > 1) {
    void *ws = nullptr;
    TDH_TRY(ws_take(static_cast<size_t>(p.splits) * M * N * sizeof(float), &ws));
    partial = static_cast<float *>(ws);
  }
  int rc = TDH_OK;
#define TDH_TILE(BM, BN, WM, WN, AV, BV)                                                  \
  rc = launch_gemm_tile<BM, BN, WM, WN, A_LANE_K, B_LANE_K, AV, BV>(a, b, epi, M, N, K, p, \
                                                                    partial, tag)
  // vector staging needs at least four floats per thread and operand
  switch (p.cfg) {
    case 0: TDH_TILE(128, 128, 2, 2, A_VEC, B_VEC); break;
    case 1: TDH_TILE(128, 64, 2, 2, A_VEC, B_VEC); break;
    case 2: TDH_TILE(64, 128, 2, 2, A_VEC, B_VEC); break;
    case 3: TDH_TILE(64, 64, 2, 2, A_VEC, B_VEC); break;
    case 4: TDH_TILE(32, 128, 1, 4, false, B_VEC); break;
    case 5: TDH_TILE(32, 256, 1, 4, false, B_VEC); break;
    case 6: TDH_TILE(32, 64, 1, 2, A_VEC, B_VEC); break;
    case 7: TDH_TILE(64, 32, 2, 1, A_VEC, B_VEC); break;
    case 8: TDH_TILE(32, 32, 1, 1, A_VEC, B_VEC); break;
    default: TDH_TILE(64, 96, 2, 1, A_VEC &&A_LANE_K, B_VEC &&B_LANE_K); break;
  }
#undef TDH_TILE
  TDH_TRY(rc);
  if (p.splits > 1) {
    // reads every partial tile once and writes the result once
    if (defer_reduce(partial, p.splits, M, N, epi)) return TDH_OK;
    ProfScope prof(reduce_tag, 4.0 * M * N * (p.splits + 1), WORK_BYTE);
    if (N % 4 == 0 && static_cast<long>(M) * N >= REDUCE_WIDE_MIN &&
        (reinterpret_cast<uintptr_t>(partial) & 15u) == 0)
      TDH_LAUNCH((splitk_reduce_wide_kernel<Epi>), dim3(static_cast<unsigned>(ceil_div_sz(static_cast<size_t>(M) * N / 4, 256))),
                 dim3(256), 0, ctx().stream, partial, p.splits, M, N, epi);
    else
      TDH_LAUNCH((splitk_reduce_kernel<Epi>), dim3(ceil_div(M * N, REDUCE_OUTPUTS)), dim3(256), 0,
                 ctx().stream, partial, p.splits, M, N, epi);
    TDH_LAUNCH_CHECK();
  }
  return TDH_OK;
}

}  // namespace tdh
