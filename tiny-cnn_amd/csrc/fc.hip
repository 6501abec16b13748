// fc.hip — fully-connected forward and backward as three fp32 MFMA GEMMs over tiny-dnn's
// [in][out] row-major weight matrix:
//   forward  Y[s][o]  = sum_c X[s][c] * W[c][o] + b[o]        M=batch N=out K=in
//   dX       dX[s][c] = sum_o dY[s][o] * W[c][o]              M=batch N=in  K=out
//   dW       dW[c][o] = sum_s X[s][c] * dY[s][o]              M=in    N=out K=batch
// dW is reduced over the batch inside the GEMM (K spans the samples) instead of being stored
// per sample and merged afterwards (fully_connected_op_internal.h:54-60, node.h:89-103).
#include "gemm_mfma.h"

namespace tdh {

size_t fc_workspace_bytes(int in, int out, int batch) {
  return gemm_workspace_bytes(batch, out, in, true) + gemm_workspace_bytes(batch, in, out, true) +
         gemm_workspace_bytes(in, out, batch, true);
}

int fc_fwd(int in, int out, int has_bias, int batch, const float *x, const float *w,
           const float *b, float *y) {
  StridedOperand A{x, in, 1, batch};   // X[s][k], k contiguous
  StridedOperand B{w, 1, out, out};    // W[k][n], n contiguous
  EpiRowMajor epi{y, out, has_bias ? b : nullptr, ActGrad(), 0};
  return launch_gemm<true, false, false, true>(A, B, epi, batch, out, in, true, "fc_fwd_gemm",
                                              "fc_fwd_splitk_reduce");
}

int fc_bwd(int in, int out, int has_bias, int batch, const float *x, const float *w,
           const float *dy, float *dx, float *dw, float *db, int accumulate, ActGrad dx_act) {
  if (dx) {
    StridedOperand A{dy, out, 1, batch};  // dY[s][k]
    StridedOperand B{w, out, 1, in};      // W[n][k], k contiguous
    EpiRowMajor epi{dx, in, nullptr, dx_act, 0};
    TDH_TRY((launch_gemm<true, true, false, false>(A, B, epi, batch, in, out, true, "fc_dx_gemm",
                                                 "fc_dx_splitk_reduce")));
  }
  if (dw) {
    StridedOperand A{x, 1, in, in};      // X[k][m], m contiguous
    StridedOperand B{dy, 1, out, out};   // dY[k][n], n contiguous
    EpiRowMajor epi{dw, out, nullptr, ActGrad(), accumulate};
    TDH_TRY((launch_gemm<false, false, true, true>(A, B, epi, in, out, batch, true, "fc_dw_gemm",
                                                   "fc_dw_splitk_reduce")));
  }
  if (db && has_bias) TDH_TRY(launch_colsum(dy, batch, out, db, accumulate));
  return TDH_OK;
}

}  // namespace tdh
