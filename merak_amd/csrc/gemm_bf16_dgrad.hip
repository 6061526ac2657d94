// dX[M,K] = dY[M,N] W[N,K]: GEMM (M, K, reduce N) with A = dY (row) and B = W read as [reduce, cols] (col).
#include "gemm_bf16_kernel.h"

int mtp_gemm_bf16_dgrad(const void* dy, const void* w, void* dx, int64_t M, int64_t N, int64_t K, int f16, void* ws,
                        hipStream_t s) {
  GemmArgs a{};
  a.A = (const uint16_t*)dy;
  a.B = (const uint16_t*)w;
  a.C = dx;
  a.M = (int)M;
  a.N = (int)K;
  a.K = (int)N;
  a.lda = N;
  a.ldb = K;
  a.ldc = K;
  a.ws = ws;
  return launch<LAY_ROW, LAY_COL, MTP_EPI_NONE, OUT_BF16>(a, s, f16);
}
