// dW[N,K] (+)= dY[M,N]^T X[M,K]: GEMM (N, K, reduce M) with both operands transposed (col).
#include "gemm_bf16_kernel.h"

// db (may be null): the bias gradient sum_m dY[m, :], in dw's dtype, produced by the same launch
int mtp_gemm_bf16_wgrad(const void* dy, const void* x, void* dw, void* db, int64_t M, int64_t N, int64_t K,
                        int dw_dtype, int accumulate, int f16, void* ws, hipStream_t s) {
  GemmArgs a{};
  a.A = (const uint16_t*)dy;
  a.B = (const uint16_t*)x;
  a.C = dw;
  a.M = (int)N;
  a.N = (int)K;
  a.K = (int)M;
  a.lda = N;
  a.ldb = K;
  a.ldc = K;
  a.accumulate = accumulate;
  a.rowsum = db;
  a.ws = ws;
  if (db) {
    if (dw_dtype == MTP_F32) return launch<LAY_COL, LAY_COL, EPI_ROWSUM, OUT_F32>(a, s, f16);
    return launch<LAY_COL, LAY_COL, EPI_ROWSUM, OUT_BF16>(a, s, f16);
  }
  if (dw_dtype == MTP_F32) return launch<LAY_COL, LAY_COL, MTP_EPI_NONE, OUT_F32>(a, s, f16);
  return launch<LAY_COL, LAY_COL, MTP_EPI_NONE, OUT_BF16>(a, s, f16);
}
