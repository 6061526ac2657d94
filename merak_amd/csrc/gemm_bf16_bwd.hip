// dX[M,K] = dY[M,N] W[N,K] and dW[N,K] (+)= dY[M,N]^T X[M,K] (+ db) of one layer in one launch, where that saves a
// round of workgroups; otherwise (and for everything the 64-deep loop does not take) the two launches of
// gemm_bf16_dgrad.hip / gemm_bf16_wgrad.hip.
#include "gemm_bf16_kernel.h"

int mtp_gemm_bf16_dgrad(const void* dy, const void* w, void* dx, int64_t M, int64_t N, int64_t K, int f16, void* ws,
                        hipStream_t s);
int mtp_gemm_bf16_wgrad(const void* dy, const void* x, void* dw, void* db, int64_t M, int64_t N, int64_t K,
                        int dw_dtype, int accumulate, int f16, void* ws, hipStream_t s);

namespace {

template <int EPI2, int OUT2, bool F16>
int launch_bwd_pair(const GemmArgs& a1, const GemmArgs& a2, int n1, int n2, hipStream_t s) {
  hipLaunchKernelGGL((gemm_q_bwd_kernel<EPI2, OUT2, F16>), dim3((unsigned)(n1 + n2)), dim3(256), 0, s, a1, a2, n1);
  MTP_CHECK_LAUNCH("gemm_bf16 backward pair");
  return MTP_OK;
}

// whole 256x256 tiles of an [rows, cols] output
int64_t tiles_of(int64_t rows, int64_t cols) { return ((rows + 255) / 256) * ((cols + 255) / 256); }

}  // namespace

// MTP_GEMM_PAIR = 0 keeps the two launches.
int mtp_gemm_bf16_bwd(const void* dy, const void* x, const void* w, void* dx, void* dw, void* db, int64_t M, int64_t N,
                      int64_t K, int dw_dtype, int accumulate, int f16, void* ws, hipStream_t s) {
  static MtpTune tune_pair("MTP_GEMM_PAIR"), tune_cfg("MTP_GEMM_CFG");
  // dgrad: C[M, K] over k = N; wgrad: C[N, K] over k = M
  GemmArgs a1{}, a2{};
  a1.A = (const uint16_t*)dy; a1.B = (const uint16_t*)w; a1.C = dx;
  a1.M = (int)M; a1.N = (int)K; a1.K = (int)N;
  a1.lda = N; a1.ldb = K; a1.ldc = K;
  a2.A = (const uint16_t*)dy; a2.B = (const uint16_t*)x; a2.C = dw;
  a2.M = (int)N; a2.N = (int)K; a2.K = (int)M;
  a2.lda = N; a2.ldb = K; a2.ldc = K;
  a2.accumulate = accumulate;
  a2.rowsum = db;
  const int64_t t1 = tiles_of(M, K), t2 = tiles_of(N, K);
  const bool saves_a_round = (t1 + t2 + 255) / 256 < (t1 + 255) / 256 + (t2 + 255) / 256;
  // both products on the 64-deep loop (whole k-tiles, rows of at least 256 bytes), each with enough k-tiles
  // for its pipeline, and nothing forced
  const bool takes = tune_pair.get(1) != 0 && !tune_cfg.is_set() && saves_a_round && q_loop_ok(a1) && q_loop_ok(a2) &&
                     a1.K >= 4 * QBK && a2.K >= 4 * QBK && t1 + t2 < (1ll << 30);
  if (!takes) {
    int rc = mtp_gemm_bf16_dgrad(dy, w, dx, M, N, K, f16, ws, s);
    if (rc) return rc;
    return mtp_gemm_bf16_wgrad(dy, x, dw, db, M, N, K, dw_dtype, accumulate, f16, ws, s);
  }
  const int n1 = (int)t1, n2 = (int)t2;
#define MTP_PAIR(E, O)                                                 \
  (f16 ? launch_bwd_pair<E, O, true>(a1, a2, n1, n2, s) : launch_bwd_pair<E, O, false>(a1, a2, n1, n2, s))
  if (db) return dw_dtype == MTP_F32 ? MTP_PAIR(EPI_ROWSUM, OUT_F32) : MTP_PAIR(EPI_ROWSUM, OUT_BF16);
  return dw_dtype == MTP_F32 ? MTP_PAIR(MTP_EPI_NONE, OUT_F32) : MTP_PAIR(MTP_EPI_NONE, OUT_BF16);
#undef MTP_PAIR
}
