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
  hipLaunchKernelGGL((gemm_q_bwd_kernel<EPI2, OUT2, F16>), dim3((unsigned)((n1 < 0 ? -n1 : n1) + n2)), dim3(256), 0, s, a1,
                     a2, n1);
  MTP_CHECK_LAUNCH("gemm_bf16 backward pair");
  return MTP_OK;
}

// whole 256x256 tiles of an [rows, cols] output
int64_t tiles_of(int64_t rows, int64_t cols) { return ((rows + 255) / 256) * ((cols + 255) / 256); }

// Time (in k-tiles) until the last tile is done when 256 compute units take c1 tiles of l1 k-tiles each and then c2
// tiles of l2, in that order, each unit taking the next tile as it falls free; a tile costs its k-tiles plus a fixed
// part (first loads, output: about six k-tiles' worth).  After the first run the units are free at one of two
// times; the second run ends at the least time by which the units' free slots hold all its tiles.
int64_t makespan(int64_t c1, int l1, int64_t c2, int l2) {
  constexpr int64_t kUnits = 256, kPerTile = 6;
  const int64_t L1 = l1 + kPerTile, L2 = l2 + kPerTile;
  const int64_t late = c1 % kUnits, early = kUnits - late;              // units that took one tile more / less
  const int64_t f_early = (c1 / kUnits) * L1, f_late = late ? f_early + L1 : f_early;
  if (c2 == 0) return f_late;
  auto capacity = [&](int64_t t) {
    const int64_t a = t > f_early ? (t - f_early) / L2 : 0, b = t > f_late ? (t - f_late) / L2 : 0;
    return early * a + late * b;
  };
  int64_t lo = f_early, hi = f_late + (c2 / kUnits + 2) * L2;           // capacity(hi) >= c2
  while (lo + 1 < hi) {
    const int64_t mid = (lo + hi) / 2;
    if (capacity(mid) >= c2) hi = mid;
    else lo = mid;
  }
  return hi > f_late ? hi : f_late;
}

}  // namespace

// MTP_GEMM_PAIR = 0 keeps the two launches, 2 takes the one launch wherever the 64-deep loop serves both products.
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
  // both products on the 64-deep loop (whole k-tiles, rows of at least 256 bytes), each with enough k-tiles
  // for its pipeline, nothing forced, and few enough tiles for the estimate below to be cheap
  bool takes = tune_pair.get(1) != 0 && !tune_cfg.is_set() && q_loop_ok(a1) && q_loop_ok(a2) && a1.K >= 4 * QBK &&
               a2.K >= 4 * QBK && t1 + t2 <= 8192;
  // the product with the longer k goes first; one launch when the estimate says it ends at least 4 % sooner than
  // the two launches one after the other
  const int k1 = a1.K / QBK, k2 = a2.K / QBK;
  const bool p1_first = k1 >= k2;
  if (takes) {
    const int64_t cl = p1_first ? t1 : t2, cs = p1_first ? t2 : t1;
    const int ll = p1_first ? k1 : k2, ls = p1_first ? k2 : k1;
    const double together = (double)makespan(cl, ll, cs, ls);
    const double apart = (double)(makespan(cl, ll, 0, 0) + makespan(cs, ls, 0, 0));
    takes = tune_pair.get(1) == 2 || together < 0.96 * apart;
  }
  if (!takes) {
    int rc = mtp_gemm_bf16_dgrad(dy, w, dx, M, N, K, f16, ws, s);
    if (rc) return rc;
    return mtp_gemm_bf16_wgrad(dy, x, dw, db, M, N, K, dw_dtype, accumulate, f16, ws, s);
  }
  // n1 > 0: dX's tiles first; n1 < 0: dW's -n1 tiles first
  const int n1 = p1_first ? (int)t1 : -(int)t2, n2 = p1_first ? (int)t2 : (int)t1;
#define MTP_PAIR(E, O)                                                 \
  (f16 ? launch_bwd_pair<E, O, true>(a1, a2, n1, n2, s) : launch_bwd_pair<E, O, false>(a1, a2, n1, n2, s))
  if (db) return dw_dtype == MTP_F32 ? MTP_PAIR(EPI_ROWSUM, OUT_F32) : MTP_PAIR(EPI_ROWSUM, OUT_BF16);
  return dw_dtype == MTP_F32 ? MTP_PAIR(MTP_EPI_NONE, OUT_F32) : MTP_PAIR(MTP_EPI_NONE, OUT_BF16);
#undef MTP_PAIR
}
