// Entry points of the linear layers: argument checks and the choice between
// the bf16 MFMA kernel, and the general fp32-MFMA kernel that serves fp32
// tensors and every bf16 shape the fast kernel does not take.
#include "mtp_common.h"

// f16 != 0: the 16-bit tensors are IEEE half instead of bf16 (same kernel, other MFMA and conversions)
// ws: stream-K scratch of MTP_LINEAR_WS_BYTES bytes, or null (every tile is then one workgroup)
int mtp_gemm_bf16_nt(const void* A, const void* B, const void* bias, void* C, void* C2, int64_t M, int64_t N,
                     int64_t K, int epilogue, int f16, void* ws, hipStream_t s);
int mtp_gemm_bf16_dgrad(const void* dy, const void* w, void* dx, int64_t M, int64_t N, int64_t K, int f16, void* ws,
                        hipStream_t s);
int mtp_gemm_bf16_wgrad(const void* dy, const void* x, void* dw, void* db, int64_t M, int64_t N, int64_t K,
                        int dw_dtype, int accumulate, int f16, void* ws, hipStream_t s);
// both of the above, in one launch where that saves a round of workgroups
int mtp_gemm_bf16_bwd(const void* dy, const void* x, const void* w, void* dx, void* dw, void* db, int64_t M, int64_t N,
                      int64_t K, int dw_dtype, int accumulate, int f16, void* ws, hipStream_t s);
// = SK_WORKSPACE_BYTES of gemm_bf16_kernel.h (checked there): 2 slots for each of 256 workgroups
#define MTP_LINEAR_WS_BYTES (2ll * 256 * 66 * 256 * 16)
int mtp_gemm_generic(const void* A, int64_t sam, int64_t sak, const void* B, int64_t sbn, int64_t sbk,
                     const void* bias, void* C, int64_t ldc, int64_t M, int64_t N, int64_t K, int dtype, int out_dtype,
                     int accumulate, hipStream_t s);
// ws: scratch for the cut along k (any size: the cut is taken when it fits), or null
int mtp_gemm_f32(int kind, const float* A, int64_t lda, const float* B, int64_t ldb, const float* bias, float* C,
                 float* rowsum, int64_t ldc, int64_t M, int64_t N, int64_t K, int accumulate, void* ws, int64_t ws_bytes,
                 hipStream_t s);
int mtp_colsum(const void* dy, void* db, int64_t M, int64_t N, int dtype, int out_dtype, int accumulate,
               hipStream_t s);
int mtp_act_fwd(const void* y, void* act, int64_t M, int64_t N, int dtype, int swiglu, hipStream_t s);

namespace {

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// the scratch is used only when it is large enough and aligned; otherwise the call runs as without one
void* usable_ws(void* ws, int64_t bytes) { return (ws && bytes >= MTP_LINEAR_WS_BYTES && aligned16(ws)) ? ws : nullptr; }
// the fp32 products take a scratch of any size (their cut along k is sized to it)
void* f32_ws(void* ws, int64_t bytes) { return (ws && bytes > 0 && aligned16(ws)) ? ws : nullptr; }

int check_dims(const char* what, int64_t M, int64_t N, int64_t K, int dtype) {
  MTP_REQUIRE(M >= 0 && N >= 1 && K >= 1, MTP_EINVAL, "%s: M=%lld N=%lld K=%lld", what, (long long)M, (long long)N,
              (long long)K);
  MTP_REQUIRE(M < (1ll << 31) && N < (1ll << 31) && K < (1ll << 31), MTP_EUNSUPPORTED,
              "%s: a dimension exceeds 2^31-1", what);
  MTP_REQUIRE(dtype == MTP_F32 || dtype == MTP_BF16 || dtype == MTP_F16, MTP_EINVAL, "%s: unknown dtype %d", what,
              dtype);
  return MTP_OK;
}

// The bf16 MFMA kernel needs 16-byte aligned rows, and tile-relative byte offsets below 2^31.
bool fast_ok(int64_t rows_ld_a, int64_t rows_ld_b, const void* a, const void* b) {
  return rows_ld_a % 8 == 0 && rows_ld_b % 8 == 0 && aligned16(a) && aligned16(b) && rows_ld_a * 2 * 256 < (1ll << 31) &&
         rows_ld_b * 2 * 256 < (1ll << 31);
}

// The fp32 MFMA kernel reads 16 bytes per lane: 16-byte aligned bases, row lengths that are multiples of 4
// floats, and (for the transposed operands, addressed from the matrix origin) matrices below 2 GiB.
bool f32_fast_ok(const void* a, const void* b, int64_t d0, int64_t d1, int64_t bytes_a, int64_t bytes_b) {
  return aligned16(a) && aligned16(b) && d0 % 4 == 0 && d1 % 4 == 0 && bytes_a < (1ll << 31) && bytes_b < (1ll << 31);
}

}  // namespace

extern "C" int64_t mtp_linear_workspace_bytes(void) { return MTP_LINEAR_WS_BYTES; }

// Scratch a product of these sizes can make use of: 0 for the (many) shapes that never touch it.  An upper bound of
// what the kernels' own planning takes (gemm_bf16_kernel.h plan_stream_k, gemm_f32.hip launch_f32): a call with
// this much never runs without scratch where it would have used some.
extern "C" int64_t mtp_linear_workspace_need(int kind, int64_t M, int64_t N, int64_t K, int dtype) {
  if (M <= 0 || N <= 0 || K <= 0 || kind < 0 || kind > 3) return 0;
  static MtpTune tune_sk("MTP_GEMM_SK"), tune_slices("MTP_GEMM_F32_SLICES");
  // (rows, columns, reduction length) of the product: forward, input gradient, weight gradient
  const int64_t dims[3][3] = {{M, N, K}, {M, K, N}, {N, K, M}};
  int64_t need = 0;
  for (int p = 0; p < 3; p++) {
    if (!(kind == p || (kind == 3 && p >= 1))) continue;
    const int64_t r = dims[p][0], c = dims[p][1], k = dims[p][2];
    if (dtype == MTP_F32) {
      // cut along k: fewer 128x128 tiles than compute units (or forced), up to 8 slices of the output and its row sums
      const int64_t tiles = ((r + 127) / 128) * ((c + 127) / 128);
      if ((tiles < 256 || tune_slices.get(0) > 1) && k >= 1024 && tune_slices.get(0) != 1) {
        const int64_t b = 8 * (r * c + r) * 4;
        need = b > need ? b : need;
      }
    } else {
      // stream-K: at most half the compute units have a 256x256 tile and k is long (or forced)
      const int64_t tiles = ((r + 255) / 256) * ((c + 255) / 256);
      const int force = tune_sk.get(-1);
      if (force != 0 && k % 64 == 0 && (force > 0 || (tiles <= 128 && k / 64 >= 32)))
        need = MTP_LINEAR_WS_BYTES > need ? MTP_LINEAR_WS_BYTES : need;
    }
  }
  return need;
}

extern "C" int mtp_linear_fwd(const void* x, const void* w, const void* bias, void* y, void* act, int64_t M,
                              int64_t N, int64_t K, int dtype, int epilogue, void* stream) {
  return mtp_linear_fwd_ws(x, w, bias, y, act, nullptr, 0, M, N, K, dtype, epilogue, stream);
}

extern "C" int mtp_linear_fwd_ws(const void* x, const void* w, const void* bias, void* y, void* act, void* workspace,
                                 int64_t workspace_bytes, int64_t M, int64_t N, int64_t K, int dtype, int epilogue,
                                 void* stream) {
  int rc = check_dims("linear_fwd", M, N, K, dtype);
  if (rc) return rc;
  MTP_REQUIRE(epilogue >= MTP_EPI_NONE && epilogue <= MTP_EPI_GELU, MTP_EINVAL, "linear_fwd: unknown epilogue %d",
              epilogue);
  const bool has_act = epilogue == MTP_EPI_BIAS_GELU || epilogue == MTP_EPI_SWIGLU || epilogue == MTP_EPI_GELU;
  if (M == 0) return MTP_OK;
  MTP_REQUIRE(has_act ? act != nullptr : act == nullptr, MTP_EINVAL,
              "linear_fwd: act must be given exactly for the activation epilogues");
  MTP_REQUIRE(has_act || y, MTP_EINVAL, "linear_fwd: null output");
  MTP_REQUIRE((epilogue != MTP_EPI_BIAS && epilogue != MTP_EPI_BIAS_GELU) || bias, MTP_EINVAL,
              "linear_fwd: bias epilogue without bias");
  MTP_REQUIRE(epilogue != MTP_EPI_SWIGLU || N % 2 == 0, MTP_EINVAL, "linear_fwd: SwiGLU needs an even N");
  MTP_REQUIRE(x && w, MTP_EINVAL, "linear_fwd: null input");
  hipStream_t s = (hipStream_t)stream;
  const void* use_bias = (epilogue == MTP_EPI_NONE || epilogue == MTP_EPI_GELU) ? nullptr : bias;

  const bool is16 = dtype == MTP_BF16 || dtype == MTP_F16;
  if (is16 && fast_ok(K, K, x, w) && N * K * 2 < (1ll << 31)) {
    int epi = epilogue;
    if (epilogue == MTP_EPI_SWIGLU && !use_bias) use_bias = nullptr;
    return mtp_gemm_bf16_nt(x, w, use_bias, y, act, M, N, K, epi, dtype == MTP_F16, usable_ws(workspace, workspace_bytes), s);
  }
  if (dtype == MTP_F32 && f32_fast_ok(x, w, K, K, 0, 0) && K * 4 * 128 < (1ll << 31)) {
    void* pre32 = y ? y : (epilogue != MTP_EPI_SWIGLU ? act : nullptr);
    MTP_REQUIRE(pre32, MTP_EUNSUPPORTED, "linear_fwd: this shape needs the pre-activation buffer y");
    rc = mtp_gemm_f32(0, (const float*)x, K, (const float*)w, K, (const float*)use_bias, (float*)pre32, nullptr, N, M, N, K, 0,
                      f32_ws(workspace, workspace_bytes), workspace_bytes, s);
    if (rc) return rc;
    if (has_act) return mtp_act_fwd(pre32, act, M, N, dtype, epilogue == MTP_EPI_SWIGLU, s);
    return MTP_OK;
  }
  // general path: GEMM (+bias) into y, then the activation as a second pass.  Without y the GELU forms
  // run in place in act; SwiGLU's act is half as wide as the pre-activation, so it needs y.
  void* pre = y;
  if (!pre && epilogue != MTP_EPI_SWIGLU) pre = act;
  MTP_REQUIRE(pre, MTP_EUNSUPPORTED, "linear_fwd: this shape needs the pre-activation buffer y");
  rc = mtp_gemm_generic(x, K, 1, w, K, 1, use_bias, pre, N, M, N, K, dtype, dtype, 0, s);
  if (rc) return rc;
  if (has_act) return mtp_act_fwd(pre, act, M, N, dtype, epilogue == MTP_EPI_SWIGLU, s);
  return MTP_OK;
}

extern "C" int mtp_linear_dgrad(const void* dy, const void* w, void* dx, int64_t M, int64_t N, int64_t K, int dtype,
                                void* stream) {
  return mtp_linear_dgrad_ws(dy, w, dx, nullptr, 0, M, N, K, dtype, stream);
}

extern "C" int mtp_linear_dgrad_ws(const void* dy, const void* w, void* dx, void* workspace, int64_t workspace_bytes,
                                   int64_t M, int64_t N, int64_t K, int dtype, void* stream) {
  int rc = check_dims("linear_dgrad", M, N, K, dtype);
  if (rc) return rc;
  if (M == 0) return MTP_OK;
  MTP_REQUIRE(dy && w && dx, MTP_EINVAL, "linear_dgrad: null pointer");
  hipStream_t s = (hipStream_t)stream;
  if ((dtype == MTP_BF16 || dtype == MTP_F16) && fast_ok(N, K, dy, w) && aligned16(dx)) {
    rc = mtp_gemm_bf16_dgrad(dy, w, dx, M, N, K, dtype == MTP_F16, usable_ws(workspace, workspace_bytes), s);
    if (rc != MTP_EUNSUPPORTED) return rc;
  }
  if (dtype == MTP_F32 && f32_fast_ok(dy, w, N, K, 0, N * K * 4) && N * 4 * 128 < (1ll << 31))
    return mtp_gemm_f32(1, (const float*)dy, N, (const float*)w, K, nullptr, (float*)dx, nullptr, K, M, K, N, 0,
                        f32_ws(workspace, workspace_bytes), workspace_bytes, s);
  // dX[m,k] = sum_n dY[m,n] W[n,k]: A = dY (N,1), B(k,n) = W[n*K + k]
  return mtp_gemm_generic(dy, N, 1, w, 1, K, nullptr, dx, K, M, K, N, dtype, dtype, 0, s);
}

extern "C" int mtp_linear_wgrad(const void* dy, const void* x, void* dw, void* db, int64_t M, int64_t N, int64_t K,
                                int dtype, int dw_dtype, int accumulate, void* stream) {
  return mtp_linear_wgrad_ws(dy, x, dw, db, nullptr, 0, M, N, K, dtype, dw_dtype, accumulate, stream);
}

extern "C" int mtp_linear_wgrad_ws(const void* dy, const void* x, void* dw, void* db, void* workspace,
                                   int64_t workspace_bytes, int64_t M, int64_t N, int64_t K, int dtype, int dw_dtype,
                                   int accumulate, void* stream) {
  int rc = check_dims("linear_wgrad", M, N, K, dtype);
  if (rc) return rc;
  MTP_REQUIRE(dw_dtype == MTP_F32 || dw_dtype == dtype, MTP_EUNSUPPORTED,
              "linear_wgrad: gradients are fp32 or of the inputs' dtype (inputs %d, dw %d)", dtype, dw_dtype);
  MTP_REQUIRE(dw, MTP_EINVAL, "linear_wgrad: null dw");
  MTP_REQUIRE(M == 0 || (dy && x), MTP_EINVAL, "linear_wgrad: null input");
  hipStream_t s = (hipStream_t)stream;
  if ((dtype == MTP_BF16 || dtype == MTP_F16) && M > 0 && fast_ok(N, K, dy, x) && aligned16(dw)) {
    rc = mtp_gemm_bf16_wgrad(dy, x, dw, db, M, N, K, dw_dtype, accumulate, dtype == MTP_F16,
                             usable_ws(workspace, workspace_bytes), s);
    if (rc != MTP_EUNSUPPORTED) return rc;
  }
  if (dtype == MTP_F32 && dw_dtype == MTP_F32 && M > 0 && f32_fast_ok(dy, x, N, K, M * N * 4, M * K * 4)) {
    // the bias gradient (column sums of dY = row sums of the A operand) rides along in the first tile column
    return mtp_gemm_f32(2, (const float*)dy, N, (const float*)x, K, nullptr, (float*)dw, (float*)db, K, N, K, M,
                        accumulate, f32_ws(workspace, workspace_bytes), workspace_bytes, s);
  }
  // dW[n,k] = sum_m dY[m,n] X[m,k]: A(n,m) = dY[m*N + n], B(k,m) = X[m*K + k]; M == 0 writes zeros
  rc = mtp_gemm_generic(dy, 1, N, x, 1, K, nullptr, dw, K, N, K, M, dtype, dw_dtype, accumulate, s);
  if (rc) return rc;
  if (db) return mtp_colsum(dy, db, M, N, dtype, dw_dtype, accumulate, s);
  return MTP_OK;
}

extern "C" int mtp_linear_bwd_ws(const void* dy, const void* x, const void* w, void* dx, void* dw, void* db,
                                 void* workspace, int64_t workspace_bytes, int64_t M, int64_t N, int64_t K, int dtype,
                                 int dw_dtype, int accumulate, void* stream) {
  int rc = check_dims("linear_bwd", M, N, K, dtype);
  if (rc) return rc;
  MTP_REQUIRE(dw_dtype == MTP_F32 || dw_dtype == dtype, MTP_EUNSUPPORTED,
              "linear_bwd: gradients are fp32 or of the inputs' dtype (inputs %d, dw %d)", dtype, dw_dtype);
  MTP_REQUIRE(dx && dw, MTP_EINVAL, "linear_bwd: null output");
  MTP_REQUIRE(M == 0 || (dy && x && w), MTP_EINVAL, "linear_bwd: null input");
  if ((dtype == MTP_BF16 || dtype == MTP_F16) && M > 0 && fast_ok(N, K, dy, w) && fast_ok(N, K, dy, x) && aligned16(dx) &&
      aligned16(dw)) {
    rc = mtp_gemm_bf16_bwd(dy, x, w, dx, dw, db, M, N, K, dw_dtype, accumulate, dtype == MTP_F16,
                           usable_ws(workspace, workspace_bytes), (hipStream_t)stream);
    if (rc != MTP_EUNSUPPORTED) return rc;
  }
  rc = mtp_linear_dgrad_ws(dy, w, dx, workspace, workspace_bytes, M, N, K, dtype, stream);
  if (rc) return rc;
  return mtp_linear_wgrad_ws(dy, x, dw, db, workspace, workspace_bytes, M, N, K, dtype, dw_dtype, accumulate, stream);
}

extern "C" int mtp_linear_bias_grad(const void* dy, void* db, int64_t M, int64_t N, int dtype, int db_dtype, int accumulate,
                                    void* stream) {
  int rc = check_dims("linear_bias_grad", M, N, 1, dtype);
  if (rc) return rc;
  MTP_REQUIRE(db_dtype == MTP_F32 || db_dtype == dtype, MTP_EUNSUPPORTED,
              "linear_bias_grad: the gradient is fp32 or of the inputs' dtype (inputs %d, db %d)", dtype, db_dtype);
  MTP_REQUIRE(db && (M == 0 || dy), MTP_EINVAL, "linear_bias_grad: null pointer");
  return mtp_colsum(dy, db, M, N, dtype, db_dtype, accumulate, (hipStream_t)stream);
}
