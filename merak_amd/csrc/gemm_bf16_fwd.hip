// Forward product Y = X W^T (+ bias, + fused activation) on the 16-bit MFMA kernel.  This file is compiled twice,
// once per element type (MTP_FWD_F16 unset: bf16 and the dispatching entry point; set: IEEE half), so that the
// longest translation unit of the build is half as long.
#include "gemm_bf16_kernel.h"

#ifdef MTP_FWD_F16
#define FWD_NAME mtp_gemm_f16_nt_impl
#define FWD_LAUNCH(EPI) launch_typed<LAY_ROW, LAY_ROW, EPI, OUT_BF16, true>(a, s)
#else
#define FWD_NAME mtp_gemm_bf16_nt
#define FWD_LAUNCH(EPI) launch_typed<LAY_ROW, LAY_ROW, EPI, OUT_BF16, false>(a, s)
int mtp_gemm_f16_nt_impl(const void* A, const void* B, const void* bias, void* C, void* C2, int64_t M, int64_t N,
                         int64_t K, int epilogue, int f16, void* ws, hipStream_t s);
#endif

int FWD_NAME(const void* A, const void* B, const void* bias, void* C, void* C2, int64_t M, int64_t N,
             int64_t K, int epilogue, int f16, void* ws, hipStream_t s) {
#ifndef MTP_FWD_F16
  if (f16) return mtp_gemm_f16_nt_impl(A, B, bias, C, C2, M, N, K, epilogue, f16, ws, s);
#endif
  GemmArgs a{};
  a.A = (const uint16_t*)A;
  a.B = (const uint16_t*)B;
  a.bias = (const uint16_t*)bias;
  a.C = C;
  a.C2 = C2;
  a.M = (int)M;
  a.N = (int)N;
  a.K = (int)K;
  a.lda = K;
  a.ldb = K;
  a.ldc = N;
  a.accumulate = 0;
  a.ws = ws;
  a.half = (int)(N / 2);
  a.ldc2 = (epilogue == MTP_EPI_SWIGLU) ? N / 2 : N;
  switch (epilogue) {
    case MTP_EPI_NONE: return FWD_LAUNCH(MTP_EPI_NONE);
    case MTP_EPI_BIAS: return FWD_LAUNCH(MTP_EPI_BIAS);
    case MTP_EPI_BIAS_GELU: return FWD_LAUNCH(MTP_EPI_BIAS_GELU);
    case MTP_EPI_GELU: return FWD_LAUNCH(MTP_EPI_GELU);
    case MTP_EPI_SWIGLU: return FWD_LAUNCH(MTP_EPI_SWIGLU);
  }
  mtp_set_error("gemm_bf16: unknown epilogue %d", epilogue);
  return MTP_EINVAL;
}
