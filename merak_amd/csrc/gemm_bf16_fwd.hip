// Forward product Y = X W^T (+ bias, + fused activation) on the bf16 MFMA kernel.
#include "gemm_bf16_kernel.h"

int mtp_gemm_bf16_nt(const void* A, const void* B, const void* bias, void* C, void* C2, int64_t M, int64_t N,
                     int64_t K, int epilogue, int f16, hipStream_t s) {
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
  a.half = (int)(N / 2);
  a.ldc2 = (epilogue == MTP_EPI_SWIGLU) ? N / 2 : N;
  switch (epilogue) {
    case MTP_EPI_NONE: return launch<LAY_ROW, LAY_ROW, MTP_EPI_NONE, OUT_BF16>(a, s, f16);
    case MTP_EPI_BIAS: return launch<LAY_ROW, LAY_ROW, MTP_EPI_BIAS, OUT_BF16>(a, s, f16);
    case MTP_EPI_BIAS_GELU: return launch<LAY_ROW, LAY_ROW, MTP_EPI_BIAS_GELU, OUT_BF16>(a, s, f16);
    case MTP_EPI_GELU: return launch<LAY_ROW, LAY_ROW, MTP_EPI_GELU, OUT_BF16>(a, s, f16);
    case MTP_EPI_SWIGLU: return launch<LAY_ROW, LAY_ROW, MTP_EPI_SWIGLU, OUT_BF16>(a, s, f16);
  }
  mtp_set_error("gemm_bf16: unknown epilogue %d", epilogue);
  return MTP_EINVAL;
}
