// The forward product on IEEE half operands: the same source as the bf16 forward, compiled for the other type.
#define MTP_FWD_F16 1
#include "gemm_bf16_fwd.hip"
