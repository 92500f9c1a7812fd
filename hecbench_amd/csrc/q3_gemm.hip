// Batched GPTQ 3-bit GEMM (placeholder until the MFMA kernel lands).
#include "hq_internal.h"

int hq_q3_gemm_launch(const void*, const int32_t*, const float*, const float*, float*, int, int, int,
                      unsigned, hipStream_t) {
  return HQ_ERR_TOO_LARGE;
}
