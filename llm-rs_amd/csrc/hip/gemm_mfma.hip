#include "gemm.h"
int llmrs_gemm_bf16_mfma(hipStream_t, const bf16*, int, const bf16*, void*, int, int, int, int, int) { return 0; }
