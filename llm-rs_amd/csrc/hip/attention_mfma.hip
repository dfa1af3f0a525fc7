#include "attention.h"
int llmrs_attention_bf16_mfma(hipStream_t, const bf16*, bf16*, const bf16*, const bf16*, const int*, const int*,
                              const int*, const int*, const int*, int, float*, size_t, const AttnArgs&) { return 0; }
