// Entry points shared between the GEMV translation units (not part of the C ABI).
#pragma once
#include "common.h"

// rows of x one MFMA-GEMV launch can take (their whole K sits in LDS); 0 = shape not
// supported by that kernel (K must be a multiple of 512 for 4-bit, 256 for 8-bit)
int exo_qmv_mfma_max_rows(int K, int bits);
int exo_qmv_mfma_launch(const bf16_t* x, const bf16_t* norm_w, float eps, const uint32_t* w,
                        const bf16_t* s, const bf16_t* b, const bf16_t* residual, bf16_t* y,
                        int M, int N, int K, int bits, hipStream_t st);
