// Internal interface between the GEMV translation units (not part of the C ABI).
#pragma once
#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

#include "common.h"

// Matrix-core GEMV for 2..16 activation rows (qmv_mfma.hip).
int exo_qmv_mfma_max_rows(int K, int bits);
size_t exo_qmv_mfma_workspace(int N);
int exo_qmv_mfma_launch(const bf16_t* x, const bf16_t* norm_w, float eps, const uint32_t* w,
                        const bf16_t* s, const bf16_t* b, const uint32_t* w2, const bf16_t* s2,
                        const bf16_t* b2, const bf16_t* residual, bf16_t* y, int M, int N, int K,
                        int bits, void* workspace, hipStream_t st);

// 4x4x4 matrix-core GEMV for 1..16 activation rows (qmv_quad.hip): rows of whole 256-byte
// slices, N a multiple of 4.  w2/s2/b2 non-null: the (gate, up) pair with SwiGLU.
bool exo_qmv_quad_ok(int M, int N, int K, int bits, bool norm);
int exo_qmv_quad_launch(const bf16_t* x, const bf16_t* norm_w, float eps, const uint32_t* w,
                        const bf16_t* s, const bf16_t* b, const uint32_t* w2, const bf16_t* s2,
                        const bf16_t* b2, const bf16_t* residual, bf16_t* y, int M, int N, int K,
                        int bits, hipStream_t st);

// 16x16x32 matrix-core GEMV for up to 16 activation rows (qmv_w16.hip): 4-bit codes, N a
// multiple of 16, rows of 4..32 whole 64-byte slices (K of 512 to 4096) - longer rows with a
// workspace (the split-K workspace of exo_qmv_mfma_workspace(N)), no fused norm and a single
// matrix: K then splits over 2..8 workgroups.  w2/s2/b2 non-null: the (gate, up) pair with SwiGLU.
bool exo_qmv_w16_ok(int M, int N, int K, int bits, bool norm, bool pair, bool has_workspace);
int exo_qmv_w16_launch(const bf16_t* x, const bf16_t* norm_w, float eps, const uint32_t* w,
                       const bf16_t* s, const bf16_t* b, const uint32_t* w2, const bf16_t* s2,
                       const bf16_t* b2, const bf16_t* residual, bf16_t* y, int M, int N, int K,
                       void* workspace, hipStream_t st);
