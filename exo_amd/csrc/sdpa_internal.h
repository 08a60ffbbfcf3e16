// Internal interface between the attention translation units (not part of the C ABI).
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

#include "common.h"

// Matrix-core causal attention for a chunk of T new tokens (sdpa_prefill.hip).
// Same arguments as exo_sdpa_prefill, already validated.
int exo_sdpa_prefill_mfma(const bf16_t* q, const bf16_t* k_cache, const bf16_t* v_cache,
                          const int32_t* pos, bf16_t* out, float scale, int B, int T, int Hq,
                          int Hkv, int D, int S_max, hipStream_t stream);
