// Layout change between the resident KV cache and the disaggregated-prefill wire format.
//
// Cache row of one layer: [Hkv, S_max, D] bf16 (head-major, so that a head's positions
// stream contiguously in attention).  Wire: [n, Hkv, D] bf16 for positions
// [start, start+n) -- the reference ships `transpose(keys[0, :, start:offset, :], (1,0,2))`
// (src/exo/worker/engines/mlx/disaggregated/adapter.py:86-135).  Pure byte movement: one
// 16-byte vector per lane, D*2/16 lanes per (token, head); reads and writes are both
// contiguous runs of D*2 bytes, which is what HBM coalescing needs at D >= 64.
#include "../../include/exo_mi355x.h"
#include "common.h"

namespace {

template <bool EXPORT>
__global__ __launch_bounds__(256) void kv_nhd_kernel(uint4* __restrict__ cache,
                                                     uint4* __restrict__ wire, int Hkv,
                                                     int S_max, int vec_per_head, int start,
                                                     long long total) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const int v = (int)(i % vec_per_head);
  const long long th = i / vec_per_head;
  const int h = (int)(th % Hkv);
  const long long t = th / Hkv;
  const long long c = ((long long)h * S_max + start + t) * vec_per_head + v;
  if (EXPORT)
    wire[i] = cache[c];
  else
    cache[c] = wire[i];
}

int launch(bool exp, const void* cache, const void* wire, int Hkv, int S_max, int D, int start,
           int n, exo_stream_t stream, const char* what) {
  EXO_REQUIRE(cache && wire, "%s: null pointer", what);
  EXO_REQUIRE(Hkv > 0 && D > 0 && D % 8 == 0 && S_max > 0, "%s: need Hkv>0, D%%8==0; got Hkv=%d D=%d",
              what, Hkv, D);
  EXO_REQUIRE(start >= 0 && n >= 0 && (long long)start + n <= S_max,
              "%s: positions [%d,%d) outside the cache of %d", what, start, start + n, S_max);
  EXO_REQUIRE(((uintptr_t)cache & 15) == 0 && ((uintptr_t)wire & 15) == 0,
              "%s: pointers must be 16-byte aligned", what);
  if (n == 0) return EXO_OK;
  const int vph = D / 8;
  const long long total = (long long)n * Hkv * vph;
  const unsigned grid = (unsigned)((total + 255) / 256);
  if (exp)
    kv_nhd_kernel<true><<<dim3(grid), 256, 0, (hipStream_t)stream>>>(
        (uint4*)cache, (uint4*)wire, Hkv, S_max, vph, start, total);
  else
    kv_nhd_kernel<false><<<dim3(grid), 256, 0, (hipStream_t)stream>>>(
        (uint4*)cache, (uint4*)wire, Hkv, S_max, vph, start, total);
  EXO_CHECK_LAUNCH(what);
  return EXO_OK;
}

}  // namespace

extern "C" int exo_kv_export_nhd(const uint16_t* cache_row, uint16_t* wire, int Hkv, int S_max,
                                 int D, int start, int n, exo_stream_t stream) {
  return launch(true, cache_row, wire, Hkv, S_max, D, start, n, stream, "exo_kv_export_nhd");
}

extern "C" int exo_kv_import_nhd(const uint16_t* wire, uint16_t* cache_row, int Hkv, int S_max,
                                 int D, int start, int n, exo_stream_t stream) {
  return launch(false, cache_row, wire, Hkv, S_max, D, start, n, stream, "exo_kv_import_nhd");
}
