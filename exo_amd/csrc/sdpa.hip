// Scaled dot-product attention over the bf16 KV cache, grouped-query.
//
// One workgroup serves ONE kv head and all G = Hq/Hkv query heads that share it, so
// every K/V byte read from HBM is used G times.  A key row (D bf16) is spread over
// D/8 lanes, 16 bytes each; a wave covers 512/D keys per load instruction and keeps
// four such loads of K and of V in flight.  Scores, softmax and the output
// accumulation are float32 (online softmax, one rescale per block of 4 keys).
//
// decode : grid (splits, Hkv, B); each split owns a contiguous key range, writes
//          (max, sum, acc[D]) per query head to the workspace; a second kernel merges
//          the splits.  The grid is fixed (positions are read on the device), so the
//          launch can be replayed from a HIP graph while the sequence grows.
// prefill: grid (T, Hkv, B); one workgroup per new token, causal limit pos+t+1,
//          writes the output directly.
#include "../../include/exo_mi355x.h"
#include "common.h"

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = 4;
constexpr int kMaxSplits = 64;
constexpr int kBlk = 4;  // keys per lane group per step

struct SdpaParams {
  const bf16_t* q;   // [B*T, Hq*D]
  const bf16_t* kc;  // [B, Hkv, S_max, D]
  const bf16_t* vc;
  const int32_t* pos;  // [B]
  bf16_t* out;         // [B*T, Hq*D]
  float* ws;           // decode partials
  float scale;
  int B, T, Hq, Hkv, S_max, splits;
};

template <int D, int G, bool DECODE>
__global__ __launch_bounds__(kThreads) void sdpa_kernel(const SdpaParams p) {
  constexpr int LPK = D / 8;     // lanes per key
  constexpr int KPI = 64 / LPK;  // keys per wave instruction
  __shared__ float red[kWaves][G][D + 2];

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int sub = lane / LPK, sl = lane % LPK;
  const int b = blockIdx.z, kvh = blockIdx.y;
  const int t = DECODE ? 0 : blockIdx.x;
  const int len = min(p.pos[b] + t + 1, p.S_max);  // keys visible to this query
  int k_begin = 0, k_end = len;
  if (DECODE) {
    int chunk = (len + p.splits - 1) / p.splits;
    chunk = (chunk + 15) & ~15;
    k_begin = min(blockIdx.x * chunk, len);
    k_end = min(k_begin + chunk, len);
  }

  // q slices for the G heads: 8 elements = 4 bf16 pairs per head per lane
  uint4 qv[G];
  const size_t qrow = (size_t)(b * p.T + t) * p.Hq * D;
#pragma unroll
  for (int g = 0; g < G; ++g)
    qv[g] = *reinterpret_cast<const uint4*>(p.q + qrow + (size_t)(kvh * G + g) * D + sl * 8);

  float m[G], l[G], o[G][8];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    m[g] = -INFINITY;
    l[g] = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) o[g][e] = 0.f;
  }

  const size_t head_base = ((size_t)b * p.Hkv + kvh) * p.S_max * D;
  const bf16_t* kb = p.kc + head_base + sl * 8;
  const bf16_t* vb = p.vc + head_base + sl * 8;

  // lane group (wave, sub) takes keys k_begin + (step*kWaves*KPI + wave*KPI + sub)*kBlk + i
  for (int k0 = k_begin + (wave * KPI + sub) * kBlk; k0 < k_end; k0 += kWaves * KPI * kBlk) {
    uint4 kk[kBlk], vv[kBlk];
#pragma unroll
    for (int i = 0; i < kBlk; ++i) {
      const int key = min(k0 + i, k_end - 1);
      kk[i] = *reinterpret_cast<const uint4*>(kb + (size_t)key * D);
      vv[i] = *reinterpret_cast<const uint4*>(vb + (size_t)key * D);
    }
    float s[G][kBlk];
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
      for (int i = 0; i < kBlk; ++i) {
        float d = dot2_bf16(qv[g].x, kk[i].x, 0.f);
        d = dot2_bf16(qv[g].y, kk[i].y, d);
        d = dot2_bf16(qv[g].z, kk[i].z, d);
        d = dot2_bf16(qv[g].w, kk[i].w, d);
#pragma unroll
        for (int off = LPK >> 1; off > 0; off >>= 1) d += __shfl_xor(d, off, 64);
        s[g][i] = (k0 + i < k_end) ? d * p.scale : -INFINITY;
      }
#pragma unroll
    for (int g = 0; g < G; ++g) {
      float bm = s[g][0];
#pragma unroll
      for (int i = 1; i < kBlk; ++i) bm = fmaxf(bm, s[g][i]);
      const float mn = fmaxf(m[g], bm);  // finite: key k0 is always valid
      const float sc = __expf(m[g] - mn);
      float pr[kBlk], ps = 0.f;
#pragma unroll
      for (int i = 0; i < kBlk; ++i) {
        pr[i] = __expf(s[g][i] - mn);
        ps += pr[i];
      }
      l[g] = l[g] * sc + ps;
      m[g] = mn;
#pragma unroll
      for (int e = 0; e < 8; ++e) o[g][e] *= sc;
#pragma unroll
      for (int i = 0; i < kBlk; ++i) {
        const uint32_t* v4 = reinterpret_cast<const uint32_t*>(&vv[i]);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          o[g][2 * e] = fmaf(pr[i], bf_lo(v4[e]), o[g][2 * e]);
          o[g][2 * e + 1] = fmaf(pr[i], bf_hi(v4[e]), o[g][2 * e + 1]);
        }
      }
    }
  }

  // merge the KPI lane groups of the wave
#pragma unroll
  for (int g = 0; g < G; ++g) {
    float mw = m[g];
#pragma unroll
    for (int off = LPK; off < 64; off <<= 1) mw = fmaxf(mw, __shfl_xor(mw, off, 64));
    const float sc = (m[g] == -INFINITY) ? 0.f : __expf(m[g] - mw);
    float lw = l[g] * sc;
#pragma unroll
    for (int off = LPK; off < 64; off <<= 1) lw += __shfl_xor(lw, off, 64);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      float ov = o[g][e] * sc;
#pragma unroll
      for (int off = LPK; off < 64; off <<= 1) ov += __shfl_xor(ov, off, 64);
      o[g][e] = ov;
    }
    if (sub == 0) {
#pragma unroll
      for (int e = 0; e < 8; ++e) red[wave][g][sl * 8 + e] = o[g][e];
      if (sl == 0) {
        red[wave][g][D] = mw;
        red[wave][g][D + 1] = lw;
      }
    }
  }
  __syncthreads();

  // merge the waves; thread -> (head, element)
  for (int idx = threadIdx.x; idx < G * D; idx += kThreads) {
    const int g = idx / D, e = idx % D;
    float mw = red[0][g][D];
#pragma unroll
    for (int w = 1; w < kWaves; ++w) mw = fmaxf(mw, red[w][g][D]);
    float acc = 0.f, lsum = 0.f;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      const float mm = red[w][g][D];
      const float sc = (mm == -INFINITY) ? 0.f : __expf(mm - mw);
      acc += red[w][g][e] * sc;
      lsum += red[w][g][D + 1] * sc;
    }
    const int h = kvh * G + g;
    if (DECODE) {
      float* dst = p.ws + ((size_t)(b * p.Hq + h) * p.splits + blockIdx.x) * (D + 2);
      dst[e] = acc;
      if (e == 0) {
        dst[D] = mw;
        dst[D + 1] = lsum;
      }
    } else {
      p.out[qrow + (size_t)h * D + e] = f2bf(acc / lsum);
    }
  }
}

template <int D>
__global__ __launch_bounds__(D) void sdpa_merge_kernel(const float* __restrict__ ws,
                                                       bf16_t* __restrict__ out, int splits) {
  const int bh = blockIdx.x, e = threadIdx.x;
  const float* src = ws + (size_t)bh * splits * (D + 2);
  float mw = -INFINITY;
  for (int s = 0; s < splits; ++s) mw = fmaxf(mw, src[(size_t)s * (D + 2) + D]);
  float acc = 0.f, lsum = 0.f;
  for (int s = 0; s < splits; ++s) {
    const float mm = src[(size_t)s * (D + 2) + D];
    const float sc = (mm == -INFINITY) ? 0.f : __expf(mm - mw);
    acc += src[(size_t)s * (D + 2) + e] * sc;
    lsum += src[(size_t)s * (D + 2) + D + 1] * sc;
  }
  out[(size_t)bh * D + e] = f2bf(acc / lsum);
}

int pick_splits(int B, int Hkv, int S_max) {
  int s = 256 / (B * Hkv);
  int cap = S_max / 64;
  if (s > cap) s = cap;
  if (s > kMaxSplits) s = kMaxSplits;
  if (s < 1) s = 1;
  return s;
}

template <int D, bool DECODE>
int launch_sdpa(const SdpaParams& p, hipStream_t st) {
  const int G = p.Hq / p.Hkv;
  dim3 grid(DECODE ? p.splits : p.T, p.Hkv, p.B);
  switch (G) {
    case 1: sdpa_kernel<D, 1, DECODE><<<grid, kThreads, 0, st>>>(p); break;
    case 2: sdpa_kernel<D, 2, DECODE><<<grid, kThreads, 0, st>>>(p); break;
    case 4: sdpa_kernel<D, 4, DECODE><<<grid, kThreads, 0, st>>>(p); break;
    case 8: sdpa_kernel<D, 8, DECODE><<<grid, kThreads, 0, st>>>(p); break;
    case 16: sdpa_kernel<D, 16, DECODE><<<grid, kThreads, 0, st>>>(p); break;
    default:
      exo_set_error("sdpa: unsupported Hq/Hkv=%d (1,2,4,8,16)", G);
      return EXO_ERR_ARG;
  }
  if (DECODE)
    sdpa_merge_kernel<D><<<dim3(p.B * p.Hq), D, 0, st>>>(p.ws, p.out, p.splits);
  return EXO_OK;
}

int check(const char* name, int B, int T, int Hq, int Hkv, int D, int S_max) {
  EXO_REQUIRE(B > 0 && T > 0 && Hq > 0 && Hkv > 0 && S_max > 0, "%s: non-positive size", name);
  EXO_REQUIRE(Hq % Hkv == 0, "%s: Hq=%d not a multiple of Hkv=%d", name, Hq, Hkv);
  EXO_REQUIRE(D == 64 || D == 128, "%s: head_dim %d not supported (64, 128)", name, D);
  EXO_REQUIRE(B <= 65535 && Hkv <= 65535, "%s: grid too large", name);
  return EXO_OK;
}

}  // namespace

extern "C" int64_t exo_sdpa_decode_workspace(int B, int Hq, int D) {
  return (int64_t)B * Hq * kMaxSplits * (D + 2) * (int64_t)sizeof(float);
}

extern "C" int exo_sdpa_decode(const uint16_t* q, const uint16_t* k_cache,
                               const uint16_t* v_cache, const int32_t* pos, uint16_t* out,
                               float* workspace, float scale, int B, int Hq, int Hkv, int D,
                               int S_max, exo_stream_t stream) {
  int rc = check("exo_sdpa_decode", B, 1, Hq, Hkv, D, S_max);
  if (rc) return rc;
  EXO_REQUIRE(q && k_cache && v_cache && pos && out && workspace,
              "exo_sdpa_decode: null pointer");
  SdpaParams p{q, k_cache, v_cache, pos, out, workspace, scale, B, 1, Hq, Hkv, S_max,
               pick_splits(B, Hkv, S_max)};
  rc = (D == 64) ? launch_sdpa<64, true>(p, (hipStream_t)stream)
                 : launch_sdpa<128, true>(p, (hipStream_t)stream);
  if (rc) return rc;
  EXO_CHECK_LAUNCH("exo_sdpa_decode");
  return EXO_OK;
}

extern "C" int exo_sdpa_prefill(const uint16_t* q, const uint16_t* k_cache,
                                const uint16_t* v_cache, const int32_t* pos, uint16_t* out,
                                float scale, int B, int T, int Hq, int Hkv, int D, int S_max,
                                exo_stream_t stream) {
  int rc = check("exo_sdpa_prefill", B, T, Hq, Hkv, D, S_max);
  if (rc) return rc;
  EXO_REQUIRE(q && k_cache && v_cache && pos && out, "exo_sdpa_prefill: null pointer");
  SdpaParams p{q, k_cache, v_cache, pos, out, nullptr, scale, B, T, Hq, Hkv, S_max, 1};
  rc = (D == 64) ? launch_sdpa<64, false>(p, (hipStream_t)stream)
                 : launch_sdpa<128, false>(p, (hipStream_t)stream);
  if (rc) return rc;
  EXO_CHECK_LAUNCH("exo_sdpa_prefill");
  return EXO_OK;
}
