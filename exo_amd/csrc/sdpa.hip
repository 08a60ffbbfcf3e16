// Scaled dot-product attention over the bf16 KV cache, grouped-query.
//
// One workgroup serves ONE kv head and all G = Hq/Hkv query heads that share it, so
// every K/V byte read from HBM is used G times.  A key row (D bf16) is spread over
// D/8 lanes, 16 bytes each; one load instruction of a wave reads 512/D consecutive
// keys (1 KiB contiguous); two tiles of four such K and V loads are in flight per lane.
// Scores, softmax and the output accumulation are float32 (online softmax, one
// rescale per block of 4 keys).
//
// decode : grid (splits, Hkv, B); each split owns a contiguous key range, writes
//          (max, sum, acc[D]) per query head to the workspace; the last workgroup of a
//          (sequence, kv head) to arrive - an atomic counter, no spinning - merges the
//          splits.  The grid is fixed (positions are read on the device), so the
//          launch can be replayed from a HIP graph while the sequence grows.
// prefill: grid (T, Hkv, B); one workgroup per new token, causal limit pos+t+1,
//          writes the output directly.
#include "../../include/exo_mi355x.h"
#include "common.h"
#include <mutex>
#include "sdpa_internal.h"

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = 4;
constexpr int kMaxSplits = 16;
// More splits than 16 were slower for every head layout measured (4 and 8 kv heads) at a few
// thousand keys: the merge by the last workgroup grows with the split count.  Contexts the
// host declares long (exo_attn_decode_hint) take up to kMaxSplitsLong (64 lost to 32 at
// every length up to 130000 keys).
constexpr int kMaxSplitsLong = 32;
constexpr int kBlk = 4;  // keys per lane group per step
#ifndef EXO_SDPA_TILES
#define EXO_SDPA_TILES 1  // decode on the interleaved-tile kernel (0: contiguous key ranges)
#endif
#ifndef EXO_SDPA_TILES_IN_FLIGHT
#define EXO_SDPA_TILES_IN_FLIGHT 2
#endif
constexpr int kTilesInFlight = EXO_SDPA_TILES_IN_FLIGHT;  // key tiles a wave keeps in flight
#ifndef EXO_SDPA_ABL
#define EXO_SDPA_ABL 0  // timing-only ablations (wrong results)
#endif
#ifndef EXO_SDPA_TILES_WAVES
#define EXO_SDPA_TILES_WAVES 4
#endif
constexpr int kTileWaves = EXO_SDPA_TILES_WAVES;  // waves per workgroup (up to 4 heads per workgroup)

struct SdpaParams {
  const bf16_t* q;   // [B*T, Hq*D]
  const bf16_t* kc;  // [B, Hkv, S_max, D]
  const bf16_t* vc;
  const int32_t* pos;  // [B]
  bf16_t* out;         // [B*T, Hq*D]
  float* ws;           // decode partials
  int* counters;       // decode: arrival counter per (sequence, kv head); zero between launches
  float scale;
  int B, T, Hq, Hkv, S_max, splits;
  // fused decode (q/k RoPE, optional head RMSNorm and the cache append done here)
  const bf16_t* qkv;        // [B, (Hq+2*Hkv)*D]
  const float* inv_freq;    // [D/2]
  const float2* rope_tab;   // [S_max, D/2] (cos, sin) per position, or null
  const bf16_t* qn;         // [D] or null
  const bf16_t* kn;
  float eps;
  // decode: the Hq/Hkv query heads of a kv head are handled by `hgroups` workgroups of G
  // heads each (blockIdx.y = kv head * hgroups + group); set by the launcher
  int hgroups;
};

// Sum over the LPK lanes of a key's lane group.  16 lanes are one DPP row: four
// full-rate VALU ops instead of four LDS-crossbar permutes.
template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}
template <int LPK>
__device__ __forceinline__ float group_sum_lpk(float d) {
  if (LPK == 16) {
    d += dpp_f<0xB1>(d);   // quad_perm [1,0,3,2]
    d += dpp_f<0x4E>(d);   // quad_perm [2,3,0,1]
    d += dpp_f<0x141>(d);  // row_half_mirror
    d += dpp_f<0x140>(d);  // row_mirror
    return d;
  }
#pragma unroll
  for (int off = LPK >> 1; off > 0; off >>= 1) d += __shfl_xor(d, off, 64);
  return d;
}
// value of the lane LPK/2 away inside the lane group (the RoPE partner)
template <int LPK>
__device__ __forceinline__ float partner_lpk(float v) {
  if (LPK == 16) return dpp_f<0x128>(v);  // row_ror:8
  return __shfl_xor(v, LPK / 2, 64);
}

__device__ __forceinline__ void st_dev(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float ld_dev(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The last workgroup's merge of the key splits of one output element: partials
// [splits][D + 2] (D sums, then the split's maximum and its sum of weights), taken sixteen
// splits at a time - all loads of a batch are issued before any is used (they miss every
// cache) - and folded into a running (maximum, sum, weighted sum).
template <int D>
__device__ __forceinline__ float merge_splits(const float* src, int splits, int e) {
  constexpr int MS = 16;
  float mw = -INFINITY, acc = 0.f, lsum = 0.f;
  for (int s0 = 0; s0 < splits; s0 += MS) {
    float pm[MS], pl[MS], po[MS];
#pragma unroll
    for (int sp = 0; sp < MS; ++sp) {
      const int spc = min(s0 + sp, splits - 1);
      pm[sp] = ld_dev(src + (size_t)spc * (D + 2) + D);
      pl[sp] = ld_dev(src + (size_t)spc * (D + 2) + D + 1);
      po[sp] = ld_dev(src + (size_t)spc * (D + 2) + e);
    }
    float mc = mw;
#pragma unroll
    for (int sp = 0; sp < MS; ++sp)
      if (s0 + sp < splits) mc = fmaxf(mc, pm[sp]);
    if (s0 > 0) {  // earlier batches move to the new maximum
      const float r = (mw == -INFINITY) ? 0.f : __expf(mw - mc);
      acc *= r;
      lsum *= r;
    }
#pragma unroll
    for (int sp = 0; sp < MS; ++sp) {
      const float sc = (s0 + sp >= splits || pm[sp] == -INFINITY) ? 0.f : __expf(pm[sp] - mc);
      acc += po[sp] * sc;
      lsum += pl[sp] * sc;
    }
    mw = mc;
  }
  return acc / lsum;
}

// One head slice (8 elements of this lane, the head spread over LPK lanes) taken from a
// fused qkv row: optional per-head RMSNorm (rounded to bf16 like a separate rms_norm),
// then rotate-half RoPE with the lane's 8 (cos, sin) pairs, rounded to bf16.
// `raw`: the lane's 16 bytes of the head; `nwv`: its 8 norm weights (HAS_NORM).
template <int D, bool ROPE>
__device__ __forceinline__ uint4 head_slice_apply(const uint4 raw, int sl, bool has_norm, const uint4 nwv,
                                                  float eps, const float (&cs)[8], const float (&sn)[8]) {
  constexpr int LPK = D / 8;
  if (!ROPE) return raw;
  const uint32_t* r4 = reinterpret_cast<const uint32_t*>(&raw);
  float x[8];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    x[2 * e] = bf_lo(r4[e]);
    x[2 * e + 1] = bf_hi(r4[e]);
  }
  if (has_norm) {
    const uint32_t* n4 = reinterpret_cast<const uint32_t*>(&nwv);
    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) ss = fmaf(x[e], x[e], ss);
    ss = group_sum_lpk<LPK>(ss);
    const float inv = rsqrtf(ss / (float)D + eps);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float w = (e & 1) ? bf_hi(n4[e >> 1]) : bf_lo(n4[e >> 1]);
      x[e] = bf2f(f2bf(x[e] * inv * w));
    }
  }
  const bool first = sl < LPK / 2;  // this lane holds elements of the first half
  uint4 out;
  uint32_t* o4 = reinterpret_cast<uint32_t*>(&out);
  float y[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float other = partner_lpk<LPK>(x[e]);
    // first half: x1*c - x2*s ; second half: x2*c + x1*s
    y[e] = first ? (x[e] * cs[e] - other * sn[e]) : (x[e] * cs[e] + other * sn[e]);
  }
#pragma unroll
  for (int e = 0; e < 4; ++e) o4[e] = pack_bf2(y[2 * e], y[2 * e + 1]);
  return out;
}
template <int D, bool ROPE>
__device__ __forceinline__ uint4 head_slice(const bf16_t* src, int sl, const bf16_t* nw,
                                            float eps, const float (&cs)[8], const float (&sn)[8]) {
  const uint4 raw = *reinterpret_cast<const uint4*>(src + sl * 8);
  uint4 nwv = make_uint4(0, 0, 0, 0);
  if (ROPE && nw) nwv = *reinterpret_cast<const uint4*>(nw + sl * 8);
  return head_slice_apply<D, ROPE>(raw, sl, nw != nullptr, nwv, eps, cs, sn);
}

// MODE 0: prefill (one workgroup per new token); 1: decode over a cache that already
// holds the new token; 2: decode fused with RoPE / head norm / cache append.
template <int D, int G, int MODE>
__global__ __launch_bounds__(kThreads) void sdpa_kernel(const SdpaParams p) {
  constexpr bool DECODE = MODE != 0;
  constexpr bool FUSED = MODE == 2;
  constexpr int LPK = D / 8;        // lanes per key
  constexpr int KPI = 64 / LPK;     // keys per wave instruction
  constexpr int STEP = KPI * kBlk;  // keys per wave per step
  __shared__ float red[kWaves][G][D + 2];
  __shared__ int s_last;

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int sub = lane / LPK, sl = lane % LPK;
  const int b = blockIdx.z;
  const int kvh = DECODE ? (int)blockIdx.y / p.hgroups : (int)blockIdx.y;
  const int hg = DECODE ? (int)blockIdx.y % p.hgroups : 0;
  const int h0 = kvh * (G * (DECODE ? p.hgroups : 1)) + hg * G;  // first query head of this workgroup
  const int t = DECODE ? 0 : blockIdx.x;
  const int len = min(p.pos[b] + t + 1, p.S_max);  // keys visible to this query
  int k_begin = 0, k_end = len;
  bool own_new = false;  // fused: this workgroup handles the new token's key/value
  if (DECODE) {
    int chunk = (len + p.splits - 1) / p.splits;
    chunk = (chunk + STEP * kWaves - 1) / (STEP * kWaves) * (STEP * kWaves);
    k_begin = min((int)blockIdx.x * chunk, len);
    k_end = min(k_begin + chunk, len);
    if (FUSED) {  // the cache holds keys [0, len-1); key len-1 comes from the qkv row
      own_new = (len - 1) / chunk == (int)blockIdx.x;
      k_begin = min(k_begin, len - 1);
      k_end = min(k_end, len - 1);
    }
  }
  // each wave owns a contiguous quarter of the workgroup's range (multiple of STEP keys)
  const int per_wave = ((k_end - k_begin + kWaves - 1) / kWaves + STEP - 1) / STEP * STEP;
  const int w_begin = min(k_begin + wave * per_wave, k_end);
  const int w_end = min(w_begin + per_wave, k_end);

  const size_t head_base = ((size_t)b * p.Hkv + kvh) * p.S_max * D;
  const bf16_t* kb = p.kc + head_base + sl * 8;
  const bf16_t* vb = p.vc + head_base + sl * 8;

  struct Tile {
    uint4 k[kBlk], v[kBlk];
  };
  // instruction i of a step reads KPI consecutive keys (KPI*D*2 contiguous bytes)
  auto load = [&](Tile& tl, int k0) {
#pragma unroll
    for (int i = 0; i < kBlk; ++i) {
      const int key = min(k0 + i * KPI + sub, w_end - 1);
      tl.k[i] = *reinterpret_cast<const uint4*>(kb + (size_t)key * D);
      tl.v[i] = *reinterpret_cast<const uint4*>(vb + (size_t)key * D);
    }
  };
  // the first K/V tile is requested before the q work so its latency overlaps it
  Tile ta, tb;
  if (w_begin < w_end) load(ta, w_begin);

  // q slices for the G heads: 8 elements = 4 bf16 pairs per head per lane
  uint4 qv[G];
  uint4 knew = make_uint4(0, 0, 0, 0), vnew = make_uint4(0, 0, 0, 0);
  const size_t qrow = (size_t)(b * p.T + t) * p.Hq * D;
  if (FUSED) {
    float cs[8], sn[8];
    if (p.rope_tab) {  // 8 consecutive (cos, sin) pairs of this position: 64 bytes
      const float4* tp = reinterpret_cast<const float4*>(
          p.rope_tab + (size_t)(len - 1) * (D / 2) + (sl * 8) % (D / 2));
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float4 v = tp[e];
        cs[2 * e] = v.x;
        sn[2 * e] = v.y;
        cs[2 * e + 1] = v.z;
        sn[2 * e + 1] = v.w;
      }
    } else {
      const float fpos = (float)(len - 1);
#pragma unroll
      for (int e = 0; e < 8; ++e)
        sincosf(fpos * p.inv_freq[(sl * 8 + e) % (D / 2)], &sn[e], &cs[e]);
    }
    const bf16_t* row = p.qkv + (size_t)b * (p.Hq + 2 * p.Hkv) * D;
#pragma unroll
    for (int g = 0; g < G; ++g)
      qv[g] = head_slice<D, true>(row + (size_t)(h0 + g) * D, sl, p.qn, p.eps, cs, sn);
    if (own_new && wave == 0) {
      knew = head_slice<D, true>(row + (size_t)(p.Hq + kvh) * D, sl, p.kn, p.eps, cs, sn);
      vnew = head_slice<D, false>(row + (size_t)(p.Hq + p.Hkv + kvh) * D, sl, nullptr, 0.f, cs, sn);
    }
  } else {
#pragma unroll
    for (int g = 0; g < G; ++g)
      qv[g] = *reinterpret_cast<const uint4*>(p.q + qrow + (size_t)(h0 + g) * D + sl * 8);
  }

  float m[G], l[G], o[G][8];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    m[g] = -INFINITY;
    l[g] = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) o[g][e] = 0.f;
  }

  auto consume = [&](const Tile& tl, int k0, int limit) {
    float s[G][kBlk];
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
      for (int i = 0; i < kBlk; ++i) {
        float d = dot2_bf16(qv[g].x, tl.k[i].x, 0.f);
        d = dot2_bf16(qv[g].y, tl.k[i].y, d);
        d = dot2_bf16(qv[g].z, tl.k[i].z, d);
        d = dot2_bf16(qv[g].w, tl.k[i].w, d);
        d = group_sum_lpk<LPK>(d);
        s[g][i] = (k0 + i * KPI + sub < limit) ? d * p.scale : -INFINITY;
      }
#pragma unroll
    for (int g = 0; g < G; ++g) {
      float bm = s[g][0];
#pragma unroll
      for (int i = 1; i < kBlk; ++i) bm = fmaxf(bm, s[g][i]);
      const float mn = fmaxf(m[g], bm);
      // a lane group that has seen no valid key yet keeps (m=-inf, l=0, o=0)
      const float base = (mn == -INFINITY) ? 0.f : mn;
      const float sc = __expf(m[g] - base);
      float pr[kBlk], ps = 0.f;
#pragma unroll
      for (int i = 0; i < kBlk; ++i) {
        pr[i] = __expf(s[g][i] - base);
        ps += pr[i];
      }
      l[g] = l[g] * sc + ps;
      m[g] = mn;
#pragma unroll
      for (int e = 0; e < 8; ++e) o[g][e] *= sc;
#pragma unroll
      for (int i = 0; i < kBlk; ++i) {
        const uint32_t* v4 = reinterpret_cast<const uint32_t*>(&tl.v[i]);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          o[g][2 * e] = fmaf(pr[i], bf_lo(v4[e]), o[g][2 * e]);
          o[g][2 * e + 1] = fmaf(pr[i], bf_hi(v4[e]), o[g][2 * e + 1]);
        }
      }
    }
  };

  if (w_begin < w_end) {
    int k0 = w_begin;
    for (;;) {
      if (k0 + STEP < w_end) load(tb, k0 + STEP);
      consume(ta, k0, w_end);
      k0 += STEP;
      if (k0 >= w_end) break;
      if (k0 + STEP < w_end) load(ta, k0 + STEP);
      consume(tb, k0, w_end);
      k0 += STEP;
      if (k0 >= w_end) break;
    }
  }
  if (FUSED && own_new && wave == 0) {
    // the new token: key/value straight from registers (only lane group 0, slot 0 is
    // valid), and appended to the cache for the following steps
    Tile tn;
#pragma unroll
    for (int i = 0; i < kBlk; ++i) {
      tn.k[i] = i == 0 ? knew : make_uint4(0, 0, 0, 0);
      tn.v[i] = i == 0 ? vnew : make_uint4(0, 0, 0, 0);
    }
    consume(tn, len - 1, len);
    if (sub == 0 && hg == 0) {  // one of the head groups appends to the cache
      const size_t o = head_base + (size_t)(len - 1) * D + sl * 8;
      *reinterpret_cast<uint4*>(const_cast<bf16_t*>(p.kc) + o) = knew;
      *reinterpret_cast<uint4*>(const_cast<bf16_t*>(p.vc) + o) = vnew;
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
    const int h = h0 + g;
    if (DECODE) {
      // device-scope (write-through) stores: the merging workgroup may run on another
      // XCD, whose L2 is not coherent with this one
      float* dst = p.ws + ((size_t)(b * p.Hq + h) * p.splits + blockIdx.x) * (D + 2);
      st_dev(dst + e, acc);
      if (e == 0) {
        st_dev(dst + D, mw);
        st_dev(dst + D + 1, lsum);
      }
    } else {
      p.out[qrow + (size_t)h * D + e] = f2bf(acc / lsum);
    }
  }
  if (!DECODE) return;

  // The last workgroup of this (sequence, kv head) to finish merges the splits.  The
  // counter returns to zero, so the launch can be replayed without re-initialising it.
  // No device-wide fence (an L2 write-back on this chip): the partials were stored and
  // are loaded at device scope; every wave waits for its own stores to complete, the
  // barrier collects the waves, and only then is the counter bumped.
  wait_own_stores_done();
  __syncthreads();
  if (threadIdx.x == 0) {
    int* cnt = &p.counters[b * p.Hkv * p.hgroups + blockIdx.y];
    const int old = __hip_atomic_fetch_add(cnt, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    s_last = (old == p.splits - 1);
    if (s_last) __hip_atomic_store(cnt, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __syncthreads();
  if (!s_last) return;
  for (int idx = threadIdx.x; idx < G * D; idx += kThreads) {
    const int g = idx / D, e = idx % D;
    const int h = h0 + g;
    const float* src = p.ws + (size_t)(b * p.Hq + h) * p.splits * (D + 2);
    p.out[qrow + (size_t)h * D + e] = f2bf(merge_splits<D>(src, p.splits, e));
  }
}

// ---------------------------------------------------------------- decode, interleaved tiles
// Decode attention with the key tiles dealt out round robin: the NWV = splits * 4 waves
// that serve one (sequence, kv head, head group) take the tiles of STEP keys in turn (wave w:
// tiles w, w + NWV, w + 2 NWV ...).  Which tile a wave starts with does not depend on the
// sequence's length, so its first two tiles are requested before the position has even been
// read - their latency runs beside the position -> rope table -> q rotation chain instead of
// behind it - and every wave gets the same number of tiles to within one, whatever the length
// (contiguous ranges rounded to whole steps left the last splits of a 2050-key context idle).
// Tiles come through buffer loads whose range ends at the last cached key: a refill past the
// end moves no data and returns zeros, so every refill is issued unconditionally and the
// number of loads in flight at each wait is a compile-time constant.
// FUSED: q/k RoPE (table or sincos), optional head RMSNorm and the cache append done here;
// the cache then holds keys [0, len-1) and key len-1 comes from the qkv row.
template <int D, int G, bool FUSED, int NW>
__global__ __launch_bounds__(64 * NW) void sdpa_tiles_kernel(const SdpaParams p) {
  constexpr int LPK = D / 8;        // lanes per key
  constexpr int KPI = 64 / LPK;     // keys per wave instruction
  constexpr int STEP = KPI * kBlk;  // keys per tile
  constexpr int NT = kTilesInFlight;
  __shared__ float red[NW][G][D + 2];
  __shared__ int s_last;

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int sub = lane / LPK, sl = lane % LPK;
  const int b = blockIdx.z;
  const int kvh = (int)blockIdx.y / p.hgroups, hg = (int)blockIdx.y % p.hgroups;
  const int h0 = kvh * (G * p.hgroups) + hg * G;  // first query head of this workgroup
  const int nwv = p.splits * NW;
  const int gwv = (int)blockIdx.x * NW + wave;

  const size_t head_base = ((size_t)b * p.Hkv + kvh) * p.S_max * D;
  struct Tile {
    uint4 k[kBlk], v[kBlk];
  };
  const int lane_ofs = (sub * D + sl * 8) * 2;  // byte offset of this lane inside an instruction's keys
  auto load_tile = [&](Tile& tl, __amdgpu_buffer_rsrc_t rk, __amdgpu_buffer_rsrc_t rv, int t) {
    const int tb = t * (STEP * D * 2);  // uniform
#pragma unroll
    for (int i = 0; i < kBlk; ++i) {
      tl.k[i] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(rk, lane_ofs + i * (KPI * D * 2), tb, 0));
      tl.v[i] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(rv, lane_ofs + i * (KPI * D * 2), tb, 0));
    }
  };
  const int len = min(p.pos[b] + 1, p.S_max);  // keys visible to the query
  const int n_keys = FUSED ? len - 1 : len;     // of which the cache holds these
  const bool own_new = FUSED && ((n_keys / STEP) % nwv) == gwv;  // this wave adds the new token
  const __amdgpu_buffer_rsrc_t rk = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<bf16_t*>(p.kc + head_base), 0, n_keys * D * 2, 0x00020000);
  const __amdgpu_buffer_rsrc_t rv = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<bf16_t*>(p.vc + head_base), 0, n_keys * D * 2, 0x00020000);

  // Order of the requests: what the q rotation needs first (rope table row, q, the new
  // token's k and v, norm weights), then the first key tiles - loads return in order, so the
  // rotation runs while the tiles are still on their way.
  uint4 qv[G];
  uint4 knew = make_uint4(0, 0, 0, 0), vnew = make_uint4(0, 0, 0, 0);
  const size_t qrow = (size_t)b * p.Hq * D;
  float4 tabv[4];
  uint4 nq = make_uint4(0, 0, 0, 0), nk = nq;
  const bf16_t* row = FUSED ? p.qkv + (size_t)b * (p.Hq + 2 * p.Hkv) * D : nullptr;
  if (FUSED) {
    if (p.rope_tab) {  // 8 consecutive (cos, sin) pairs of this position: 64 bytes
      const float4* tp = reinterpret_cast<const float4*>(
          p.rope_tab + (size_t)(len - 1) * (D / 2) + (sl * 8) % (D / 2));
#pragma unroll
      for (int e = 0; e < 4; ++e) tabv[e] = tp[e];
    }
#pragma unroll
    for (int g = 0; g < G; ++g)
      qv[g] = *reinterpret_cast<const uint4*>(row + (size_t)(h0 + g) * D + sl * 8);
    if (own_new) {
      knew = *reinterpret_cast<const uint4*>(row + (size_t)(p.Hq + kvh) * D + sl * 8);
      vnew = *reinterpret_cast<const uint4*>(row + (size_t)(p.Hq + p.Hkv + kvh) * D + sl * 8);
    }
    if (p.qn) nq = *reinterpret_cast<const uint4*>(p.qn + sl * 8);
    if (p.kn) nk = *reinterpret_cast<const uint4*>(p.kn + sl * 8);
  } else {
#pragma unroll
    for (int g = 0; g < G; ++g)
      qv[g] = *reinterpret_cast<const uint4*>(p.q + qrow + (size_t)(h0 + g) * D + sl * 8);
  }
  Tile tl[NT];
#pragma unroll
  for (int n = 0; n < NT; ++n) load_tile(tl[n], rk, rv, gwv + n * nwv);
  if (FUSED) {
    float cs[8], sn[8];
    if (p.rope_tab) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        cs[2 * e] = tabv[e].x;
        sn[2 * e] = tabv[e].y;
        cs[2 * e + 1] = tabv[e].z;
        sn[2 * e + 1] = tabv[e].w;
      }
    } else {
      const float fpos = (float)(len - 1);
#pragma unroll
      for (int e = 0; e < 8; ++e)
        sincosf(fpos * p.inv_freq[(sl * 8 + e) % (D / 2)], &sn[e], &cs[e]);
    }
#pragma unroll
    for (int g = 0; g < G; ++g)
      qv[g] = head_slice_apply<D, true>(qv[g], sl, p.qn != nullptr, nq, p.eps, cs, sn);
    if (own_new) knew = head_slice_apply<D, true>(knew, sl, p.kn != nullptr, nk, p.eps, cs, sn);
  }

  float m[G], l[G], o[G][8];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    m[g] = -INFINITY;
    l[g] = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) o[g][e] = 0.f;
  }

  // keys [k0, k0 + STEP) of the tile against the G heads; keys from `limit` on do not count
  // (MASKV: and their value rows are replaced by zeros - what the tile holds there is whatever
  // the cache row held, not necessarily finite)
  auto consume = [&](const Tile& tile, int k0, int limit, bool maskv) {
    float s[G][kBlk];
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
      for (int i = 0; i < kBlk; ++i) {
        float d = dot2_bf16(qv[g].x, tile.k[i].x, 0.f);
        d = dot2_bf16(qv[g].y, tile.k[i].y, d);
        d = dot2_bf16(qv[g].z, tile.k[i].z, d);
        d = dot2_bf16(qv[g].w, tile.k[i].w, d);
        d = group_sum_lpk<LPK>(d);
        s[g][i] = (k0 + i * KPI + sub < limit) ? d * p.scale : -INFINITY;
      }
    uint4 vv[kBlk];
#pragma unroll
    for (int i = 0; i < kBlk; ++i) {
      vv[i] = tile.v[i];
      if (maskv && !(k0 + i * KPI + sub < limit)) vv[i] = make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int g = 0; g < G; ++g) {
      float bm = s[g][0];
#pragma unroll
      for (int i = 1; i < kBlk; ++i) bm = fmaxf(bm, s[g][i]);
      const float mn = fmaxf(m[g], bm);
      // a lane group that has seen no valid key yet keeps (m=-inf, l=0, o=0)
      const float base = (mn == -INFINITY) ? 0.f : mn;
      const float sc = __expf(m[g] - base);
      float pr[kBlk], ps = 0.f;
#pragma unroll
      for (int i = 0; i < kBlk; ++i) {
        pr[i] = __expf(s[g][i] - base);
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
  };

  // the tiles of this wave in turn; every refill is issued (past the end: out of range)
  {
    int t = gwv;
    bool more = t * STEP < n_keys;
    while (more) {
#pragma unroll
      for (int n = 0; n < NT; ++n) {
        if (more) {
          const int k0 = t * STEP;
          consume(tl[n], k0, n_keys, k0 + STEP > n_keys);
        }
        load_tile(tl[n], rk, rv, t + NT * nwv);
        t += nwv;
        more = more && t * STEP < n_keys;
      }
    }
  }
  if (own_new) {
    // the new token: key/value straight from registers (only lane group 0, slot 0 is
    // valid), and appended to the cache for the following steps
    Tile tn;
#pragma unroll
    for (int i = 0; i < kBlk; ++i) {
      tn.k[i] = i == 0 ? knew : make_uint4(0, 0, 0, 0);
      tn.v[i] = i == 0 ? vnew : make_uint4(0, 0, 0, 0);
    }
    consume(tn, len - 1, len, false);
    if (sub == 0 && hg == 0) {  // one of the head groups appends to the cache
      const size_t o = head_base + (size_t)(len - 1) * D + sl * 8;
      *reinterpret_cast<uint4*>(const_cast<bf16_t*>(p.kc) + o) = knew;
      *reinterpret_cast<uint4*>(const_cast<bf16_t*>(p.vc) + o) = vnew;
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

  // merge the waves; thread -> (head, element); partial results at device scope (the merging
  // workgroup may run on another XCD, whose L2 is not coherent with this one)
  for (int idx = threadIdx.x; idx < G * D; idx += 64 * NW) {
    const int g = idx / D, e = idx % D;
    float mw = red[0][g][D];
#pragma unroll
    for (int w = 1; w < NW; ++w) mw = fmaxf(mw, red[w][g][D]);
    float acc = 0.f, lsum = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      const float mm = red[w][g][D];
      const float sc = (mm == -INFINITY) ? 0.f : __expf(mm - mw);
      acc += red[w][g][e] * sc;
      lsum += red[w][g][D + 1] * sc;
    }
#if (EXO_SDPA_ABL & 1)  // timing only: no hand-over, every split writes its own result
    p.out[qrow + (size_t)(h0 + g) * D + e] = f2bf(acc / lsum);
    continue;
#endif
    float* dst = p.ws + ((size_t)(b * p.Hq + h0 + g) * p.splits + blockIdx.x) * (D + 2);
    st_dev(dst + e, acc);
    if (e == 0) {
      st_dev(dst + D, mw);
      st_dev(dst + D + 1, lsum);
    }
  }
#if (EXO_SDPA_ABL & 1)
  return;
#endif
  // the last workgroup of this (sequence, kv head, head group) to finish merges the splits
  // (see sdpa_kernel); the counter returns to zero
  wait_own_stores_done();
  __syncthreads();
  if (threadIdx.x == 0) {
    int* cnt = &p.counters[b * p.Hkv * p.hgroups + blockIdx.y];
    const int old = __hip_atomic_fetch_add(cnt, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    s_last = (old == p.splits - 1);
    if (s_last) __hip_atomic_store(cnt, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __syncthreads();
  if (!s_last) return;
  for (int idx = threadIdx.x; idx < G * D; idx += 64 * NW) {
    const int g = idx / D, e = idx % D;
    const int h = h0 + g;
    const float* src = p.ws + (size_t)(b * p.Hq + h) * p.splits * (D + 2);
    p.out[qrow + (size_t)h * D + e] = f2bf(merge_splits<D>(src, p.splits, e));
  }
}

typedef short short4_t __attribute__((ext_vector_type(4)));
// ds_read_b64_tr_b16: four consecutive rows of one column out of a row-major bf16 tile
__device__ __forceinline__ uint2 lds_read_tr16(const bf16_t* p) {
  const short4_t v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
      (short4_t __attribute__((address_space(3)))*)p);
  return __builtin_bit_cast(uint2, v);
}

// ---------------------------------------------------------------- matrix-core decode
// Fused decode attention (RoPE, head norm, cache append, attention) for D = 128 with the
// two products on v_mfma_f32_32x32x16_bf16.  The scalar kernel above spends ~10 vector
// instructions per (query head, key) and lane group; with several sequences in the step
// that - not the K/V bytes - bounds it.  Here one wave multiplies a tile
// of 32 keys by ALL G query heads of the kv head at once (they are columns of the B operand,
// the unused ones zero):
//   S^T[key][head] = K . Q^T     A = K rows from the wave's LDS tile, B = Q^T from registers
//   O^T[d][head]  += V^T . P^T   A = V^T: 8 keys of one d per lane, out of the row-major V
//                                tile with two transposing LDS reads; B = the S^T registers
// as in the prefill kernel (same permuted key order, same per-lane softmax state).
// Work split: grid (splits, Hkv, B); a workgroup's four waves take a quarter of the split's
// keys each, in tiles of 32 that go global -> registers -> the wave's own LDS region (no
// block barrier in the loop).  The new token's key and value come from registers / LDS and
// are added by wave 0 of the split that owns position len-1.  The partial results leave in
// the layout of the scalar kernel, so the merge of waves and splits is the same code.
template <int G>
__global__ __launch_bounds__(kThreads, 2) void sdpa_decode_mfma_kernel(const SdpaParams p) {
  constexpr int D = 128;
  constexpr int TK = 32;          // keys per tile
  constexpr int KS = D + 8;       // LDS row stride (bf16)
  constexpr int STEPS = D / 16, DT = D / 32;
  constexpr int VS = D + 16;      // V rows: 32 bytes past a multiple of the 256-byte bank span
  constexpr int TILE = TK * KS;   // bf16 elements of a K tile
  constexpr int WAVE_TILES = TK * KS + TK * VS;  // K tile + V tile of one wave
  constexpr int TILE_BYTES = kWaves * WAVE_TILES * 2;
  constexpr int RED_BYTES = kWaves * G * (D + 2) * 4;
  constexpr int SMEM = TILE_BYTES > RED_BYTES ? TILE_BYTES : RED_BYTES;
  __shared__ __attribute__((aligned(16))) char smem[SMEM];
  __shared__ __attribute__((aligned(16))) bf16_t q_lds[G * D];
  __shared__ __attribute__((aligned(16))) bf16_t kv_new[2 * D];
  __shared__ int s_last;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 31, kq = lane >> 5;
  const int b = blockIdx.z, kvh = blockIdx.y;
  const int h0 = kvh * G;
  const int len = min(p.pos[b] + 1, p.S_max);
  // the cache holds keys [0, len-1); key len-1 comes from the qkv row
  int chunk = (len + p.splits - 1) / p.splits;
  chunk = (chunk + TK * kWaves - 1) / (TK * kWaves) * (TK * kWaves);
  const bool own_new = (len - 1) / chunk == (int)blockIdx.x;
  const int k_begin = min(min((int)blockIdx.x * chunk, len), len - 1);
  const int k_end = min(min((int)blockIdx.x * chunk + chunk, len), len - 1);
  const int per_wave = ((k_end - k_begin + kWaves - 1) / kWaves + TK - 1) / TK * TK;
  const int w_begin = min(k_begin + wave * per_wave, k_end);
  const int w_end = min(w_begin + per_wave, k_end);

  const size_t head_base = ((size_t)b * p.Hkv + kvh) * p.S_max * D;
  const bf16_t* kb = p.kc + head_base;
  const bf16_t* vb = p.vc + head_base;
  // tile loads: 16-byte chunk vi = lane + 64*i of the tile is (key vi/16, chunk vi%16)
  // (always executed, with clamped keys, so that the tile registers are plain values: a
  // conditional refill made the compiler keep them in scratch memory and wait for every
  // load right after issuing it)
  // (eight named registers each, not arrays: those stayed in scratch memory here)
  uint4 k0r, k1r, k2r, k3r, k4r, k5r, k6r, k7r, v0r, v1r, v2r, v3r, v4r, v5r, v6r, v7r;
#define EXO_LOAD1(I, K0)                                                                \
  {                                                                                     \
    const int vi = lane + 64 * I;                                                       \
    const int key = max(min((K0) + (vi >> 4), w_end - 1), 0); /* past the range: masked */ \
    k##I##r = *reinterpret_cast<const uint4*>(kb + (size_t)key * D + (vi & 15) * 8);    \
    v##I##r = *reinterpret_cast<const uint4*>(vb + (size_t)key * D + (vi & 15) * 8);    \
  }
#define EXO_LOAD_TILE(K0) \
  EXO_LOAD1(0, K0) EXO_LOAD1(1, K0) EXO_LOAD1(2, K0) EXO_LOAD1(3, K0) EXO_LOAD1(4, K0) EXO_LOAD1(5, K0) EXO_LOAD1(6, K0) EXO_LOAD1(7, K0)
#define EXO_STORE1(I)                                                                  \
  {                                                                                    \
    const int vi = lane + 64 * I;                                                      \
    *reinterpret_cast<uint4*>(&k_t[(vi >> 4) * KS + (vi & 15) * 8]) = k##I##r;         \
    *reinterpret_cast<uint4*>(&v_t[(vi >> 4) * VS + (vi & 15) * 8]) = v##I##r;         \
  }
  EXO_LOAD_TILE(w_begin)  // in flight during the q work

  // ---- q of the G heads (RoPE, optional head norm) -> LDS; the new token's k and v
  {
    const int sub = lane >> 4, sl = lane & 15;
    float cs[8], sn[8];
    if (p.rope_tab) {
      const float4* tp = reinterpret_cast<const float4*>(
          p.rope_tab + (size_t)(len - 1) * (D / 2) + (sl * 8) % (D / 2));
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float4 v = tp[e];
        cs[2 * e] = v.x;
        sn[2 * e] = v.y;
        cs[2 * e + 1] = v.z;
        sn[2 * e + 1] = v.w;
      }
    } else {
      const float fpos = (float)(len - 1);
#pragma unroll
      for (int e = 0; e < 8; ++e) sincosf(fpos * p.inv_freq[(sl * 8 + e) % (D / 2)], &sn[e], &cs[e]);
    }
    const bf16_t* row = p.qkv + (size_t)b * (p.Hq + 2 * p.Hkv) * D;
#if (EXO_SDPA_ABL & 8)  // timing only: no table, no rotation
    for (int e = 0; e < 8; ++e) cs[e] = 1.f, sn[e] = 0.f;
#endif
    for (int g = wave * 4 + sub; g < G; g += 4 * kWaves)  // a 16-lane group per head
      *reinterpret_cast<uint4*>(&q_lds[g * D + sl * 8]) =
          head_slice<D, true>(row + (size_t)(h0 + g) * D, sl, p.qn, p.eps, cs, sn);
    if (own_new && wave == kWaves - 1 && sub < 2) {
      const uint4 t = sub == 0 ? head_slice<D, true>(row + (size_t)(p.Hq + kvh) * D, sl, p.kn, p.eps, cs, sn)
                               : head_slice<D, false>(row + (size_t)(p.Hq + p.Hkv + kvh) * D, sl, nullptr, 0.f, cs, sn);
      *reinterpret_cast<uint4*>(&kv_new[sub * D + sl * 8]) = t;
      // appended to the cache for the following steps
      bf16_t* dst = const_cast<bf16_t*>(sub == 0 ? p.kc : p.vc) + head_base + (size_t)(len - 1) * D + sl * 8;
      *reinterpret_cast<uint4*>(dst) = t;
    }
  }
  __syncthreads();

  // Q^T operand: lane (head n, half kq) takes d = 16*st + 8*kq .. +8 of its head for step
  // st - re-read from LDS for every tile (32 registers fewer to carry through the loop;
  // lanes beyond the G heads read head 0 and their columns are never stored)
  const bf16_t* qrow_lds = &q_lds[(n < G ? n : 0) * D + kq * 8];

  bf16_t* k_t = reinterpret_cast<bf16_t*>(smem) + (size_t)wave * WAVE_TILES;
  bf16_t* v_t = k_t + TILE;
  // A-operand row r of the 32-key tile holds this key, so that D registers 8s..8s+7 of
  // lane half kq are keys 16s + 8kq .. +8
  const int jr = n >> 3;
  const int key_of_row = 16 * (jr >> 1) + 8 * ((n >> 2) & 1) + 4 * (jr & 1) + (n & 3);
  const float scale_log2e = p.scale * 1.4426950408889634f;

  floatx16 o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int e = 0; e < 16; ++e) o[dt][e] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;  // log2 domain

  for (int k0 = w_begin; k0 < w_end; k0 += TK) {
    EXO_STORE1(0) EXO_STORE1(1) EXO_STORE1(2) EXO_STORE1(3) EXO_STORE1(4) EXO_STORE1(5) EXO_STORE1(6) EXO_STORE1(7)
    // the tile is private to the wave: its writes are complete before its reads
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_wave_barrier();
    EXO_LOAD_TILE(k0 + TK)

#if (EXO_SDPA_ABL & 4)  // timing only: tiles travel to LDS, nothing is computed
    o[0][0] += bf2f(k_t[lane]) + bf2f(v_t[lane]);
    continue;
#endif
    floatx16 sc;
#pragma unroll
    for (int e = 0; e < 16; ++e) sc[e] = 0.f;
    {
      const bf16_t* kr = &k_t[key_of_row * KS + kq * 8];
#pragma unroll
      for (int st = 0; st < STEPS; ++st) {
        const uint4 a = *reinterpret_cast<const uint4*>(kr + st * 16);
        const uint4 qv = *reinterpret_cast<const uint4*>(qrow_lds + st * 16);
        sc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                     __builtin_bit_cast(bf16x8_t, qv), sc, 0, 0, 0);
      }
    }
    const int vis = w_end - k0;  // keys [0, vis) of the tile are real
    float mx = -INFINITY;
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int key = 16 * (e >> 3) + 8 * kq + (e & 7);
      const float x = key < vis ? sc[e] * scale_log2e : -INFINITY;
      sc[e] = x;
      mx = fmaxf(mx, x);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(m_run, mx);  // finite: key 0 of the tile is real
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
    float sum = 0.f;
    uint4 pb[2];
    {
      float pr[16];
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        pr[e] = __builtin_amdgcn_exp2f(sc[e] - m_new);
        sum += pr[e];
      }
#pragma unroll
      for (int st = 0; st < 2; ++st) {
        pb[st].x = pack_bf2(pr[8 * st + 0], pr[8 * st + 1]);
        pb[st].y = pack_bf2(pr[8 * st + 2], pr[8 * st + 3]);
        pb[st].z = pack_bf2(pr[8 * st + 4], pr[8 * st + 5]);
        pb[st].w = pack_bf2(pr[8 * st + 6], pr[8 * st + 7]);
      }
    }
    sum += __shfl_xor(sum, 32, 64);
    l_run = l_run * alpha + sum;
    m_run = m_new;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
      for (int e = 0; e < 16; ++e) o[dt][e] *= alpha;
      // V^T operand: lane (d = 32*dt + n, half kq) takes keys 16*st + 8*kq .. +8 of that d,
      // four at a time with the transposing LDS read: a block of 16 lanes whose lane r
      // points at V[key0 + r/4][d0 + 4*(r%4) ..+4] gets V[key0 .. key0+4][d0 + i] in lane i
      const bf16_t* vr = &v_t[(kq * 8 + ((lane & 15) >> 2)) * VS + dt * 32 + ((lane >> 4) & 1) * 16 +
                              (lane & 3) * 4];
#pragma unroll
      for (int st = 0; st < 2; ++st) {
        const uint2 lo = lds_read_tr16(vr + (st * 16) * VS);
        const uint2 hi = lds_read_tr16(vr + (st * 16 + 4) * VS);
        const uint4 a = make_uint4(lo.x, lo.y, hi.x, hi.y);
        o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                        __builtin_bit_cast(bf16x8_t, pb[st]),
                                                        o[dt], 0, 0, 0);
      }
    }
  }

  if (own_new && wave == 0) {
    // the new token: one more key for every head, from LDS; this lane's half of the dot
    float part = 0.f;
#pragma unroll
    for (int st = 0; st < STEPS; ++st) {
      const uint4 kn4 = *reinterpret_cast<const uint4*>(&kv_new[st * 16 + kq * 8]);
      const uint4 qv = *reinterpret_cast<const uint4*>(qrow_lds + st * 16);
      part = dot2_bf16(qv.x, kn4.x, part);
      part = dot2_bf16(qv.y, kn4.y, part);
      part = dot2_bf16(qv.z, kn4.z, part);
      part = dot2_bf16(qv.w, kn4.w, part);
    }
    const float sv = (part + __shfl_xor(part, 32, 64)) * scale_log2e;
    const float m_new = fmaxf(m_run, sv);
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
    const float pn = __builtin_amdgcn_exp2f(sv - m_new);
    l_run = l_run * alpha + pn;
    m_run = m_new;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int d = dt * 32 + 8 * (r >> 2) + 4 * kq + (r & 3);
        o[dt][r] = o[dt][r] * alpha + pn * bf2f(kv_new[D + d]);
      }
  }

#undef EXO_LOAD_TILE
#undef EXO_LOAD1
#undef EXO_STORE1
  // ---- partial results of the waves, in the scalar kernel's layout: red[wave][head][d],
  // then (max, sum) in natural-log units
  __syncthreads();  // every wave is done with its tiles: the memory changes hands
  float (*red)[G][D + 2] = reinterpret_cast<float (*)[G][D + 2]>(smem);
  if (n < G) {
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        red[wave][n][dt * 32 + 8 * (r >> 2) + 4 * kq + (r & 3)] = o[dt][r];
    if (kq == 0) {
      red[wave][n][D] = m_run * 0.6931471805599453f;
      red[wave][n][D + 1] = l_run;
    }
  }
  __syncthreads();

  const size_t qrow = (size_t)b * p.Hq * D;
  for (int idx = threadIdx.x; idx < G * D; idx += kThreads) {
    const int g = idx / D, e = idx % D;
    float mw = red[0][g][D];
#pragma unroll
    for (int w = 1; w < kWaves; ++w) mw = fmaxf(mw, red[w][g][D]);
    float acc = 0.f, lsum = 0.f;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      const float mm = red[w][g][D];
      const float scw = (mm == -INFINITY) ? 0.f : __expf(mm - mw);
      acc += red[w][g][e] * scw;
      lsum += red[w][g][D + 1] * scw;
    }
#if (EXO_SDPA_ABL & 2)  // timing only: no hand-over, every split writes its own result
    p.out[qrow + (size_t)(h0 + g) * D + e] = f2bf(acc / lsum);
    continue;
#endif
    float* dst = p.ws + ((size_t)(b * p.Hq + h0 + g) * p.splits + blockIdx.x) * (D + 2);
    st_dev(dst + e, acc);
    if (e == 0) {
      st_dev(dst + D, mw);
      st_dev(dst + D + 1, lsum);
    }
  }
#if (EXO_SDPA_ABL & 2)
  return;
#endif
  // the last workgroup of this (sequence, kv head) merges the splits (see sdpa_kernel)
  wait_own_stores_done();
  __syncthreads();
  if (threadIdx.x == 0) {
    int* cnt = &p.counters[b * p.Hkv + blockIdx.y];
    const int old = __hip_atomic_fetch_add(cnt, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    s_last = (old == p.splits - 1);
    if (s_last) __hip_atomic_store(cnt, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __syncthreads();
  if (!s_last) return;
  for (int idx = threadIdx.x; idx < G * D; idx += kThreads) {
    const int g = idx / D, e = idx % D;
    const int h = h0 + g;
    const float* src = p.ws + (size_t)(b * p.Hq + h) * p.splits * (D + 2);
    p.out[qrow + (size_t)h * D + e] = f2bf(merge_splits<D>(src, p.splits, e));
  }
}

// Decode work split.  The G = Hq/Hkv query heads of a kv head are spread over `hgroups`
// workgroups (each re-reads the K/V range from L2, but the per-key arithmetic, the register
// footprint and the in-wave merge of a workgroup shrink with its head count): as many as
// keep (sequences x kv heads x groups) within 64, so that at least 4 key splits remain at
// about 256 workgroups in total.  Batch 1: one head per workgroup, 8 splits (measured on
// Llama-3.1-8B and Qwen3: faster than 2 or 4 heads per workgroup; 128 and 512 workgroups
// slower).  Batch 8 with 8 kv heads: all 4 heads in one workgroup, 4 splits.
int pick_hgroups(int B, int Hq, int Hkv) {
  const int G = Hq / Hkv;
  int h = 1;
  while (h * 2 <= G && G % (h * 2) == 0 && B * Hkv * h * 2 <= 64) h *= 2;
  return h;
}
#ifndef EXO_SDPA_SPLIT_WGS
#define EXO_SDPA_SPLIT_WGS 256
#endif
int pick_splits(int B, int Hq, int Hkv, int S_max) {
  int s = EXO_SDPA_SPLIT_WGS / (B * Hkv * pick_hgroups(B, Hq, Hkv));
  int cap = S_max / 64;
  if (s > cap) s = cap;
  if (s > kMaxSplits) s = kMaxSplits;
  if (s < 1) s = 1;
  return s;
}

template <int D, int MODE>
int launch_sdpa(const SdpaParams& p0, hipStream_t st) {
  SdpaParams p = p0;
  int G = p.Hq / p.Hkv;
  p.hgroups = 1;
  if (MODE != 0) {
    p.hgroups = pick_hgroups(p.B, p.Hq, p.Hkv);
    G /= p.hgroups;
  }
  dim3 grid(MODE != 0 ? p.splits : p.T, p.Hkv * p.hgroups, p.B);
  if (MODE != 0 && EXO_SDPA_TILES) {
    constexpr bool FUSED = MODE == 2;
    exo_note_variant("sdpa_tiles<%d,%d,%s> grid=%dx%dx%d", D, G, FUSED ? "true" : "false", (int)grid.x,
                     (int)grid.y, (int)grid.z);
    switch (G) {
      case 1:
        // few splits (many kv-head groups): eight waves per workgroup halve a wave's tiles
        // (64 query / 4 kv heads at 4100 keys: 13.4 -> 12.4 us; with 8 splits four waves win)
        if (p.splits <= 4 && kTileWaves == 4)
          sdpa_tiles_kernel<D, 1, FUSED, 8><<<grid, 512, 0, st>>>(p);
        else
          sdpa_tiles_kernel<D, 1, FUSED, kTileWaves><<<grid, 64 * kTileWaves, 0, st>>>(p);
        break;
      case 2: sdpa_tiles_kernel<D, 2, FUSED, kTileWaves><<<grid, 64 * kTileWaves, 0, st>>>(p); break;
      case 4: sdpa_tiles_kernel<D, 4, FUSED, kTileWaves><<<grid, 64 * kTileWaves, 0, st>>>(p); break;
      case 8: sdpa_tiles_kernel<D, 8, FUSED, 4><<<grid, 256, 0, st>>>(p); break;
      case 16: sdpa_tiles_kernel<D, 16, FUSED, 4><<<grid, 256, 0, st>>>(p); break;
      default:
        exo_set_error("sdpa: unsupported Hq/Hkv=%d (1,2,4,8,16)", G);
        return EXO_ERR_ARG;
    }
    return EXO_OK;
  }
  exo_note_variant("sdpa_kernel<%d,%d,%d> grid=%dx%dx%d", D, G, MODE, (int)grid.x, (int)grid.y, (int)grid.z);
  switch (G) {
    case 1: sdpa_kernel<D, 1, MODE><<<grid, kThreads, 0, st>>>(p); break;
    case 2: sdpa_kernel<D, 2, MODE><<<grid, kThreads, 0, st>>>(p); break;
    case 4: sdpa_kernel<D, 4, MODE><<<grid, kThreads, 0, st>>>(p); break;
    case 8: sdpa_kernel<D, 8, MODE><<<grid, kThreads, 0, st>>>(p); break;
    case 16: sdpa_kernel<D, 16, MODE><<<grid, kThreads, 0, st>>>(p); break;
    default:
      exo_set_error("sdpa: unsupported Hq/Hkv=%d (1,2,4,8,16)", G);
      return EXO_ERR_ARG;
  }
  return EXO_OK;
}

// chunks of at least this many tokens take the matrix-core kernel; shorter ones the
// one-workgroup-per-token kernel below
constexpr int kMfmaPrefillMinT = 8;

int check(const char* name, int B, int T, int Hq, int Hkv, int D, int S_max) {
  EXO_REQUIRE(B > 0 && T > 0 && Hq > 0 && Hkv > 0 && S_max > 0, "%s: non-positive size", name);
  EXO_REQUIRE(Hq % Hkv == 0, "%s: Hq=%d not a multiple of Hkv=%d", name, Hq, Hkv);
  EXO_REQUIRE(D == 64 || D == 128, "%s: head_dim %d not supported (64, 128)", name, D);
  EXO_REQUIRE(B <= 65535 && Hkv <= 65535, "%s: grid too large", name);
  return EXO_OK;
}

// Workspace: one int counter per (sequence, query head) first, then the partials of
// (query heads x splits): kMaxSplits splits for any launch; a long-context launch has up to
// kMaxSplitsLong splits but at most 256 workgroups of at most 16 heads each.
constexpr int64_t kLongHeadSplits = 256 * 16;
int64_t ws_counter_floats(int B, int Hq) { return ((int64_t)B * Hq + 63) / 64 * 64; }
int64_t ws_head_splits(int B, int Hq) {
  const int64_t heads = (int64_t)B * Hq;
  const int64_t lng = heads * kMaxSplitsLong < kLongHeadSplits ? heads * kMaxSplitsLong : kLongHeadSplits;
  return heads * kMaxSplits > lng ? heads * kMaxSplits : lng;
}

}  // namespace

extern "C" int64_t exo_sdpa_decode_workspace(int B, int Hq, int D) {
  return (ws_counter_floats(B, Hq) + ws_head_splits(B, Hq) * (D + 2)) * (int64_t)sizeof(float);
}

extern "C" int exo_sdpa_decode(const uint16_t* q, const uint16_t* k_cache,
                               const uint16_t* v_cache, const int32_t* pos, uint16_t* out,
                               float* workspace, float scale, int B, int Hq, int Hkv, int D,
                               int S_max, exo_stream_t stream) {
  int rc = check("exo_sdpa_decode", B, 1, Hq, Hkv, D, S_max);
  if (rc) return rc;
  EXO_REQUIRE(q && k_cache && v_cache && pos && out && workspace,
              "exo_sdpa_decode: null pointer");
  SdpaParams p{q, k_cache, v_cache, pos, out, workspace + ws_counter_floats(B, Hq),
               reinterpret_cast<int*>(workspace), scale, B, 1, Hq,
               Hkv, S_max, pick_splits(B, Hq, Hkv, S_max), nullptr, nullptr, nullptr, nullptr, nullptr,
               0.f};
  rc = (D == 64) ? launch_sdpa<64, 1>(p, (hipStream_t)stream)
                 : launch_sdpa<128, 1>(p, (hipStream_t)stream);
  if (rc) return rc;
  EXO_CHECK_LAUNCH("exo_sdpa_decode");
  return EXO_OK;
}

// ---------------------------------------------------------------- no-allocation variant
// exo_sdpa_decode for callers that cannot allocate (code under graph capture, serving
// loops, harnesses that forbid it): the split-KV partials and arrival counters live in a
// file-scope device array instead of a caller workspace.  The array's name is only a
// host-side handle; its device address is looked up once per device and kept.
constexpr int kStaticMaxHeads = EXO_SDPA_DECODE_STATIC_MAX_HEADS;  // B * Hq of one call
constexpr int kStaticMaxD = 128;
constexpr int64_t kStaticFloats =  // the counters, then kMaxSplits partials per head
    (kStaticMaxHeads + 63) / 64 * 64 + (int64_t)kStaticMaxHeads * kMaxSplits * (kStaticMaxD + 2);
static __device__ __align__(256) float scratch[kStaticFloats];

constexpr int kMaxDevices = 64;
static float* g_scratch_ptr[kMaxDevices];  // device address of `scratch`, per device
static std::mutex g_scratch_mutex;

// device address of this device's copy of `scratch` (resolved on first use)
static int scratch_address(float** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    exo_set_error("exo_sdpa_decode_static: cannot identify the current device: %s",
                  e != hipSuccess ? hipGetErrorString(e) : "index out of range");
    return EXO_ERR_HIP;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) {
      exo_set_error("exo_sdpa_decode_static: hipGetSymbolAddress failed on device %d: %s", dev,
                    hipGetErrorString(e));
      return EXO_ERR_HIP;
    }
    g_scratch_ptr[dev] = static_cast<float*>(ptr);
  }
  *out = g_scratch_ptr[dev];
  return EXO_OK;
}

__global__ __launch_bounds__(256) void zero_ints_kernel(int* __restrict__ p, int n) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) p[i] = 0;
}

extern "C" int exo_sdpa_decode_static(const uint16_t* q, const uint16_t* k_cache,
                                      const uint16_t* v_cache, const int32_t* pos,
                                      uint16_t* out, float scale, int B, int Hq, int Hkv, int D,
                                      int S_max, exo_stream_t stream) {
  int rc = check("exo_sdpa_decode_static", B, 1, Hq, Hkv, D, S_max);
  if (rc) return rc;
  EXO_REQUIRE((int64_t)B * Hq <= kStaticMaxHeads,
              "exo_sdpa_decode_static: B*Hq = %lld query heads exceed the static scratch "
              "(at most %d); use exo_sdpa_decode with a workspace",
              (long long)B * Hq, kStaticMaxHeads);
  EXO_REQUIRE(q && k_cache && v_cache && pos && out, "exo_sdpa_decode_static: null pointer");
  float* ws = nullptr;
  rc = scratch_address(&ws);
  if (rc) return rc;
  // The counters of this call's layout reach as far as its head count, where an earlier
  // call with fewer heads may have left partial sums: they are cleared by a small kernel
  // (no memset node, so the call can be captured into a graph).
  const int n_cnt = B * Hq;
  int* cnt = reinterpret_cast<int*>(ws);
  zero_ints_kernel<<<dim3(exo_ceil_div(n_cnt, 256)), 256, 0, (hipStream_t)stream>>>(cnt, n_cnt);
  EXO_CHECK_LAUNCH("exo_sdpa_decode_static");
  return exo_sdpa_decode(q, k_cache, v_cache, pos, out, ws, scale, B, Hq, Hkv, D, S_max, stream);
}

__global__ __launch_bounds__(256) void rope_table_kernel(const float* __restrict__ inv_freq,
                                                         float2* __restrict__ tab, int n,
                                                         int half) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  float sn, cs;
  sincosf((float)(i / half) * inv_freq[i % half], &sn, &cs);
  tab[i] = make_float2(cs, sn);
}

extern "C" int exo_rope_table(const float* inv_freq, float* table, int S_max, int D,
                              exo_stream_t stream) {
  EXO_REQUIRE(inv_freq && table && S_max > 0 && (D == 64 || D == 128),
              "exo_rope_table: bad argument (D must be 64 or 128)");
  const int n = S_max * (D / 2);
  rope_table_kernel<<<dim3(exo_ceil_div(n, 256)), 256, 0, (hipStream_t)stream>>>(
      inv_freq, reinterpret_cast<float2*>(table), n, D / 2);
  EXO_CHECK_LAUNCH("exo_rope_table");
  return EXO_OK;
}

// Contexts the host declares long (keys_hint) take the matrix-core kernel whatever the head
// count.  One sequence of 32 query heads, us per launch, scalar kernel with 8 splits | the
// matrix-core kernel with 16 | 32 | 64 splits per kv head:
//   8 kv heads:   2050 keys 9.3 | 10.6;  8000 keys 17.0 | 15.5 | 17.0 | 23.9;  16000 keys
//                 - | 24.1 | 22.3 | 28.4;  32000 keys 51.1 | 37.3 | 35.8 | 37.6;  130000 keys
//                 178 | 110 | 107 | 111
//   4 kv heads:   2050 keys 9.3 | 12.6;  8000 keys 15.4 | 16.2 | 18.7 | 27.5;  32000 keys
//                 49.2 | 37.0 | 31.1 | 34.7;  130000 keys 172 | 104 | 69 | 72
//   64 query / 4 kv heads: 8000 keys 24.2 | 21.9 | 28.0 | 44.5;  32000 keys 88.6 | 44.5 |
//                 41.5 | 51.8;  130000 keys 328 | 115 | 81 | 88
// (a wave has one tile of 32 keys, 16 KB of K and V, in flight: over tens of thousands of keys
// more workgroups keep the memory busier, until the last workgroup's merge of the splits
// costs more than that returns).  Hence: from kAttnLongKeys keys the matrix-core kernel with
// up to 16 splits, from kAttnVeryLongKeys with up to 32.
constexpr int kAttnLongKeys = EXO_ATTN_LONG_KEYS;
constexpr int kAttnVeryLongKeys = EXO_ATTN_VERY_LONG_KEYS;

extern "C" int exo_attn_decode_hint(const uint16_t* qkv, uint16_t* k_cache, uint16_t* v_cache,
                                    const int32_t* pos, const float* inv_freq,
                                    const float* rope_table, const uint16_t* q_norm_w,
                                    const uint16_t* k_norm_w, float eps, uint16_t* out,
                                    float* workspace, float scale, int B, int Hq, int Hkv, int D,
                                    int S_max, int keys_hint, exo_stream_t stream) {
  int rc = check("exo_attn_decode", B, 1, Hq, Hkv, D, S_max);
  if (rc) return rc;
  EXO_REQUIRE(qkv && k_cache && v_cache && pos && inv_freq && out && workspace,
              "exo_attn_decode: null pointer");
  EXO_REQUIRE(keys_hint >= 0, "exo_attn_decode: keys_hint=%d is negative", keys_hint);
  SdpaParams p{nullptr, k_cache, v_cache, pos, out, workspace + ws_counter_floats(B, Hq),
               reinterpret_cast<int*>(workspace), scale, B, 1, Hq,
               Hkv, S_max, pick_splits(B, Hq, Hkv, S_max), qkv, inv_freq,
               reinterpret_cast<const float2*>(rope_table), q_norm_w, k_norm_w, eps};
  // 128 or more query heads per step (4+ sequences of 32 heads): the scalar kernel is bound
  // by its vector instructions there and the matrix-core kernel is ahead (measured at 2050
  // keys, 32 query / 8 kv heads: 4 sequences 16.9 -> 15.7 us, 8 sequences 24.4 -> 21.0 us; 2
  // sequences level; one sequence with 8 or 16 heads per kv head 8.4 -> 11.8 and 10.5 -> 16.7
  // us, two sequences of 64 query / 4 kv heads 13.7 -> 17.6 us, so those stay with the
  // scalar kernel: it also takes 16 or more (sequence, kv head) pairs to fill the chip with
  // the matrix-core kernel's workgroups; 32 / 4 heads: 4 sequences level, 8 sequences
  // 22.7 -> 18.4 us; 64 / 4 heads: 4 sequences 21.1 -> 19.2, 8 sequences 34.2 -> 23.5 us)
  const int G = Hq / Hkv;
  // (two sequences of 32 / 8 heads - 16 (sequence, kv head) pairs, enough workgroups for the
  // matrix-core kernel - are level at 2050 keys and ahead beyond: 3000 keys 15.5 -> 14.2 us,
  // 4096 keys 18.9 -> 16.1, 6144 keys 25.5 -> 19.4)
  const int long_keys = B * Hkv >= 16 ? EXO_ATTN_MID_KEYS : kAttnLongKeys;
  const bool long_ctx = keys_hint >= long_keys && S_max >= long_keys;
  if (D == 128 && (G == 4 || G == 8 || G == 16) &&
      ((B * Hq >= 128 && B * Hkv >= 16) || long_ctx)) {
    const int max_sp = keys_hint >= kAttnVeryLongKeys && S_max >= kAttnVeryLongKeys ? kMaxSplitsLong : kMaxSplits;
    int sp = 256 / (B * Hkv);
    sp = sp > max_sp ? max_sp : (sp < 1 ? 1 : sp);
    if (sp > S_max / 128) sp = S_max / 128 > 0 ? S_max / 128 : 1;
    p.splits = sp;
    p.hgroups = 1;
    const dim3 grid(p.splits, Hkv, B);
    exo_note_variant("sdpa_decode_mfma<%d> grid=%dx%dx%d", G, (int)grid.x, (int)grid.y, (int)grid.z);
    if (G == 4)
      sdpa_decode_mfma_kernel<4><<<grid, kThreads, 0, (hipStream_t)stream>>>(p);
    else if (G == 8)
      sdpa_decode_mfma_kernel<8><<<grid, kThreads, 0, (hipStream_t)stream>>>(p);
    else
      sdpa_decode_mfma_kernel<16><<<grid, kThreads, 0, (hipStream_t)stream>>>(p);
    EXO_CHECK_LAUNCH("exo_attn_decode");
    return EXO_OK;
  }
  rc = (D == 64) ? launch_sdpa<64, 2>(p, (hipStream_t)stream)
                 : launch_sdpa<128, 2>(p, (hipStream_t)stream);
  if (rc) return rc;
  EXO_CHECK_LAUNCH("exo_attn_decode");
  return EXO_OK;
}

extern "C" int exo_attn_decode(const uint16_t* qkv, uint16_t* k_cache, uint16_t* v_cache,
                               const int32_t* pos, const float* inv_freq, const float* rope_table,
                               const uint16_t* q_norm_w, const uint16_t* k_norm_w, float eps,
                               uint16_t* out, float* workspace, float scale, int B, int Hq,
                               int Hkv, int D, int S_max, exo_stream_t stream) {
  return exo_attn_decode_hint(qkv, k_cache, v_cache, pos, inv_freq, rope_table, q_norm_w, k_norm_w,
                              eps, out, workspace, scale, B, Hq, Hkv, D, S_max, 0, stream);
}

extern "C" int exo_sdpa_prefill(const uint16_t* q, const uint16_t* k_cache,
                                const uint16_t* v_cache, const int32_t* pos, uint16_t* out,
                                float scale, int B, int T, int Hq, int Hkv, int D, int S_max,
                                exo_stream_t stream) {
  int rc = check("exo_sdpa_prefill", B, T, Hq, Hkv, D, S_max);
  if (rc) return rc;
  EXO_REQUIRE(q && k_cache && v_cache && pos && out, "exo_sdpa_prefill: null pointer");
  if (T >= kMfmaPrefillMinT) {
    rc = exo_sdpa_prefill_mfma(q, k_cache, v_cache, pos, out, scale, B, T, Hq, Hkv, D, S_max,
                               (hipStream_t)stream);
    if (rc) return rc;
    EXO_CHECK_LAUNCH("exo_sdpa_prefill");
    return EXO_OK;
  }
  SdpaParams p{q, k_cache, v_cache, pos, out, nullptr, nullptr, scale, B, T, Hq, Hkv, S_max, 1,
               nullptr, nullptr, nullptr, nullptr, nullptr, 0.f};
  rc = (D == 64) ? launch_sdpa<64, 0>(p, (hipStream_t)stream)
                 : launch_sdpa<128, 0>(p, (hipStream_t)stream);
  if (rc) return rc;
  EXO_CHECK_LAUNCH("exo_sdpa_prefill");
  return EXO_OK;
}
