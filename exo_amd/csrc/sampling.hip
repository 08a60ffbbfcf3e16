// The sampling step of decode on the device: logits processors (token bans, repetition /
// presence / frequency penalties), log-normaliser, temperature / top-p / min-p / top-k
// filtering, a seeded draw, and the 20 most likely tokens with their log-probabilities -
// everything `_patched_step` of the reference does between the model call and the next
// token (src/exo/worker/engines/mlx/patches/opt_batch_gen.py:67-107), as a fixed sequence
// of launches that can sit at the end of a captured decode graph.
//
// The row of logits ([V] bf16, 250-300 KB, L2 resident: the lm_head GEMV has just written
// it) is cut into 64 slices, one workgroup each; every pass streams it once:
//   edits    one workgroup per row lists the few tokens the processors touch (banned ids
//            and the tokens of the penalty contexts, <= 264) with their edited values; the
//            streaming passes patch those positions through a slice bitmap, so the logits
//            themselves are never rewritten;
//   stats    per slice (max, argmax, sum exp(x - max));
//   coarse   (only with top-p / top-k / top-logprobs) every value is a bf16, i.e. a 16-bit
//   fine     order-preserving key.  Count and probability mass (2^-40 fixed point: integer sums
//            are exact, so nothing depends on arrival order) are first accumulated per BUCKET
//            of 128 keys (sign and exponent: 512 buckets) - in LDS per slice, then the few
//            non-empty buckets with global atomics.  A scan of the 512 buckets from the top
//            finds the bucket in which the running count reaches k (and 20), and the one in
//            which the running mass reaches top_p; a second pass histograms only the values of
//            those buckets by their low 7 key bits, and a scan of those 128 entries, continued
//            from the totals above the bucket, gives the exact keys: the k-th largest value,
//            the nucleus edge, the 20th largest value.  (A flat 65536-entry table took 85 us to
//            fill with 2 atomics per logit and 115 us to scan and clear; the two levels take a few
//            microseconds each.)
//   weights  per slice the sum of exp((x - max) / T) over the kept tokens (x >= threshold);
//            tokens at or above the 20th largest key are appended to a candidate list;
//   select   one workgroup per row: uniform from Philox-4x32-10 (key = request seed,
//            counter = draws so far), the slice in which the running sum crosses u * total,
//            then the token inside it (inverse CDF in vocabulary order); ranks the
//            candidates; appends the token to the history ring; advances the cache position.
// All filters compose to one value threshold: token i is kept iff x_i >= max(t_top_p,
// t_min_p, t_top_k).
#include "../../include/exo_mi355x.h"
#include "common.h"

namespace {

constexpr int kBlocks = 64;      // slices per row
constexpr int kMaxSlice = 4096;  // elements per slice (two 8-element chunks per thread)
constexpr int kMaxEdits = EXO_SAMPLER_MAX_CONTEXT + EXO_SAMPLER_MAX_BANNED;
constexpr int kTop = EXO_SAMPLER_TOP_LOGPROBS;
constexpr int kMaxCand = 32;    // values strictly above the 20th largest: 19 at most
constexpr int kBuckets = 512;  // key >> 7: sign and exponent
constexpr int kFine = 128;     // key & 127: mantissa, in value order inside a bucket
constexpr int kTargets = 3;    // 0: k-th largest (top-k), 1: nucleus edge (top-p), 2: 20th largest
constexpr float kBan = -1e9f;

struct RowWs {
  float part[kBlocks][4];  // max, argmax (int bits), sum exp(x - max), kept weight
  int n_edit;
  float thr;    // value threshold from top-p / top-k (-inf: none)
  int key_top;  // key of the 20th largest value
  int cand_n;
  // per target: the bucket in which the running count / mass from the top crosses it (-1:
  // never), and the count and mass of the buckets above it
  int bkt[kTargets];
  unsigned int above_c[kTargets];
  unsigned long long above_m[kTargets];
  int edit_idx[kMaxEdits];
  float edit_val[kMaxEdits];
  unsigned long long cand[kMaxCand];  // key << 32 | index, values strictly above the 20th largest
  // tokens whose value EQUALS the 20th largest, per slice: the first kTop of them in
  // vocabulary order (a flat row has thousands; which of them make the list must not depend
  // on the order in which workgroups arrive)
  int tie_n[kBlocks];
  int tie_idx[kBlocks][kTop];
};
constexpr size_t kRowWsBytes = (sizeof(RowWs) + 255) / 256 * 256;

// mass and count per bucket, and per low key of each target's bucket; zero between steps
struct Tables {
  unsigned long long cm[kBuckets];
  unsigned long long fm[kTargets][kFine];
  unsigned int cc[kBuckets];
  unsigned int fc[kTargets][kFine];
};
constexpr size_t kTablesBytes = (sizeof(Tables) + 255) / 256 * 256;

// Workspace: one self-contained region per row (the row's RowWs, then its tables), so
// launches of different row counts can share one workspace.
constexpr size_t kRowStride = kRowWsBytes + kTablesBytes;
__device__ __forceinline__ RowWs* row_ws(void* ws, int row) {
  return reinterpret_cast<RowWs*>(static_cast<char*>(ws) + (size_t)row * kRowStride);
}
__device__ __forceinline__ Tables* row_tables(void* ws, int row) {
  return reinterpret_cast<Tables*>(static_cast<char*>(ws) + (size_t)row * kRowStride + kRowWsBytes);
}

// order-preserving 16-bit key of a bf16 value and back
__device__ __forceinline__ int key_of(float x) {
  const uint32_t b = __builtin_bit_cast(uint32_t, x) >> 16;
  return (b & 0x8000u) ? (~b & 0xffffu) : (b | 0x8000u);
}
__device__ __forceinline__ float value_of(int key) {
  const uint32_t b = (key & 0x8000) ? (key & 0x7fff) : (~key & 0xffff);
  return __builtin_bit_cast(float, b << 16);
}
__device__ __forceinline__ float bf16r(float v) { return bf2f(f2bf(v)); }

// ---- slices -------------------------------------------------------------------
struct SliceGeom {
  int per, lo, hi;
  bool vec;
};
__device__ __forceinline__ SliceGeom slice_geom(const bf16_t* logits, int V, int block) {
  SliceGeom g;
  g.vec = (V & 7) == 0 && ((uintptr_t)logits & 15) == 0;
  g.per = ((((V + 7) >> 3) + kBlocks - 1) / kBlocks) << 3;
  g.lo = min(block * g.per, V);
  g.hi = min(g.lo + g.per, V);
  return g;
}

// The slice's edited positions as a bitmap in LDS and the edit list next to it.
struct EditLds {
  uint32_t bm[kMaxSlice / 32];
  int idx[kMaxEdits];
  float val[kMaxEdits];
  int n;
};
__device__ __forceinline__ void stage_edits(const RowWs* w, const SliceGeom& g, EditLds& e) {
  const int n = w->n_edit;
  if (threadIdx.x == 0) e.n = n;
  if (n > 0) {
    for (int i = threadIdx.x; i < kMaxSlice / 32; i += blockDim.x) e.bm[i] = 0;
    __syncthreads();
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
      const int t = w->edit_idx[i];
      e.idx[i] = t;
      e.val[i] = w->edit_val[i];
      if (t >= g.lo && t < g.hi) atomicOr(&e.bm[(t - g.lo) >> 5], 1u << ((t - g.lo) & 31));
    }
  }
  __syncthreads();
}
__device__ __forceinline__ float edited_value(const EditLds& e, int index, float x) {
  for (int i = 0; i < e.n; ++i)
    if (e.idx[i] == index) return e.val[i];
  return x;
}

// This thread's share of the slice: chunk u (0, 1) holds the 8 elements from index
// i0[u]; positions outside the slice read -inf.  Edits are applied.
__device__ __forceinline__ void load_share(const bf16_t* src, const SliceGeom& g, const EditLds& e,
                                           float (&xv)[16], int (&i0)[2]) {
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    i0[u] = g.lo + ((int)threadIdx.x + 256 * u) * 8;
    if (g.vec) {
      uint4 v = make_uint4(0xff80ff80u, 0xff80ff80u, 0xff80ff80u, 0xff80ff80u);  // -inf
      if (i0[u] < g.hi) v = *reinterpret_cast<const uint4*>(src + i0[u]);
      const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        xv[8 * u + 2 * k] = bf_lo(w[k]);
        xv[8 * u + 2 * k + 1] = bf_hi(w[k]);
      }
    } else {
#pragma unroll
      for (int k = 0; k < 8; ++k)
        xv[8 * u + k] = (i0[u] + k < g.hi) ? bf2f(src[i0[u] + k]) : -INFINITY;
    }
    if (e.n > 0 && i0[u] < g.hi) {
      const int o = i0[u] - g.lo;  // multiple of 8: the chunk's bits sit in one byte
      const uint32_t bits = (e.bm[o >> 5] >> (o & 31)) & 0xffu;
      if (bits) {
#pragma unroll
        for (int k = 0; k < 8; ++k)
          if (bits & (1u << k)) xv[8 * u + k] = edited_value(e, i0[u] + k, xv[8 * u + k]);
      }
    }
  }
}

// (max, lowest index holding it, sum exp(x - max)) over the row from the slice partials;
// every wave computes it for itself (64 partials = one per lane).
__device__ __forceinline__ void merge_stats(const RowWs* w, float& mx, int& mi, float& lse) {
  const int lane = threadIdx.x & 63;
  const float bm = w->part[lane][0], bs = w->part[lane][2];
  mx = bm;
  mi = __float_as_int(w->part[lane][1]);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(mx, o, 64);
    const int oi = __shfl_xor(mi, o, 64);
    if (ov > mx || (ov == mx && oi < mi)) {
      mx = ov;
      mi = oi;
    }
  }
  float se = (bm > -INFINITY) ? bs * expf(bm - mx) : 0.f;
  se = wave_sum(se);
  lse = mx + logf(se);
}

// ---- edits --------------------------------------------------------------------
__global__ __launch_bounds__(512) void sampler_edits_kernel(
    const bf16_t* __restrict__ logits, const exo_sampler_params* __restrict__ params,
    const int32_t* __restrict__ history, const int32_t* __restrict__ hist_len, void* ws, int V,
    int hist_cap) {
  __shared__ int s_tok[kMaxEdits];
  __shared__ int s_n;
  const int row = blockIdx.x, c = threadIdx.x;
  const exo_sampler_params p = params[row];
  RowWs* w = row_ws(ws, row);
  const bool rep_on = p.repetition_penalty != 0.f && p.repetition_penalty != 1.f;
  const bool pres_on = p.presence_penalty != 0.f;
  const bool freq_on = p.frequency_penalty != 0.f;
  const int len = hist_len[row];
  const int n_hist = min(len, hist_cap);
  const int rep_ctx = rep_on ? min(max(p.repetition_context, 0), n_hist) : 0;
  const int pres_ctx = pres_on ? min(max(p.presence_context, 0), n_hist) : 0;
  const int freq_ctx = freq_on ? min(max(p.frequency_context, 0), n_hist) : 0;
  const int max_ctx = max(rep_ctx, max(pres_ctx, freq_ctx));
  const int nb = min(max(p.n_banned, 0), EXO_SAMPLER_MAX_BANNED);
  const int32_t* hrow = history + (size_t)row * hist_cap;
  // candidate c: banned id c, or the token j = c - MAX_BANNED positions back in the history
  int tok = -1;
  if (c < nb) {
    tok = p.banned[c];
  } else if (c >= EXO_SAMPLER_MAX_BANNED && c - EXO_SAMPLER_MAX_BANNED < max_ctx) {
    const int j = c - EXO_SAMPLER_MAX_BANNED;
    tok = hrow[(len - 1 - j) % hist_cap];
  }
  if (tok >= V) tok = -1;
  if (c < kMaxEdits) s_tok[c] = tok;
  if (c == 0) s_n = 0;
  __syncthreads();
  if (c < kMaxEdits && tok >= 0) {
    bool first = true;
    for (int o = 0; o < c; ++o) first = first && (s_tok[o] != tok);
    if (first) {
      bool banned = false;
      for (int o = 0; o < nb; ++o) banned = banned || (s_tok[o] == tok);
      bool in_rep = false, in_pres = false;
      int cf = 0;
      for (int j = 0; j < max_ctx; ++j) {
        const bool hit = s_tok[EXO_SAMPLER_MAX_BANNED + j] == tok;
        in_rep = in_rep || (hit && j < rep_ctx);
        in_pres = in_pres || (hit && j < pres_ctx);
        cf += (hit && j < freq_ctx) ? 1 : 0;
      }
      float v = bf2f(logits[(size_t)row * V + tok]);
      if (banned) v = bf16r(kBan);
      if (in_rep) v = bf16r(v < 0.f ? __fmul_rn(v, p.repetition_penalty) : __fdiv_rn(v, p.repetition_penalty));
      if (in_pres) v = bf16r(__fsub_rn(v, p.presence_penalty));
      if (cf > 0) v = bf16r(__fsub_rn(v, __fmul_rn(p.frequency_penalty, (float)cf)));
      const int slot = atomicAdd(&s_n, 1);
      w->edit_idx[slot] = tok;
      w->edit_val[slot] = v;
    }
  }
  __syncthreads();
  if (c == 0) w->n_edit = s_n;
}

// ---- stats --------------------------------------------------------------------
__global__ __launch_bounds__(256) void sample_stats_kernel(const bf16_t* __restrict__ logits,
                                                           void* ws, int V, int has_edits) {
  __shared__ EditLds ed;
  __shared__ float smax[4], ssum[4];
  __shared__ int sidx[4];
  const int row = blockIdx.y;
  RowWs* w = row_ws(ws, row);
  if (blockIdx.x == 0 && threadIdx.x == 0) {  // per-step fields of the row
    w->thr = -INFINITY;
    w->key_top = 0;
    w->cand_n = 0;
    if (!has_edits) w->n_edit = 0;
  }
  if (!has_edits && threadIdx.x == 0) ed.n = 0;
  const SliceGeom g = slice_geom(logits, V, blockIdx.x);
  if (has_edits)
    stage_edits(w, g, ed);
  else
    __syncthreads();
  float xv[16];
  int i0[2];
  load_share(logits + (size_t)row * V, g, ed, xv, i0);
  float mx = -INFINITY;
  int mi = 0x7fffffff;
#pragma unroll
  for (int u = 0; u < 2; ++u)
#pragma unroll
    for (int k = 0; k < 8; ++k)
      if (xv[8 * u + k] > mx) {
        mx = xv[8 * u + k];
        mi = i0[u] + k;
      }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(mx, o, 64);
    const int oi = __shfl_xor(mi, o, 64);
    if (ov > mx || (ov == mx && oi < mi)) {
      mx = ov;
      mi = oi;
    }
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) {
    smax[wave] = mx;
    sidx[wave] = mi;
  }
  __syncthreads();
  float bm = smax[0];
  int bi = sidx[0];
#pragma unroll
  for (int wv = 1; wv < 4; ++wv)
    if (smax[wv] > bm || (smax[wv] == bm && sidx[wv] < bi)) {
      bm = smax[wv];
      bi = sidx[wv];
    }
  float se = 0.f;
  if (bm > -INFINITY) {
#pragma unroll
    for (int k = 0; k < 16; ++k) se += expf(xv[k] - bm);  // padding is -inf: exp = 0
  }
  se = wave_sum(se);
  if (lane == 0) ssum[wave] = se;
  __syncthreads();
  if (threadIdx.x == 0) {
    w->part[blockIdx.x][0] = bm;
    w->part[blockIdx.x][1] = __int_as_float(bi);
    w->part[blockIdx.x][2] = ssum[0] + ssum[1] + ssum[2] + ssum[3];
    w->part[blockIdx.x][3] = 0.f;
  }
}

// ---- key table ----------------------------------------------------------------
constexpr double kMassOne = 1099511627776.0;  // 2^40

__device__ __forceinline__ bool row_needs_table(const exo_sampler_params& p, bool want_top) {
  const bool sampling = p.temperature != 0.f;
  return want_top || (sampling && (p.top_k > 0 || (p.top_p > 0.f && p.top_p < 1.f)));
}

// what a row asks of the tables
struct Wanted {
  unsigned int kk;             // top-k (0: none)
  bool use_p;                  // top-p
  unsigned long long target;   // top_p of the mass, fixed point
  bool top;                    // the 20 most likely
};
__device__ __forceinline__ Wanted wanted_of(const exo_sampler_params& p, bool want_top) {
  const bool sampling = p.temperature != 0.f;
  Wanted q;
  q.kk = (sampling && p.top_k > 0) ? (unsigned int)p.top_k : 0u;
  q.use_p = sampling && p.top_p > 0.f && p.top_p < 1.f;
  q.target = q.use_p ? (unsigned long long)((double)p.top_p * kMassOne) : 0ull;
  q.top = want_top;
  return q;
}

__device__ __forceinline__ unsigned long long shfl_up_u64(unsigned long long v, int o) {
  const unsigned int lo = __shfl_up((unsigned int)v, o, 64), hi = __shfl_up((unsigned int)(v >> 32), o, 64);
  return ((unsigned long long)hi << 32) | lo;
}
__device__ __forceinline__ unsigned long long shfl_u64(unsigned long long v, int src) {
  const unsigned int lo = __shfl((unsigned int)v, src, 64), hi = __shfl((unsigned int)(v >> 32), src, 64);
  return ((unsigned long long)hi << 32) | lo;
}

// One wave walks N = 64 * PER entries from the highest index down (lane t owns entries
// N-1 - PER*t .. downwards), the running (count, mass) starting at (c0, m0).  For each target:
// the entry at which the running count reaches kk / 20 (count before it below, count with it
// at or above), or the running mass reaches `target`; found[] = entry index or -1, and
// (fc, fm) = the totals strictly above that entry.  Every lane returns the same values.
template <int PER>
__device__ __forceinline__ void scan_down(const unsigned long long* __restrict__ mt,
                                          const unsigned int* __restrict__ ct, const Wanted& q,
                                          const unsigned int (&c0)[kTargets],
                                          const unsigned long long (&m0)[kTargets],
                                          const bool (&active)[kTargets], int (&found)[kTargets],
                                          unsigned int (&fc)[kTargets],
                                          unsigned long long (&fm)[kTargets]) {
  const int lane = threadIdx.x & 63;
  const int hi = 64 * PER - 1 - PER * lane;
  unsigned long long m[PER], msum = 0;
  unsigned int c[PER], csum = 0;
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    m[i] = mt[hi - i];
    c[i] = ct[hi - i];
    msum += m[i];
    csum += c[i];
  }
  unsigned long long minc = msum;
  unsigned int cinc = csum;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const unsigned long long mu = shfl_up_u64(minc, o);
    const unsigned int cu = __shfl_up(cinc, o, 64);
    if (lane >= o) {
      minc += mu;
      cinc += cu;
    }
  }
  const unsigned long long mex = minc - msum;  // totals of the lanes above (higher entries)
  const unsigned int cex = cinc - csum;
#pragma unroll
  for (int j = 0; j < kTargets; ++j) {
    int f = -1;
    unsigned int fcj = 0;
    unsigned long long fmj = 0;
    if (active[j]) {
      unsigned long long ma = m0[j] + mex;
      unsigned int ca = c0[j] + cex;
      const unsigned int want_c = j == 0 ? q.kk : (unsigned int)kTop;
#pragma unroll
      for (int i = 0; i < PER; ++i) {
        if (c[i]) {
          const bool hit = (j == 1) ? (ma < q.target && ma + m[i] >= q.target)
                                    : (ca < want_c && ca + c[i] >= want_c);
          if (hit) {
            f = hi - i;
            fcj = ca;
            fmj = ma;
          }
        }
        ma += m[i];
        ca += c[i];
      }
    }
    const unsigned long long mask = __ballot(f >= 0);
    if (mask) {
      const int src = __ffsll((long long)mask) - 1;
      found[j] = __shfl(f, src, 64);
      fc[j] = __shfl(fcj, src, 64);
      fm[j] = shfl_u64(fmj, src);
    } else {
      found[j] = -1;
      fc[j] = 0;
      fm[j] = 0;
    }
  }
}

// ---- coarse: count and mass per bucket ------------------------------------------------
__global__ __launch_bounds__(256) void sample_coarse_kernel(
    const bf16_t* __restrict__ logits, const exo_sampler_params* __restrict__ params, void* ws,
    int V, int want_top) {
  __shared__ EditLds ed;
  __shared__ unsigned long long hm[kBuckets];
  __shared__ unsigned int hc[kBuckets];
  const int row = blockIdx.y;
  if (!row_needs_table(params[row], want_top != 0)) return;
  RowWs* w = row_ws(ws, row);
  const SliceGeom g = slice_geom(logits, V, blockIdx.x);
  for (int b = threadIdx.x; b < kBuckets; b += 256) {
    hm[b] = 0;
    hc[b] = 0;
  }
  stage_edits(w, g, ed);  // (ends in a barrier)
  float mx, lse;
  int mi;
  merge_stats(w, mx, mi, lse);
  float xv[16];
  int i0[2];
  load_share(logits + (size_t)row * V, g, ed, xv, i0);
#pragma unroll
  for (int u = 0; u < 2; ++u)
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const float x = xv[8 * u + k];
      if (i0[u] + k < g.hi) {  // -inf logits are real values too (key 0x007f)
        const int b = key_of(x) >> 7;
        atomicAdd(&hc[b], 1u);
        const unsigned long long q = (unsigned long long)((double)expf(x - lse) * kMassOne);
        if (q) atomicAdd(&hm[b], q);
      }
    }
  __syncthreads();
  Tables* T = row_tables(ws, row);
  for (int b = threadIdx.x; b < kBuckets; b += 256) {
    if (hc[b]) atomicAdd(&T->cc[b], hc[b]);
    if (hm[b]) atomicAdd(&T->cm[b], hm[b]);
  }
}

// ---- fine: the buckets that hold a target, by their low key bits ----------------------
__global__ __launch_bounds__(256) void sample_fine_kernel(
    const bf16_t* __restrict__ logits, const exo_sampler_params* __restrict__ params, void* ws,
    int V, int want_top) {
  __shared__ EditLds ed;
  __shared__ unsigned long long hm[kTargets][kFine];
  __shared__ unsigned int hc[kTargets][kFine];
  const int row = blockIdx.y;
  const exo_sampler_params p = params[row];
  if (!row_needs_table(p, want_top != 0)) return;
  RowWs* w = row_ws(ws, row);
  Tables* T = row_tables(ws, row);
  const Wanted q = wanted_of(p, want_top != 0);
  // every wave finds the target buckets for itself (512 entries, L2 resident)
  int bkt[kTargets];
  unsigned int ac[kTargets];
  unsigned long long am[kTargets];
  {
    const unsigned int c0[kTargets] = {0u, 0u, 0u};
    const unsigned long long m0[kTargets] = {0ull, 0ull, 0ull};
    const bool active[kTargets] = {q.kk != 0, q.use_p, q.top};
    scan_down<kBuckets / 64>(T->cm, T->cc, q, c0, m0, active, bkt, ac, am);
  }
  if (blockIdx.x == 0 && threadIdx.x == 0) {
#pragma unroll
    for (int j = 0; j < kTargets; ++j) {
      w->bkt[j] = bkt[j];
      w->above_c[j] = ac[j];
      w->above_m[j] = am[j];
    }
  }
  if (bkt[0] < 0 && bkt[1] < 0 && bkt[2] < 0) return;  // (uniform over the workgroup)
  const SliceGeom g = slice_geom(logits, V, blockIdx.x);
  for (int i = threadIdx.x; i < kTargets * kFine; i += 256) {
    (&hm[0][0])[i] = 0;
    (&hc[0][0])[i] = 0;
  }
  stage_edits(w, g, ed);
  float mx, lse;
  int mi;
  merge_stats(w, mx, mi, lse);
  float xv[16];
  int i0[2];
  load_share(logits + (size_t)row * V, g, ed, xv, i0);
#pragma unroll
  for (int u = 0; u < 2; ++u)
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const float x = xv[8 * u + k];
      if (i0[u] + k < g.hi) {
        const int key = key_of(x), b = key >> 7, f = key & (kFine - 1);
        if (b == bkt[0] || b == bkt[1] || b == bkt[2]) {
          const unsigned long long qm = (unsigned long long)((double)expf(x - lse) * kMassOne);
#pragma unroll
          for (int j = 0; j < kTargets; ++j)
            if (b == bkt[j]) {
              atomicAdd(&hc[j][f], 1u);
              if (qm) atomicAdd(&hm[j][f], qm);
            }
        }
      }
    }
  __syncthreads();
  for (int i = threadIdx.x; i < kTargets * kFine; i += 256) {
    const unsigned int c = (&hc[0][0])[i];
    const unsigned long long m = (&hm[0][0])[i];
    if (c) atomicAdd(&T->fc[0][0] + i, c);
    if (m) atomicAdd(&T->fm[0][0] + i, m);
  }
}

// The exact keys from the fine tables (one wave; the same values in every lane): the value
// threshold of top-k / top-p (-inf: none) and the key of the 20th largest value (0: none).
__device__ __forceinline__ void fine_thresholds(const RowWs* w, const Tables* T, const Wanted& q,
                                                float& thr, int& key_top) {
  thr = -INFINITY;
  key_top = 0;
#pragma unroll
  for (int j = 0; j < kTargets; ++j) {
    const int b = w->bkt[j];
    if (b < 0) continue;  // fewer than k (20) tokens in all, or the mass never reaches top_p
    const unsigned int c0[kTargets] = {w->above_c[j], w->above_c[j], w->above_c[j]};
    const unsigned long long m0[kTargets] = {w->above_m[j], w->above_m[j], w->above_m[j]};
    const bool active[kTargets] = {j == 0, j == 1, j == 2};
    int f[kTargets];
    unsigned int fc[kTargets];
    unsigned long long fm[kTargets];
    scan_down<kFine / 64>(T->fm[j], T->fc[j], q, c0, m0, active, f, fc, fm);
    if (f[j] >= 0) {
      const int key = (b << 7) | f[j];
      if (j == 2)
        key_top = key;
      else
        thr = fmaxf(thr, value_of(key));
    }
  }
}

// ---- weights ------------------------------------------------------------------
__device__ __forceinline__ float keep_threshold(const exo_sampler_params& p, float table_thr,
                                                float mx) {
  float thr = table_thr;
  if (p.min_p > 0.f) thr = fmaxf(thr, mx + logf(p.min_p));
  return thr;
}

__global__ __launch_bounds__(256) void sample_weights_kernel(
    const bf16_t* __restrict__ logits, const exo_sampler_params* __restrict__ params, void* ws,
    int V, int want_top) {
  __shared__ EditLds ed;
  __shared__ float ssum[4];
  const int row = blockIdx.y;
  const exo_sampler_params p = params[row];
  const bool sampling = p.temperature != 0.f;
  if (!sampling && !want_top) return;
  RowWs* w = row_ws(ws, row);
  // the exact keys of this step from the fine tables (every wave for itself); the first
  // workgroup leaves them for the select launch and clears the bucket table, whose last
  // reader was the previous launch
  float table_thr = -INFINITY;
  int kt = 0;
  if (row_needs_table(p, want_top != 0)) {
    Tables* T = row_tables(ws, row);
    fine_thresholds(w, T, wanted_of(p, want_top != 0), table_thr, kt);
    if (blockIdx.x == 0) {
      if (threadIdx.x == 0) {
        w->thr = table_thr;
        w->key_top = kt;
      }
      for (int b = threadIdx.x; b < kBuckets; b += 256) {
        T->cm[b] = 0;
        T->cc[b] = 0;
      }
    }
  }
  const SliceGeom g = slice_geom(logits, V, blockIdx.x);
  stage_edits(w, g, ed);
  float mx, lse;
  int mi;
  merge_stats(w, mx, mi, lse);
  float xv[16];
  int i0[2];
  load_share(logits + (size_t)row * V, g, ed, xv, i0);
  if (want_top) {
    // strictly above the 20th largest value: at most 19 tokens in the whole row, any order
    // (the select launch ranks them); equal to it: this slice's first kTop in vocabulary
    // order, by a scan over the threads (chunk 0 of every thread precedes chunk 1 of any)
    __shared__ int s_tiew[4];
    int base = 0;
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      int mine = 0;
#pragma unroll
      for (int k = 0; k < 8; ++k)
        if (i0[u] + k < g.hi) {
          const int key = key_of(xv[8 * u + k]);
          if (key > kt) {
            const int slot = atomicAdd(&w->cand_n, 1);
            if (slot < kMaxCand)
              w->cand[slot] = ((unsigned long long)key << 32) | (unsigned int)(i0[u] + k);
          } else if (key == kt) {
            ++mine;
          }
        }
      int inc = mine;
      const int ln = threadIdx.x & 63, wv = threadIdx.x >> 6;
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        const int up = __shfl_up(inc, o, 64);
        if (ln >= o) inc += up;
      }
      if (ln == 63) s_tiew[wv] = inc;
      __syncthreads();
      int before = base;
      for (int q = 0; q < wv; ++q) before += s_tiew[q];
      const int round_total = s_tiew[0] + s_tiew[1] + s_tiew[2] + s_tiew[3];
      int at = before + inc - mine;  // ties of this slice in front of this thread's chunk
      if (mine > 0 && at < kTop) {
#pragma unroll
        for (int k = 0; k < 8; ++k)
          if (i0[u] + k < g.hi && key_of(xv[8 * u + k]) == kt) {
            if (at < kTop) w->tie_idx[blockIdx.x][at] = i0[u] + k;
            ++at;
          }
      }
      __syncthreads();
      base += round_total;
    }
    if (threadIdx.x == 0) w->tie_n[blockIdx.x] = min(base, kTop);
  }
  if (!sampling) return;
  const float thr = keep_threshold(p, table_thr, mx);
  const float inv_t = 1.f / p.temperature;
  float s = 0.f;
#pragma unroll
  for (int k = 0; k < 16; ++k)
    if (xv[k] >= thr) s += expf((xv[k] - mx) * inv_t);
  s = wave_sum(s);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) ssum[wave] = s;
  __syncthreads();
  if (threadIdx.x == 0) w->part[blockIdx.x][3] = ssum[0] + ssum[1] + ssum[2] + ssum[3];
}

// ---- select -------------------------------------------------------------------
__device__ __forceinline__ void philox4x32_10(uint32_t (&c)[4], uint32_t k0, uint32_t k1) {
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    const unsigned long long p0 = 0xD2511F53ull * c[0], p1 = 0xCD9E8D57ull * c[2];
    const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c[1] ^ k0, n1 = (uint32_t)p1;
    const uint32_t n2 = (uint32_t)(p0 >> 32) ^ c[3] ^ k1, n3 = (uint32_t)p0;
    c[0] = n0;
    c[1] = n1;
    c[2] = n2;
    c[3] = n3;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
}

__global__ __launch_bounds__(256) void sample_select_kernel(
    const bf16_t* __restrict__ logits, const exo_sampler_params* __restrict__ params,
    int32_t* __restrict__ history, int32_t* __restrict__ hist_len, uint32_t* __restrict__ draws,
    int32_t* __restrict__ token, float* __restrict__ logprob, float* __restrict__ lse_out,
    int32_t* __restrict__ top_idx, float* __restrict__ top_val, int32_t* __restrict__ feedback,
    int32_t* __restrict__ pos_inc, void* ws, int V, int hist_cap, int want_top) {
  __shared__ EditLds ed;
  __shared__ float s_wsum[4], s_rem;
  __shared__ int s_block, s_tok, s_last_kept;
  __shared__ float s_x;
  const int row = blockIdx.x, tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const exo_sampler_params p = params[row];
  RowWs* w = row_ws(ws, row);
  if (row_needs_table(p, want_top != 0)) {  // the weights launch was the fine tables' last reader
    Tables* T = row_tables(ws, row);
    for (int i = tid; i < kTargets * kFine; i += 256) {
      (&T->fm[0][0])[i] = 0;
      (&T->fc[0][0])[i] = 0;
    }
  }
  float mx, lse;
  int mi;
  merge_stats(w, mx, mi, lse);
  int tok = mi;
  float x_tok = mx;
  if (p.temperature != 0.f) {
    if (tid == 0) {
      // the slice in which the running sum of kept weights crosses u * total (slices in
      // order, sums in float32, the same order every time)
      float total = 0.f;
      for (int b = 0; b < kBlocks; ++b) total += w->part[b][3];
      uint32_t c[4] = {draws[row], 0u, 0u, 0u};
      philox4x32_10(c, p.seed_lo, p.seed_hi);
      const float u = (float)(c[0] >> 8) * 0x1p-24f;
      const float target = u * total;
      float run = 0.f;
      int blk = -1, last = 0;
      float rem = 0.f;
      for (int b = 0; b < kBlocks; ++b) {
        const float wb = w->part[b][3];
        if (wb > 0.f) {
          last = b;
          if (blk < 0 && run + wb > target) {
            blk = b;
            rem = target - run;
          }
        }
        run += wb;
      }
      if (blk < 0) {  // rounding at the very end of the distribution
        blk = last;
        rem = INFINITY;
      }
      s_block = blk;
      s_rem = rem;
      s_tok = -1;
      s_last_kept = -1;
    }
    __syncthreads();
    const SliceGeom g = slice_geom(logits, V, s_block);
    stage_edits(w, g, ed);
    float xv[16];
    int i0[2];
    load_share(logits + (size_t)row * V, g, ed, xv, i0);
    const float thr = keep_threshold(p, w->thr, mx);
    const float inv_t = 1.f / p.temperature;
    float rem = s_rem;
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      // chunk u of every thread, in thread order = vocabulary order
      float wk[8], local = 0.f;
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        wk[k] = (xv[8 * u + k] >= thr) ? expf((xv[8 * u + k] - mx) * inv_t) : 0.f;
        local += wk[k];
        if (wk[k] > 0.f) atomicMax(&s_last_kept, i0[u] + k);
      }
      // inclusive scan of `local` over the 256 threads; the intervals [excl, incl) of
      // consecutive threads tile the line exactly (excl is the neighbour's incl, bit for bit)
      float inc = local;
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        const float up = __shfl_up(inc, o, 64);
        if (lane >= o) inc += up;
      }
      const float prev = __shfl_up(inc, 1, 64);
      if (lane == 63) s_wsum[wave] = inc;
      __syncthreads();
      float before = 0.f;
      for (int wv = 0; wv < wave; ++wv) before += s_wsum[wv];
      const float round_total = ((s_wsum[0] + s_wsum[1]) + s_wsum[2]) + s_wsum[3];
      const float excl = lane > 0 ? before + prev : before;
      const float incl = before + inc;
      if (excl <= rem && rem < incl) {  // exactly one thread
        float run = excl;
        int sel = -1, last = -1;
#pragma unroll
        for (int k = 0; k < 8; ++k) {
          if (wk[k] > 0.f) {
            last = k;
            if (sel < 0 && run + wk[k] > rem) sel = k;
          }
          run += wk[k];
        }
        if (sel < 0) sel = last;  // the in-thread sum rounds differently from the scan
        if (sel >= 0) {
          s_tok = i0[u] + sel;
          float xs = 0.f;
#pragma unroll
          for (int k = 0; k < 8; ++k)
            if (k == sel) xs = xv[8 * u + k];
          s_x = xs;
        }
      }
      __syncthreads();
      if (s_tok >= 0) break;
      rem -= round_total;
    }
    __syncthreads();
    if (s_tok < 0) {  // float32 rounding put the target past the last kept token
      const int lk = s_last_kept;
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int k = 0; k < 8; ++k)
          if (i0[u] + k == lk) {
            s_tok = lk;
            s_x = xv[8 * u + k];
          }
      __syncthreads();
    }
    tok = s_tok;
    x_tok = s_x;
    if (tok < 0 || tok >= V) {  // no token was kept (min_p above 1, logits that are not numbers)
      tok = mi;
      x_tok = mx;
    }
  }
  tok = min(max(tok, 0), V - 1);
  if (want_top && top_idx && top_val) {
    // the tokens strictly above the 20th largest value, ranked: higher key first, lower index
    // first among equals; then the tokens equal to it, lowest ids first (slices in order)
    const int n = min(w->cand_n, kTop - 1);
    for (int c = tid; c < n; c += 256) {
      const unsigned long long me = w->cand[c];
      const unsigned int mk = (unsigned int)(me >> 32), mi2 = (unsigned int)me;
      int rank = 0;
      for (int o = 0; o < n; ++o) {
        const unsigned long long ot = w->cand[o];
        const unsigned int ok = (unsigned int)(ot >> 32), oi = (unsigned int)ot;
        rank += (ok > mk || (ok == mk && oi < mi2)) ? 1 : 0;
      }
      top_idx[(size_t)row * kTop + rank] = (int)mi2;
      top_val[(size_t)row * kTop + rank] = value_of((int)mk) - lse;
    }
    if (tid == 0) {
      int at = n;
      const float tv = value_of(w->key_top) - lse;
      for (int b = 0; b < kBlocks && at < kTop; ++b)
        for (int j = 0; j < w->tie_n[b] && at < kTop; ++j, ++at) {
          top_idx[(size_t)row * kTop + at] = w->tie_idx[b][j];
          top_val[(size_t)row * kTop + at] = tv;
        }
      for (; at < kTop; ++at) {  // vocabularies of fewer than 20 tokens
        top_idx[(size_t)row * kTop + at] = -1;
        top_val[(size_t)row * kTop + at] = -INFINITY;
      }
    }
  }
  if (tid == 0) {
    token[row] = tok;
    if (logprob) logprob[row] = x_tok - lse;
    if (lse_out) lse_out[row] = lse;
    if (feedback) feedback[row] = tok;
    if (history && hist_len) {
      const int len = hist_len[row];
      history[(size_t)row * hist_cap + len % hist_cap] = tok;
      hist_len[row] = len + 1;
    }
    if (draws && p.temperature != 0.f) draws[row] += 1;
    if (pos_inc) pos_inc[row] += 1;
  }
}

}  // namespace

extern "C" int64_t exo_sample_workspace(int rows) {
  if (rows <= 0) return 0;
  return (int64_t)rows * (int64_t)kRowStride;
}

extern "C" int exo_sample(const uint16_t* logits, const exo_sampler_params* params,
                          int32_t* history, int32_t* hist_len, uint32_t* draws, int32_t* token,
                          float* logprob, float* lse, int32_t* top_idx, float* top_val,
                          int32_t* feedback, int32_t* pos_inc, void* workspace,
                          int64_t workspace_bytes, int rows, int V, int hist_cap, int mode,
                          exo_stream_t stream) {
  EXO_REQUIRE(rows >= 0 && rows <= 65535 && V > 0, "exo_sample: bad size rows=%d V=%d", rows, V);
  EXO_REQUIRE(V <= kBlocks * kMaxSlice, "exo_sample: V=%d exceeds %d", V, kBlocks * kMaxSlice);
  EXO_REQUIRE(hist_cap >= 0 && hist_cap <= EXO_SAMPLER_MAX_CONTEXT,
              "exo_sample: hist_cap=%d outside [0,%d]", hist_cap, EXO_SAMPLER_MAX_CONTEXT);
  EXO_REQUIRE((mode & ~(EXO_SAMPLE_EDITS | EXO_SAMPLE_DRAW | EXO_SAMPLE_TABLE | EXO_SAMPLE_TOP)) == 0,
              "exo_sample: unknown mode bits 0x%x", mode);
  EXO_REQUIRE(logits && params && token && workspace, "exo_sample: null pointer");
  EXO_REQUIRE(workspace_bytes >= exo_sample_workspace(rows) && ((uintptr_t)workspace & 255) == 0,
              "exo_sample: workspace of %lld bytes, need %lld (256-byte aligned)",
              (long long)workspace_bytes, (long long)exo_sample_workspace(rows));
  const bool edits = mode & EXO_SAMPLE_EDITS, want_top = mode & EXO_SAMPLE_TOP;
  EXO_REQUIRE(!edits || hist_cap == 0 || (history && hist_len),
              "exo_sample: the penalty processors need the history ring");
  EXO_REQUIRE(!history || hist_cap > 0, "exo_sample: a history ring of zero entries (hist_cap=0)");
  EXO_REQUIRE(!want_top || (top_idx && top_val), "exo_sample: top-logprob outputs missing");
  EXO_REQUIRE(!(mode & EXO_SAMPLE_DRAW) || draws, "exo_sample: draw counters missing");
  if (rows == 0) return EXO_OK;
  const hipStream_t st = (hipStream_t)stream;
  const bf16_t* lg = logits;
  if (edits)
    sampler_edits_kernel<<<dim3(rows), 512, 0, st>>>(lg, params, history, hist_len, workspace, V,
                                                     hist_cap > 0 ? hist_cap : 1);
  sample_stats_kernel<<<dim3(kBlocks, rows), 256, 0, st>>>(lg, workspace, V, edits ? 1 : 0);
  if (mode & (EXO_SAMPLE_TABLE | EXO_SAMPLE_TOP)) {
    sample_coarse_kernel<<<dim3(kBlocks, rows), 256, 0, st>>>(lg, params, workspace, V,
                                                             want_top ? 1 : 0);
    sample_fine_kernel<<<dim3(kBlocks, rows), 256, 0, st>>>(lg, params, workspace, V,
                                                           want_top ? 1 : 0);
  }
  // (the weights launch also resolves and clears the tables: it runs whenever they were filled)
  if (mode & (EXO_SAMPLE_DRAW | EXO_SAMPLE_TOP | EXO_SAMPLE_TABLE))
    sample_weights_kernel<<<dim3(kBlocks, rows), 256, 0, st>>>(lg, params, workspace, V,
                                                              want_top ? 1 : 0);
  sample_select_kernel<<<dim3(rows), 256, 0, st>>>(lg, params, history, hist_len, draws, token,
                                                   logprob, lse, top_idx, top_val, feedback,
                                                   pos_inc, workspace, V,
                                                   hist_cap > 0 ? hist_cap : 1, want_top ? 1 : 0);
  EXO_CHECK_LAUNCH("exo_sample");
  return EXO_OK;
}
