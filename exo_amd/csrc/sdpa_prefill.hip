// Causal attention for a chunk of T new tokens (prefill) on the matrix cores.
//
// Flash-attention recurrence with both products on v_mfma_f32_32x32x16_bf16, written
// transposed so that every per-query quantity (running max, sum, rescale factor) is a
// per-LANE scalar:
//   S^T[key][query] = K . Q^T          A = K rows from LDS,      B = Q^T from registers
//   O^T[d][query]  += V^T . P^T        A = V^T rows from LDS,    B = P^T = the S^T registers
// The D-operand layout of the first product puts, in lane (query, half), registers that
// are 8 consecutive keys per 16-key step once the K rows are fed in a permuted order;
// they are rounded to bf16 and used as the B operand of the second product without any
// data movement.  V is transposed on its way into LDS (2-byte stores), K goes in as is.  (A
// row-major V tile read back through ds_read_b64_tr_b16 was measured and is slower here:
// 2046 tokens 100 -> 164 us.)
//
// Work split: a wave owns 32 query tokens of ONE query head; the four waves of a
// workgroup take four consecutive (token tile, head) units of one kv head, so with GQA
// (4, 8, 16 query heads per kv head) they share every K/V tile they stage.  Key tiles of
// 64 in two LDS buffers: while a tile is computed, the next one goes from registers into the
// other buffer and the one after that is on its way from memory; one barrier per tile.
//
// SPLIT (launches of at most one workgroup per CU, i.e. prompts of about a thousand tokens):
// eight waves, two teams of four that take the first and the second half of the
// workgroup's key tiles for the same four units, each with tile buffers of its own; at the end
// the second team's (O^T, max, sum) pass through LDS and are merged into the first's.  The
// causal triangle gives a launch of one round workgroups of 1 to N tiles; without the split
// the heavy ones run on alone, one wave per SIMD, for most of the launch.
#include "../../include/exo_mi355x.h"
#include "common.h"
#include "sdpa_internal.h"

namespace {

constexpr int kBN = 64;   // keys per tile
constexpr int kBM = 32;   // query tokens per wave
constexpr int kPadK = 8;  // bf16 of padding per K row / V^T row in LDS

struct FaParams {
  const bf16_t* q;    // [B*T, Hq*D] (already rotated)
  const bf16_t* k;    // [B, Hkv, S_max, D]
  const bf16_t* v;
  const int32_t* pos;  // [B] tokens in the cache before this chunk
  bf16_t* out;         // [B*T, Hq*D]
  float scale_log2e;
  int T, Hq, Hkv, S_max, G, units;  // units = token tiles * G
};

template <int D>
constexpr int fa_lds_bytes() {
  return 2 * (kBN * (D + kPadK) + D * (kBN + kPadK)) * 2;
}

template <int D, bool SPLIT>
__global__ __launch_bounds__(SPLIT ? 512 : 256, SPLIT ? 1 : 2) void fa_prefill_kernel(const FaParams p) {
  constexpr int STEPS = D / 16;  // MFMA steps over d for S^T
  constexpr int DT = D / 32;     // 32-row tiles of O^T
  constexpr int KS = D + kPadK;  // LDS row stride of K (bf16)
  constexpr int VS = kBN + kPadK;  // LDS row stride of V^T (bf16)
  constexpr int VEC = D / 8;     // 16-byte vectors per K/V row
  constexpr int LOADS = kBN * VEC / 256;
  constexpr int BUF = kBN * KS + D * VS;  // bf16 elements of one (K, V^T) tile pair
  extern __shared__ __attribute__((aligned(16))) bf16_t fa_lds[];  // [2][BUF] per team

  const int tid = threadIdx.x & 255, lane = tid & 63;  // within the team
  const int team = SPLIT ? __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 8) : 0;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  bf16_t* const lds = fa_lds + team * (2 * BUF);
  const int n = lane & 31, kq = lane >> 5;
  const int kvh = blockIdx.y, b = blockIdx.z;
  // Heavy (late) token tiles first - but a launch of up to two workgroups per CU is one round
  // with nothing left to balance it, and the dispatcher hands a CU its second workgroup 256
  // positions after its first: every other run of 256 then takes the light tiles first, so
  // that the two workgroups of a CU are a heavy and a light one (2046 tokens, 32 / 8 heads:
  // 129 -> 109 us; with 2048 launches the same order lost 10 %).
  const int row = (int)blockIdx.y + (int)gridDim.y * (int)blockIdx.z;
  const int rows_per_run = max(1, 256 / (int)gridDim.x);
  const bool one_round = !SPLIT && gridDim.x * gridDim.y * gridDim.z <= 512;  // (longer launches balance
  const bool light_first = one_round && ((row / rows_per_run) & 1);  //  themselves, heavy first)
  const int u0 = (light_first ? (int)blockIdx.x : (int)gridDim.x - 1 - (int)blockIdx.x) * 4;
  const int u = u0 + wave;
  const bool active = u < p.units;
  const int uc = active ? u : p.units - 1;
  const int tt = uc / p.G, g = uc % p.G;
  const int hq = kvh * p.G + g;
  const int pos = p.pos[b];
  const int t_lane = min(tt * kBM + n, p.T - 1);            // this lane's query token
  const int last_w = pos + min(tt * kBM + kBM - 1, p.T - 1);  // last key any row of the wave sees
  const int tt_max = min(u0 + 3, p.units - 1) / p.G;
  const int last_wg = min(pos + min(tt_max * kBM + kBM - 1, p.T - 1), p.S_max - 1);
  const int n_all = last_wg / kBN + 1;  // key tiles of the workgroup
  // SPLIT: team 0 takes tiles [0, n_all / 2), team 1 the rest - at least as many, and the
  // ones with the causal edge; the workgroup's barriers are counted by team 1's tiles
  const int t_first = (SPLIT && team) ? n_all / 2 : 0;
  const int n_tiles = !SPLIT ? n_all : team ? n_all - n_all / 2 : n_all / 2;
  const int n_iter = SPLIT ? n_all - n_all / 2 : n_all;

  // Q^T operand: lane (query n, half kq) holds d = step*16 + kq*8 .. +8 for every step
  uint4 qreg[STEPS];
  {
    const bf16_t* qp = p.q + ((size_t)b * p.T + t_lane) * ((size_t)p.Hq * D) + (size_t)hq * D + kq * 8;
#pragma unroll
    for (int s = 0; s < STEPS; ++s) qreg[s] = *reinterpret_cast<const uint4*>(qp + s * 16);
  }

  // K/V tiles come through buffer loads: one descriptor per (sequence, kv head) that ends
  // with the cache (rows past it read as zero; they are masked), a lane offset that never
  // changes and the tile as the scalar offset - no 64-bit address per load in registers.
  // A K tile is one contiguous block (16 bytes per thread and load); a V load takes key
  // tid % 64, chunk tid / 64 + 4 i, so that a thread's stores into V^T are 8 rows of one key.
  const size_t head_off = ((size_t)b * p.Hkv + kvh) * (size_t)p.S_max * D;
  const uint32_t head_bytes = (uint32_t)p.S_max * D * 2;
  const __amdgpu_buffer_rsrc_t rk =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(p.k + head_off), 0, head_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t rv =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(p.v + head_off), 0, head_bytes, 0x00020000);
  const uint32_t koff = tid * 16, voff = (tid & (kBN - 1)) * (D * 2) + (tid / kBN) * 16;
  uint4 kreg[LOADS], vreg[LOADS];
  auto load_tile = [&](int kt) {
    const uint32_t tile = (uint32_t)(t_first + kt) * (kBN * D * 2);
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
      kreg[i] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(rk, koff, tile + i * 4096, 0));
      vreg[i] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(rv, voff + i * 64, tile, 0));
    }
  };
  auto store_tile = [&](int buf) {
    bf16_t* kl = lds + buf * BUF;
    bf16_t* vl = kl + kBN * KS;
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
      const int vi = tid + i * 256;
      *reinterpret_cast<uint4*>(&kl[(vi / VEC) * KS + (vi % VEC) * 8]) = kreg[i];
      const int key = vi & (kBN - 1), c = vi / kBN;
      const uint32_t w[4] = {vreg[i].x, vreg[i].y, vreg[i].z, vreg[i].w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        vl[(c * 8 + 2 * j) * VS + key] = (bf16_t)(w[j] & 0xFFFFu);
        vl[(c * 8 + 2 * j + 1) * VS + key] = (bf16_t)(w[j] >> 16);
      }
    }
  };

  // A-operand row r of a 32-key sub-tile holds this key, so that D registers 8s..8s+7
  // of lane half kq are keys 16s + 8kq .. +8
  const int jr = n >> 3;
  const int key_of_row = 16 * (jr >> 1) + 8 * ((n >> 2) & 1) + 4 * (jr & 1) + (n & 3);

  floatx16 o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int e = 0; e < 16; ++e) o[dt][e] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;

  if (!SPLIT || n_tiles > 0) {
    load_tile(0);
    store_tile(0);
  }
  // Every load so far (the Q operand among them) has landed before the loop is entered: left
  // to itself the compiler requests Q last and then waits, in EVERY iteration, for as many
  // loads as were issued after each Q register - which in the loop are the tile loads just
  // requested, so the prefetch would be waited for on the spot.
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
  if (n_tiles > 1) load_tile(1);
  for (int kt = 0; kt < n_iter; ++kt) {
    // tile kt is complete in its buffer, and every wave is done reading the other buffer
    __syncthreads();
    if (SPLIT && kt >= n_tiles) continue;  // (team 0 when the tile count is odd)
    if (kt + 1 < n_tiles) {
      store_tile((kt + 1) & 1);
      if (kt + 2 < n_tiles) load_tile(kt + 2);
    }
    const int key0 = (t_first + kt) * kBN;
    if (key0 > last_w) continue;  // wave-uniform: nothing visible to this wave's rows
    const bf16_t* k_lds = lds + (kt & 1) * BUF;
    const bf16_t* v_lds = k_lds + kBN * KS;

    // ---- S^T = K Q^T for the two 32-key sub-tiles
    floatx16 s[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
      for (int e = 0; e < 16; ++e) s[ks][e] = 0.f;
      const bf16_t* kr = &k_lds[(ks * 32 + key_of_row) * KS + kq * 8];
#pragma unroll
      for (int st = 0; st < STEPS; ++st) {
        const uint4 a = *reinterpret_cast<const uint4*>(kr + st * 16);
        s[ks] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                        __builtin_bit_cast(bf16x8_t, qreg[st]),
                                                        s[ks], 0, 0, 0);
      }
    }
    // ---- online softmax over this lane's 32 keys (+ the partner half's 32)
    const bool diag = key0 + kBN - 1 > pos + tt * kBM;  // some (query, key) pair is masked
    const int vis = pos + t_lane - key0;                  // keys 0..vis of the tile are visible
    float mx = -INFINITY;
#pragma unroll
    for (int ks = 0; ks < 2; ++ks)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        float x = s[ks][e] * p.scale_log2e;
        if (diag) {
          const int key = ks * 32 + 16 * (e >> 3) + 8 * kq + (e & 7);
          if (key > vis) x = -INFINITY;
        }
        s[ks][e] = x;
        mx = fmaxf(mx, x);
      }
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(m_run, mx);
    // m_new is finite: key 0 is visible to every query, and tiles come in key order
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
    float sum = 0.f;
    uint4 pb[2][2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      float pr[16];
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        pr[e] = __builtin_amdgcn_exp2f(s[ks][e] - m_new);
        sum += pr[e];
      }
#pragma unroll
      for (int st = 0; st < 2; ++st) {
        pb[ks][st].x = pack_bf2(pr[8 * st + 0], pr[8 * st + 1]);
        pb[ks][st].y = pack_bf2(pr[8 * st + 2], pr[8 * st + 3]);
        pb[ks][st].z = pack_bf2(pr[8 * st + 4], pr[8 * st + 5]);
        pb[ks][st].w = pack_bf2(pr[8 * st + 6], pr[8 * st + 7]);
      }
    }
    sum += __shfl_xor(sum, 32, 64);
    l_run = l_run * alpha + sum;
    m_run = m_new;
    // ---- O^T = alpha * O^T + V^T P^T
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
      for (int e = 0; e < 16; ++e) o[dt][e] *= alpha;
      const bf16_t* vr = &v_lds[(dt * 32 + n) * VS + kq * 8];
#pragma unroll
      for (int ks = 0; ks < 2; ++ks)
#pragma unroll
        for (int st = 0; st < 2; ++st) {
          const uint4 a = *reinterpret_cast<const uint4*>(vr + ks * 32 + st * 16);
          o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                          __builtin_bit_cast(bf16x8_t, pb[ks][st]),
                                                          o[dt], 0, 0, 0);
        }
    }
  }

  if (SPLIT) {
    // the second team's sums: through LDS (lane-contiguous floats per register), merged into
    // the first team's, which goes on alone
    float* ex = reinterpret_cast<float*>(fa_lds) + wave * ((DT * 16 + 2) * 64);
    __syncthreads();  // both teams have finished with their tile buffers
    if (team == 1) {
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int e = 0; e < 16; ++e) ex[(dt * 16 + e) * 64 + lane] = o[dt][e];
      ex[(DT * 16) * 64 + lane] = m_run;
      ex[(DT * 16 + 1) * 64 + lane] = l_run;
    }
    __syncthreads();
    if (team == 1) return;  // (no workgroup barrier after this point)
    const float m1 = ex[(DT * 16) * 64 + lane], l1 = ex[(DT * 16 + 1) * 64 + lane];
    const float m = fmaxf(m_run, m1);  // finite: key 0 is visible to one of the teams
    const float a0 = m_run == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m_run - m);
    const float a1 = m1 == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m1 - m);
    l_run = l_run * a0 + l1 * a1;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int e = 0; e < 16; ++e) o[dt][e] = o[dt][e] * a0 + ex[(dt * 16 + e) * 64 + lane] * a1;
  }

  // ---- out[token][hq*D + d] = O^T[d][token] / l
  if (!active || tt * kBM + n >= p.T) return;
  const float inv = 1.f / l_run;
  bf16_t* op = p.out + ((size_t)b * p.T + t_lane) * ((size_t)p.Hq * D) + (size_t)hq * D;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      uint2 w;
      w.x = pack_bf2(o[dt][4 * j + 0] * inv, o[dt][4 * j + 1] * inv);
      w.y = pack_bf2(o[dt][4 * j + 2] * inv, o[dt][4 * j + 3] * inv);
      *reinterpret_cast<uint2*>(op + dt * 32 + 8 * j + 4 * kq) = w;
    }
}

}  // namespace

int exo_sdpa_prefill_mfma(const bf16_t* q, const bf16_t* k_cache, const bf16_t* v_cache,
                          const int32_t* pos, bf16_t* out, float scale, int B, int T, int Hq,
                          int Hkv, int D, int S_max, hipStream_t stream) {
  FaParams p;
  p.q = q;
  p.k = k_cache;
  p.v = v_cache;
  p.pos = pos;
  p.out = out;
  p.scale_log2e = scale * 1.4426950408889634f;
  p.T = T;
  p.Hq = Hq;
  p.Hkv = Hkv;
  p.S_max = S_max;
  p.G = Hq / Hkv;
  p.units = ((T + kBM - 1) / kBM) * p.G;
  const dim3 grid((p.units + 3) / 4, Hkv, B);
  // the split variant where its eight-wave workgroups are one round of one per CU (their two
  // teams' tile buffers leave room for one) and the heaviest has enough tiles to share out:
  // 1022 tokens of 32 / 4 heads (256 workgroups) 34.9 -> 30.3 us; with 512 workgroups it is
  // two rounds and loses to two four-wave workgroups per CU (2046 tokens, 32 / 8: 75 -> 106 us)
  const bool split = (int64_t)grid.x * grid.y * grid.z <= 256 && T >= 256;
  // more than 64 KiB of LDS per workgroup: raised once per kernel instance
  auto raise = [](const void* fn, int bytes, bool* done) {
    if (*done || bytes <= 64 * 1024) return EXO_OK;
    const hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e != hipSuccess) {
      exo_set_error("exo_sdpa_prefill: cannot raise dynamic LDS limit: %s", hipGetErrorString(e));
      return EXO_ERR_HIP;
    }
    *done = true;
    return EXO_OK;
  };
  static bool done[4] = {false, false, false, false};
  const int lds = (D == 64 ? fa_lds_bytes<64>() : fa_lds_bytes<128>()) * (split ? 2 : 1);
  int rc;
  exo_note_variant("fa_prefill<%d,%s> grid=%dx%dx%d", D, split ? "true" : "false", (int)grid.x, (int)grid.y,
                   (int)grid.z);
  if (D == 64 && !split) {
    if ((rc = raise(reinterpret_cast<const void*>(fa_prefill_kernel<64, false>), lds, &done[0]))) return rc;
    fa_prefill_kernel<64, false><<<grid, 256, lds, stream>>>(p);
  } else if (D == 64) {
    if ((rc = raise(reinterpret_cast<const void*>(fa_prefill_kernel<64, true>), lds, &done[1]))) return rc;
    fa_prefill_kernel<64, true><<<grid, 512, lds, stream>>>(p);
  } else if (!split) {
    if ((rc = raise(reinterpret_cast<const void*>(fa_prefill_kernel<128, false>), lds, &done[2]))) return rc;
    fa_prefill_kernel<128, false><<<grid, 256, lds, stream>>>(p);
  } else {
    if ((rc = raise(reinterpret_cast<const void*>(fa_prefill_kernel<128, true>), lds, &done[3]))) return rc;
    fa_prefill_kernel<128, true><<<grid, 512, lds, stream>>>(p);
  }
  return EXO_OK;
}
