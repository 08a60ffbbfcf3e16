// Quantised matmul for prefill (any M): y[M,N] = x[M,K] @ dq(W)[N,K]^T.
//
// Matrix-core design for gfx950: a 256x128 (128x128 for M <= 128) output tile per
// 256-thread workgroup, one 64-wide K step per iteration = exactly one quantisation group,
// so every packed row segment needs a single (scale, bias).  Each thread dequantises 32 (4-bit) or
// 2x16 (8-bit) codes to bf16 in registers - bf16(fma(s, q, b)), codes converted with
// v_cvt_f32_ubyteN - and stores them to LDS next to the activation tile; the four
// waves (2x2) then issue v_mfma_f32_32x32x16_bf16 on 128x64 (64x64) sub-tiles with float32
// accumulators: the taller tile halves both the dequantisation work and the LDS bytes
// read per MFMA.  Global loads of the next K step are issued before the MFMAs of the
// current one.  LDS rows are padded by 16 bytes to keep ds_read_b128 conflict-free.
#include "../../include/exo_mi355x.h"
#include "common.h"

namespace {

constexpr int BK = 64;
constexpr int LDS_STRIDE = BK + 8;  // bf16 elements per LDS row

struct QmmParams {
  const bf16_t* x;
  const uint32_t* w;
  const bf16_t* s;
  const bf16_t* b;
  const bf16_t* residual;
  bf16_t* y;
  int M, N, K;
  // grouped mode (MoE experts, rows sorted by expert): blockIdx.y is a tile of
  // tiles[]; row r of the tile is pair sorted[start + r]; it reads activation row
  // pair / x_div and writes output row pair; the tile multiplies by expert e's matrix
  const int32_t* sorted;  // [pairs]
  const int32_t* tiles;   // [max_tiles][3] = expert (-1: unused), start, rows
  int x_div;
  size_t w_stride, s_stride;  // elements between consecutive experts
};

template <int BITS>
struct WFrag {  // one thread's share of the packed W tile for one K step
  uint4 q[BITS / 4];  // 4-bit: 16 B = 32 codes; 8-bit: 2 x 16 B = 2 x 16 codes
  float s, b;
};

__device__ __forceinline__ float ubyte_f(uint32_t v, int i) {
  return (float)((v >> (8 * i)) & 0xffu);  // v_cvt_f32_ubyteN
}

// The workgroup is 2 x WN waves; a wave computes (32*MI) x 64 outputs, so the tile is
// (64*MI) x (64*WN).  STAGES = K steps whose global loads are in flight (held in
// registers) while the current step is multiplied.
template <int BITS, int MI, int WN, int STAGES, bool GROUPED = false>
__global__ __launch_bounds__(128 * WN, 2) void qmm_kernel(const QmmParams p) {
  constexpr int kThreads = 128 * WN;
  constexpr int BM = 64 * MI, BN = 64 * WN;
  constexpr int XR = BM * 8 / kThreads;  // 16-byte x loads per thread and K step
  __shared__ __attribute__((aligned(16))) bf16_t xs[BM * LDS_STRIDE];
  __shared__ __attribute__((aligned(16))) bf16_t ws[BN * LDS_STRIDE];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n0 = blockIdx.x * BN;
  const int wm = (wave / WN) * (32 * MI), wn = (wave % WN) * 64;
  const int G = p.K >> 6;
  const int wpr = p.K * BITS / 32;
  int m0 = blockIdx.y * BM, m_end = p.M;
  size_t w_off = 0, s_off = 0;
  __shared__ int row_pair[GROUPED ? BM : 1];  // pair index of every row of the tile
  if (GROUPED) {
    const int32_t* ti = p.tiles + 3 * (size_t)blockIdx.y;
    const int e = ti[0];
    if (e < 0) return;  // whole workgroup: tile slot not in use
    m0 = 0;
    m_end = ti[2];
    for (int r = tid; r < BM; r += kThreads) row_pair[r] = r < m_end ? p.sorted[ti[1] + r] : -1;
    w_off = (size_t)e * p.w_stride;
    s_off = (size_t)e * p.s_stride;
    __syncthreads();
  }

  // W: thread -> (row, part): 2 parts of 32 codes per row and K step
  const int w_row = tid >> 1, w_part = tid & 1;
  const bool w_ok = (n0 + w_row) < p.N;
  const uint32_t* wsrc = p.w + w_off + (size_t)(n0 + (w_ok ? w_row : 0)) * wpr + w_part * (BITS);
  const bf16_t* ssrc = p.s + s_off + (size_t)(n0 + (w_ok ? w_row : 0)) * G;
  const bf16_t* bsrc = p.b + s_off + (size_t)(n0 + (w_ok ? w_row : 0)) * G;

  struct Stage {
    uint4 xa[XR];
    WFrag<BITS> wf;
  };

  auto load_global = [&](Stage& st, int k0) {
#pragma unroll
    for (int r = 0; r < XR; ++r) {
      const int id = tid + kThreads * r;
      const int row = id >> 3, kp = id & 7;
      if (m0 + row < m_end) {
        const size_t src = GROUPED ? (size_t)(row_pair[row] / p.x_div) : (size_t)(m0 + row);
        st.xa[r] = *reinterpret_cast<const uint4*>(p.x + src * p.K + k0 + kp * 8);
      } else
        st.xa[r] = make_uint4(0, 0, 0, 0);
    }
    const int kw = k0 * BITS / 32;  // word offset of this K step
#pragma unroll
    for (int i = 0; i < BITS / 4; ++i)
      st.wf.q[i] = *reinterpret_cast<const uint4*>(wsrc + kw + i * 4);
    st.wf.s = bf2f(ssrc[k0 >> 6]);
    st.wf.b = bf2f(bsrc[k0 >> 6]);
    if (!w_ok) {
      st.wf.s = 0.f;
      st.wf.b = 0.f;
    }
  };

  auto store_lds = [&](const Stage& st) {
#pragma unroll
    for (int r = 0; r < XR; ++r) {
      const int id = tid + kThreads * r;
      const int row = id >> 3, kp = id & 7;
      *reinterpret_cast<uint4*>(&xs[row * LDS_STRIDE + kp * 8]) = st.xa[r];
    }
    bf16_t* dst = &ws[w_row * LDS_STRIDE + w_part * 32];
    const float s = st.wf.s, b = st.wf.b;
    const uint32_t* qw = reinterpret_cast<const uint32_t*>(&st.wf.q[0]);
    if (BITS == 4) {
#pragma unroll
      for (int h = 0; h < 2; ++h) {  // 2 words = 16 codes = two 16-byte LDS stores
        uint4 o[2];
        uint32_t* o4 = reinterpret_cast<uint32_t*>(o);
#pragma unroll
        for (int wi = 0; wi < 2; ++wi) {
          const uint32_t v = qw[h * 2 + wi];
          const uint32_t ev = v & 0x0f0f0f0fu, od = (v >> 4) & 0x0f0f0f0fu;
#pragma unroll
          for (int e = 0; e < 4; ++e)
            o4[wi * 4 + e] = pack_bf2(fmaf(s, ubyte_f(ev, e), b), fmaf(s, ubyte_f(od, e), b));
        }
        *reinterpret_cast<uint4*>(dst + h * 16) = o[0];
        *reinterpret_cast<uint4*>(dst + h * 16 + 8) = o[1];
      }
    } else {
#pragma unroll
      for (int h = 0; h < 4; ++h) {  // 8 codes (2 words) per 16-byte LDS store
        uint4 o;
        uint32_t* o4 = reinterpret_cast<uint32_t*>(&o);
#pragma unroll
        for (int wi = 0; wi < 2; ++wi) {
          const uint32_t v = qw[h * 2 + wi];
          o4[wi * 2] = pack_bf2(fmaf(s, ubyte_f(v, 0), b), fmaf(s, ubyte_f(v, 1), b));
          o4[wi * 2 + 1] = pack_bf2(fmaf(s, ubyte_f(v, 2), b), fmaf(s, ubyte_f(v, 3), b));
        }
        *reinterpret_cast<uint4*>(dst + h * 8) = o;
      }
    }
  };

  floatx16 acc[MI][2];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  const int frow = lane & 31, fk = (lane >> 5) * 8;
  auto multiply = [&]() {
#pragma unroll
    for (int ks = 0; ks < BK; ks += 16) {
      bf16x8_t a[MI], bq[2];
#pragma unroll
      for (int i = 0; i < MI; ++i)
        a[i] = *reinterpret_cast<const bf16x8_t*>(&xs[(wm + i * 32 + frow) * LDS_STRIDE + ks + fk]);
#pragma unroll
      for (int j = 0; j < 2; ++j)
        bq[j] = *reinterpret_cast<const bf16x8_t*>(&ws[(wn + j * 32 + frow) * LDS_STRIDE + ks + fk]);
#pragma unroll
      for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], bq[j], acc[i][j], 0, 0, 0);
    }
  };

  // one K step: stage `st` (loaded STAGES steps ago) goes to LDS, is refilled with the
  // step STAGES ahead, and the tile is multiplied
  auto step = [&](Stage& st, int k0) {
    __syncthreads();  // previous step's LDS reads are done
    store_lds(st);
    __syncthreads();
    if (k0 + STAGES * BK < p.K) load_global(st, k0 + STAGES * BK);
    multiply();
  };

  Stage st[STAGES];
#pragma unroll
  for (int i = 0; i < STAGES; ++i)
    if (i * BK < p.K) load_global(st[i], i * BK);
  for (int k0 = 0; k0 < p.K; k0 += STAGES * BK) {
#pragma unroll
    for (int i = 0; i < STAGES; ++i)
      if (k0 + i * BK < p.K) step(st[i], k0 + i * BK);
  }

  // D[i][j]: column j = lane%32 (W row n), rows 8*(r/4) + 4*(lane/32) + r%4 (token m)
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int n = n0 + wn + j * 32 + (lane & 31);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + wm + i * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
        if (m < m_end && n < p.N) {
          const size_t o = (size_t)(GROUPED ? row_pair[m] : m) * p.N + n;
          float v = acc[i][j][r];
          if (p.residual) v = bf2f(f2bf(v)) + bf2f(p.residual[o]);
          p.y[o] = f2bf(v);
        }
      }
    }
}

template <int BITS>
void launch_qmm(const QmmParams& p, hipStream_t st) {
  const int M = p.M, N = p.N;
  // up to 128 rows: little arithmetic per K step, so several steps' loads are kept in
  // flight; taller inputs: 256-row tiles halve the dequantisation work per output
  if (M <= 128)
    qmm_kernel<BITS, 2, 2, 2><<<dim3(exo_ceil_div(N, 128), exo_ceil_div(M, 128)), 256, 0, st>>>(p);
  else
    qmm_kernel<BITS, 4, 2, 1><<<dim3(exo_ceil_div(N, 128), exo_ceil_div(M, 256)), 256, 0, st>>>(p);
}

constexpr int kGroupBM = 128;  // rows per tile of the grouped GEMM
constexpr int kGroupMaxE = 256;

// Sort the (token, slot) pairs by expert and cut every expert's run into tiles of
// kGroupBM rows.  One workgroup: counts in LDS, a serial scan over the experts, a second
// pass that scatters the pair indices.  The order inside an expert's run depends on
// atomic arrival order; every output row is computed independently of its tile position,
// so results do not.
__global__ __launch_bounds__(1024) void moe_group_kernel(const int32_t* __restrict__ idx, int P,
                                                         int E, int32_t* __restrict__ sorted,
                                                         int32_t* __restrict__ tiles,
                                                         int max_tiles) {
  __shared__ int cnt[kGroupMaxE], off[kGroupMaxE], cur[kGroupMaxE], tile0[kGroupMaxE + 1];
  const int tid = threadIdx.x;
  for (int e = tid; e < E; e += 1024) cnt[e] = 0;
  __syncthreads();
  for (int i = tid; i < P; i += 1024) {
    const int e = idx[i];
    if (e >= 0 && e < E) atomicAdd(&cnt[e], 1);
  }
  __syncthreads();
  if (tid == 0) {
    int o = 0, t = 0;
    for (int e = 0; e < E; ++e) {
      off[e] = o;
      cur[e] = o;
      tile0[e] = t;
      o += cnt[e];
      t += (cnt[e] + kGroupBM - 1) / kGroupBM;
    }
    tile0[E] = t;
  }
  __syncthreads();
  for (int i = tid; i < P; i += 1024) {
    const int e = idx[i];
    if (e >= 0 && e < E) sorted[atomicAdd(&cur[e], 1)] = i;
  }
  for (int e = tid; e < E; e += 1024) {
    const int nt = tile0[e + 1] - tile0[e];
    for (int j = 0; j < nt; ++j) {
      int32_t* t = tiles + 3 * (size_t)(tile0[e] + j);
      t[0] = e;
      t[1] = off[e] + j * kGroupBM;
      t[2] = min(kGroupBM, cnt[e] - j * kGroupBM);
    }
  }
  for (int t = tile0[E] + tid; t < max_tiles; t += 1024) tiles[3 * (size_t)t] = -1;
}

int group_max_tiles(int64_t pairs, int E) { return (int)((pairs + kGroupBM - 1) / kGroupBM) + E; }

}  // namespace

extern "C" int64_t exo_moe_group_workspace(int T, int topk, int E) {
  if (T <= 0 || topk <= 0 || E <= 0) return 0;
  const int64_t pairs = (int64_t)T * topk;
  return (pairs + 3 * (int64_t)group_max_tiles(pairs, E)) * 4;
}

extern "C" int exo_moe_group(const int32_t* idx, int T, int topk, int E, void* workspace,
                             int64_t workspace_bytes, exo_stream_t stream) {
  EXO_REQUIRE(idx && workspace, "exo_moe_group: null pointer");
  EXO_REQUIRE(T > 0 && topk > 0 && E > 0 && E <= kGroupMaxE && (int64_t)T * topk < (1ll << 30),
              "exo_moe_group: need T>0, topk>0, 0<E<=%d; got T=%d topk=%d E=%d", kGroupMaxE, T,
              topk, E);
  EXO_REQUIRE(workspace_bytes >= exo_moe_group_workspace(T, topk, E),
              "exo_moe_group: workspace of %lld bytes, need %lld", (long long)workspace_bytes,
              (long long)exo_moe_group_workspace(T, topk, E));
  const int P = T * topk;
  int32_t* sorted = reinterpret_cast<int32_t*>(workspace);
  moe_group_kernel<<<1, 1024, 0, (hipStream_t)stream>>>(idx, P, E, sorted, sorted + P,
                                                       group_max_tiles(P, E));
  EXO_CHECK_LAUNCH("exo_moe_group");
  return EXO_OK;
}

extern "C" int exo_gather_qmm(const uint16_t* x, const uint32_t* w, const uint16_t* scales,
                              const uint16_t* biases, const void* workspace, uint16_t* y, int T,
                              int topk, int x_rows, int E, int N, int K, int bits,
                              int group_size, exo_stream_t stream) {
  EXO_REQUIRE(bits == 4 || bits == 8, "exo_gather_qmm: bits must be 4 or 8, got %d", bits);
  EXO_REQUIRE(group_size == 64, "exo_gather_qmm: group_size must be 64, got %d", group_size);
  EXO_REQUIRE(N > 0 && K > 0 && K % 64 == 0, "exo_gather_qmm: bad shape N=%d K=%d", N, K);
  EXO_REQUIRE(T > 0 && topk > 0 && E > 0 && E <= kGroupMaxE && (int64_t)T * topk < (1ll << 30),
              "exo_gather_qmm: bad T=%d topk=%d E=%d", T, topk, E);
  EXO_REQUIRE(x_rows == 1 || x_rows == topk, "exo_gather_qmm: x_rows must be 1 or topk, got %d",
              x_rows);
  EXO_REQUIRE(x && w && scales && biases && workspace && y, "exo_gather_qmm: null pointer");
  const int P = T * topk;
  const int max_tiles = group_max_tiles(P, E);
  EXO_REQUIRE(max_tiles <= 65535, "exo_gather_qmm: %d row tiles exceed the grid limit", max_tiles);
  QmmParams p{x, w, scales, biases, nullptr, y, P, N, K};
  p.sorted = reinterpret_cast<const int32_t*>(workspace);
  p.tiles = p.sorted + P;
  p.x_div = x_rows == 1 ? topk : 1;
  p.w_stride = (size_t)N * (K * bits / 32);
  p.s_stride = (size_t)N * (K / 64);
  const dim3 grid(exo_ceil_div(N, 128), max_tiles);
  if (bits == 4)
    qmm_kernel<4, 2, 2, 2, true><<<grid, 256, 0, (hipStream_t)stream>>>(p);
  else
    qmm_kernel<8, 2, 2, 2, true><<<grid, 256, 0, (hipStream_t)stream>>>(p);
  EXO_CHECK_LAUNCH("exo_gather_qmm");
  return EXO_OK;
}

extern "C" int exo_qmm(const uint16_t* x, const uint32_t* w, const uint16_t* scales,
                       const uint16_t* biases, const uint16_t* residual, uint16_t* y, int M,
                       int N, int K, int bits, int group_size, exo_stream_t stream) {
  EXO_REQUIRE(bits == 4 || bits == 8, "exo_qmm: bits must be 4 or 8, got %d", bits);
  EXO_REQUIRE(group_size == 64, "exo_qmm: group_size must be 64, got %d", group_size);
  EXO_REQUIRE(M >= 0 && N > 0 && K > 0 && K % 64 == 0, "exo_qmm: bad shape M=%d N=%d K=%d", M, N,
              K);
  EXO_REQUIRE(x && w && scales && biases && y, "exo_qmm: null pointer");
  if (M == 0) return EXO_OK;
  QmmParams p{x, w, scales, biases, residual, y, M, N, K};
  p.sorted = nullptr;
  p.tiles = nullptr;
  p.x_div = 1;
  p.w_stride = p.s_stride = 0;
  EXO_REQUIRE(exo_ceil_div(M, 128) <= 65535, "exo_qmm: M=%d too large", M);
  if (bits == 4)
    launch_qmm<4>(p, (hipStream_t)stream);
  else
    launch_qmm<8>(p, (hipStream_t)stream);
  EXO_CHECK_LAUNCH("exo_qmm");
  return EXO_OK;
}
