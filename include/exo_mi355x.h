/* libexo_mi355x.so - C ABI of the MI355X (gfx950) kernels for exo's per-shard
 * transformer forward on MLX affine-quantised weights.
 *
 * The reference has no FFI on this path: its engine calls mlx / mlx_lm Python
 * operators.  Each entry point below replaces one of those operators and cites
 * the place the reference states or calls it (paths relative to the reference
 * tree).  All pointers are DEVICE pointers unless noted; `stream` is a
 * hipStream_t passed as void*.  No entry point allocates, frees or synchronises;
 * all are asynchronous on `stream`.  Return value: 0 ok, -1 bad argument,
 * -2 HIP launch error; exo_last_error() gives the message (thread-local).
 *
 * Tensor conventions (MLX checkpoint layout, untouched):
 *   packed weight  uint32 [N, K*bits/32], element i of a row in word i/(32/bits),
 *                  bits [bits*(i mod 32/bits), +bits)     (.typings/mlx/core/__init__.pyi:4180-4184)
 *   scales/biases  bf16   [N, K/group_size]               (src/exo/worker/engines/mlx/auto_parallel.py:880-881)
 *   activations    bf16 row-major
 * group_size must be 64 and bits 4 or 8.
 */
#ifndef EXO_MI355X_H
#define EXO_MI355X_H
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

typedef void* exo_stream_t;

int exo_abi_version(void);
const char* exo_last_error(void);
/* Diagnostic, no reference counterpart: the kernel instance and launch shape that the
 * calling thread's latest exo_qmv* / exo_qmm* / exo_gather_* / exo_attn_decode* /
 * exo_sdpa_* call selected, as text (e.g. "qmm wide ring4 pair bits=4 ..."); thread-local,
 * empty before the first such call.  Tests use it to assert that a shape reached the
 * instance it targets. */
const char* exo_last_variant(void);
/* 1 if dequantised bf16 weights are formed as bf16(bf16(s*q)+b), 0 if bf16(fma(s,q,b)). */
int exo_dequant_two_roundings(void);

/* K0: packed words -> one uint8 code per element.  (.typings/mlx/core/__init__.pyi:4180-4184) */
int exo_unpack_codes(const uint32_t* w, uint8_t* out, int64_t n_words, int bits,
                     exo_stream_t stream);

/* mx.dequantize(w, scales, biases, group_size, bits) -> bf16 [rows, K].
 * (.typings/mlx/core/__init__.pyi:2413-2451) */
int exo_dequantize(const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                   uint16_t* out, int64_t rows, int K, int bits, int group_size,
                   exo_stream_t stream);

/* K4: nn.QuantizedEmbedding.__call__: out[i,:] = dequantize(row ids[i]).
 * ids int32 [n_ids] on device.  (.typings/mlx/nn/layers/quantized.pyi:42-85) */
int exo_embed_dequant(const int32_t* ids, const uint32_t* w, const uint16_t* scales,
                      const uint16_t* biases, uint16_t* out, int n_ids, int vocab, int K,
                      int bits, int group_size, exo_stream_t stream);

/* K1: mx.quantized_matmul(x, w, scales, biases, transpose=True) for M <= 16 rows of
 * x (decode): y[M,N] = x[M,K] @ dq(w)[N,K]^T, float32 accumulation, bf16 out.
 * Optional fused epilogue: if `residual` is non-null, y = bf16(residual + bf16(acc))
 * (the `h + r` of a transformer block).  (.typings/mlx/core/__init__.pyi:4198-4234,
 * reached through nn.QuantizedLinear.__call__ .typings/mlx/nn/layers/quantized.pyi:87-118) */
int exo_qmv(const uint16_t* x, const uint32_t* w, const uint16_t* scales,
            const uint16_t* biases, const uint16_t* residual, uint16_t* y, int M, int N,
            int K, int bits, int group_size, exo_stream_t stream);

/* K1+K8: fused gate/up projection and SwiGLU for M <= 16:
 * y[M,N] = silu(x @ dq(wg)^T) * (x @ dq(wu)^T), each projection rounded to bf16
 * first, as two QuantizedLinear calls followed by swiglu would.
 * (.typings/mlx_lm/models/switch_layers.pyi:52-57) */
int exo_qmv_swiglu(const uint16_t* x, const uint32_t* wg, const uint16_t* sg,
                   const uint16_t* bg, const uint32_t* wu, const uint16_t* su,
                   const uint16_t* bu, uint16_t* y, int M, int N, int K, int bits,
                   int group_size, exo_stream_t stream);

/* K5+K1 fused: the same two operators with mx.fast.rms_norm applied to the input rows
 * on the fly (no separate pass over HBM): x <- bf16(x * rsqrt(mean(x^2)+eps) * norm_weight),
 * norm_weight bf16 [K]; null norm_weight = no normalisation.  This is how a transformer
 * block's `proj(norm(h))` runs in decode.  (rms_norm + nn.QuantizedLinear.__call__) */
int exo_norm_qmv(const uint16_t* x, const uint16_t* norm_weight, float eps, const uint32_t* w,
                 const uint16_t* scales, const uint16_t* biases, const uint16_t* residual,
                 uint16_t* y, int M, int N, int K, int bits, int group_size,
                 exo_stream_t stream);

/* K1 with a workspace for 2 <= M <= 16 rows per tile: K is split over several workgroups
 * per block of 32 output rows and the float32 partial sums meet in `workspace`, so that 16
 * rows fit the LDS at any K and a small N still fills the chip.  exo_qmv_workspace(N)
 * bytes, 256-byte aligned; its first 64 KiB are arrival counters, which the caller zeroes
 * once (every launch leaves them zero; one workspace serves launches of any N up to the N
 * it was sized for).  Launches that share a workspace must be ordered
 * on one stream.  workspace == NULL behaves like exo_norm_qmv.  M == 1 never touches it,
 * nor does M == 2 with K <= 8192 (two rows ride the single-row kernel's two-row tile). */
int64_t exo_qmv_workspace(int N);
int exo_norm_qmv_ws(const uint16_t* x, const uint16_t* norm_weight, float eps,
                    const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                    const uint16_t* residual, uint16_t* y, void* workspace,
                    int64_t workspace_bytes, int M, int N, int K, int bits, int group_size,
                    exo_stream_t stream);
int exo_norm_qmv_swiglu(const uint16_t* x, const uint16_t* norm_weight, float eps,
                        const uint32_t* wg, const uint16_t* sg, const uint16_t* bg,
                        const uint32_t* wu, const uint16_t* su, const uint16_t* bu, uint16_t* y,
                        int M, int N, int K, int bits, int group_size, exo_stream_t stream);
/* exo_norm_qmv_swiglu with the workspace of exo_norm_qmv_ws, sized for both matrices:
 * exo_qmv_workspace(2 * N) bytes.  For 2 <= M <= 16 rows both projections and the
 * SwiGLU (.typings/mlx_lm/models/switch_layers.pyi:52-57) run as one matrix-core launch.
 * workspace == NULL behaves like exo_norm_qmv_swiglu. */
int exo_norm_qmv_swiglu_ws(const uint16_t* x, const uint16_t* norm_weight, float eps,
                           const uint32_t* wg, const uint16_t* sg, const uint16_t* bg,
                           const uint32_t* wu, const uint16_t* su, const uint16_t* bu,
                           uint16_t* y, void* workspace, int64_t workspace_bytes, int M, int N,
                           int K, int bits, int group_size, exo_stream_t stream);

/* K2: the same operator for any M (prefill): weights are dequantised to bf16 in
 * registers and multiplied on the matrix cores, float32 accumulation, bf16 out.
 * (.typings/mlx/core/__init__.pyi:4198-4234) */
int exo_qmm(const uint16_t* x, const uint32_t* w, const uint16_t* scales,
            const uint16_t* biases, const uint16_t* residual, uint16_t* y, int M, int N,
            int K, int bits, int group_size, exo_stream_t stream);
/* exo_qmm with a workspace for launches of few output tiles (fewer than 256 tiles of
 * 128 x 128: a short prompt, or a narrow matrix such as a MoE router under a long one): the
 * tiles alone do not fill the chip, so K is split over up to 8 workgroups per tile, the
 * float32 partial tiles go to `workspace` and a second small launch adds them in a fixed
 * order.  Inputs of up to 32 rows (64 on matrices of 8192 rows or more; matrices of at most
 * 32768 rows) take a 256-column tile whose four waves own 64 weight rows each, with K split
 * up to 16 ways.  exo_qmm_workspace(M, N) bytes (0: this shape never splits),
 * 256-byte aligned, no initialisation needed.  Launches that share a workspace must be
 * ordered on one stream.  workspace == NULL behaves like exo_qmm. */
int64_t exo_qmm_workspace(int M, int N);
int exo_qmm_ws(const uint16_t* x, const uint32_t* w, const uint16_t* scales,
               const uint16_t* biases, const uint16_t* residual, uint16_t* y, void* workspace,
               int64_t workspace_bytes, int M, int N, int K, int bits, int group_size,
               exo_stream_t stream);

/* K2 + K8 for a (gate, up) pair, any M (the prefill form of exo_qmv_swiglu): y[M,N] =
 * silu(x @ dq(w_gate)^T) * (x @ dq(w_up)^T), both projections rounded to bf16 before the
 * SwiGLU - the bits of two exo_qmm calls followed by exo_swiglu, without writing either
 * projection.  Both matrices [N,K].  (mlx_lm llama MLP `down(silu(gate(x)) * up(x))`;
 * `swiglu` .typings/mlx_lm/models/switch_layers.pyi:52-57) */
int exo_qmm_swiglu(const uint16_t* x, const uint32_t* w_gate, const uint16_t* s_gate,
                   const uint16_t* b_gate, const uint32_t* w_up, const uint16_t* s_up,
                   const uint16_t* b_up, uint16_t* y, int M, int N, int K, int bits,
                   int group_size, exo_stream_t stream);
/* exo_qmm_swiglu with a workspace, for inputs of up to 128 rows whose output tiles leave
 * half of the chip or more idle (the MLP of a small model under a short prompt): K is split
 * over up to 8 workgroups per tile, the float32 partials of both projections go to
 * `workspace` and a second small launch adds them in a fixed order, rounds each projection to
 * bf16 and applies the SwiGLU.  exo_qmm_swiglu_workspace(M, N) bytes (0: this shape never
 * splits), 256-byte aligned, no initialisation needed; launches that share it must be ordered
 * on one stream.  workspace == NULL behaves like exo_qmm_swiglu. */
int64_t exo_qmm_swiglu_workspace(int M, int N);
int exo_qmm_swiglu_ws(const uint16_t* x, const uint32_t* w_gate, const uint16_t* s_gate,
                      const uint16_t* b_gate, const uint32_t* w_up, const uint16_t* s_up,
                      const uint16_t* b_up, uint16_t* y, void* workspace,
                      int64_t workspace_bytes, int M, int N, int K, int bits, int group_size,
                      exo_stream_t stream);

/* K3 for prefill-sized T: the same operator as exo_gather_qmv on the matrix cores.  The
 * (token, slot) pairs are first sorted by expert (exo_moe_group, once per routing
 * decision; its workspace of exo_moe_group_workspace(T, topk, E) bytes then serves every
 * exo_gather_qmm of the layer), and each expert's run of rows is multiplied by that
 * expert's matrix in tiles of 128 rows.  x bf16 [T, x_rows, K] with x_rows == 1 or topk;
 * y bf16 [T, topk, N].  What `sorted_indices=True` asks of mx.gather_qmm
 * (.typings/mlx/core/__init__.pyi:2957-3006; .typings/mlx_lm/models/switch_layers.pyi:10-31). */
int64_t exo_moe_group_workspace(int T, int topk, int E);
int exo_moe_group(const int32_t* idx, int T, int topk, int E, void* workspace,
                  int64_t workspace_bytes, exo_stream_t stream);
int exo_gather_qmm(const uint16_t* x, const uint32_t* w, const uint16_t* scales,
                   const uint16_t* biases, const void* workspace, uint16_t* y, int T, int topk,
                   int x_rows, int E, int N, int K, int bits, int group_size,
                   exo_stream_t stream);
/* SwitchGLU's gate and up projections with their swiglu for prefill-sized T, one launch:
 * y[t,j,:] = silu(x @ dq(w_gate[e])^T) * (x @ dq(w_up[e])^T), e = the expert of pair (t,j),
 * both projections rounded to bf16 first - the bits of two exo_gather_qmm calls followed by
 * exo_swiglu.  Same workspace and shapes as exo_gather_qmm; both matrices [E,N,K].
 * (.typings/mlx_lm/models/switch_layers.pyi:52-73) */
int exo_gather_qmm_swiglu(const uint16_t* x, const uint32_t* w_gate, const uint16_t* s_gate,
                          const uint16_t* b_gate, const uint32_t* w_up, const uint16_t* s_up,
                          const uint16_t* b_up, const void* workspace, uint16_t* y, int T,
                          int topk, int x_rows, int E, int N, int K, int bits, int group_size,
                          exo_stream_t stream);

/* K3: mx.gather_qmm(x, w, scales, biases, rhs_indices=idx, transpose=True) as
 * QuantizedSwitchLinear calls it: w uint32 [E,N,K*bits/32]; idx int32 [T,topk];
 * x bf16 [T, x_rows, K] with x_rows == 1 (same row for every slot) or topk;
 * y bf16 [T, topk, N].  Decode-sized T (grouped GEMV).
 * (.typings/mlx/core/__init__.pyi:2957-3006; .typings/mlx_lm/models/switch_layers.pyi:10-31) */
int exo_gather_qmv(const uint16_t* x, const uint32_t* w, const uint16_t* scales,
                   const uint16_t* biases, const int32_t* idx, uint16_t* y, int T, int topk,
                   int x_rows, int E, int N, int K, int bits, int group_size,
                   exo_stream_t stream);

/* K3+K8: SwitchGLU gate/up + swiglu in one pass: y[T,topk,N] =
 * silu(x @ dq(wg[e])^T) * (x @ dq(wu[e])^T), x bf16 [T,K].
 * (.typings/mlx_lm/models/switch_layers.pyi:59-73) */
int exo_gather_qmv_swiglu(const uint16_t* x, const uint32_t* wg, const uint16_t* sg,
                          const uint16_t* bg, const uint32_t* wu, const uint16_t* su,
                          const uint16_t* bu, const int32_t* idx, uint16_t* y, int T,
                          int topk, int E, int N, int K, int bits, int group_size,
                          exo_stream_t stream);

/* exo_gather_qmv_swiglu with rms_norm(x, norm_weight, eps) applied to every token row
 * first (norm_weight == NULL: no norm), so that a MoE block's post-attention norm needs no
 * launch of its own in decode. */
int exo_norm_gather_qmv_swiglu(const uint16_t* x, const uint16_t* norm_weight, float eps,
                               const uint32_t* wg, const uint16_t* sg, const uint16_t* bg,
                               const uint32_t* wu, const uint16_t* su, const uint16_t* bu,
                               const int32_t* idx, uint16_t* y, int T, int topk, int E, int N,
                               int K, int bits, int group_size, exo_stream_t stream);

/* K9+K3+K8 for decode: exo_router_topk and exo_norm_gather_qmv_swiglu in one launch.  Every
 * wave repeats the routing of its token from router_logits bf16 [T,E] (same arithmetic as
 * exo_router_topk: E <= 256, topk <= 16) and streams the expert of its slot; idx_out int32
 * [T,topk] and scores_out bf16 [T,topk] are written for the down projection
 * (exo_gather_qmv_combine).  (qwen3_moe's gate + SwitchGLU,
 * .typings/mlx_lm/models/switch_layers.pyi:59-73) */
int exo_norm_route_gather_qmv_swiglu(const uint16_t* x, const uint16_t* norm_weight, float eps,
                                     const uint16_t* router_logits, int renorm,
                                     int32_t* idx_out, uint16_t* scores_out, const uint32_t* wg,
                                     const uint16_t* sg, const uint16_t* bg, const uint32_t* wu,
                                     const uint16_t* su, const uint16_t* bu, uint16_t* y, int T,
                                     int topk, int E, int N, int K, int bits, int group_size,
                                     exo_stream_t stream);

/* K5: mx.fast.rms_norm with the preceding residual add fused:
 *   h = residual ? bf16(x + residual) : x ;  h_out = h (may be null) ;
 *   n_out = bf16(h * rsqrt(mean(h^2)+eps) * weight).
 * rows x H bf16.  (called by mlx_lm llama/qwen3_moe blocks; no stub in the reference) */
int exo_add_rmsnorm(const uint16_t* x, const uint16_t* residual, const uint16_t* weight,
                    uint16_t* h_out, uint16_t* n_out, int rows, int H, float eps,
                    exo_stream_t stream);

/* K6+K10 (+ Qwen3 q/k-norm): split a fused qkv row into heads, optionally RMS-normalise
 * each q/k head (q_norm_w/k_norm_w bf16 [D] or null), rotate q and k (rotate-half
 * RoPE, angle (pos[b]+t)*inv_freq[i]) and append k,v to the cache at pos[b]+t.
 *   qkv      bf16 [B*T, (Hq+2*Hkv)*D]
 *   q_out    bf16 [B*T, Hq*D]
 *   k_cache/v_cache bf16 [B, Hkv, S_max, D]
 *   pos      int32 [B] on device: tokens already cached per sequence
 *   inv_freq float [D/2]
 * (mx.fast.rope, KVCache.update_and_fetch .typings/mlx_lm/models/cache.pyi:150-169,
 *  rope_utils .typings/mlx_lm/models/rope_utils.pyi:20-51) */
int exo_rope_kv_append(const uint16_t* qkv, uint16_t* q_out, uint16_t* k_cache,
                       uint16_t* v_cache, const int32_t* pos, const float* inv_freq,
                       const uint16_t* q_norm_w, const uint16_t* k_norm_w, float eps, int B,
                       int T, int Hq, int Hkv, int D, int S_max, exo_stream_t stream);

/* The same with the angles' (cos, sin) read from the table exo_rope_table wrote (float
 * [table_rows, D/2, 2]) for positions inside it; positions beyond it, or rope_table == NULL,
 * compute them from inv_freq - the same values either way. */
int exo_rope_kv_append_tab(const uint16_t* qkv, uint16_t* q_out, uint16_t* k_cache,
                           uint16_t* v_cache, const int32_t* pos, const float* inv_freq,
                           const float* rope_table, int table_rows, const uint16_t* q_norm_w,
                           const uint16_t* k_norm_w, float eps, int B, int T, int Hq, int Hkv,
                           int D, int S_max, exo_stream_t stream);

/* K7 decode: scaled_dot_product_attention for one new token per sequence over the
 * cache, grouped-query: q bf16 [B, Hq*D]; lens int32 [B] = pos[b]+1 valid keys;
 * out bf16 [B, Hq*D].  `workspace`: exo_sdpa_decode_workspace(B,Hq,D) bytes, zeroed ONCE
 * by the caller before its first use (it starts with arrival counters that every launch
 * leaves at zero); launches that share a workspace must not overlap.
 * (.typings/mlx_lm/models/base.pyi:39-47) */
int64_t exo_sdpa_decode_workspace(int B, int Hq, int D);
int exo_sdpa_decode(const uint16_t* q, const uint16_t* k_cache, const uint16_t* v_cache,
                    const int32_t* pos, uint16_t* out, float* workspace, float scale, int B,
                    int Hq, int Hkv, int D, int S_max, exo_stream_t stream);

/* exo_sdpa_decode for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid allocation).  No counterpart in the
 * reference.  Same arguments and same results, bit for bit, as exo_sdpa_decode, minus the
 * workspace: the split-KV partials and arrival counters live in a static device array
 * inside the library (about 2.1 MB per GPU, held until the process ends).  The call
 * allocates and frees nothing.  Limit: B * Hq <= EXO_SDPA_DECODE_STATIC_MAX_HEADS query
 * heads per call (head_dim <= 128); larger calls return -1 with a message.  All calls on
 * one GPU share that array: calls that overlap on one GPU (two streams, two threads) race;
 * order them on one stream.  The first call on a device looks the array's address up and
 * must not run under stream capture; later ones may be captured. */
#define EXO_SDPA_DECODE_STATIC_MAX_HEADS 256
int exo_sdpa_decode_static(const uint16_t* q, const uint16_t* k_cache, const uint16_t* v_cache,
                           const int32_t* pos, uint16_t* out, float scale, int B, int Hq,
                           int Hkv, int D, int S_max, exo_stream_t stream);

/* K6+K10+K7 fused for decode: one launch per layer does what exo_rope_kv_append followed
 * by exo_sdpa_decode do for T == 1: q and k heads of the fused qkv row [B,(Hq+2Hkv)*D] are
 * (head-normalised and) rotated at position pos[b], the new k,v are appended to the
 * cache at pos[b], and attention runs over pos[b]+1 keys (pos[b] < S_max, and < the
 * table's S_max when rope_table is given).  Same workspace contract as
 * exo_sdpa_decode.  No separate reference operator: it is rope + update_and_fetch +
 * scaled_dot_product_attention of one attention block. */
int exo_attn_decode(const uint16_t* qkv, uint16_t* k_cache, uint16_t* v_cache,
                    const int32_t* pos, const float* inv_freq, const float* rope_table,
                    const uint16_t* q_norm_w, const uint16_t* k_norm_w, float eps, uint16_t* out,
                    float* workspace, float scale, int B, int Hq, int Hkv, int D, int S_max,
                    exo_stream_t stream);

/* exo_attn_decode with the host's knowledge of the context: keys_hint = the number of keys
 * the longest sequence of this step holds, as far as the host knows (0: unknown, which is
 * exo_attn_decode).  From EXO_ATTN_LONG_KEYS keys on (in a cache at least that long) the
 * launch is laid out for long contexts: the matrix-core kernel whatever the head count
 * (already from EXO_ATTN_MID_KEYS on when B * n_kv_heads is 16 or more); from
 * EXO_ATTN_VERY_LONG_KEYS on with the keys of a kv head over up to 32 workgroups instead of
 * 16.  The hint only selects the layout - any value gives a correct result for any pos[] -
 * so a captured launch stays valid while the context grows; the layouts round differently
 * (within the tolerance of the attention tests). */
#define EXO_ATTN_MID_KEYS 3072
#define EXO_ATTN_LONG_KEYS 6144
#define EXO_ATTN_VERY_LONG_KEYS 12288
int exo_attn_decode_hint(const uint16_t* qkv, uint16_t* k_cache, uint16_t* v_cache,
                         const int32_t* pos, const float* inv_freq, const float* rope_table,
                         const uint16_t* q_norm_w, const uint16_t* k_norm_w, float eps,
                         uint16_t* out, float* workspace, float scale, int B, int Hq, int Hkv,
                         int D, int S_max, int keys_hint, exo_stream_t stream);

/* (cos, sin) of position*inv_freq[i] for every position < S_max: float [S_max, D/2, 2],
 * the same sincosf values the RoPE kernels compute inline.  Passing it to
 * exo_attn_decode (may be null there) replaces 8 sincosf per lane by one 64-byte load. */
int exo_rope_table(const float* inv_freq, float* table, int S_max, int D, exo_stream_t stream);

/* K7 prefill: causal attention of T new tokens per sequence (already appended to the
 * cache) over pos[b]+T keys.  q bf16 [B*T, Hq*D] -> out same shape. */
int exo_sdpa_prefill(const uint16_t* q, const uint16_t* k_cache, const uint16_t* v_cache,
                     const int32_t* pos, uint16_t* out, float scale, int B, int T, int Hq,
                     int Hkv, int D, int S_max, exo_stream_t stream);

/* Disaggregated prefill, export: positions [start, start+n) of one layer's cache row
 * ([Hkv, S_max, D] bf16) -> wire layout [n, Hkv, D] bf16, the `bhsd_to_nhd` transpose of
 * src/exo/worker/engines/mlx/disaggregated/adapter.py:74-77,103-109.  D % 8 == 0,
 * 16-byte aligned pointers. */
int exo_kv_export_nhd(const uint16_t* cache_row, uint16_t* wire, int Hkv, int S_max, int D,
                      int start, int n, exo_stream_t stream);

/* Disaggregated prefill, ingest: wire [n, Hkv, D] -> positions [start, start+n) of a cache
 * row (`nhd_to_bhsd` + `inject_kv_chunk`, adapter.py:80-83,182-201). */
int exo_kv_import_nhd(const uint16_t* wire, uint16_t* cache_row, int Hkv, int S_max, int D,
                      int start, int n, exo_stream_t stream);

/* K8: swiglu(gate, up) = silu(gate)*up elementwise, n elements.
 * (.typings/mlx_lm/models/switch_layers.pyi:52-57) */
int exo_swiglu(const uint16_t* gate, const uint16_t* up, uint16_t* out, int64_t n,
               exo_stream_t stream);

/* K9: Qwen3-MoE routing: softmax over E experts (float32, rounded to bf16), the k
 * largest (ties to the lower id, slots in descending score), optional renormalisation.
 * logits bf16 [rows,E] -> idx int32 [rows,k], scores bf16 [rows,k].  E <= 256, k <= 16. */
int exo_router_topk(const uint16_t* logits, int32_t* idx, uint16_t* scores, int rows, int E,
                    int k, int renorm, exo_stream_t stream);

/* K3 (down projection of SwitchGLU, decode) fused with the block's weighted sum over
 * the top-k experts and the residual: out[t,:] = bf16(bf16(sum_j bf16(bf16(x[t,j,:] @
 * dq(w[idx[t,j]])^T) * scores[t,j])) + residual[t,:]), the rounding points of
 * exo_gather_qmv followed by exo_moe_combine.  x bf16 [T,topk,K], out bf16 [T,N].
 * Shapes outside the fused kernel (topk > 8, or rows of more than 4 chunks per lane) run
 * those two calls through `scratch` (bf16 [T,topk,N]); scratch may be NULL otherwise.
 * (.typings/mlx/core/__init__.pyi:2957-3006; .typings/mlx_lm/models/switch_layers.pyi:59-73) */
int exo_gather_qmv_combine(const uint16_t* x, const uint32_t* w, const uint16_t* scales,
                           const uint16_t* biases, const int32_t* idx, const uint16_t* scores,
                           const uint16_t* residual, uint16_t* out, uint16_t* scratch, int T,
                           int topk, int E, int N, int K, int bits, int group_size,
                           exo_stream_t stream);

/* MoE combine: out[t,:] = bf16( sum_j bf16(y[t,j,:] * scores[t,j]) ) (+ residual[t,:]
 * added in bf16 when non-null).  y bf16 [T,topk,H]. */
int exo_moe_combine(const uint16_t* y, const uint16_t* scores, const uint16_t* residual,
                    uint16_t* out, int T, int topk, int H, exo_stream_t stream);

/* A9 (src/exo/worker/engines/mlx/patches/opt_batch_gen.py:67-88, greedy sampler):
 * per row of bf16 logits [rows,V]: token = argmax (lowest index on ties),
 * lse = logsumexp (float32), logprob of the token.  `workspace` float,
 * exo_argmax_workspace(rows) bytes.  If pos_inc is non-null, pos_inc[r] += 1 for
 * every row (advances the per-sequence cache position for the next graph replay). */
int64_t exo_argmax_workspace(int rows);
int exo_argmax_logsumexp(const uint16_t* logits, int32_t* token, float* lse, float* logprob,
                         float* workspace, int32_t* pos_inc, int rows, int V,
                         exo_stream_t stream);

/* A9, whole: everything between the model call and the next token in the reference's
 * decode step (src/exo/worker/engines/mlx/patches/opt_batch_gen.py:67-107): the logits
 * processors of each sequence (token bans src/exo/worker/engines/mlx/generator/
 * generate.py:465-473; repetition / presence / frequency penalties, make_logits_processors
 * .typings/mlx_lm/sample_utils.pyi:47-72 as called at generate.py:599-608),
 * logprobs = logits - logsumexp(logits), the sequence's sampler (make_sampler
 * .typings/mlx_lm/sample_utils.pyi:10-45 with the defaults of generate.py:614-619:
 * temperature, top-p, min-p, top-k) and the 20 most likely tokens (opt_batch_gen.py:93-107).
 *
 * Per row r of bf16 logits [rows, V]:
 *   x = logits[r] with the processors applied, each rounding its result to bf16: banned ids
 *       -> -1e9; tokens among the last repetition_context of the history: x/penalty if
 *       x >= 0 else x*penalty; among the last presence_context: x - presence_penalty;
 *       x - frequency_penalty * (occurrences among the last frequency_context);
 *   lse = logsumexp(x) (float32);
 *   temperature == 0: token = argmax x (lowest id on ties);
 *   else token i is kept iff x_i >= max(t_p, t_m, t_k): t_p the smallest value whose tokens
 *       of strictly larger value hold less than top_p of the probability mass, t_m =
 *       max(x) + log(min_p), t_k the k-th largest value; token = inverse CDF, in vocabulary
 *       order, of the weights exp((x - max) / temperature) over the kept tokens at the
 *       uniform u = (first word of Philox-4x32-10(counter = (draws[r],0,0,0), key =
 *       (seed_lo, seed_hi)) >> 8) * 2^-24; draws[r] += 1;
 *   logprob[r] = x[token] - lse;  top_idx/top_val [rows,20]: the 20 largest x, descending
 *       (lower id first among equals), as ids and x - lse;
 *   history[r][hist_len[r] % hist_cap] = token, hist_len[r] += 1 (history int32
 *       [rows, hist_cap]: a ring of the sequence's latest tokens, prompt included);
 *   feedback[r] = token (the next step's input id), pos_inc[r] += 1 - each when non-null.
 * `mode` says which launches the rows need (rows whose parameters do not ask for a stage
 * pass through it untouched): EDITS if any row bans or penalises, DRAW if any row has
 * temperature != 0, TABLE if any sampling row uses top_p in (0,1) or top_k > 0, TOP for
 * the top-20 outputs.  workspace: exo_sample_workspace(rows) bytes, 256-byte aligned,
 * zeroed ONCE by the caller (every call leaves its tables zero); calls that share it must
 * be ordered on one stream.  V <= 262144; contexts <= hist_cap <= 256. */
#define EXO_SAMPLER_MAX_CONTEXT 256
#define EXO_SAMPLER_MAX_BANNED 8
#define EXO_SAMPLER_TOP_LOGPROBS 20
#define EXO_SAMPLE_EDITS 1
#define EXO_SAMPLE_DRAW 2
#define EXO_SAMPLE_TABLE 4
#define EXO_SAMPLE_TOP 8
typedef struct exo_sampler_params {
  float temperature;        /* 0: greedy */
  float top_p;              /* in (0,1): nucleus filter; anything else: off */
  float min_p;              /* > 0: keep p >= min_p * max p */
  int32_t top_k;            /* > 0: keep the k most likely */
  float repetition_penalty; /* 0 or 1: off */
  int32_t repetition_context;
  float presence_penalty;   /* 0: off */
  int32_t presence_context;
  float frequency_penalty;  /* 0: off */
  int32_t frequency_context;
  uint32_t seed_lo, seed_hi;
  int32_t n_banned;         /* <= EXO_SAMPLER_MAX_BANNED */
  int32_t banned[EXO_SAMPLER_MAX_BANNED];
} exo_sampler_params;
int64_t exo_sample_workspace(int rows);
int exo_sample(const uint16_t* logits, const exo_sampler_params* params, int32_t* history,
               int32_t* hist_len, uint32_t* draws, int32_t* token, float* logprob, float* lse,
               int32_t* top_idx, float* top_val, int32_t* feedback, int32_t* pos_inc,
               void* workspace, int64_t workspace_bytes, int rows, int V, int hist_cap, int mode,
               exo_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif
