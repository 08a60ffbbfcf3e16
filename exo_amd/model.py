"""The per-shard transformer forward over a contiguous layer range.

What the reference obtains from mlx_lm's ``llama.Model`` / ``qwen3_moe.Model`` after
``pipeline_auto_parallel`` has kept ``layers[start:end]``
(src/exo/worker/engines/mlx/auto_parallel.py:276-395), behind the ``Model`` protocol
of src/exo/worker/engines/mlx/types.py:29-37: ``model(tokens, cache,
input_embeddings=None)``.  The first shard embeds the tokens, every other shard
receives the hidden state [B,T,H] (what PipelineFirstLayer would ``recv_like``,
auto_parallel.py:132-139); the last shard applies the final norm and lm_head, every
other one returns the hidden state leaving its last local layer.

Every operator is a HIP kernel reached through the C ABI (exo_amd.ops).  Single-token
steps (B*T <= 16 rows) use the fused dequant-GEMV family and can be replayed from a
HIP graph (``decode_step``); longer inputs use the matrix-core GEMM and the causal
prefill attention.
"""

from __future__ import annotations

import contextlib
import gc
import math

import torch

from . import ops
from .cache import ShardKVCache
from .config import ModelConfig
from .ops import QuantizedWeight

GEMV_MAX_ROWS = ops.QMV_MAX_M


@contextlib.contextmanager
def capture_graph(graph: "torch.cuda.CUDAGraph"):
    """``torch.cuda.graph(graph)`` with Python's garbage collector held off while the stream
    records: a collected object that owns pinned host memory, an event or another graph makes
    runtime calls in its destructor that a recording stream does not allow, and the process
    aborts.  What is garbage by then waits for the first collection after the recording.  (No
    forced collection in front of it either: the memory that one hands back moves the
    allocations that follow, and launches timed afterwards ran 5 % slower.)"""
    was_on = gc.isenabled()
    gc.disable()
    try:
        with torch.cuda.graph(graph):
            yield
    finally:
        if was_on:
            gc.enable()


def rope_inv_freq(cfg: ModelConfig) -> torch.Tensor:
    """Per-pair inverse frequencies (float32, CPU): theta^(-2i/d), with the llama3
    piecewise rescale of mlx_lm's Llama3RoPE (.typings/mlx_lm/models/rope_utils.pyi:20-51)."""
    d = cfg.head_dim
    inv = 1.0 / (cfg.rope_theta ** (torch.arange(0, d, 2, dtype=torch.float64) / d))
    sc = cfg.rope_scaling
    if sc and sc.get("rope_type", sc.get("type")) == "llama3":
        factor = float(sc["factor"])
        lo = float(sc.get("low_freq_factor", 1.0))
        hi = float(sc.get("high_freq_factor", 4.0))
        old = float(sc.get("original_max_position_embeddings", 8192))
        wl = 2 * math.pi / inv
        scaled = torch.where(wl > old / lo, inv / factor, inv)
        smooth = (old / wl - lo) / (hi - lo)
        mid = (1 - smooth) * inv / factor + smooth * inv
        is_mid = (wl <= old / lo) & (wl >= old / hi)
        inv = torch.where(is_mid, mid, scaled)
    elif sc and sc.get("rope_type", sc.get("type")) not in (None, "default", "linear"):
        raise ValueError(f"rope_scaling {sc} not supported")
    if sc and sc.get("rope_type", sc.get("type")) == "linear":
        inv = inv / float(sc["factor"])
    return inv.to(torch.float32)


def _qw(w: dict, prefix: str, cfg: ModelConfig) -> QuantizedWeight:
    """The (weight, scales, biases) triple under ``prefix``; the bit width comes from the
    tensor shapes, so per-module overrides of the checkpoint's quantisation are honoured
    and a malformed tensor fails here, at load, not at the first forward."""
    return QuantizedWeight.from_tensors(w[prefix + ".weight"], w[prefix + ".scales"],
                                        w[prefix + ".biases"], cfg.group_size, prefix)


class _Layer:
    """Weights of one transformer block (device resident)."""

    def __init__(self, cfg: ModelConfig, w: dict, i: int):
        p = f"model.layers.{i}."

        def q(name: str) -> QuantizedWeight:
            return _qw(w, p + name, cfg)

        self.index = i
        self.in_norm = w[p + "input_layernorm.weight"]
        self.post_norm = w[p + "post_attention_layernorm.weight"]
        qp, kp, vp = q("self_attn.q_proj"), q("self_attn.k_proj"), q("self_attn.v_proj")
        if not (qp.bits == kp.bits == vp.bits):
            raise ValueError(f"{p}self_attn: q/k/v projections quantised at different widths "
                             f"({qp.bits}/{kp.bits}/{vp.bits} bits) cannot share one launch")
        bits = qp.bits
        # q|k|v concatenated along the output rows: one launch instead of three
        self.qkv = QuantizedWeight(
            torch.cat([qp.weight, kp.weight, vp.weight]).contiguous(),
            torch.cat([qp.scales, kp.scales, vp.scales]).contiguous(),
            torch.cat([qp.biases, kp.biases, vp.biases]).contiguous(), bits, cfg.group_size)
        self.o = q("self_attn.o_proj")
        self.q_norm = w.get(p + "self_attn.q_norm.weight")
        self.k_norm = w.get(p + "self_attn.k_norm.weight")
        if cfg.is_moe:
            self.router = q("mlp.gate")
            self.gate = q("mlp.switch_mlp.gate_proj")
            self.up = q("mlp.switch_mlp.up_proj")
            self.down = q("mlp.switch_mlp.down_proj")
        else:
            self.gate, self.up, self.down = q("mlp.gate_proj"), q("mlp.up_proj"), q("mlp.down_proj")

    def nbytes(self) -> int:
        n = self.qkv.nbytes + self.o.nbytes + self.gate.nbytes + self.up.nbytes + self.down.nbytes
        return n + (self.router.nbytes if hasattr(self, "router") else 0)


class _Buffers:
    """Activation workspace for R = B*T rows."""

    def __init__(self, m: "ShardModel", R: int, B: int, device):
        c = m.cfg
        bf = dict(dtype=torch.bfloat16, device=device)
        Hq, Hkv, D = c.num_attention_heads, c.num_key_value_heads, c.head_dim
        self.R = R
        self.tokens = torch.zeros(R, dtype=torch.int32, device=device)
        self.h = torch.empty(R, c.hidden_size, **bf)
        self.n = torch.empty(R, c.hidden_size, **bf)
        self.qkv = torch.empty(R, (Hq + 2 * Hkv) * D, **bf)
        self.q = torch.empty(R, Hq * D, **bf)
        self.attn = torch.empty(R, Hq * D, **bf)
        if c.is_moe:
            k, Ie = c.num_experts_per_tok, c.moe_intermediate_size
            self.router_logits = torch.empty(R, c.num_experts, **bf)
            self.act = torch.empty(R, k, Ie, **bf)
            self.expert_out = torch.empty(R, k, c.hidden_size, **bf)
            self.gate = self.up = None
        else:
            self.act = torch.empty(R, c.intermediate_size, **bf)
            self.gate = self.up = None
        self.sdpa_ws = ops.sdpa_decode_workspace(B, Hq, D, device)
        # sampling outputs (last shard)
        self.logits = None
        self.next_token = torch.zeros(B, dtype=torch.int32, device=device)
        self.lse = torch.zeros(B, dtype=torch.float32, device=device)
        self.logprob = torch.zeros(B, dtype=torch.float32, device=device)
        self.argmax_ws = ops.argmax_workspace(B, device)


class ShardModel:
    def __init__(self, cfg: ModelConfig, weights: dict[str, torch.Tensor], start_layer: int = 0,
                 end_layer: int | None = None, device="cuda:0"):
        self.cfg = cfg
        self.device = torch.device(device)
        self.start_layer = start_layer
        self.end_layer = cfg.num_hidden_layers if end_layer is None else end_layer
        if not (0 <= self.start_layer < self.end_layer <= cfg.num_hidden_layers):
            raise ValueError(f"bad layer range [{start_layer},{end_layer}) of {cfg.num_hidden_layers}")
        self.layers = [_Layer(cfg, weights, i) for i in range(self.start_layer, self.end_layer)]
        self.embed_tokens = None
        if self.is_first or (self.is_last and cfg.tie_word_embeddings):
            self.embed_tokens = _qw(weights, "model.embed_tokens", cfg)
        self.norm = self.lm_head = None
        if self.is_last:
            self.norm = weights["model.norm.weight"]
            self.lm_head = self.embed_tokens if cfg.tie_word_embeddings else _qw(
                weights, "lm_head", cfg)
        self.inv_freq = rope_inv_freq(cfg).to(self.device)
        self.scale = cfg.head_dim ** -0.5
        # inputs of up to this many rows take the GEMV family with fused norms; 8-bit
        # weights switch to the GEMM (separate norm launch) above 8 rows, where it is faster
        self.gemv_rows = GEMV_MAX_ROWS if cfg.bits == 4 else 8
        self._bufs: dict[tuple[int, int], _Buffers] = {}
        self._graphs: dict[int, tuple] = {}
        self._rope_tab: torch.Tensor | None = None
        self._retired_rope_tabs: list[torch.Tensor] = []

    # ------------------------------------------------------------------ properties
    @property
    def is_first(self) -> bool:
        return self.start_layer == 0

    @property
    def is_last(self) -> bool:
        return self.end_layer == self.cfg.num_hidden_layers

    def _rope_table(self, n: int) -> torch.Tensor:
        """(cos, sin) table covering n positions, built once on the device."""
        if self._rope_tab is None or self._rope_tab.shape[0] < n:
            if self._rope_tab is not None:  # a captured graph may still point at the old table
                self._retired_rope_tabs.append(self._rope_tab)
            self._rope_tab = ops.rope_table(self.inv_freq, n, self.cfg.head_dim)
        return self._rope_tab

    def weight_bytes(self) -> int:
        n = sum(l.nbytes() for l in self.layers)
        if self.lm_head is not None:
            n += self.lm_head.nbytes
        return n

    def make_cache(self, batch: int = 1, max_seq: int = 4096) -> ShardKVCache:
        c = self.cfg
        return ShardKVCache(len(self.layers), batch, c.num_key_value_heads, c.head_dim, max_seq,
                            self.device)

    def _buffers(self, B: int, T: int) -> _Buffers:
        key = (B, T)
        if key not in self._bufs:
            if T > 1 and len(self._bufs) > 8:  # prefill shapes vary; do not hoard them
                for k in [k for k in self._bufs if k[1] > 1]:
                    del self._bufs[k]
            self._bufs[key] = _Buffers(self, B * T, B, self.device)
        return self._bufs[key]

    # ------------------------------------------------------------------ the forward
    def _mlp(self, L: _Layer, bf: _Buffers, R: int) -> None:
        """h <- h + mlp(post_norm(h)) in place; bf.n holds the normed input."""
        c = self.cfg
        gemv = R <= (GEMV_MAX_ROWS if c.is_moe else self.gemv_rows)
        if not c.is_moe:
            if gemv:  # post-attention norm and SwiGLU fused into the gate/up GEMV pair
                ops.qmv_swiglu(bf.h, L.gate, L.up, out=bf.act, norm_weight=L.post_norm,
                               eps=c.rms_norm_eps)
            elif R >= 64:  # one GEMM launch for both projections, SwiGLU in its epilogue
                ops.qmm_swiglu(bf.n, L.gate, L.up, out=bf.act)
            else:  # up to 63 rows: the 256-column split-K GEMM per projection is faster
                #   (8192x2048 at 126 rows: pair 27 us, two GEMMs + SwiGLU 44 us; at 32 rows 28 / 29
                #   us; 14336x4096 at 32 rows 58 / 46 us, at 64 rows 57 / 59 us)
                if bf.gate is None:
                    bf.gate = torch.empty_like(bf.act)
                    bf.up = torch.empty_like(bf.act)
                ops.quantized_matmul(bf.n, L.gate, out=bf.gate)
                ops.quantized_matmul(bf.n, L.up, out=bf.up)
                ops.swiglu(bf.gate, bf.up, out=bf.act)
            ops.quantized_matmul(bf.act, L.down, residual=bf.h, out=bf.h)
            return
        if gemv:  # decode: the post-attention norm is fused into both consumers of it
            ops.quantized_matmul(bf.h, L.router, out=bf.router_logits, norm_weight=L.post_norm,
                                 eps=c.rms_norm_eps)
        else:
            ops.quantized_matmul(bf.n, L.router, out=bf.router_logits)
        k = c.num_experts_per_tok
        if gemv and c.num_experts <= 256 and k <= 16:
            # decode: the gate/up launch routes by itself (every wave repeats the top-k of its
            # token from the logits), one launch fewer per layer.  Qwen3-30B, separate top-k
            # launch -> routing inside: batch 1 543 -> 574 tok/s on the build that introduced
            # it; 2 rows 973 -> 1025, 4 rows 1399 -> 1455, 8 rows 2115 -> 2178, 16 rows
            # 2987 -> 3050 on the current one.
            idx, sc, _ = ops.route_gather_qmv_swiglu(
                bf.h, bf.router_logits, k, c.norm_topk_prob, L.gate, L.up, out=bf.act,
                norm_weight=L.post_norm, eps=c.rms_norm_eps)
            ops.gather_qmv_combine(bf.act, L.down, idx, sc, residual=bf.h, out=bf.h,
                                   scratch=bf.expert_out, check_indices=False)
            return
        idx, sc = ops.router_topk(bf.router_logits, c.num_experts_per_tok, c.norm_topk_prob)
        if not gemv:  # prefill: rows sorted by expert; gate, up and SwiGLU in one grouped GEMM
            ws = ops.moe_group(idx, c.num_experts, check_indices=False)  # ids from router_topk
            ops.grouped_qmm_swiglu(bf.n.view(R, 1, -1), L.gate, L.up, ws, k, out=bf.act)
            ops.grouped_qmm(bf.act, L.down, ws, k, out=bf.expert_out)
            ops.moe_combine(bf.expert_out, sc, residual=bf.h, out=bf.h)
            return
        ops.gather_qmv_swiglu(bf.h, L.gate, L.up, idx, out=bf.act, norm_weight=L.post_norm,
                              eps=c.rms_norm_eps, check_indices=False)
        ops.gather_qmv_combine(bf.act, L.down, idx, sc, residual=bf.h, out=bf.h,
                               scratch=bf.expert_out, check_indices=False)

    @staticmethod
    def _keys_hint(cache: ShardKVCache, rsl: slice) -> int:
        """The context regime of a decode step from the host's count of the longest sequence
        (0 or the threshold reached): the attention launch is laid out per regime, and a
        captured step stays valid inside one."""
        n = max(cache.offsets[rsl]) + 1
        return (ops.ATTN_VERY_LONG_KEYS if n >= ops.ATTN_VERY_LONG_KEYS else
                ops.ATTN_LONG_KEYS if n >= ops.ATTN_LONG_KEYS else
                ops.ATTN_MID_KEYS if n >= ops.ATTN_MID_KEYS else 0)

    def _run(self, B: int, T: int, cache: ShardKVCache, bf: _Buffers, logits_mode: str,
             rows: slice | None = None):
        """Launch the shard forward for B sequences x T tokens on the current stream.
        Input: bf.tokens (first shard) or bf.h (other shards).  KV rows ``rows`` of the
        cache are used (default: the first B)."""
        c = self.cfg
        R = B * T
        Hq, Hkv, D = c.num_attention_heads, c.num_key_value_heads, c.head_dim
        rsl = rows if rows is not None else slice(0, B)
        pos = cache.pos[rsl]
        keys_hint = self._keys_hint(cache, rsl)
        if self.is_first:
            ops.embed(bf.tokens, self.embed_tokens, out=bf.h)
        gemv = R <= self.gemv_rows                                       # qkv, o, lm_head
        mlp_gemv = R <= (GEMV_MAX_ROWS if c.is_moe else self.gemv_rows)  # see _mlp
        for li, L in enumerate(self.layers):
            kc, vc = cache.k[li][rsl], cache.v[li][rsl]
            if gemv:  # input norm fused into the q|k|v GEMV
                ops.quantized_matmul(bf.h, L.qkv, out=bf.qkv, norm_weight=L.in_norm,
                                     eps=c.rms_norm_eps)
            else:
                ops.rms_norm(bf.h, L.in_norm, c.rms_norm_eps, out=bf.n)
                ops.quantized_matmul(bf.n, L.qkv, out=bf.qkv)
            if T == 1:  # rope + append + attention in one launch
                ops.attn_decode(bf.qkv, kc, vc, pos, self.inv_freq, bf.attn, bf.sdpa_ws, self.scale,
                                B, Hq, Hkv, D, L.q_norm, L.k_norm, c.rms_norm_eps,
                                rope_tab=self._rope_table(cache.max_seq), keys_hint=keys_hint)
            else:
                ops.rope_kv_append(bf.qkv, bf.q, kc, vc, pos, self.inv_freq, B, T, Hq, Hkv, D,
                                   L.q_norm, L.k_norm, c.rms_norm_eps,
                                   rope_tab=self._rope_table(cache.max_seq))
                ops.sdpa_prefill(bf.q, kc, vc, pos, bf.attn, self.scale, B, T, Hq, Hkv, D)
            ops.quantized_matmul(bf.attn, L.o, residual=bf.h, out=bf.h)
            if not mlp_gemv:
                ops.rms_norm(bf.h, L.post_norm, c.rms_norm_eps, out=bf.n)
            self._mlp(L, bf, R)
        if not self.is_last or logits_mode == "none":
            return bf.h
        hl = bf.h.view(B, T, -1)[:, -1].contiguous() if (logits_mode == "last" and T > 1) else bf.h
        rows = hl.shape[0]
        if bf.logits is None or bf.logits.shape[0] != rows:
            bf.logits = torch.empty(rows, c.vocab_size, dtype=torch.bfloat16, device=self.device)
        if rows <= self.gemv_rows:  # final norm fused into the lm_head GEMV
            ops.quantized_matmul(hl, self.lm_head, out=bf.logits, norm_weight=self.norm,
                                 eps=c.rms_norm_eps)
        else:
            n = ops.rms_norm(hl, self.norm, c.rms_norm_eps)
            ops.quantized_matmul(n, self.lm_head, out=bf.logits)
        return bf.logits

    def __call__(self, tokens: torch.Tensor | None, cache: ShardKVCache,
                 input_embeddings: torch.Tensor | None = None, logits: str = "all",
                 rows: slice | None = None) -> torch.Tensor:
        """tokens int [B,T] (first shard) or input_embeddings bf16 [B,T,H] (other shards).
        Appends T entries to the cache rows.  Returns bf16 logits [B,T,V] ("all"),
        [B,1,V] ("last") on the last shard, else the hidden state [B,T,H]."""
        if self.is_first:
            assert tokens is not None
            B, T = tokens.shape
        else:
            assert input_embeddings is not None
            B, T = input_embeddings.shape[:2]
        nrows = (rows.stop - rows.start) if rows is not None else B
        if nrows != B or B > cache.batch:
            raise ValueError(f"batch {B} does not match cache rows {nrows} (cache batch {cache.batch})")
        r0 = rows.start if rows is not None else 0
        if max(cache.offsets[r0 : r0 + B]) + T > cache.max_seq:
            raise ValueError(f"KV cache overflow: {max(cache.offsets[r0:r0 + B])}+{T} > {cache.max_seq}")
        bf = self._buffers(B, T)
        if self.is_first:
            bf.tokens.copy_(tokens.reshape(-1).to(torch.int32))
        else:
            bf.h.copy_(input_embeddings.reshape(B * T, -1))
        out = self._run(B, T, cache, bf, logits if self.is_last else "none", rows)
        cache.pos[r0 : r0 + B] += T
        cache.advance_host(T, range(r0, r0 + B))
        if self.is_last and logits != "none":
            return out.view(B, -1, self.cfg.vocab_size).clone()
        return out.view(B, T, -1).clone()

    # ------------------------------------------------------------------ graph decode
    def decode_step(self, cache: ShardKVCache, B: int, use_graph: bool = True,
                    feedback: bool = False, sampler=None, mode: int = 0, row0: int = 0) -> _Buffers:
        """One single-token step for cache rows [row0, row0+B): reads ``bufs.tokens`` (first shard)
        or ``bufs.h``, leaves logits / next_token / lse / logprob (last shard) or the
        hidden state in the returned buffers, advances the device positions.  The kernel
        sequence is captured once per B into a HIP graph and replayed.  ``feedback``
        (last shard): the graph also writes the chosen token into ``tokens``, so steps
        can be chained without the host.  ``sampler`` (a DeviceSampler, last shard): the step
        ends in the device sampling kernels with the stages ``mode`` names instead of the
        plain argmax; results are then in the sampler's ``token`` / ``logprob`` / ``top_*``."""
        bf = self._buffers(B, 1)
        rsl = slice(row0, row0 + B)
        if row0 < 0 or row0 + B > cache.batch:
            raise ValueError(f"rows [{row0}, {row0 + B}) outside the cache's {cache.batch} rows")
        if max(cache.offsets[rsl]) + 1 > cache.max_seq:
            raise ValueError("KV cache overflow")
        if sampler is not None and not self.is_last:
            raise ValueError("sampling needs the shard that holds the lm_head")
        if sampler is not None and row0 != 0:
            raise ValueError("the sampling state is indexed by cache row: row0 must be 0 with a sampler")

        def body():
            out = self._run(B, 1, cache, bf, "all", rsl if row0 else None)
            if self.is_last and sampler is not None:
                sampler.sample(out, B, mode, feedback=bf.tokens if feedback else None,
                               pos_inc=cache.pos[rsl])
            elif self.is_last:
                ops.argmax_logsumexp(out, bf.next_token, bf.lse, bf.logprob, bf.argmax_ws,
                                     cache.pos[rsl])
                if feedback:
                    bf.tokens.copy_(bf.next_token)
            else:
                cache.pos[rsl] += 1

        if not use_graph:
            body()
        else:
            key = (B, feedback, sampler is not None, mode, row0, self._keys_hint(cache, rsl))
            hit = self._graphs.get(key)
            if hit is None or hit[1] is not cache or hit[2] is not sampler:
                # warm up outside capture (lazy module loads, attribute settings), then
                # restore what the warm-up changed: the positions it advanced, the hidden
                # state a later shard adds its residuals into in place, the input tokens
                # the feedback overwrote, the sampler's counters and history ring
                saved = cache.pos.clone()
                saved_in = bf.tokens.clone() if self.is_first else bf.h.clone()
                saved_sampler = sampler.snapshot() if sampler is not None else None
                s = torch.cuda.Stream()
                s.wait_stream(torch.cuda.current_stream())
                with torch.cuda.stream(s):
                    body()
                torch.cuda.current_stream().wait_stream(s)
                torch.cuda.synchronize()
                cache.pos.copy_(saved)
                (bf.tokens if self.is_first else bf.h).copy_(saved_in)
                if sampler is not None:
                    sampler.restore(saved_sampler)
                g = torch.cuda.CUDAGraph()
                with capture_graph(g):
                    body()
                cache.pos.copy_(saved)
                self._graphs[key] = (g, cache, sampler)
            self._graphs[key][0].replay()
        cache.advance_host(1, range(row0, row0 + B))
        return bf
