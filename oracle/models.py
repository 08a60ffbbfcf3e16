"""Llama and Qwen3-MoE shard forward + the reference's generation protocol (CPU).

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

Restates, for a contiguous layer range [start, end):
  * the model forward the reference obtains from mlx_lm (module tree corroborated by
    src/exo/worker/engines/mlx/auto_parallel.py:209-243,638-648,1249-1259), with the
    layer slicing of pipeline_auto_parallel (auto_parallel.py:276-395): the first
    shard embeds, the last applies the final norm and lm_head, every other boundary
    passes the hidden state [B,T,H];
  * one KV cache per LOCAL layer (src/exo/worker/engines/mlx/cache.py:560-581);
  * prefill / trim(2) / re-feed of the last two prompt tokens
    (src/exo/worker/engines/mlx/generator/generate.py:282-396,666-733).

Weights are a dict of numpy arrays keyed by MLX checkpoint tensor names
(``model.layers.{i}.self_attn.q_proj.{weight,scales,biases}`` ...).  Activations are
float32 arrays holding bf16-representable values; every op rounds once to bf16.
"""

from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np

from . import affine, ops
from .affine import act_round as bf16_round
from .affine import bf16_bits_to_f32


@dataclass
class Config:
    model_type: str = "llama"
    hidden_size: int = 64
    num_hidden_layers: int = 2
    num_attention_heads: int = 4
    num_key_value_heads: int = 2
    head_dim: int = 16
    intermediate_size: int = 128
    vocab_size: int = 256
    rms_norm_eps: float = 1e-5
    rope_theta: float = 500000.0
    rope_scaling: dict | None = None
    tie_word_embeddings: bool = False
    group_size: int = 64
    bits: int = 4
    num_experts: int = 0
    num_experts_per_tok: int = 0
    moe_intermediate_size: int = 0
    norm_topk_prob: bool = True

    @staticmethod
    def from_json(d: dict) -> "Config":
        q = d.get("quantization", d.get("quantization_config", {})) or {}
        hd = d.get("head_dim") or d["hidden_size"] // d["num_attention_heads"]
        return Config(
            model_type=d["model_type"],
            hidden_size=d["hidden_size"],
            num_hidden_layers=d["num_hidden_layers"],
            num_attention_heads=d["num_attention_heads"],
            num_key_value_heads=d.get("num_key_value_heads", d["num_attention_heads"]),
            head_dim=hd,
            intermediate_size=d.get("intermediate_size", 0),
            vocab_size=d["vocab_size"],
            rms_norm_eps=d.get("rms_norm_eps", 1e-5),
            rope_theta=d.get("rope_theta", 10000.0),
            rope_scaling=d.get("rope_scaling"),
            tie_word_embeddings=d.get("tie_word_embeddings", False),
            group_size=q.get("group_size", 64),
            bits=q.get("bits", 4),
            num_experts=d.get("num_experts", 0),
            num_experts_per_tok=d.get("num_experts_per_tok", 0),
            moe_intermediate_size=d.get("moe_intermediate_size", 0),
            norm_topk_prob=d.get("norm_topk_prob", True),
        )


@dataclass
class LayerKV:
    """Plain bf16 KV cache for one layer (mlx_lm KVCache: update_and_fetch / trim,
    .typings/mlx_lm/models/cache.pyi:150-169)."""

    k: np.ndarray | None = None  # [B,Hkv,S,D]
    v: np.ndarray | None = None
    offset: int = 0

    def update_and_fetch(self, k, v):
        if self.k is None or self.offset == 0:
            self.k, self.v = k, v
        else:
            self.k = np.concatenate([self.k[:, :, : self.offset], k], axis=2)
            self.v = np.concatenate([self.v[:, :, : self.offset], v], axis=2)
        self.offset = self.k.shape[2]
        return self.k, self.v

    def trim(self, n: int) -> int:
        n = min(n, self.offset)
        self.offset -= n
        if self.k is not None:
            self.k = self.k[:, :, : self.offset]
            self.v = self.v[:, :, : self.offset]
        return n


def make_kv_cache(n_local_layers: int) -> list[LayerKV]:
    return [LayerKV() for _ in range(n_local_layers)]


@dataclass
class ShardModel:
    cfg: Config
    weights: dict
    start_layer: int = 0
    end_layer: int | None = None
    dequant_mode: str = "M1"
    # A matmul with more than `gemm_rows` input rows multiplies by weights rounded to
    # bf16 (one rounding of the float32 fma), the way a kernel that dequantises into
    # bf16 operands for the matrix cores does; fewer rows use the un-rounded float32
    # weights of a fused GEMV.  None = un-rounded everywhere.  Which of the two MLX's
    # own kernels do is PARITY UNPINNED; both are within the stated tolerance.
    gemm_rows: int | None = None
    # use the C restatement (oracle/qmm_ref.c) for matmuls of at most 16 rows: same
    # arithmetic, no dequantised copy of the matrix, OpenMP over output rows
    use_c: bool = False
    _dq: dict = field(default_factory=dict)
    router_margins: list = field(default_factory=list)  # (layer, logit gap per token)

    def __post_init__(self):
        if self.end_layer is None:
            self.end_layer = self.cfg.num_hidden_layers
        self.inv_freq = ops.rope_inv_freq(
            self.cfg.head_dim, self.cfg.rope_theta, self.cfg.rope_scaling
        )

    # -- helpers
    @property
    def n_local_layers(self) -> int:
        return self.end_layer - self.start_layer

    @property
    def is_first(self) -> bool:
        return self.start_layer == 0

    @property
    def is_last(self) -> bool:
        return self.end_layer == self.cfg.num_hidden_layers

    def _bits(self, prefix: str) -> int:
        """Bit width of one tensor from its shapes: a row of K elements is K*bits/32 words
        and K/group_size scales (.typings/mlx/core/__init__.pyi:4180-4188).  Checkpoints may
        quantise single modules at another width than the default of config.json."""
        words = self.weights[prefix + ".weight"].shape[-1]
        groups = self.weights[prefix + ".scales"].shape[-1]
        bits, rem = divmod(32 * words, self.cfg.group_size * groups)
        assert rem == 0 and bits in (4, 8), (prefix, words, groups)
        return bits

    def _wd(self, prefix: str, expert: int | None = None) -> np.ndarray:
        """float32 dequantised matrix (cached)."""
        key = (prefix, expert)
        if key not in self._dq:
            w = self.weights[prefix + ".weight"]
            s = self.weights[prefix + ".scales"]
            b = self.weights[prefix + ".biases"]
            if expert is not None:
                w, s, b = w[expert], s[expert], b[expert]
            self._dq[key] = affine.dequantize_f32(
                w, s, b, self.cfg.group_size, self._bits(prefix)
            )
        return self._dq[key]

    def linear(self, x: np.ndarray, prefix: str) -> np.ndarray:
        rows = int(np.prod(x.shape[:-1]))
        # (in exact mode - no bf16 rounding of the weights for long inputs - the C
        # restatement serves every row count: no float32 copy of the matrix is formed)
        if self.use_c and (rows <= 16 or self.gemm_rows is None):
            from . import cref

            y = cref.qmm_t(
                affine.f32_to_bf16_bits(x.reshape(rows, -1)), self.weights[prefix + ".weight"],
                self.weights[prefix + ".scales"], self.weights[prefix + ".biases"], self._bits(prefix))
            return bf16_bits_to_f32(y).reshape(*x.shape[:-1], -1)
        w = self._wd(prefix)
        if self.gemm_rows is not None and rows > self.gemm_rows:
            key = (prefix, "bf16")
            if key not in self._dq:
                self._dq[key] = bf16_round(w)
            w = self._dq[key]
        return bf16_round(x.astype(np.float32) @ w.T)

    def _norm_w(self, name: str) -> np.ndarray:
        return bf16_bits_to_f32(self.weights[name])

    # -- blocks
    def attention(self, x, i: int, kv: LayerKV):
        c = self.cfg
        B, T, _ = x.shape
        p = f"model.layers.{i}.self_attn."
        q = self.linear(x, p + "q_proj").reshape(B, T, c.num_attention_heads, c.head_dim)
        k = self.linear(x, p + "k_proj").reshape(B, T, c.num_key_value_heads, c.head_dim)
        v = self.linear(x, p + "v_proj").reshape(B, T, c.num_key_value_heads, c.head_dim)
        if c.model_type == "qwen3_moe":  # per-head RMSNorm before RoPE
            q = ops.rms_norm(q, self._norm_w(p + "q_norm.weight"), c.rms_norm_eps)
            k = ops.rms_norm(k, self._norm_w(p + "k_norm.weight"), c.rms_norm_eps)
        q = q.transpose(0, 2, 1, 3)
        k = k.transpose(0, 2, 1, 3)
        v = v.transpose(0, 2, 1, 3)
        off = kv.offset
        q = ops.rope(q, self.inv_freq, off)
        k = ops.rope(k, self.inv_freq, off)
        kk, vv = kv.update_and_fetch(k, v)
        S = kk.shape[2]
        o = ops.sdpa(q, kk, vv, c.head_dim**-0.5, S - T)
        o = o.transpose(0, 2, 1, 3).reshape(B, T, c.num_attention_heads * c.head_dim)
        return self.linear(o, p + "o_proj")

    def mlp(self, x, i: int):
        p = f"model.layers.{i}.mlp."
        g = self.linear(x, p + "gate_proj")
        u = self.linear(x, p + "up_proj")
        return self.linear(ops.swiglu(g, u), p + "down_proj")

    def moe(self, x, i: int):
        c = self.cfg
        B, T, H = x.shape
        p = f"model.layers.{i}.mlp."
        xf = x.reshape(B * T, H)
        logits = self.linear(xf, p + "gate")
        idx, sc = ops.router_topk(logits, c.num_experts_per_tok, c.norm_topk_prob)
        # how close the k-th and (k+1)-th expert were, per token: a caller comparing
        # against another implementation can tell a routing near-tie from an error
        srt = -np.sort(-logits.astype(np.float32), axis=-1)
        k = c.num_experts_per_tok
        if srt.shape[-1] > k:
            self.router_margins.append((i, srt[:, k - 1] - srt[:, k]))
        out = np.zeros((B * T, H), np.float32)
        for t in range(B * T):
            acc = np.zeros(H, np.float32)
            for j in range(c.num_experts_per_tok):
                e = int(idx[t, j])
                g = bf16_round(self._wd(p + "switch_mlp.gate_proj", e) @ xf[t])
                u = bf16_round(self._wd(p + "switch_mlp.up_proj", e) @ xf[t])
                d = bf16_round(self._wd(p + "switch_mlp.down_proj", e) @ ops.swiglu(g, u))
                acc += bf16_round(d * sc[t, j])
            out[t] = bf16_round(acc)
        return out.reshape(B, T, H)

    def layer(self, h, i: int, kv: LayerKV):
        c = self.cfg
        p = f"model.layers.{i}."
        r = self.attention(
            ops.rms_norm(h, self._norm_w(p + "input_layernorm.weight"), c.rms_norm_eps), i, kv
        )
        h = bf16_round(h + r)
        xn = ops.rms_norm(h, self._norm_w(p + "post_attention_layernorm.weight"), c.rms_norm_eps)
        r = self.moe(xn, i) if c.model_type == "qwen3_moe" else self.mlp(xn, i)
        return bf16_round(h + r)

    # -- the shard forward
    def __call__(self, tokens, cache: list[LayerKV], input_hidden=None) -> np.ndarray:
        """tokens int [B,T].  First shard embeds ``tokens``; any other shard takes
        ``input_hidden`` [B,T,H] (what PipelineFirstLayer would have received,
        auto_parallel.py:132-139).  Returns logits [B,T,V] on the last shard, else
        the hidden state leaving the last local layer."""
        c = self.cfg
        if self.is_first:
            tokens = np.asarray(tokens)
            B, T = tokens.shape
            h = affine.embed(
                tokens.reshape(-1),
                self.weights["model.embed_tokens.weight"],
                self.weights["model.embed_tokens.scales"],
                self.weights["model.embed_tokens.biases"],
                c.group_size,
                self._bits("model.embed_tokens"),
                self.dequant_mode,
            ).reshape(B, T, c.hidden_size)
        else:
            assert input_hidden is not None
            h = np.asarray(input_hidden, np.float32)
        for li, i in enumerate(range(self.start_layer, self.end_layer)):
            h = self.layer(h, i, cache[li])
        if not self.is_last:
            return h
        h = ops.rms_norm(h, self._norm_w("model.norm.weight"), c.rms_norm_eps)
        head = "model.embed_tokens" if c.tie_word_embeddings else "lm_head"
        return self.linear(h, head)


# ------------------------------------------------------------------ generation


def prefill(model: ShardModel, tokens, cache, step: int = 4096, faithful: bool = False):
    """Reference ``prefill`` (generate.py:282-396) for a batch-1 token list: after it the
    cache holds len(tokens)-1 entries.  ``faithful`` also runs the two single-token
    forwards whose cache entries trim(2) then discards (the sampled token is the
    argmax); they change no result, only cost."""
    n = len(tokens)
    if n == 0:
        return
    toks = np.asarray(tokens, np.int64)
    done = 0
    while n - done > 1:
        m = min(step, n - done - 1)
        model(toks[None, done : done + m], cache)
        done += m
    if faithful:
        lg = model(toks[None, done : done + 1], cache)
        nxt = int(np.argmax(lg[0, -1]))
        model(np.array([[nxt]]), cache)
        for c in cache:
            c.trim(2)


def greedy_generate(model: ShardModel, prompt, max_tokens: int, faithful: bool = False):
    """``mlx_generate`` at temperature 0 (generate.py:532-827): prefill on
    prompt[:-1] (cache N-2), then feed prompt[-2] and prompt[-1] as single-token
    forwards, then one single-token forward per generated token.
    Returns (tokens, per-step logits [max_tokens, V])."""
    cache = make_kv_cache(model.n_local_layers)
    prefill(model, list(prompt[:-1]), cache, faithful=faithful)
    assert cache[0].offset == max(len(prompt) - 2, 0)
    out, all_logits = [], []
    if len(prompt) >= 2:
        model(np.array([[prompt[-2]]]), cache)
    tok = int(prompt[-1])
    for _ in range(max_tokens):
        lg = model(np.array([[tok]]), cache)[0, -1]
        all_logits.append(lg)
        tok = int(np.argmax(lg))
        out.append(tok)
    return out, np.stack(all_logits)
