"""Bandwidth-bound transformer ops restated on the CPU (numpy float32).

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

The reference reaches these through mlx_lm model code; exo itself only names them
at the call sites cited per function.  ``mx.fast.*`` has no stub in the reference,
so each op is the textbook definition; the tests pin them against the
``transformers`` / ``torch.nn.functional`` routines of the same name.

Convention: every op takes float32 arrays holding bf16-representable values,
computes in float32 and rounds its result to bf16 once (returned as float32).
"""

from __future__ import annotations

import math

import numpy as np

from .affine import act_round as bf16_round


def rms_norm(x: np.ndarray, weight: np.ndarray, eps: float) -> np.ndarray:
    """mx.fast.rms_norm(x, w, eps): x * rsqrt(mean(x^2) + eps) * w over the last axis.
    Multiplication by w happens in float32 before the single rounding."""
    x = x.astype(np.float32)
    ms = np.mean(x.astype(np.float64) ** 2, axis=-1, keepdims=True)
    inv = (1.0 / np.sqrt(ms + eps)).astype(np.float32)
    return bf16_round(x * inv * weight.astype(np.float32))


def rope_inv_freq(head_dim: int, theta: float, scaling: dict | None = None) -> np.ndarray:
    """Per-pair inverse frequencies [head_dim/2] float32.

    default : theta^(-2i/d).
    llama3  : the piecewise rescale of mlx_lm's Llama3RoPE
              (.typings/mlx_lm/models/rope_utils.pyi:20-51), same rule as
              transformers' _compute_llama3_parameters.
    """
    i = np.arange(0, head_dim, 2, dtype=np.float64)
    inv = 1.0 / (theta ** (i / head_dim))
    if scaling and scaling.get("rope_type", scaling.get("type")) == "llama3":
        factor = float(scaling["factor"])
        lo = float(scaling.get("low_freq_factor", 1.0))
        hi = float(scaling.get("high_freq_factor", 4.0))
        old = float(scaling.get("original_max_position_embeddings", 8192))
        wavelen = 2 * math.pi / inv
        low_wl = old / lo
        high_wl = old / hi
        out = np.where(wavelen > low_wl, inv / factor, inv)
        smooth = (old / wavelen - lo) / (hi - lo)
        mid = (1 - smooth) * inv / factor + smooth * inv
        is_mid = (wavelen <= low_wl) & (wavelen >= high_wl)
        inv = np.where(is_mid, mid, out)
    return inv.astype(np.float32)


def rope(x: np.ndarray, inv_freq: np.ndarray, offset: int) -> np.ndarray:
    """mx.fast.rope(x, dims=D, traditional=False, offset=offset): rotate the pairs
    (x[i], x[i+D/2]) of the last axis by angle (offset+t)*inv_freq[i].
    x: [B, H, T, D]."""
    B, H, T, D = x.shape
    pos = (np.arange(T, dtype=np.float32) + np.float32(offset))[:, None]
    ang = pos * inv_freq[None, :].astype(np.float32)  # float32 product, like the kernel
    c = np.cos(ang.astype(np.float64)).astype(np.float32)
    s = np.sin(ang.astype(np.float64)).astype(np.float32)
    x1 = x[..., : D // 2].astype(np.float32)
    x2 = x[..., D // 2 :].astype(np.float32)
    o1 = x1 * c - x2 * s
    o2 = x2 * c + x1 * s
    return bf16_round(np.concatenate([o1, o2], axis=-1))


def sdpa(q, k, v, scale: float, causal_offset: int | None) -> np.ndarray:
    """mx.fast.scaled_dot_product_attention with grouped-query broadcast
    (.typings/mlx_lm/models/base.pyi:39-47).

    q [B,Hq,T,D], k/v [B,Hkv,S,D]; query t may attend keys j <= causal_offset + t
    when causal_offset is not None (causal_offset = S - T for a cache holding the
    new tokens at its end), all keys otherwise.  float32 softmax.
    """
    B, Hq, T, D = q.shape
    Hkv, S = k.shape[1], k.shape[2]
    rep = Hq // Hkv
    kk = np.repeat(k.astype(np.float32), rep, axis=1)
    vv = np.repeat(v.astype(np.float32), rep, axis=1)
    s = np.einsum("bhtd,bhsd->bhts", q.astype(np.float32), kk) * np.float32(scale)
    if causal_offset is not None:
        t = np.arange(T)[:, None]
        j = np.arange(S)[None, :]
        s = np.where(j <= t + causal_offset, s, -np.inf)
    s = s - s.max(-1, keepdims=True)
    p = np.exp(s)
    p = p / p.sum(-1, keepdims=True)
    return bf16_round(np.einsum("bhts,bhsd->bhtd", p, vv))


def swiglu(gate: np.ndarray, up: np.ndarray) -> np.ndarray:
    """silu(gate) * up (.typings/mlx_lm/models/switch_layers.pyi:52-57), one rounding."""
    g = gate.astype(np.float32)
    return bf16_round(g / (1.0 + np.exp(-g)) * up.astype(np.float32))


def router_topk(logits: np.ndarray, k: int, norm_topk_prob: bool):
    """Qwen3-MoE routing as mlx_lm's Qwen3MoeSparseMoeBlock does it: softmax over
    experts in float32 (rounded to bf16 because the logits are bf16), the k largest
    by value (ties to the lower expert id; order of the k slots = descending score),
    optional renormalisation by their sum (a bf16 sum, then a bf16 division).
    -> (indices int32 [R,k], scores float32-holding-bf16 [R,k])."""
    x = logits.astype(np.float32)
    x = x - x.max(-1, keepdims=True)
    p = np.exp(x)
    p = bf16_round(p / p.sum(-1, keepdims=True))
    order = np.argsort(-p, axis=-1, kind="stable")[:, :k]
    sc = np.take_along_axis(p, order, axis=-1)
    if norm_topk_prob:
        tot = np.zeros((sc.shape[0], 1), np.float32)
        for j in range(k):  # float32 running sum in slot order
            tot = (tot + sc[:, j : j + 1]).astype(np.float32)
        sc = bf16_round(sc / bf16_round(tot))
    return order.astype(np.int32), sc


def logsumexp(x: np.ndarray) -> np.ndarray:
    x = x.astype(np.float32)
    m = x.max(-1, keepdims=True)
    return (m + np.log(np.exp(x - m).sum(-1, keepdims=True))).astype(np.float32)
