"""Shared helpers for the tests: bf16 <-> numpy bits, seeded quantised matrices,
tolerance rule.  Imports the oracle (tests are allowed to)."""

from __future__ import annotations

import numpy as np

from oracle import affine

RTOL = 2e-2  # north-star tolerance for bf16 activations / logits


def rng(seed):
    return np.random.default_rng(seed)


def rand_bf16(shape, seed, scale=1.0) -> np.ndarray:
    """float32 array of bf16-representable N(0, scale) values."""
    return affine.bf16_round((rng(seed).standard_normal(shape) * scale).astype(np.float32))


def rand_quantized(N, K, bits, seed, scale=0.02, E=None):
    """(w uint32, scales bf16-bits, biases bf16-bits) from N(0, scale) weights."""
    if E is None:
        w = (rng(seed).standard_normal((N, K)) * scale).astype(np.float32)
        return affine.quantize(w, 64, bits)
    parts = [rand_quantized(N, K, bits, seed * 1000 + e, scale) for e in range(E)]
    return tuple(np.stack([p[i] for p in parts]) for i in range(3))


def assert_close(got: np.ndarray, want: np.ndarray, rtol=RTOL, what="", tail_frac=0.0):
    """|got - want| <= rtol*|want| + atol with atol = rtol * rms(want).  ``tail_frac`` (for
    outputs of several hundred thousand elements, where the far tail of the rounding-flip
    distribution shows): that fraction of the elements may lie outside the bound, none
    outside twice the bound."""
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    assert got.shape == want.shape, (got.shape, want.shape)
    atol = rtol * float(np.sqrt(np.mean(want**2))) if want.size else 0.0
    err = np.abs(got - want)
    bound = rtol * np.abs(want) + atol
    bad = err > bound
    if tail_frac and bad.sum() <= tail_frac * bad.size and not (err > 2 * bound).any():
        if bad.any():
            print(f"[parity] {what}: {bad.sum()}/{bad.size} elements between one and two bounds (tail)")
        return float(err.max()), atol
    if bad.any():
        i = np.unravel_index(np.argmax(err - bound), err.shape)
        raise AssertionError(
            f"{what}: {bad.sum()}/{bad.size} outside rtol={rtol} atol={atol:.3e}; "
            f"worst at {i}: got {got[i]} want {want[i]}"
        )
    return float(err.max()), atol


def assert_close_stat(got, want, rtol=RTOL, max_rel_rms=RTOL, max_outlier_frac=5e-3, what=""):
    """Criterion for tensors that passed through SEVERAL bf16-rounded layers.

    Every op rounds its output to bf16; two correct implementations that accumulate
    in a different order flip a fraction of those roundings, and the flips propagate,
    so elementwise agreement at rtol 2e-2 cannot hold for every element of a deep
    stack (the oracle disagrees with itself by the same amount when its weights are
    rounded to bf16 first).  Required here: relative RMS error <= max_rel_rms and at
    most max_outlier_frac of the elements outside |d| <= rtol*|want| + rtol*rms(want).
    Single ops and single layers are held to the elementwise bound (assert_close)."""
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    assert got.shape == want.shape, (got.shape, want.shape)
    rms = float(np.sqrt(np.mean(want**2)))
    err = np.abs(got - want)
    rel_rms = float(np.sqrt(np.mean(err**2))) / rms
    frac = float(np.mean(err > rtol * np.abs(want) + rtol * rms))
    print(f"[parity] {what}: rel-rms {rel_rms:.3e} outliers {frac:.3e} max|e|/rms {err.max() / rms:.3e}")
    assert rel_rms <= max_rel_rms, f"{what}: relative RMS error {rel_rms:.3e} > {max_rel_rms}"
    assert frac <= max_outlier_frac, f"{what}: {frac:.3e} of elements outside the elementwise bound"
    return rel_rms, frac


# ---- torch side (imported lazily so CPU-only oracle tests do not need torch)


def t_bf16(a: np.ndarray, device):
    """float32 numpy (bf16-representable) or uint16 bits -> torch bf16 on device."""
    import torch

    bits = a if a.dtype == np.uint16 else affine.f32_to_bf16_bits(a)
    return torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16).to(device)


def t_u32(a: np.ndarray, device):
    import torch

    return torch.from_numpy(a.view(np.int32).copy()).to(device)


def n_f32(t) -> np.ndarray:
    """torch bf16/float tensor -> float32 numpy."""
    return t.detach().float().cpu().numpy()


def n_bits(t) -> np.ndarray:
    """torch bf16 tensor -> uint16 bits."""
    import torch

    return t.detach().contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


def t_qw(triple, bits, device):
    from exo_amd.ops import QuantizedWeight

    w, s, b = triple
    return QuantizedWeight(t_u32(w, device), t_bf16(s, device), t_bf16(b, device), bits)


# ---- checkpoints shared by the oracle and the GPU engine


def load_checkpoint_numpy(path):
    """MLX-layout safetensors -> {name: numpy} (uint32 words, uint16 bf16 bits) plus the
    oracle Config."""
    import json
    from pathlib import Path

    import torch
    from safetensors.torch import load_file

    from oracle.models import Config

    path = Path(path)
    out = {}
    for f in sorted(path.glob("*.safetensors")):
        for k, v in load_file(str(f)).items():
            if v.dtype == torch.uint32:
                out[k] = v.view(torch.int32).numpy().view(np.uint32)
            elif v.dtype == torch.bfloat16:
                out[k] = v.view(torch.int16).numpy().view(np.uint16)
            else:
                raise TypeError(f"{k}: {v.dtype}")
    with open(path / "config.json") as fh:
        cfg = Config.from_json(json.load(fh))
    return cfg, out


def tiny_config(kind: str, bits: int = 4):
    from exo_amd.config import LLAMA3_SCALING, ModelConfig

    if kind == "llama":
        return ModelConfig("llama", 256, 3, 8, 2, 64, 512, 1000, 1e-5, 5e5,
                           dict(LLAMA3_SCALING, factor=32.0), False, 64, bits)
    if kind == "llama_tied_d128":
        return ModelConfig("llama", 512, 2, 4, 2, 128, 1024, 777, 1e-5, 5e5,
                           dict(LLAMA3_SCALING, factor=8.0), True, 64, bits)
    if kind == "qwen3_moe":
        return ModelConfig("qwen3_moe", 256, 2, 8, 2, 128, 0, 600, 1e-6, 1e6, None, False, 64, bits,
                           8, 2, 128, True)
    if kind == "qwen3_moe_router8":  # 4-bit experts and attention, router kept at 8 bits
        c = tiny_config("qwen3_moe", 4)
        c.quant_overrides = {f"model.layers.{i}.mlp.gate": {"group_size": 64, "bits": 8}
                             for i in range(c.num_hidden_layers)}
        return c
    raise KeyError(kind)


def check_tokens(got, want, om, what):
    """Per-token statistical parity.  For MoE models a token whose k-th and (k+1)-th
    router logits are within bf16 noise may legitimately pick another expert; such
    tokens (and later ones, through the KV cache) are exempt when the oracle's router
    gap shows the near-tie."""
    got, want = got.reshape(-1, got.shape[-1]), want.reshape(-1, want.shape[-1])
    gaps = None
    if om.router_margins:
        T = want.shape[0]
        gaps = np.min(np.stack([g[-T:] for _, g in om.router_margins[-om.n_local_layers:]]), axis=0)
    tied_before = False
    for t in range(want.shape[0]):
        rms = float(np.sqrt(np.mean(want[t] ** 2)))
        rel = float(np.sqrt(np.mean((got[t] - want[t]) ** 2))) / rms
        if gaps is not None and gaps[t] <= 2.0 ** -6 * max(1.0, rms):
            tied_before = True
        if rel > 2e-2:
            gap = "n/a" if gaps is None else f"{float(np.min(gaps[: t + 1])):.3e}"
            assert tied_before, (f"{what}: token {t} rel-rms {rel:.3e} with no router near-tie "
                                 f"(smallest router gap so far {gap})")
            print(f"[parity] {what}: token {t} rel-rms {rel:.3e} after a router near-tie (exempt)")
    return tied_before


def weights_to_numpy(weights: dict) -> dict:
    """{name: torch tensor} of a synthesised shard -> the oracle's numpy layout (uint32
    words, uint16 bf16 bits)."""
    import torch

    out = {}
    for k, v in weights.items():
        v = v.detach().cpu()
        if v.dtype in (torch.uint32, torch.int32):
            out[k] = v.view(torch.int32).numpy().view(np.uint32)
        elif v.dtype == torch.bfloat16:
            out[k] = v.view(torch.int16).numpy().view(np.uint16)
        else:
            raise TypeError(f"{k}: {v.dtype}")
    return out
