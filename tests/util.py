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


def assert_close(got: np.ndarray, want: np.ndarray, rtol=RTOL, what=""):
    """|got - want| <= rtol*|want| + atol with atol = rtol * rms(want)."""
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    assert got.shape == want.shape, (got.shape, want.shape)
    atol = rtol * float(np.sqrt(np.mean(want**2))) if want.size else 0.0
    err = np.abs(got - want)
    bound = rtol * np.abs(want) + atol
    bad = err > bound
    if bad.any():
        i = np.unravel_index(np.argmax(err - bound), err.shape)
        raise AssertionError(
            f"{what}: {bad.sum()}/{bad.size} outside rtol={rtol} atol={atol:.3e}; "
            f"worst at {i}: got {got[i]} want {want[i]}"
        )
    return float(err.max()), atol


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
