"""MLX affine group quantisation: packing, quantise, dequantise, quantised matmul.

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).  numpy, float32/float64.

Follows the operator documentation carried by the reference:
  packing + quantise formula   .typings/mlx/core/__init__.pyi:4166-4188
  dequantise formula           .typings/mlx/core/__init__.pyi:2444-2450
  quantized_matmul             .typings/mlx/core/__init__.pyi:4198-4234
  gather_qmm                   .typings/mlx/core/__init__.pyi:2957-3006
  tensor shapes                src/exo/worker/engines/mlx/auto_parallel.py:880-881

bf16 values are carried as numpy uint16 bit patterns ("bf16 bits") wherever bit
equality matters, and as float32 holding bf16-representable values elsewhere.
"""

from __future__ import annotations

import numpy as np

# ----------------------------------------------------------------------------- bf16


def bf16_round(x: np.ndarray) -> np.ndarray:
    """float32 -> nearest bf16 (ties to even), returned as float32."""
    return bf16_bits_to_f32(f32_to_bf16_bits(x))


_EXACT_ACTIVATIONS = False


class exact_activations:
    """Context manager for the tests that pin the STRUCTURE of the oracle against
    float32 library models: while active, ``act_round`` is the identity, so the
    oracle computes the same real-valued function without bf16 rounding between ops."""

    def __enter__(self):
        global _EXACT_ACTIVATIONS
        self._old = _EXACT_ACTIVATIONS
        _EXACT_ACTIVATIONS = True

    def __exit__(self, *a):
        global _EXACT_ACTIVATIONS
        _EXACT_ACTIVATIONS = self._old


def act_round(x: np.ndarray) -> np.ndarray:
    """Rounding of an ACTIVATION to bf16 at an op boundary."""
    if _EXACT_ACTIVATIONS:
        return np.asarray(x, np.float32)
    return bf16_round(x)


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    bias = ((u >> 16) & 1) + np.uint32(0x7FFF)
    r = ((u.astype(np.uint64) + bias) >> 16).astype(np.uint16)
    nan = np.isnan(x)
    if np.any(nan):
        r = np.where(nan, np.uint16(0x7FC0), r)
    return r


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(
        np.float32
    )


# -------------------------------------------------------------------------- packing


def pack_codes(codes: np.ndarray, bits: int) -> np.ndarray:
    """uint8 codes [..., K] -> uint32 words [..., K*bits/32], first element in the
    least significant bits (.pyi:4180-4184)."""
    assert bits in (4, 8)
    per = 32 // bits
    K = codes.shape[-1]
    assert K % per == 0
    c = codes.astype(np.uint32).reshape(*codes.shape[:-1], K // per, per)
    shifts = (np.arange(per, dtype=np.uint32) * bits).astype(np.uint32)
    return np.bitwise_or.reduce(c << shifts, axis=-1).astype(np.uint32)


def unpack_codes(w: np.ndarray, bits: int) -> np.ndarray:
    """uint32 words [..., W] -> uint8 codes [..., W*32/bits]."""
    assert bits in (4, 8)
    per = 32 // bits
    shifts = (np.arange(per, dtype=np.uint32) * bits).astype(np.uint32)
    mask = np.uint32((1 << bits) - 1)
    c = (w.astype(np.uint32)[..., None] >> shifts) & mask
    return c.reshape(*w.shape[:-1], w.shape[-1] * per).astype(np.uint8)


# ------------------------------------------------------------------------- quantise


def quantize(w: np.ndarray, group_size: int = 64, bits: int = 4, rule: str = "mlx"):
    """float32 [N,K] -> (packed uint32 [N,K*bits/32], scales bf16-bits [N,K/g],
    biases bf16-bits [N,K/g]).

    rule="doc": exactly the documented formula (.pyi:4167-4178):
        alpha=max, beta=min, s=(alpha-beta)/(2^b-1), q=round((w-beta)/s).
    rule="mlx": the edge-snapping variant recalled from the mlx sources (sign of s
        chosen toward the larger-magnitude edge, that edge made exactly
        representable, s clamped away from 0).  PARITY UNPINNED: only mx.quantize
        can confirm it.  It only affects which synthetic weights are generated,
        never kernel parity, because kernels consume already-packed tensors.
    Scales/biases are rounded to bf16 BEFORE the codes are computed, so that the
    stored triple is self-consistent.
    """
    N, K = w.shape
    assert K % group_size == 0
    nb = float((1 << bits) - 1)
    g = w.astype(np.float32).reshape(N, K // group_size, group_size)
    wmax = g.max(-1)
    wmin = g.min(-1)
    if rule == "doc":
        s = (wmax - wmin) / nb
        s = np.where(s == 0, np.float32(1e-7), s)
        beta = wmin
    elif rule == "mlx":
        eps = np.float32(1e-7)
        s = np.maximum((wmax - wmin) / nb, eps)
        side = np.abs(wmin) > np.abs(wmax)
        s = np.where(side, s, -s)
        edge = np.where(side, wmin, wmax)
        q0 = np.rint(edge / s)
        nz = q0 != 0
        s = np.where(nz, edge / np.where(nz, q0, 1), s)
        beta = np.where(nz, edge, np.float32(0))
    else:
        raise ValueError(rule)
    s = bf16_round(s.astype(np.float32))
    beta = bf16_round(beta.astype(np.float32))
    s_safe = np.where(s == 0, np.float32(1e-7), s)
    q = np.rint((g - beta[..., None]) / s_safe[..., None])
    q = np.clip(q, 0, nb).astype(np.uint8).reshape(N, K)
    return pack_codes(q, bits), f32_to_bf16_bits(s), f32_to_bf16_bits(beta)


# ----------------------------------------------------------------------- dequantise


def dequantize_f32(w, scales, biases, group_size: int = 64, bits: int = 4):
    """Exact real-valued s*q+beta evaluated in float32 with a single rounding per
    element (float32 fma semantics via float64).  Shape [..., N, K] float32."""
    q = unpack_codes(w, bits).astype(np.float64)
    s = bf16_bits_to_f32(scales).astype(np.float64)
    b = bf16_bits_to_f32(biases).astype(np.float64)
    s = np.repeat(s, group_size, axis=-1)
    b = np.repeat(b, group_size, axis=-1)
    return (s * q + b).astype(np.float32)


def dequantize(w, scales, biases, group_size: int = 64, bits: int = 4, mode="M1"):
    """-> bf16 bits [..., N, K] of w_i = s*q_i + beta (.pyi:2444-2450).

    The formula is documented; the rounding order to bf16 is PARITY UNPINNED:
      M1  bf16(bf16(s*q) + beta)   two roundings (bf16 arithmetic per operation)
      M2  bf16(fma(s, q, beta))    one rounding
    """
    q = unpack_codes(w, bits).astype(np.float32)
    s = np.repeat(bf16_bits_to_f32(scales), group_size, axis=-1)
    b = np.repeat(bf16_bits_to_f32(biases), group_size, axis=-1)
    if mode == "M1":
        # s (8-bit mantissa) * q (<= 8 bits) is exact in float32.
        return f32_to_bf16_bits(bf16_round(s * q) + b)
    if mode == "M2":
        return f32_to_bf16_bits(dequantize_f32(w, scales, biases, group_size, bits))
    raise ValueError(mode)


# --------------------------------------------------------------- quantised matmuls


def qmm(x, w, scales, biases, group_size: int = 64, bits: int = 4, out_bf16=True):
    """quantized_matmul(x, w, scales, biases, transpose=True): y = x @ dq(w).T
    x float32 (bf16-representable) [..., K]; returns float32 [..., N], rounded to
    bf16 when out_bf16.  Accumulation is float32 over the un-rounded dequantised
    weights (no intermediate bf16 weight is formed in a fused kernel)."""
    wd = dequantize_f32(w, scales, biases, group_size, bits)  # [N,K]
    y = np.asarray(x, np.float32) @ wd.T
    return act_round(y) if out_bf16 else y


def gather_qmm(x, w, scales, biases, rhs_indices, group_size=64, bits=4, out_bf16=True):
    """gather_qmm(x, w, s, b, rhs_indices=idx, transpose=True) as SwitchLinear calls
    it (.typings/mlx_lm/models/switch_layers.pyi:10-31).

    x  float32 [T, R, K] with R == 1 (broadcast over slots) or R == top_k
    w  uint32 [E, N, K*bits/32];  rhs_indices int [T, top_k]
    -> float32 [T, top_k, N]:  y[t, j] = x[t, j or 0] @ dq(w[idx[t, j]]).T
    """
    T, topk = rhs_indices.shape
    N = w.shape[1]
    y = np.zeros((T, topk, N), np.float32)
    cache: dict[int, np.ndarray] = {}
    for t in range(T):
        for j in range(topk):
            e = int(rhs_indices[t, j])
            if e not in cache:
                cache[e] = dequantize_f32(w[e], scales[e], biases[e], group_size, bits)
            xv = x[t, j if x.shape[1] > 1 else 0].astype(np.float32)
            y[t, j] = cache[e] @ xv
    return act_round(y) if out_bf16 else y


def embed(ids, w, scales, biases, group_size: int = 64, bits: int = 4, mode="M1"):
    """QuantizedEmbedding.__call__ (.typings/mlx/nn/layers/quantized.pyi:42-85): row
    gather followed by dequantize -> float32 holding bf16 values [len(ids), K]."""
    ids = np.asarray(ids).reshape(-1)
    return bf16_bits_to_f32(
        dequantize(w[ids], scales[ids], biases[ids], group_size, bits, mode)
    )
