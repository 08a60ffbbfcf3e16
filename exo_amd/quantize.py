"""MLX affine group quantisation of a float matrix (torch, runs on any device).

Used to synthesise checkpoints in the MLX layout (benchmarks, tests); inference never
quantises.  Implements ``mx.quantize(w, group_size, bits)``
(.typings/mlx/core/__init__.pyi:4126-4196): per group of ``group_size`` consecutive
elements of a row, codes ``q = round((w - beta) / s)`` packed LSB-first into uint32.
The edge rule (which edge of the group range is represented exactly, sign of the
scale) follows the rule recalled from the mlx sources; the documented min/max rule is
available as ``rule="doc"``.
"""

from __future__ import annotations

import torch


def pack_codes(codes: torch.Tensor, bits: int) -> torch.Tensor:
    """uint8 codes [..., K] -> int32 words [..., K*bits/32] (uint32 bit pattern)."""
    per = 32 // bits
    c = codes.to(torch.int64).reshape(*codes.shape[:-1], codes.shape[-1] // per, per)
    shifts = torch.arange(per, device=codes.device, dtype=torch.int64) * bits
    w = (c << shifts).sum(-1)
    w = torch.where(w >= 2**31, w - 2**32, w)
    return w.to(torch.int32)


def quantize(w: torch.Tensor, group_size: int = 64, bits: int = 4, rule: str = "mlx"):
    """float [N,K] -> (int32 words [N,K*bits/32], bf16 scales [N,K/g], bf16 biases)."""
    N, K = w.shape
    assert K % group_size == 0
    nb = float((1 << bits) - 1)
    g = w.float().reshape(N, K // group_size, group_size)
    wmax = g.amax(-1)
    wmin = g.amin(-1)
    if rule == "doc":
        s = (wmax - wmin) / nb
        s = torch.where(s == 0, torch.full_like(s, 1e-7), s)
        beta = wmin
    elif rule == "mlx":
        s = torch.clamp((wmax - wmin) / nb, min=1e-7)
        side = wmin.abs() > wmax.abs()
        s = torch.where(side, s, -s)
        edge = torch.where(side, wmin, wmax)
        q0 = torch.round(edge / s)
        nz = q0 != 0
        s = torch.where(nz, edge / torch.where(nz, q0, torch.ones_like(q0)), s)
        beta = torch.where(nz, edge, torch.zeros_like(edge))
    else:
        raise ValueError(rule)
    s = s.bfloat16()
    beta = beta.bfloat16()
    sf = s.float()
    sf = torch.where(sf == 0, torch.full_like(sf, 1e-7), sf)
    q = torch.round((g - beta.float()[..., None]) / sf[..., None]).clamp_(0, nb)
    return pack_codes(q.to(torch.uint8).reshape(N, K), bits), s, beta
