"""Operator layer: MLX-named operators on torch device tensors, executed by the HIP
kernels of libexo_mi355x.so through its C ABI.

Names and argument meaning follow the MLX operators the reference calls
(.typings/mlx/core/__init__.pyi: quantized_matmul :4198-4234, gather_qmm :2957-3006,
dequantize :2413-2451; mx.fast.rms_norm / rope / scaled_dot_product_attention).
torch is used for device memory and streams only; every function launches on torch's
current stream and never synchronises.  Errors: ValueError for bad arguments (the C
ABI's -1), NativeError for HIP failures or a missing library.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from . import native
from .native import check

GROUP_SIZE = 64


def _ptr(t: torch.Tensor | None) -> int | None:
    if t is None:
        return None
    assert t.is_cuda and t.is_contiguous(), "device-resident contiguous tensor required"
    return t.data_ptr()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> int:
    """Handle of the current HIP stream of the current device.  Asked once per launch, so the
    raw getter (a fraction of a microsecond) is used where this torch build has it;
    ``torch.cuda.current_stream()`` builds a Stream object and costs about 8 us, most of the
    host time of a launch from Python."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


@dataclass
class QuantizedWeight:
    """MLX affine-quantised matrix: ``weight`` uint32 words viewed as int32
    [..., N, K*bits/32], ``scales`` / ``biases`` bf16 [..., N, K/64]."""

    weight: torch.Tensor
    scales: torch.Tensor
    biases: torch.Tensor
    bits: int
    group_size: int = GROUP_SIZE

    def __post_init__(self):
        if self.weight.dtype == torch.uint32:
            self.weight = self.weight.view(torch.int32)
        assert self.weight.dtype == torch.int32
        assert self.scales.dtype == torch.bfloat16 and self.biases.dtype == torch.bfloat16
        assert self.bits in (4, 8) and self.group_size == GROUP_SIZE

    @property
    def N(self) -> int:
        return self.weight.shape[-2]

    @property
    def K(self) -> int:
        return self.weight.shape[-1] * 32 // self.bits

    @property
    def nbytes(self) -> int:
        return (
            self.weight.numel() * 4 + self.scales.numel() * 2 + self.biases.numel() * 2
        )

    @staticmethod
    def from_tensors(weight: torch.Tensor, scales: torch.Tensor, biases: torch.Tensor,
                     group_size: int = GROUP_SIZE, name: str = "") -> "QuantizedWeight":
        """Bits of this tensor from its own shapes (a checkpoint may quantise single modules
        at another width than the ``quantization.bits`` of its config.json, through per-path
        entries there): a row of K elements is K*bits/32 words and K/group_size scales."""
        words, groups = weight.shape[-1], scales.shape[-1]
        bits, rem = divmod(32 * words, group_size * groups)
        if rem or bits not in (4, 8) or scales.shape != biases.shape or \
                weight.shape[:-1] != scales.shape[:-1]:
            raise ValueError(
                f"{name or 'quantised tensor'}: weight {tuple(weight.shape)} with scales "
                f"{tuple(scales.shape)} / biases {tuple(biases.shape)} is not an affine "
                f"group-{group_size} tensor of 4 or 8 bits")
        return QuantizedWeight(weight, scales, biases, bits, group_size)

    def to(self, device) -> "QuantizedWeight":
        return QuantizedWeight(
            self.weight.to(device).contiguous(),
            self.scales.to(device).contiguous(),
            self.biases.to(device).contiguous(),
            self.bits,
            self.group_size,
        )

    def __getitem__(self, rows: slice) -> "QuantizedWeight":
        return QuantizedWeight(
            self.weight[rows], self.scales[rows], self.biases[rows], self.bits, self.group_size
        )


# ------------------------------------------------------------------ format ops


def unpack_codes(weight: torch.Tensor, bits: int) -> torch.Tensor:
    """uint32 words [..., W] -> uint8 codes [..., W*32/bits]."""
    lib = native.load()
    w = weight.view(torch.int32) if weight.dtype == torch.uint32 else weight
    out = torch.empty(
        *w.shape[:-1], w.shape[-1] * (32 // bits), dtype=torch.uint8, device=w.device
    )
    check(lib.exo_unpack_codes(_ptr(w), _ptr(out), w.numel(), bits, _stream()), "unpack_codes")
    return out


def dequantize(qw: QuantizedWeight) -> torch.Tensor:
    """mx.dequantize -> bf16 [..., N, K]."""
    lib = native.load()
    rows = qw.weight.numel() // qw.weight.shape[-1]
    out = torch.empty(*qw.weight.shape[:-1], qw.K, dtype=torch.bfloat16, device=qw.weight.device)
    check(
        lib.exo_dequantize(
            _ptr(qw.weight), _ptr(qw.scales), _ptr(qw.biases), _ptr(out), rows, qw.K, qw.bits,
            qw.group_size, _stream(),
        ),
        "dequantize",
    )
    return out


def embed(ids: torch.Tensor, qw: QuantizedWeight, out: torch.Tensor | None = None) -> torch.Tensor:
    """QuantizedEmbedding.__call__: ids int32 [n] -> bf16 [n, K]."""
    lib = native.load()
    assert ids.dtype == torch.int32
    n = ids.numel()
    if out is None:
        out = torch.empty(n, qw.K, dtype=torch.bfloat16, device=ids.device)
    check(
        lib.exo_embed_dequant(
            _ptr(ids), _ptr(qw.weight), _ptr(qw.scales), _ptr(qw.biases), _ptr(out), n, qw.N,
            qw.K, qw.bits, qw.group_size, _stream(),
        ),
        "embed",
    )
    return out


# ------------------------------------------------------------------ matmuls

QMV_MAX_M = 16


_QMV_WS: dict = {}


def qmv_workspace(N: int, device) -> torch.Tensor:
    """Split-K workspace for the 2..16-row GEMV, one per device (this engine issues all
    its work in stream order), grown to the largest N seen.  A replaced buffer stays
    alive: a captured graph may still point at it.  Zeroed once; the kernel leaves its
    counters zero."""
    key = torch.device(device).index or 0
    need = native.load().exo_qmv_workspace(N)
    cur = _QMV_WS.get(key)
    if cur is None or cur[-1].numel() < need:
        buf = torch.zeros(need, dtype=torch.uint8, device=device)
        _QMV_WS.setdefault(key, []).append(buf)
        cur = _QMV_WS[key]
    return cur[-1]


_QMM_WS: dict[int, list[torch.Tensor]] = {}


def qmm_workspace(M: int, N: int, device, pair: bool = False) -> torch.Tensor | None:
    """Split-K workspace of the GEMM (``pair``: of the gate/up pair GEMM) for launches of few
    output tiles (None for the others), one per device, grown on demand; a replaced buffer
    stays alive (a captured graph may still point at it)."""
    lib = native.load()
    need = lib.exo_qmm_swiglu_workspace(M, N) if pair else lib.exo_qmm_workspace(M, N)
    if need == 0:
        return None
    key = torch.device(device).index or 0
    cur = _QMM_WS.get(key)
    if cur is None or cur[-1].numel() < need:
        buf = torch.empty(need, dtype=torch.uint8, device=device)
        _QMM_WS.setdefault(key, []).append(buf)
        cur = _QMM_WS[key]
    return cur[-1]


def quantized_matmul(
    x: torch.Tensor,
    qw: QuantizedWeight,
    residual: torch.Tensor | None = None,
    out: torch.Tensor | None = None,
    norm_weight: torch.Tensor | None = None,
    eps: float = 0.0,
) -> torch.Tensor:
    """mx.quantized_matmul(x, w, scales, biases, transpose=True): x bf16 [M,K] ->
    bf16 [M,N].  M <= 16 runs the fused dequant-GEMV, larger M the MFMA GEMM.
    ``residual`` (bf16 [M,N]) fuses the block's ``h + r``; ``norm_weight`` (M <= 16
    only) fuses a preceding rms_norm(x, norm_weight, eps)."""
    lib = native.load()
    assert x.dtype == torch.bfloat16 and x.dim() == 2
    M, K = x.shape
    if K != qw.K:
        raise ValueError(f"quantized_matmul: x has K={K}, weight has K={qw.K}")
    if out is None:
        out = torch.empty(M, qw.N, dtype=torch.bfloat16, device=x.device)
    if norm_weight is not None and M > QMV_MAX_M:
        raise ValueError("fused rms_norm is only available on the GEMV path (M <= 16)")
    # 9..16 rows: the matrix-core GEMV needs its 16-row variant there, which the split-K
    # GEMM matches or beats for 8-bit weights (measured on the Llama-8B shapes)
    gemm_rows = M > 8 and norm_weight is None and qw.bits == 8
    # a matrix of up to 1 MiB without a residual (a MoE router): the library runs its
    # single-row kernel once per row in one launch, whatever the bit width
    if residual is None and qw.N * K * qw.bits // 8 <= (1 << 20):
        gemm_rows = False
    if 2 <= M <= QMV_MAX_M and not gemm_rows:
        ws = qmv_workspace(qw.N, x.device)
        check(
            lib.exo_norm_qmv_ws(
                _ptr(x), _ptr(norm_weight), eps, _ptr(qw.weight), _ptr(qw.scales),
                _ptr(qw.biases), _ptr(residual), _ptr(out), _ptr(ws), ws.numel(), M, qw.N, K,
                qw.bits, qw.group_size, _stream(),
            ),
            "quantized_matmul(rows 2..16)",
        )
        return out
    if norm_weight is not None:
        check(
            lib.exo_norm_qmv(
                _ptr(x), _ptr(norm_weight), eps, _ptr(qw.weight), _ptr(qw.scales),
                _ptr(qw.biases), _ptr(residual), _ptr(out), M, qw.N, K, qw.bits, qw.group_size,
                _stream(),
            ),
            "quantized_matmul(norm)",
        )
        return out
    if M > QMV_MAX_M or gemm_rows:
        ws = qmm_workspace(M, qw.N, x.device)
        check(
            lib.exo_qmm_ws(
                _ptr(x), _ptr(qw.weight), _ptr(qw.scales), _ptr(qw.biases), _ptr(residual),
                _ptr(out), _ptr(ws), 0 if ws is None else ws.numel(), M, qw.N, K, qw.bits,
                qw.group_size, _stream(),
            ),
            "quantized_matmul(gemm)",
        )
        return out
    check(
        lib.exo_qmv(
            _ptr(x), _ptr(qw.weight), _ptr(qw.scales), _ptr(qw.biases), _ptr(residual), _ptr(out),
            M, qw.N, K, qw.bits, qw.group_size, _stream(),
        ),
        "quantized_matmul",
    )
    return out


def qmm_swiglu(x, gate: QuantizedWeight, up: QuantizedWeight, out=None,
               split_k: bool = True) -> torch.Tensor:
    """silu(x @ gate^T) * (x @ up^T) on the matrix cores (any M): one launch, or a K-split
    launch plus a reduce + SwiGLU launch where few output tiles would leave the chip idle
    (``split_k=False``: never)."""
    lib = native.load()
    M, K = x.shape
    if K != gate.K or gate.K != up.K or gate.N != up.N or gate.bits != up.bits:
        raise ValueError("qmm_swiglu: gate and up must have the same shape and bits as x's K")
    if out is None:
        out = torch.empty(M, gate.N, dtype=torch.bfloat16, device=x.device)
    ws = qmm_workspace(M, gate.N, x.device, pair=True) if split_k else None
    check(
        lib.exo_qmm_swiglu_ws(
            _ptr(x), _ptr(gate.weight), _ptr(gate.scales), _ptr(gate.biases), _ptr(up.weight),
            _ptr(up.scales), _ptr(up.biases), _ptr(out), _ptr(ws), 0 if ws is None else ws.numel(),
            M, gate.N, K, gate.bits, gate.group_size, _stream(),
        ),
        "qmm_swiglu",
    )
    return out


def qmm(x, qw: QuantizedWeight, residual=None, out=None) -> torch.Tensor:
    """Force the matrix-core path (any M)."""
    lib = native.load()
    M, K = x.shape
    if out is None:
        out = torch.empty(M, qw.N, dtype=torch.bfloat16, device=x.device)
    check(
        lib.exo_qmm(
            _ptr(x), _ptr(qw.weight), _ptr(qw.scales), _ptr(qw.biases), _ptr(residual), _ptr(out),
            M, qw.N, K, qw.bits, qw.group_size, _stream(),
        ),
        "qmm",
    )
    return out


def qmv_swiglu(x, gate: QuantizedWeight, up: QuantizedWeight, out=None, norm_weight=None,
               eps: float = 0.0) -> torch.Tensor:
    """silu(x @ gate^T) * (x @ up^T) for M <= 16, optionally on rms_norm(x)."""
    lib = native.load()
    M, K = x.shape
    assert gate.N == up.N and gate.K == up.K == K and gate.bits == up.bits
    if out is None:
        out = torch.empty(M, gate.N, dtype=torch.bfloat16, device=x.device)
    if 2 <= M <= QMV_MAX_M:
        ws = qmv_workspace(2 * gate.N, x.device)
        check(
            lib.exo_norm_qmv_swiglu_ws(
                _ptr(x), _ptr(norm_weight), eps, _ptr(gate.weight), _ptr(gate.scales),
                _ptr(gate.biases), _ptr(up.weight), _ptr(up.scales), _ptr(up.biases), _ptr(out),
                _ptr(ws), ws.numel(), M, gate.N, K, gate.bits, gate.group_size, _stream(),
            ),
            "qmv_swiglu(rows 2..16)",
        )
        return out
    check(
        lib.exo_norm_qmv_swiglu(
            _ptr(x), _ptr(norm_weight), eps, _ptr(gate.weight), _ptr(gate.scales), _ptr(gate.biases), _ptr(up.weight),
            _ptr(up.scales), _ptr(up.biases), _ptr(out), M, gate.N, K, gate.bits,
            gate.group_size, _stream(),
        ),
        "qmv_swiglu",
    )
    return out


def check_expert_ids(idx: torch.Tensor, E: int, what: str) -> None:
    """Reject expert ids outside [0, E).  Reads the indices back (a host synchronisation),
    so it is skipped while the stream is being captured into a graph; callers whose indices
    come straight from ``router_topk`` (in range by construction) pass
    ``check_indices=False``.  The kernels clamp the id only so that a bad one cannot
    address memory outside the weight tensor."""
    if idx.numel() == 0 or torch.cuda.is_current_stream_capturing():
        return
    lo, hi = int(idx.min()), int(idx.max())
    if lo < 0 or hi >= E:
        raise ValueError(f"{what}: expert ids span [{lo}, {hi}], outside [0, {E})")


def gather_qmm(x: torch.Tensor, qw: QuantizedWeight, rhs_indices: torch.Tensor, out=None,
               check_indices: bool = True):
    """mx.gather_qmm(x, w, s, b, rhs_indices=idx, transpose=True) for decode-sized
    inputs: x bf16 [T, R, K] (R == 1 or topk), idx int32 [T, topk] -> bf16 [T, topk, N]."""
    lib = native.load()
    T, R, K = x.shape
    topk = rhs_indices.shape[1]
    assert rhs_indices.dtype == torch.int32 and rhs_indices.shape[0] == T
    E = qw.weight.shape[0]
    if check_indices:
        check_expert_ids(rhs_indices, E, "gather_qmm")
    if out is None:
        out = torch.empty(T, topk, qw.N, dtype=torch.bfloat16, device=x.device)
    check(
        lib.exo_gather_qmv(
            _ptr(x), _ptr(qw.weight), _ptr(qw.scales), _ptr(qw.biases), _ptr(rhs_indices),
            _ptr(out), T, topk, R, E, qw.N, K, qw.bits, qw.group_size, _stream(),
        ),
        "gather_qmm",
    )
    return out


def gather_qmv_combine(x, qw: QuantizedWeight, idx, scores, residual=None, out=None, scratch=None,
                       check_indices: bool = True):
    """SwitchGLU's down projection for decode-sized inputs fused with the weighted sum over
    the top-k experts and the residual: x bf16 [T,topk,K], idx int32 [T,topk], scores bf16
    [T,topk], residual bf16 [T,N] -> bf16 [T,N].  ``scratch`` (bf16 [T,topk,N]) serves the
    shapes the fused kernel does not take."""
    lib = native.load()
    T, topk, K = x.shape
    E = qw.weight.shape[0]
    if check_indices:
        check_expert_ids(idx, E, "gather_qmv_combine")
    if out is None:
        out = torch.empty(T, qw.N, dtype=torch.bfloat16, device=x.device)
    check(
        lib.exo_gather_qmv_combine(
            _ptr(x), _ptr(qw.weight), _ptr(qw.scales), _ptr(qw.biases), _ptr(idx), _ptr(scores),
            _ptr(residual), _ptr(out), _ptr(scratch), T, topk, E, qw.N, K, qw.bits,
            qw.group_size, _stream(),
        ),
        "gather_qmv_combine",
    )
    return out


def moe_group(idx: torch.Tensor, E: int, check_indices: bool = True) -> torch.Tensor:
    """Sort the (token, slot) pairs of idx int32 [T, topk] by expert; the returned workspace
    feeds grouped_qmm for every projection that shares this routing decision."""
    lib = native.load()
    T, topk = idx.shape
    assert idx.dtype == torch.int32 and idx.is_contiguous()
    if check_indices:
        check_expert_ids(idx, E, "moe_group")
    nbytes = lib.exo_moe_group_workspace(T, topk, E)
    ws = torch.empty(nbytes // 4, dtype=torch.int32, device=idx.device)
    check(lib.exo_moe_group(_ptr(idx), T, topk, E, _ptr(ws), nbytes, _stream()), "moe_group")
    return ws


def grouped_qmm(x: torch.Tensor, qw: QuantizedWeight, group_ws: torch.Tensor, topk: int, out=None):
    """mx.gather_qmm for prefill-sized inputs on the matrix cores: x bf16 [T, R, K] (R == 1
    or topk), routing prepared by moe_group -> bf16 [T, topk, N]."""
    lib = native.load()
    T, R, K = x.shape
    E = qw.weight.shape[0]
    if K != qw.K:
        raise ValueError(f"grouped_qmm: x has K={K}, weight has K={qw.K}")
    if out is None:
        out = torch.empty(T, topk, qw.N, dtype=torch.bfloat16, device=x.device)
    check(
        lib.exo_gather_qmm(
            _ptr(x), _ptr(qw.weight), _ptr(qw.scales), _ptr(qw.biases), _ptr(group_ws), _ptr(out),
            T, topk, R, E, qw.N, K, qw.bits, qw.group_size, _stream(),
        ),
        "grouped_qmm",
    )
    return out


def grouped_qmm_swiglu(x: torch.Tensor, gate: QuantizedWeight, up: QuantizedWeight,
                       group_ws: torch.Tensor, topk: int, out=None):
    """SwitchGLU's gate/up + swiglu for prefill-sized inputs, one launch: x bf16 [T, R, K]
    (R == 1 or topk), routing prepared by moe_group -> bf16 [T, topk, N]."""
    lib = native.load()
    T, R, K = x.shape
    E = gate.weight.shape[0]
    if K != gate.K or gate.K != up.K or gate.N != up.N or gate.bits != up.bits:
        raise ValueError("grouped_qmm_swiglu: gate and up must have the same shape and bits as x's K")
    if out is None:
        out = torch.empty(T, topk, gate.N, dtype=torch.bfloat16, device=x.device)
    check(
        lib.exo_gather_qmm_swiglu(
            _ptr(x), _ptr(gate.weight), _ptr(gate.scales), _ptr(gate.biases), _ptr(up.weight),
            _ptr(up.scales), _ptr(up.biases), _ptr(group_ws), _ptr(out), T, topk, R, E, gate.N, K,
            gate.bits, gate.group_size, _stream(),
        ),
        "grouped_qmm_swiglu",
    )
    return out


def gather_qmv_swiglu(x, gate: QuantizedWeight, up: QuantizedWeight, idx, out=None,
                      norm_weight=None, eps: float = 0.0, check_indices: bool = True):
    """SwitchGLU's gate/up + swiglu: x bf16 [T,K], idx int32 [T,topk] -> [T,topk,N];
    ``norm_weight`` fuses a preceding rms_norm(x, norm_weight, eps)."""
    lib = native.load()
    T, K = x.shape
    topk = idx.shape[1]
    E = gate.weight.shape[0]
    if check_indices:
        check_expert_ids(idx, E, "gather_qmv_swiglu")
    if out is None:
        out = torch.empty(T, topk, gate.N, dtype=torch.bfloat16, device=x.device)
    check(
        lib.exo_norm_gather_qmv_swiglu(
            _ptr(x), _ptr(norm_weight), eps, _ptr(gate.weight), _ptr(gate.scales),
            _ptr(gate.biases), _ptr(up.weight), _ptr(up.scales), _ptr(up.biases), _ptr(idx),
            _ptr(out), T, topk, E, gate.N, K, gate.bits, gate.group_size, _stream(),
        ),
        "gather_qmv_swiglu",
    )
    return out


def route_gather_qmv_swiglu(x, router_logits, k: int, renorm: bool, gate: QuantizedWeight,
                            up: QuantizedWeight, out=None, norm_weight=None, eps: float = 0.0):
    """router_topk + gather_qmv_swiglu in one launch (decode): x bf16 [T,K], router_logits
    bf16 [T,E] -> (idx int32 [T,k], scores bf16 [T,k], out [T,k,N])."""
    lib = native.load()
    T, K = x.shape
    E = gate.weight.shape[0]
    if router_logits.shape != (T, E):
        raise ValueError(f"router_logits {tuple(router_logits.shape)} != ({T}, {E})")
    idx = torch.empty(T, k, dtype=torch.int32, device=x.device)
    sc = torch.empty(T, k, dtype=torch.bfloat16, device=x.device)
    if out is None:
        out = torch.empty(T, k, gate.N, dtype=torch.bfloat16, device=x.device)
    check(
        lib.exo_norm_route_gather_qmv_swiglu(
            _ptr(x), _ptr(norm_weight), eps, _ptr(router_logits), int(renorm), _ptr(idx), _ptr(sc),
            _ptr(gate.weight), _ptr(gate.scales), _ptr(gate.biases), _ptr(up.weight),
            _ptr(up.scales), _ptr(up.biases), _ptr(out), T, k, E, gate.N, K, gate.bits,
            gate.group_size, _stream(),
        ),
        "route_gather_qmv_swiglu",
    )
    return idx, sc, out


# ------------------------------------------------------------------ small ops


def add_rms_norm(x, residual, weight, eps: float, h_out=None, n_out=None):
    """h = x (+ residual, bf16 add); returns (h, rms_norm(h) * weight)."""
    lib = native.load()
    rows, H = x.shape
    if n_out is None:
        n_out = torch.empty_like(x)
    if residual is not None and h_out is None:
        h_out = torch.empty_like(x)
    check(
        lib.exo_add_rmsnorm(
            _ptr(x), _ptr(residual), _ptr(weight), _ptr(h_out), _ptr(n_out), rows, H, eps,
            _stream(),
        ),
        "add_rms_norm",
    )
    return (h_out if residual is not None else x), n_out


def rms_norm(x, weight, eps: float, out=None):
    """mx.fast.rms_norm over the last axis of x [rows, H]."""
    return add_rms_norm(x, None, weight, eps, None, out)[1]


def rope_kv_append(qkv, q_out, k_cache, v_cache, pos, inv_freq, B, T, Hq, Hkv, D,
                   q_norm_w=None, k_norm_w=None, eps: float = 0.0, rope_tab=None):
    """Split fused qkv [B*T,(Hq+2Hkv)*D]; (q/k head norm;) RoPE at pos[b]+t; q -> q_out
    [B*T,Hq*D]; k,v -> caches [B,Hkv,S_max,D].  ``rope_tab`` (from rope_table): the angles'
    cosines and sines are read from it for positions inside it."""
    lib = native.load()
    S_max = k_cache.shape[2]
    check(
        lib.exo_rope_kv_append_tab(
            _ptr(qkv), _ptr(q_out), _ptr(k_cache), _ptr(v_cache), _ptr(pos), _ptr(inv_freq),
            _ptr(rope_tab), 0 if rope_tab is None else rope_tab.shape[0],
            _ptr(q_norm_w), _ptr(k_norm_w), eps, B, T, Hq, Hkv, D, S_max, _stream(),
        ),
        "rope_kv_append",
    )


def sdpa_decode_workspace(B: int, Hq: int, D: int, device) -> torch.Tensor:
    n = native.load().exo_sdpa_decode_workspace(B, Hq, D)
    return torch.zeros(n // 4, dtype=torch.float32, device=device)  # counters start at 0


def sdpa_decode(q, k_cache, v_cache, pos, out, workspace, scale, B, Hq, Hkv, D):
    lib = native.load()
    check(
        lib.exo_sdpa_decode(
            _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(pos), _ptr(out), _ptr(workspace), scale,
            B, Hq, Hkv, D, k_cache.shape[2], _stream(),
        ),
        "sdpa_decode",
    )


def rope_table(inv_freq: torch.Tensor, S_max: int, D: int) -> torch.Tensor:
    """float32 [S_max, D/2, 2]: (cos, sin) of position * inv_freq."""
    lib = native.load()
    tab = torch.empty(S_max, D // 2, 2, dtype=torch.float32, device=inv_freq.device)
    check(lib.exo_rope_table(_ptr(inv_freq), _ptr(tab), S_max, D, _stream()), "rope_table")
    return tab


ATTN_MID_KEYS = 3072         # EXO_ATTN_MID_KEYS of the C header
ATTN_LONG_KEYS = 6144        # EXO_ATTN_LONG_KEYS
ATTN_VERY_LONG_KEYS = 12288  # EXO_ATTN_VERY_LONG_KEYS


def attn_decode(qkv, k_cache, v_cache, pos, inv_freq, out, workspace, scale, B, Hq, Hkv, D,
                q_norm_w=None, k_norm_w=None, eps: float = 0.0, rope_tab=None, keys_hint: int = 0):
    """rope (+ head norm) + cache append + attention for one new token per sequence.
    ``keys_hint``: keys the longest sequence holds as far as the host knows (0: unknown); from
    ATTN_LONG_KEYS and again from ATTN_VERY_LONG_KEYS on the launch is laid out for longer
    contexts."""
    lib = native.load()
    if rope_tab is not None and rope_tab.shape[0] < k_cache.shape[2]:
        raise ValueError("rope table shorter than the cache")
    check(
        lib.exo_attn_decode_hint(
            _ptr(qkv), _ptr(k_cache), _ptr(v_cache), _ptr(pos), _ptr(inv_freq), _ptr(rope_tab),
            _ptr(q_norm_w),
            _ptr(k_norm_w), eps, _ptr(out), _ptr(workspace), scale, B, Hq, Hkv, D,
            k_cache.shape[2], int(keys_hint), _stream(),
        ),
        "attn_decode",
    )


def sdpa_prefill(q, k_cache, v_cache, pos, out, scale, B, T, Hq, Hkv, D):
    lib = native.load()
    check(
        lib.exo_sdpa_prefill(
            _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(pos), _ptr(out), scale, B, T, Hq, Hkv,
            D, k_cache.shape[2], _stream(),
        ),
        "sdpa_prefill",
    )


def kv_export_nhd(cache_row, start: int, n: int, out=None):
    """Positions [start, start+n) of one layer's cache row [Hkv,S_max,D] -> [n,Hkv,D]."""
    lib = native.load()
    Hkv, S_max, D = cache_row.shape
    if not cache_row.is_contiguous():
        raise ValueError("kv_export_nhd: cache row must be contiguous")
    if out is None:
        out = torch.empty(n, Hkv, D, dtype=cache_row.dtype, device=cache_row.device)
    if n == 0 and 0 <= start <= S_max:
        return out
    check(lib.exo_kv_export_nhd(_ptr(cache_row), _ptr(out), Hkv, S_max, D, start, n, _stream()),
          "kv_export_nhd")
    return out


def kv_import_nhd(wire, cache_row, start: int):
    """wire [n,Hkv,D] -> positions [start, start+n) of cache_row [Hkv,S_max,D] (in place)."""
    lib = native.load()
    Hkv, S_max, D = cache_row.shape
    n = wire.shape[0]
    if tuple(wire.shape[1:]) != (Hkv, D) or wire.dtype != cache_row.dtype:
        raise ValueError(f"kv_import_nhd: wire {tuple(wire.shape)} does not fit cache row "
                         f"{tuple(cache_row.shape)}")
    if not (cache_row.is_contiguous() and wire.is_contiguous()):
        raise ValueError("kv_import_nhd: tensors must be contiguous")
    if n == 0 and 0 <= start <= S_max:
        return cache_row
    check(lib.exo_kv_import_nhd(_ptr(wire), _ptr(cache_row), Hkv, S_max, D, start, n, _stream()),
          "kv_import_nhd")
    return cache_row


def swiglu(gate, up, out=None):
    lib = native.load()
    if out is None:
        out = torch.empty_like(gate)
    check(lib.exo_swiglu(_ptr(gate), _ptr(up), _ptr(out), gate.numel(), _stream()), "swiglu")
    return out


def router_topk(logits, k: int, renorm: bool):
    """-> (idx int32 [rows,k], scores bf16 [rows,k])."""
    lib = native.load()
    rows, E = logits.shape
    idx = torch.empty(rows, k, dtype=torch.int32, device=logits.device)
    sc = torch.empty(rows, k, dtype=torch.bfloat16, device=logits.device)
    check(
        lib.exo_router_topk(_ptr(logits), _ptr(idx), _ptr(sc), rows, E, k, int(renorm), _stream()),
        "router_topk",
    )
    return idx, sc


def moe_combine(y, scores, residual=None, out=None):
    lib = native.load()
    T, topk, H = y.shape
    if out is None:
        out = torch.empty(T, H, dtype=torch.bfloat16, device=y.device)
    check(
        lib.exo_moe_combine(_ptr(y), _ptr(scores), _ptr(residual), _ptr(out), T, topk, H, _stream()),
        "moe_combine",
    )
    return out


def argmax_workspace(rows: int, device) -> torch.Tensor:
    n = native.load().exo_argmax_workspace(rows)
    return torch.empty(n // 4, dtype=torch.float32, device=device)


def argmax_logsumexp(logits, token, lse, logprob, workspace, pos_inc=None):
    """Greedy sampler + log-normaliser over bf16 logits [rows, V]."""
    lib = native.load()
    rows, V = logits.shape
    check(
        lib.exo_argmax_logsumexp(
            _ptr(logits), _ptr(token), _ptr(lse), _ptr(logprob), _ptr(workspace), _ptr(pos_inc),
            rows, V, _stream(),
        ),
        "argmax_logsumexp",
    )
