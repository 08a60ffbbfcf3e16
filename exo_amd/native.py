"""ctypes binding of libexo_mi355x.so (the C ABI declared in include/exo_mi355x.h).

The library is the only compute path: if it is missing, loading raises and every
operator of this package fails loudly.  There is no CPU or eager-PyTorch fallback.
"""

from __future__ import annotations

import ctypes as C
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "libexo_mi355x.so"

_vp = C.c_void_p
_i = C.c_int
_i64 = C.c_int64
_f = C.c_float

# name -> (restype, argtypes); mirrors include/exo_mi355x.h one to one
SIGNATURES: dict[str, tuple] = {
    "exo_abi_version": (_i, []),
    "exo_last_error": (C.c_char_p, []),
    "exo_last_variant": (C.c_char_p, []),
    "exo_dequant_two_roundings": (_i, []),
    "exo_unpack_codes": (_i, [_vp, _vp, _i64, _i, _vp]),
    "exo_dequantize": (_i, [_vp, _vp, _vp, _vp, _i64, _i, _i, _i, _vp]),
    "exo_embed_dequant": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "exo_qmv": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "exo_qmv_swiglu": (_i, [_vp] * 8 + [_i, _i, _i, _i, _i, _vp]),
    "exo_norm_qmv": (_i, [_vp, _vp, _f, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "exo_qmv_workspace": (_i64, [_i]),
    "exo_norm_qmv_ws": (_i, [_vp, _vp, _f, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i, _i, _i, _i, _i, _vp]),
    "exo_norm_qmv_swiglu": (_i, [_vp, _vp, _f] + [_vp] * 7 + [_i, _i, _i, _i, _i, _vp]),
    "exo_norm_qmv_swiglu_ws": (_i, [_vp, _vp, _f] + [_vp] * 8 + [_i64, _i, _i, _i, _i, _i, _vp]),
    "exo_moe_group_workspace": (_i64, [_i, _i, _i]),
    "exo_moe_group": (_i, [_vp, _i, _i, _i, _vp, _i64, _vp]),
    "exo_gather_qmm": (_i, [_vp] * 6 + [_i] * 8 + [_vp]),
    "exo_gather_qmm_swiglu": (_i, [_vp] * 9 + [_i] * 8 + [_vp]),
    "exo_qmm": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "exo_qmm_workspace": (_i64, [_i, _i]),
    "exo_qmm_ws": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i, _i, _i, _i, _i, _vp]),
    "exo_qmm_swiglu": (_i, [_vp] * 8 + [_i, _i, _i, _i, _i, _vp]),
    "exo_qmm_swiglu_workspace": (_i64, [_i, _i]),
    "exo_qmm_swiglu_ws": (_i, [_vp] * 9 + [_i64, _i, _i, _i, _i, _i, _vp]),
    "exo_gather_qmv": (_i, [_vp] * 6 + [_i] * 8 + [_vp]),
    "exo_gather_qmv_combine": (_i, [_vp] * 9 + [_i] * 7 + [_vp]),
    "exo_gather_qmv_swiglu": (_i, [_vp] * 9 + [_i] * 7 + [_vp]),
    "exo_norm_gather_qmv_swiglu": (_i, [_vp, _vp, _f] + [_vp] * 8 + [_i] * 7 + [_vp]),
    "exo_norm_route_gather_qmv_swiglu": (_i, [_vp, _vp, _f, _vp, _i] + [_vp] * 9 + [_i] * 7 + [_vp]),
    "exo_add_rmsnorm": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _f, _vp]),
    "exo_rope_kv_append": (_i, [_vp] * 8 + [_f] + [_i] * 6 + [_vp]),
    "exo_rope_kv_append_tab": (_i, [_vp] * 7 + [_i] + [_vp] * 2 + [_f] + [_i] * 6 + [_vp]),
    "exo_sdpa_decode_workspace": (_i64, [_i, _i, _i]),
    "exo_sdpa_decode": (_i, [_vp] * 6 + [_f] + [_i] * 5 + [_vp]),
    "exo_sdpa_decode_static": (_i, [_vp] * 5 + [_f] + [_i] * 5 + [_vp]),
    "exo_attn_decode": (_i, [_vp] * 8 + [_f, _vp, _vp, _f] + [_i] * 5 + [_vp]),
    "exo_attn_decode_hint": (_i, [_vp] * 8 + [_f, _vp, _vp, _f] + [_i] * 6 + [_vp]),
    "exo_rope_table": (_i, [_vp, _vp, _i, _i, _vp]),
    "exo_sdpa_prefill": (_i, [_vp] * 5 + [_f] + [_i] * 6 + [_vp]),
    "exo_kv_export_nhd": (_i, [_vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "exo_kv_import_nhd": (_i, [_vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "exo_swiglu": (_i, [_vp, _vp, _vp, _i64, _vp]),
    "exo_router_topk": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "exo_moe_combine": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _vp]),
    "exo_argmax_workspace": (_i64, [_i]),
    "exo_argmax_logsumexp": (_i, [_vp] * 6 + [_i, _i, _vp]),
    "exo_sample_workspace": (_i64, [_i]),
    "exo_sample": (_i, [_vp] * 13 + [_i64, _i, _i, _i, _i, _vp]),
}


class NativeError(RuntimeError):
    pass


_lib = None


def load() -> C.CDLL:
    """Load the shared library (once).  Raises NativeError when it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise NativeError(
            f"{LIB_PATH} not found: build it with `python -m exo_amd.build` "
            "(there is no fallback path)"
        )
    lib = C.CDLL(str(LIB_PATH))
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().exo_last_error().decode("utf-8", "replace")
        if rc == -1:
            raise ValueError(f"{what}: {msg}")
        raise NativeError(f"{what}: {msg} (rc={rc})")


def last_variant() -> str:
    """The kernel instance the calling thread's latest matmul / attention call selected."""
    return load().exo_last_variant().decode("utf-8", "replace")
