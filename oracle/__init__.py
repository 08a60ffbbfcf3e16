"""CPU oracle for the per-shard transformer forward on MLX affine-quantized weights.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package (``exo_amd``) may import
this directory; it is the checker used by ``tests/``, ``__graft_entry__.smoke()``
and the ``cpu_baseline`` leg of ``bench.py``.

The arithmetic it restates lives in two third-party dependencies of the reference
that are not vendored under the reference tree: ``mlx`` 0.32.0 (uv.lock:1376-1378)
and ``mlx-lm`` 0.31.3 (uv.lock:1547-1549).  The restatement follows the operator
documentation the reference carries in ``.typings/mlx/core/__init__.pyi`` and the
call sites in ``src/exo/worker/engines/mlx``.

Pin status per function (what, other than the formula itself, checks it):

* ``pack_codes`` / ``unpack_codes``   pinned  - hand-written words from the docstring
  example (.pyi:4180-4184) + exhaustive code/slot round trip.
* ``dequantize``                      pinned for the formula ``s*q+beta`` by hand
  computed values; the ROUNDING ORDER to bf16 (modes M1/M2 below) is
  "parity unpinned": only ``mx.dequantize`` itself could decide it.
* ``quantize``                        "parity unpinned" (edge rules of mx.quantize);
  documented formula pinned by reconstruction-error bound and exact recovery of
  representable grids.  Used only to synthesise weights.
* ``qmm`` / ``gather_qmm``            pinned - equals dense float64 matmul of the
  dequantised matrix (library routine); gather form by brute-force loops.
* ``rms_norm``, ``rope``, ``sdpa``, ``swiglu``, ``router_topk``
                                      pinned - against ``transformers`` /
  ``torch.nn.functional`` routines and closed-form invariants.
* ``llama_forward`` / ``qwen3_moe_forward``  pinned against ``transformers``
  ``LlamaForCausalLM`` / ``Qwen3MoeForCausalLM`` built from config objects and fed
  the dequantised weights; mlx_lm-specific rounding points (where bf16 rounding
  happens between ops) are "parity unpinned".
* generation protocol (prefill / trim 2 / re-feed last two tokens)  pinned by the
  cache-length invariants the reference's tests state
  (src/exo/worker/tests/unittests/test_mlx/test_kv_prefix_cache.py:157,374).
"""
