"""The decode attention entry point that allocates nothing (static device scratch) against
the workspace-taking entry point it is a variant of, through the C ABI: bit-identical
output on two calls in a row, the second with a smaller input (its arrival counters then
sit where the first call left partial sums)."""

import numpy as np
import pytest
import torch

from exo_amd import native

pytestmark = pytest.mark.gpu


def _case(lib, dev, B, Hq, Hkv, D, S_max, lens, seed):
    g = torch.Generator(device=dev).manual_seed(seed)
    q = torch.randn(B, Hq * D, device=dev, generator=g).bfloat16()
    kc = torch.randn(B, Hkv, S_max, D, device=dev, generator=g).bfloat16()
    vc = torch.randn(B, Hkv, S_max, D, device=dev, generator=g).bfloat16()
    pos = torch.tensor([n - 1 for n in lens], dtype=torch.int32, device=dev)  # lens = pos + 1 keys
    scale = D ** -0.5
    st = torch.cuda.current_stream().cuda_stream
    ws = torch.zeros(lib.exo_sdpa_decode_workspace(B, Hq, D) // 4, dtype=torch.float32, device=dev)
    want = torch.empty(B, Hq * D, dtype=torch.bfloat16, device=dev)
    rc = lib.exo_sdpa_decode(q.data_ptr(), kc.data_ptr(), vc.data_ptr(), pos.data_ptr(),
                             want.data_ptr(), ws.data_ptr(), scale, B, Hq, Hkv, D, S_max, st)
    assert rc == 0, lib.exo_last_error()
    got = torch.full_like(want, float("nan"))
    before = torch.cuda.memory_allocated(dev)
    rc = lib.exo_sdpa_decode_static(q.data_ptr(), kc.data_ptr(), vc.data_ptr(), pos.data_ptr(),
                                    got.data_ptr(), scale, B, Hq, Hkv, D, S_max, st)
    assert rc == 0, lib.exo_last_error()
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated(dev) == before
    assert torch.equal(got.view(torch.int16), want.view(torch.int16)), (B, Hq, Hkv, D, lens)
    assert bool(torch.isfinite(got.float()).all())


def test_static_scratch_decode_attention_matches_workspace_variant(device):
    lib = native.load()
    print("no-alloc case 1: B=4 Hq=32 Hkv=8 D=128 S_max=1024", flush=True)
    _case(lib, device, 4, 32, 8, 128, 1024, [1000, 513, 64, 1], seed=1)
    print("no-alloc case 2 (smaller): B=2 Hq=8 Hkv=2 D=64 S_max=512", flush=True)
    _case(lib, device, 2, 8, 2, 64, 512, [300, 17], seed=2)
    print("no-alloc case 3: the largest size the scratch takes, B=8 Hq=32", flush=True)
    _case(lib, device, 8, 32, 8, 128, 256, [256, 200, 100, 50, 25, 12, 6, 3], seed=3)
    # beyond the limit: a clear error, nothing launched
    rc = lib.exo_sdpa_decode_static(1, 1, 1, 1, 1, 1.0, 9, 32, 8, 128, 256, None)
    assert rc == -1 and b"exceed the static scratch" in lib.exo_last_error()
