"""The allocation-free attention entry point, dc_gather_attn_static_bf16, through the C ABI.

It shares the kernels of dc_gather_attn_bf16 and keeps the per-split softmax partials in a
static device array inside the library instead of a caller's workspace, so its output must
equal dc_gather_attn_bf16's bit for bit.  Two calls in a row share that array; the second
one here is smaller, so it runs over what the first one left behind.
"""
import math

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _case(hip, g, b, h, grp, hd, n, n_idx, sink, recent, new_tok, per_unit):
    k = torch.randn((b, h, n, hd), generator=g, device=DEV).to(torch.bfloat16)
    v = torch.randn((b, h, n, hd), generator=g, device=DEV).to(torch.bfloat16)
    q = torch.randn((b, h * grp, hd), generator=g, device=DEV).to(torch.bfloat16)
    nk = torch.randn((b, h, hd), generator=g, device=DEV).to(torch.bfloat16) if new_tok else None
    nv = torch.randn((b, h, hd), generator=g, device=DEV).to(torch.bfloat16) if new_tok else None
    lo, hi = sink, n - recent
    idx = torch.stack([torch.randperm(hi - lo, generator=g, device=DEV)[:n_idx] for _ in range(b * h)]).to(torch.int32)
    n_unit = None
    if per_unit:
        n_unit = torch.randint(0, n_idx + 1, (b * h,), generator=g, device=DEV).to(torch.int32)
    return k, v, q, nk, nv, idx, n_unit, lo, hi


def _static_call(hip, k, v, q, nk, nv, idx, n_unit, lo, hi, sink, recent, out, lse):
    b, h, n, hd = k.shape
    grp = q.shape[1] // h
    p = lambda t: None if t is None else t.data_ptr()
    return hip.lib.dc_gather_attn_static_bf16(
        p(q), p(k), p(v), p(idx), p(nk), p(nv), p(out), p(lse), b, h, grp, hd, idx.shape[1], idx.stride(0),
        p(n_unit), lo, sink, hi, recent, None, k.stride(0), k.stride(1), k.stride(2), v.stride(0), v.stride(1),
        v.stride(2), 1.0 / math.sqrt(hd), torch.cuda.current_stream().cuda_stream)


def test_static_scratch_attention_matches_the_workspace_entry_point():
    from diffcache_amd import _hip as hip
    g = torch.Generator(device=DEV).manual_seed(99)
    cases = [
        # b, h, grp, hd, n, n_idx, sink, recent, new token, per-unit sizes
        (2, 8, 4, 128, 9000, 2048, 4, 64, True, False),      # 16 units x 17 splits
        (1, 3, 4, 128, 3000, 300, 4, 64, True, True),        # smaller: runs over the first call's partials
        (1, 2, 7, 128, 2000, 500, 2, 9, False, False),
        (1, 2, 1, 64, 500, 70, 0, 0, False, False),
        (1, 1, 8, 256, 400, 33, 1, 1, True, True),
    ]
    for case in cases:
        print("static attention case", case, flush=True)
        b, h, grp, hd, n, n_idx, sink, recent, new_tok, per_unit = case
        k, v, q, nk, nv, idx, n_unit, lo, hi = _case(hip, g, *case)
        want_lse = torch.empty((b, h * grp), dtype=torch.float32, device=DEV)
        want = hip.gather_attn(q, k, v, idx, n_idx, lo, sink, hi, recent, nk, nv, lse=want_lse, n_idx_unit=n_unit)
        out = torch.full_like(want, float("nan"))
        lse = torch.full_like(want_lse, float("nan"))
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated()
        free_before = torch.cuda.mem_get_info()[0]          # the driver's count: sees a hipMalloc inside the library too
        rc = _static_call(hip, k, v, q, nk, nv, idx, n_unit, lo, hi, sink, recent, out, lse)
        assert rc == 0, hip.lib.dc_last_error().decode()
        assert torch.cuda.memory_allocated() == before
        torch.cuda.synchronize()
        if case is not cases[0]:    # (the first call on a device resolves the array's address: the code object may be loaded then)
            assert torch.cuda.mem_get_info()[0] == free_before, case
        assert torch.equal(out.view(torch.int16), want.view(torch.int16)), case
        assert torch.equal(lse, want_lse), case


def test_static_scratch_attention_rejects_sizes_beyond_its_scratch():
    from diffcache_amd import _hip as hip
    # 4096 units x 1100 attended rows x 4 heads x 128: 9 splits x 2 KiB x 4096 = 75 MB > 32 MiB
    b, h, grp, hd, n = 512, 8, 4, 128, 8
    k = torch.zeros((1, 1, n, hd), dtype=torch.bfloat16, device=DEV)   # never read: the call must refuse first
    q = torch.zeros((b, h * grp, hd), dtype=torch.bfloat16, device=DEV)
    out = torch.full_like(q, 7.0)
    idx = torch.zeros((b * h, 1024), dtype=torch.int32, device=DEV)
    p = lambda t: t.data_ptr()
    need = hip.lib.dc_attn_workspace_bytes(b * h, grp, hd, 1024 + 4 + 64 + 1)
    assert need > (32 << 20)
    rc = hip.lib.dc_gather_attn_static_bf16(
        p(q), p(k), p(k), p(idx), None, None, p(out), None, b, h, grp, hd, 1024, 1024, None, 4, 4, 4, 0, None,
        0, 0, hd, 0, 0, hd, 0.1, torch.cuda.current_stream().cuda_stream)
    assert rc == -12, rc
    msg = hip.lib.dc_last_error().decode()
    assert "scratch" in msg and str(need) in msg, msg
    torch.cuda.synchronize()
    assert bool((out == 7.0).all())                  # nothing was launched
    # a size that fits is accepted right after the refusal
    test_static_scratch_attention_matches_the_workspace_entry_point()
