"""flash_forward_splitkv_static -- the split-KV entry point that allocates nothing (its partials live in a scratch array
built into the library) -- against flash_forward_splitkv with a caller-owned workspace: same kernels, so the outputs must
be bit-identical, on two calls in a row of which the second is smaller (it reuses the array the first one filled)."""
import ctypes as C

import numpy as np
import pytest

from helpers import check_o_lse, oracle_forward_batched, randn_f16_gpu

pytestmark = pytest.mark.gpu


def _both(fa, q, k, v, S, **kw):
    """(O, LSE) through the workspace entry point and through the static-scratch one, called through the C ABI."""
    import torch
    from flash_attn_amd import binding

    B, H, Nq, d = q.shape
    o_ws, lse_ws = fa.flash_forward_splitkv(q, k, v, num_splits=S, **kw)
    o = torch.full((B, H, Nq, d), float("nan"), dtype=torch.float16, device=q.device)
    lse = torch.full((B, H, Nq), float("nan"), dtype=torch.float32, device=q.device)
    p = binding.make_params(q, k, v, o, lse, None, kw.get("causal", False), kw.get("window", (-1, -1)),
                            kw.get("alibi_slopes"), 0.0, 0, 0, S)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = fa.lib().flash_forward_splitkv_static(C.byref(p), stream)
    assert rc == 0, fa.lib().flash_strerror(rc)
    torch.cuda.synchronize()
    return (o_ws, lse_ws), (o, lse)


@pytest.mark.parametrize("first,second", [
    # decode stream: 8 MiB of partials, then 25 KiB
    (dict(B=4, H=32, Hk=32, Nq=1, Nk=8192, d=128, S=16), dict(B=1, H=4, Hk=4, Nq=1, Nk=1000, d=128, S=3)),
    # tiled split kernel with masks, ragged sizes; then grouped decode (heads as rows of the tiled kernel)
    (dict(B=2, H=4, Hk=4, Nq=300, Nk=1021, d=64, S=5, causal=True), dict(B=2, H=8, Hk=2, Nq=1, Nk=700, d=128, S=4)),
    # 8-wave split kernel, then a problem that resolves to one split (no partials at all)
    (dict(B=1, H=2, Hk=2, Nq=600, Nk=900, d=128, S=3, causal=True), dict(B=1, H=2, Hk=2, Nq=70, Nk=100, d=32, S=4)),
])
def test_static_scratch_matches_workspace_entry_point(fa, oracle, first, second):
    import torch
    for c in (first, second):
        c = dict(c)
        B, H, Hk, Nq, Nk, d, S = (c.pop(x) for x in ("B", "H", "Hk", "Nq", "Nk", "d", "S"))
        q = randn_f16_gpu((B, H, Nq, d), 51)
        k = randn_f16_gpu((B, Hk, Nk, d), 52)
        v = randn_f16_gpu((B, Hk, Nk, d), 53)
        (o_ws, lse_ws), (o, lse) = _both(fa, q, k, v, S, **c)
        assert torch.equal(o, o_ws), "O differs from the workspace entry point"
        assert torch.equal(lse, lse_ws), "LSE differs from the workspace entry point"
        kr, vr = (t.repeat_interleave(H // Hk, dim=1).contiguous() for t in (k, v))
        O, L = oracle_forward_batched(oracle, q, kr, vr, **c)
        check_o_lse(o, lse, O, L, f"static scratch {Nq}x{Nk} S={S}")


def test_static_scratch_rejects_what_does_not_fit(fa):
    """B=64, H=64, 128 splits of one query row at d=128 need 270 MB of partials: an error code, nothing launched (K and V
    point at a buffer far smaller than the shape says, which a launch would overrun)."""
    import torch

    q = torch.zeros((64, 64, 1, 128), dtype=torch.float16, device="cuda")
    kv = torch.zeros(4096, dtype=torch.float16, device="cuda")
    o = torch.full_like(q, 7.0)
    lse = torch.zeros((64, 64, 1), dtype=torch.float32, device="cuda")
    p = fa.FlashParams()
    p.Q, p.K, p.V, p.O, p.LSE = q.data_ptr(), kv.data_ptr(), kv.data_ptr(), o.data_ptr(), lse.data_ptr()
    p.B, p.H, p.Nq, p.Nk, p.d = 64, 64, 1, 16384, 128
    p.softmax_scale = 0.1
    p.window_left = p.window_right = -1
    p.num_splits = 128
    rc = fa.lib().flash_forward_splitkv_static(C.byref(p), None)
    assert rc == -8 and b"scratch" in fa.lib().flash_strerror(rc)
    torch.cuda.synchronize()
    assert bool((o == 7.0).all())
