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
    """B=1, H=16, 2048 rows, 4 splits at d=128 need 64 MiB of partials, twice the scratch: an error code and nothing
    launched.  Every buffer has the size the shape says, so that a regression of the check shows as a wrong return code
    or a changed output, not as a kernel reading out of bounds."""
    import torch

    B, H, Nq, Nk, d, S = 1, 16, 2048, 512, 128, 4
    q = randn_f16_gpu((B, H, Nq, d), 61)
    k = randn_f16_gpu((B, H, Nk, d), 62)
    v = randn_f16_gpu((B, H, Nk, d), 63)
    assert sum(fa.workspace_bytes(B, H, Nq, Nk, d, S)) > fa.FLASH_STATIC_SCRATCH_BYTES
    o = torch.full((B, H, Nq, d), 7.0, dtype=torch.float16, device="cuda")
    lse = torch.full((B, H, Nq), 7.0, dtype=torch.float32, device="cuda")
    from flash_attn_amd import binding
    p = binding.make_params(q, k, v, o, lse, None, False, (-1, -1), None, 0.0, 0, 0, S)
    rc = fa.lib().flash_forward_splitkv_static(C.byref(p), None)
    assert rc == -8 and b"scratch" in fa.lib().flash_strerror(rc)
    torch.cuda.synchronize()
    assert bool((o == 7.0).all()) and bool((lse == 7.0).all())
    # one split fewer rows: 32 MiB + 256 KiB still does not fit; half the rows do
    p.Nq = 1024
    assert fa.lib().flash_forward_splitkv_static(C.byref(p), None) == -8
    p.Nq = 1000
    assert fa.lib().flash_forward_splitkv_static(C.byref(p), None) == 0
    torch.cuda.synchronize()
    # (the static call read rows 0..999 of every head slice at the stride of 1000 rows: compare on a contiguous copy)
    qc = q.reshape(-1)[:B * H * 1000 * d].view(B, H, 1000, d)
    o_c, lse_c = fa.flash_forward_splitkv(qc.contiguous(), k, v, num_splits=S)
    assert torch.equal(o.reshape(-1)[:B * H * 1000 * d].view(B, H, 1000, d), o_c)
    assert torch.equal(lse.reshape(-1)[:B * H * 1000].view(B, H, 1000), lse_c)


def test_static_entry_point_allocates_nothing_and_replays_from_a_graph(fa):
    """The two promises beyond bit-identical results: no device memory is allocated or freed by the call (the free
    memory the runtime reports and the bytes PyTorch holds are the same before and after), and the call can be captured
    into a HIP graph -- three replays with new inputs in between, each compared with an eager call of the workspace
    entry point."""
    import torch
    from flash_attn_amd import binding

    B, H, Hk, Nq, Nk, d, S = 2, 8, 8, 1, 6000, 128, 6
    q = randn_f16_gpu((B, H, Nq, d), 71)
    k = randn_f16_gpu((B, Hk, Nk, d), 72)
    v = randn_f16_gpu((B, Hk, Nk, d), 73)
    o = torch.empty((B, H, Nq, d), dtype=torch.float16, device="cuda")
    lse = torch.empty((B, H, Nq), dtype=torch.float32, device="cuda")
    p = binding.make_params(q, k, v, o, lse, None, False, (-1, -1), None, 0.0, 0, 0, S)
    L = fa.lib()

    def call():
        rc = L.flash_forward_splitkv_static(C.byref(p), C.c_void_p(torch.cuda.current_stream().cuda_stream))
        assert rc == 0, L.flash_strerror(rc)

    call()  # first call on the device and of this shape class: symbol look-up, kernel attributes
    torch.cuda.synchronize()
    free0, held0 = torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated()
    for _ in range(3):
        call()
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0 and torch.cuda.memory_allocated() == held0

    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        call()
    for rep in range(3):
        q.copy_(randn_f16_gpu((B, H, Nq, d), 300 + rep))
        k.copy_(randn_f16_gpu((B, Hk, Nk, d), 400 + rep))
        o.zero_()
        lse.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        o_e, lse_e = fa.flash_forward_splitkv(q, k, v, num_splits=S)  # eager, workspace of its own
        torch.cuda.synchronize()
        assert torch.equal(o, o_e) and torch.equal(lse, lse_e), f"replay {rep} differs from the eager call"
