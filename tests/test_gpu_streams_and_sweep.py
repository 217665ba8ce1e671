"""GPU tests of how the entry points behave as a library: launches on a caller's stream, capture into a HIP graph
(the entry points allocate nothing and keep no state, so a captured launch can be replayed), and a seeded sweep over
random shapes and mask combinations against the CPU oracle."""
import numpy as np
import pytest

from helpers import check_o_lse, oracle_forward_batched, randn_f16_gpu

pytestmark = pytest.mark.gpu


def test_launch_on_a_side_stream_matches_default_stream(fa):
    import torch

    q, k, v = (randn_f16_gpu((2, 4, 300, 128), s) for s in (1, 2, 3))
    o0, l0 = fa.flash_forward(q, k, v, causal=True)
    torch.cuda.synchronize()
    s = torch.cuda.Stream()  # default priority
    o1 = torch.empty_like(o0)
    l1 = torch.empty_like(l0)
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        fa.flash_forward(q, k, v, causal=True, out=o1, lse=l1, stream=s)
    s.synchronize()
    assert torch.equal(o0, o1) and torch.equal(l0, l1)


@pytest.mark.parametrize("mode", ["prefill_d128", "prefill_d64", "decode_split"])
def test_graph_capture_and_replay(fa, mode):
    """A captured launch replays correctly: three replays, new inputs copied into the captured buffers in between,
    each replay compared with an eager launch on the same inputs."""
    import torch

    if mode == "prefill_d128":
        shape_q, shape_k, kw, split = (2, 4, 384, 128), (2, 4, 384, 128), dict(causal=True), False
    elif mode == "prefill_d64":
        shape_q, shape_k, kw, split = (2, 4, 200, 64), (2, 4, 333, 64), dict(window=(64, 8)), False
    else:
        shape_q, shape_k, kw, split = (2, 8, 1, 128), (2, 2, 4096, 128), dict(), True
    q, k, v = randn_f16_gpu(shape_q, 11), randn_f16_gpu(shape_k, 12), randn_f16_gpu(shape_k, 13)
    B, H, Nq, d = shape_q
    o = torch.empty(shape_q, dtype=torch.float16, device="cuda")
    lse = torch.empty((B, H, Nq), dtype=torch.float32, device="cuda")
    S = 8
    ws = (torch.empty((B, H, S, Nq, d), dtype=torch.float32, device="cuda"),
          torch.empty((B, H, S, Nq), dtype=torch.float32, device="cuda")) if split else None

    def launch(out, out_lse):
        if split:
            fa.flash_forward_splitkv(q, k, v, num_splits=S, workspace=ws, out=out, lse=out_lse, **kw)
        else:
            fa.flash_forward(q, k, v, out=out, lse=out_lse, **kw)

    launch(o, lse)  # warm-up outside the capture: one-time kernel attribute calls happen here
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        launch(o, lse)
    o_e, lse_e = torch.empty_like(o), torch.empty_like(lse)
    for rep in range(3):
        q.copy_(randn_f16_gpu(shape_q, 100 + rep))
        k.copy_(randn_f16_gpu(shape_k, 200 + rep))
        o.zero_()
        lse.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        launch(o_e, lse_e)  # eager, same inputs
        torch.cuda.synchronize()
        assert torch.equal(o, o_e), f"{mode}: replay {rep} differs from the eager launch"
        assert torch.equal(lse, lse_e)


def test_random_shape_sweep(fa, oracle):
    """200 seeded random problems: sizes around the tile edges and beyond the 8-wave kernel's thresholds, every mask
    family, ALiBi, non-default scales, dropout, grouped K/V heads, with explicit, automatic and no key splits."""
    import torch

    rng = np.random.default_rng(2024)
    dims = [8, 16, 31, 32, 40, 64, 64, 72, 96, 100, 128, 128, 128]
    for case in range(200):
        d = int(rng.choice(dims))
        B, Hk = int(rng.integers(1, 3)), int(rng.integers(1, 3))
        H = Hk * int(rng.choice([1, 1, 2, 4, 8]))
        Nq = int(rng.choice([1, 1, 7, 64, 65, 129, 200, 257, 300, 511, 640, 1025, 1100, 1400]))
        Nk = Nq if rng.random() < 0.5 else int(rng.integers(1, 1600))
        fam = int(rng.integers(0, 4))
        kw, okw = {}, {}
        if fam == 1:
            kw = okw = dict(causal=True)
        elif fam == 2:
            w = (int(rng.integers(0, 700)), int(rng.integers(0, 700)))
            kw, okw = dict(window=w), dict(window=w)
        elif fam == 3:
            w = (int(rng.integers(0, 800)), -1)
            kw, okw = dict(causal=True, window=w), dict(causal=True, window=w)
        if rng.random() < 0.3:
            sl = oracle.alibi_slopes(H)
            kw = dict(kw, alibi_slopes=torch.from_numpy(sl).cuda())
            okw = dict(okw, slopes=sl)
        if rng.random() < 0.15:
            sc = float(rng.choice([0.02, 0.3, -0.1]))
            kw, okw = dict(kw, softmax_scale=sc), dict(okw, scale=sc)
        q = randn_f16_gpu((B, H, Nq, d), 1000 + case)
        k = randn_f16_gpu((B, Hk, Nk, d), 2000 + case)
        v = randn_f16_gpu((B, Hk, Nk, d), 3000 + case)
        kr, vr = (t.repeat_interleave(H // Hk, dim=1).contiguous() for t in (k, v))
        what = f"case {case}: B{B} H{H}/{Hk} Nq{Nq} Nk{Nk} d{d} {sorted(kw)}"
        S = int(rng.integers(0, 6))  # 0: the library chooses
        if rng.random() < 0.25:
            p = float(rng.choice([0.1, 0.5, 0.77]))
            seed, off = int(rng.integers(0, 2 ** 40)), int(rng.integers(0, 2 ** 33))
            keep = oracle.dropout_keep_mask(seed, off, p, B, H, Nq, Nk)
            okw = dict(okw, keep_mask=torch.from_numpy(keep), p_drop=p)
            kw = dict(kw, dropout_p=p, seed=seed, offset=off)
            what += f" dropout {p}"
        O, L = oracle_forward_batched(oracle, q, kr, vr, **okw)
        o, lse = fa.flash_forward(q, k, v, **kw)
        check_o_lse(o, lse, O, L, what)
        o, lse = fa.flash_forward_splitkv(q, k, v, num_splits=S, **kw)
        check_o_lse(o, lse, O, L, what + f" split {S}")
