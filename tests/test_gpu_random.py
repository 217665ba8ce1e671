"""GPU parity on random requests: shapes, head dims (any value 1 ... 128), grouped heads, every mask family, ALiBi,
dropout, scales, split counts and kernel hints drawn from a seeded generator, each compared with the CPU oracle on
the same inputs (O within 2e-3 + 1e-2 relative, LSE within 1e-4: helpers.check_o_lse).  The named edge cases live in
test_gpu_edge_cases.py; this sweep is for the combinations nobody thought of."""
import numpy as np
import pytest

from helpers import check_o_lse, oracle_forward_batched, randn_f16_gpu

pytestmark = pytest.mark.gpu


def _draw(rng, oracle, case):
    import torch
    d = int(rng.choice([int(rng.integers(1, 129)), int(rng.integers(97, 129)), 128, 64, 31, 100]))
    Hk = int(rng.choice([1, 2, 3]))
    G = int(rng.choice([1, 1, 2, 4, 8]))
    H = Hk * G
    B = int(rng.choice([1, 2]))
    Nq = int(rng.choice([1, 1, 2, 17, 64, 127, 128, 129, 200, 257, 300, 513]))
    Nk = Nq if rng.random() < 0.4 else int(rng.choice([1, 5, 63, 64, 65, 128, 200, 333, 512, 777]))
    fam = int(rng.integers(0, 5))
    kw = {}
    if fam == 1:
        kw = dict(causal=True)
    elif fam == 2:
        kw = dict(causal=True, window=(int(rng.choice([0, 7, 64, 100, 256])), -1))
    elif fam == 3:
        kw = dict(window=(int(rng.choice([0, 5, 32, 128, 300])), int(rng.choice([0, 9, 64, 200]))))
    elif fam == 4:
        kw = dict(window=(-1, int(rng.choice([0, 33, 128]))))
    okw = dict(kw)
    if rng.random() < 0.3:
        sl = oracle.alibi_slopes(H)
        kw["alibi_slopes"], okw["slopes"] = torch.from_numpy(sl).cuda(), sl
    p = float(rng.choice([0.0, 0.0, 0.0, 0.1, 0.5]))
    if rng.random() < 0.1:
        sc = float(rng.choice([-0.3, 0.0, 0.05, 1.0]))
        kw["softmax_scale"], okw["scale"] = sc, sc
    if p > 0.0:
        keep = oracle.dropout_keep_mask(case, 3, p, B, H, Nq, Nk)
        kw.update(dropout_p=p, seed=case, offset=3)
        okw.update(keep_mask=torch.from_numpy(keep), p_drop=p)
    hint = int(rng.choice([0, 0, 1, 2]))
    S = int(rng.choice([1, 1, 0, 2, 3, 5, 8]))
    return B, H, Hk, Nq, Nk, d, kw, okw, hint, S


@pytest.mark.parametrize("seed", [101, 102, 103, 104])
def test_random_requests_match_the_oracle(fa, oracle, seed):
    rng = np.random.default_rng(seed)
    for case in range(100):
        B, H, Hk, Nq, Nk, d, kw, okw, hint, S = _draw(rng, oracle, 1000 * seed + case)
        q = randn_f16_gpu((B, H, Nq, d), 10 * case + 1)
        k = randn_f16_gpu((B, Hk, Nk, d), 10 * case + 2)
        v = randn_f16_gpu((B, Hk, Nk, d), 10 * case + 3)
        kr, vr = (t.repeat_interleave(H // Hk, dim=1).contiguous() for t in (k, v))
        what = (f"seed {seed} case {case}: B{B} H{H}/{Hk} Nq{Nq} Nk{Nk} d{d} splits {S} hint {hint} "
                f"{ {a: b for a, b in kw.items() if a != 'alibi_slopes'} } alibi {'alibi_slopes' in kw}")
        O, L = oracle_forward_batched(oracle, q, kr, vr, **okw)
        o, lse = fa.flash_forward_splitkv(q, k, v, num_splits=S, kernel_hint=hint, **kw)
        check_o_lse(o, lse, O, L, what)
        if S == 1:
            o, lse = fa.flash_forward(q, k, v, kernel_hint=hint, **kw)
            check_o_lse(o, lse, O, L, what + " (flash_forward)")
