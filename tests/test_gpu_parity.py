"""GPU parity: the HIP path, called through the C ABI, against the CPU oracle on identical seeded inputs.
The five cases named cfgN are the configurations of the benchmark contract at full size."""
import numpy as np
import pytest

from helpers import check_o_lse, oracle_forward_batched, randn_f16_gpu, to_f32_np

pytestmark = pytest.mark.gpu


def _qkv(B, H, Nq, Nk, d, seed=0):
    return (randn_f16_gpu((B, H, Nq, d), 3 * seed + 1), randn_f16_gpu((B, H, Nk, d), 3 * seed + 2),
            randn_f16_gpu((B, H, Nk, d), 3 * seed + 3))


def test_cfg1_plain(fa, oracle):
    q, k, v = _qkv(1, 2, 128, 128, 64)
    o, lse = fa.flash_forward(q, k, v)
    O, L = oracle_forward_batched(oracle, q, k, v)
    check_o_lse(o, lse, O, L, "cfg1")


def test_cfg2_causal_prefill(fa, oracle):
    q, k, v = _qkv(4, 16, 2048, 2048, 128)
    o, lse = fa.flash_forward(q, k, v, causal=True)
    O, L = oracle_forward_batched(oracle, q, k, v, causal=True)
    check_o_lse(o, lse, O, L, "cfg2")


def test_cfg3_local_alibi(fa, oracle):
    import torch

    B, H = 2, 16
    q, k, v = _qkv(B, H, 4096, 4096, 64)
    slopes = oracle.alibi_slopes(H)
    o, lse = fa.flash_forward(q, k, v, window=(256, 0), alibi_slopes=torch.from_numpy(slopes).cuda())
    O, L = oracle_forward_batched(oracle, q, k, v, window=(256, 0), slopes=slopes)
    check_o_lse(o, lse, O, L, "cfg3")


def test_cfg4_odd_causal_dropout(fa, oracle):
    B, H, N, d = 8, 32, 1000, 96
    q, k, v = _qkv(B, H, N, N, d)
    o, lse, km = fa.flash_forward(q, k, v, causal=True, dropout_p=0.1, seed=1234, offset=0, return_keep_mask=True)
    keep = oracle.dropout_keep_mask(1234, 0, 0.1, B, H, N, N)
    km = km.cpu().numpy()
    tri = np.tril(np.ones((N, N), dtype=bool))
    # the mask the fused kernel applied, bit-exact against the CPU Philox replica (causal part is all it visits)
    assert np.array_equal(km[..., tri], keep[..., tri])
    # and the separately launched mask kernel over the full rectangle
    km2 = fa.dropout_keep_mask(B, H, N, N, 0.1, 1234, 0).cpu().numpy()
    assert np.array_equal(km2, keep)
    import torch
    O, L = oracle_forward_batched(oracle, q, k, v, causal=True, keep_mask=torch.from_numpy(keep), p_drop=0.1)
    check_o_lse(o, lse, O, L, "cfg4")


def test_cfg5_splitkv_decode(fa, oracle):
    B, H, Nk, d, S = 16, 32, 16384, 128, 16
    q, k, v = _qkv(B, H, 1, Nk, d)
    o, lse, (op, lp) = fa.flash_forward_splitkv(q, k, v, num_splits=S, return_partials=True)
    O, L = oracle_forward_batched(oracle, q, k, v)
    check_o_lse(o, lse, O, L, "cfg5")
    # per-split partials against the oracle's restatement of the reference split kernel, one batch entry
    Ot, Ls, Ms, LSEp = oracle.splitkv_partials(to_f32_np(q[:1]), to_f32_np(k[:1]), to_f32_np(v[:1]), S)
    assert np.abs(to_f32_np(op[:1]) - Ot).max() <= 2e-3
    assert np.abs(to_f32_np(lp[:1]) - LSEp).max() <= 1e-4
