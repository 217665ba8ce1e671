"""Shared helpers of the parity tests: seeded inputs, tolerances of the contract, oracle in batches."""
import numpy as np

# Contract tolerances: fp16 O within max-abs 2e-3 plus relative 1e-2 of the CPU path, fp32 LSE within 1e-4.
O_ATOL, O_RTOL, LSE_ATOL = 2e-3, 1e-2, 1e-4


def randn_f16_gpu(shape, seed, device="cuda"):
    """fp16 tensor = RN_fp16(N(0,1)) from the portable counter-based generator of the oracle (a pure function of seed and
    element index: the bench + verify driver's `--fill normal --seed` and the benchmark draw the same bits), filled on
    the host and copied to the device."""
    import torch
    from oracle import cpu_oracle

    return torch.from_numpy(cpu_oracle.normal_f16(tuple(shape), seed)).to(device)


def to_f32_np(t):
    return t.detach().float().cpu().numpy()


def check_o_lse(o_gpu, lse_gpu, o_ref, lse_ref, what=""):
    """o_gpu fp16 / lse_gpu fp32 (numpy or torch) against the oracle's fp32 arrays."""
    o_gpu = o_gpu if isinstance(o_gpu, np.ndarray) else to_f32_np(o_gpu)
    lse_gpu = lse_gpu if isinstance(lse_gpu, np.ndarray) else to_f32_np(lse_gpu)
    assert np.isfinite(o_gpu).all(), f"{what}: non-finite O"
    err = np.abs(o_gpu - o_ref)
    bound = O_ATOL + O_RTOL * np.abs(o_ref)
    worst = float((err - bound).max())
    assert worst <= 0.0, f"{what}: O off by {float(err.max()):.3e} (max |err|), worst excess {worst:.3e}"
    fin = np.isfinite(lse_ref)
    assert np.array_equal(np.isneginf(lse_gpu), np.isneginf(lse_ref)), f"{what}: -inf pattern of LSE differs"
    if fin.any():
        lerr = float(np.abs(lse_gpu[fin] - lse_ref[fin]).max())
        assert lerr <= LSE_ATOL, f"{what}: LSE off by {lerr:.3e}"
    return float(err.max())


def oracle_forward_batched(oracle, q, k, v, **kw):
    """Oracle over torch fp16 device tensors, one batch entry at a time to bound host memory.
    A keep_mask given as a torch tensor is sliced alongside."""
    B = q.shape[0]
    keep = kw.pop("keep_mask", None)
    Os, Ls = [], []
    for b in range(B):
        km = None if keep is None else keep[b:b + 1].cpu().numpy()
        O, L = oracle.attention_forward(to_f32_np(q[b:b + 1]), to_f32_np(k[b:b + 1]), to_f32_np(v[b:b + 1]),
                                        keep_mask=km, **kw)
        Os.append(O)
        Ls.append(L)
    return np.concatenate(Os), np.concatenate(Ls)
