#!/usr/bin/env python3
"""Writes the golden vectors under tests/golden/ from the reference's own CPU functions.

Run in the authoring container, where the reference checkout exists and `make -C oracle` has produced
oracle/_ref/libref_cpu.so (the reference's verfiy / attention_forward_cpu / num_splits_heuristic, src/main.cu:254-422,
compiled unmodified).  The vectors are data only: seeded fp16 inputs, the fp32 outputs the reference computed for
them, and argument/result tables.  The GPU box and CI never need the reference: tests read these files.

    python tests/golden/make_golden.py
"""
import ctypes as C
import json
import os
import sys
import tempfile

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

from oracle import cpu_oracle as co  # noqa: E402


def slopes_pos(H):
    # 2^(-8 (h+1) / H): the formula of src/main.cu:66 with the sign the operator contract uses
    return np.array([2.0 ** (-8.0 / H * (i + 1)) for i in range(H)], dtype=np.float32)


def attention_cases():
    out = {}
    rng = np.random.default_rng(20240611)
    # A: the CPU-verifier configuration (B=1, H=2, N=128, d=64)
    # B: ragged sizes (N=77, d=40, H=3)
    for tag, (B, H, N, d) in {"A": (1, 2, 128, 64), "B": (1, 3, 77, 40)}.items():
        q, k, v = [rng.standard_normal((B, H, N, d)).astype(np.float16) for _ in range(3)]
        out[f"{tag}_q"], out[f"{tag}_k"], out[f"{tag}_v"] = q, k, v
        scale = np.float32(1.0 / np.sqrt(d))
        out[f"{tag}_scale"] = scale
        sl = slopes_pos(H)
        out[f"{tag}_slopes"] = sl
        variants = {"plain": {}, "causal": {"causal": True}}
        if tag == "B":
            variants.update({"window9": {"window_size": 9}, "alibi": {"slopes": sl},
                             "causal_alibi_window20": {"causal": True, "slopes": sl, "window_size": 20}})
        for name, kw in variants.items():
            out[f"{tag}_O_{name}"] = co.ref_attention_forward_cpu(q.astype(np.float32), k.astype(np.float32),
                                                                  v.astype(np.float32), scale, **kw)
    return out


def heuristic_table():
    rows = []
    for sms in (108, 256):
        for bhm in (1, 2, 4, 8, 16, 32, 48, 64, 100, 128, 200, 256, 512, 1023, 1024, 2048):
            for nblk in (1, 2, 3, 4, 7, 8, 16, 31, 32, 64, 128):
                for max_splits in (nblk, 128):
                    seq = nblk * 128
                    rows.append([bhm, sms, nblk, max_splits, seq,
                                 co.ref_num_splits_heuristic(bhm, sms, nblk, max_splits, seq)])
    # the reference's checked-in run (B=1, H=8, N=1021, d=31; src/main.cu:39-49,125) and the benchmark shapes
    for args in ((8 * 8, 108, 8, 8, 1024), (8 * 8, 256, 8, 8, 1024), (1024, 256, 16, 16, 2048), (512, 256, 128, 128, 16384),
                 (512, 108, 128, 128, 16384)):
        rows.append(list(args) + [co.ref_num_splits_heuristic(*args)])
    return rows


def verfiy_cases():
    """verfiy prints its error count; capture it from stdout (src/main.cu:264-275)."""
    R = co.ref_lib()
    R.ref_verfiy.restype = None
    f32p = C.POINTER(C.c_float)
    R.ref_verfiy.argtypes = [f32p, f32p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_float]
    rng = np.random.default_rng(5)
    cases = []
    libc = C.CDLL(None)
    for n, tol in ((64, 0.06), (64, 0.01), (32, 0.5)):
        cpu = rng.standard_normal(n).astype(np.float32)
        dev = (cpu * (1 + 0.1 * rng.standard_normal(n))).astype(np.float32)
        dev[3] = np.nan
        dev[7] = np.inf
        with tempfile.TemporaryFile() as tf:
            sys.stdout.flush()
            saved = os.dup(1)
            os.dup2(tf.fileno(), 1)
            try:
                R.ref_verfiy(cpu.ctypes.data_as(f32p), dev.ctypes.data_as(f32p), 1, 1, n, 1, tol)
                libc.fflush(None)
            finally:
                os.dup2(saved, 1)
                os.close(saved)
            tf.seek(0)
            text = tf.read().decode()
        count = int(text.strip().splitlines()[-1].split("error:")[1].split("=")[0])
        cases.append({"cpu": cpu.tolist(), "dev": [float(x) if np.isfinite(x) else str(x) for x in dev], "tol": tol,
                      "count": count})
    return cases


def main():
    if co.ref_lib() is None:
        sys.exit("oracle/_ref/libref_cpu.so missing: run `make -C oracle` where the reference checkout exists")
    np.savez(os.path.join(HERE, "reference_cpu_vectors.npz"), **attention_cases())
    with open(os.path.join(HERE, "heuristic_table.json"), "w") as f:
        json.dump({"columns": ["batch_nheads_mblocks", "num_SMs", "num_n_blocks", "max_splits", "seq_len", "result"],
                   "rows": heuristic_table()}, f, separators=(",", ":"))
    with open(os.path.join(HERE, "verfiy_cases.json"), "w") as f:
        json.dump(verfiy_cases(), f, separators=(",", ":"))
    print("golden vectors written")


if __name__ == "__main__":
    main()
