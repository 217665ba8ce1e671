#!/usr/bin/env python3
"""Benchmark of the FlashAttention-forward hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--only-main]

A step is one pass of the hot path over one batch of synthetic input already resident in HBM.  The headline
workload is the causal prefill configuration (B=4, H=16, Nq=Nk=2048, d=128); the split-KV decode configuration
(B=16, H=32, Nq=1, Nk=16384, d=128, 16 splits) and the remaining configurations are timed beside it and reported
in extra keys of the same JSON line.  Timing protocol: warm-up launches, then K back-to-back launches between two
HIP events on the launch stream (the reference's protocol, src/main.cu:187-213), plus a host clock around the same
region for ms_per_step.
"""
import argparse
import json
import math
import os
import subprocess
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_F16_TFLOPS = 2500.0  # MI355X dense fp16 MFMA
PEAK_HBM_GBPS = 8000.0    # MI355X HBM3E
METRIC = "fwd attention TFLOP/s + % fp16 MFMA peak; split-KV decode HBM GB/s"


def unmasked_pairs(Nq, Nk, causal, wl, wr):
    """Number of (i, j) pairs a head attends to (row index i + Nk - Nq)."""
    shift = Nk - Nq
    total = 0
    for i in range(Nq):
        ii = i + shift
        lo = max(0, ii - wl) if wl >= 0 else 0
        hi = Nk - 1
        if causal:
            hi = min(hi, ii)
        if wr >= 0:
            hi = min(hi, ii + wr)
        total += max(0, hi - lo + 1)
    return total


CONFIGS = {
    "cfg1": dict(B=1, H=2, Nq=128, Nk=128, d=64, causal=False, window=(-1, -1), alibi=False, p=0.0, splits=0),
    "cfg2": dict(B=4, H=16, Nq=2048, Nk=2048, d=128, causal=True, window=(-1, -1), alibi=False, p=0.0, splits=0),
    "cfg3": dict(B=2, H=16, Nq=4096, Nk=4096, d=64, causal=False, window=(256, 0), alibi=True, p=0.0, splits=0),
    "cfg4": dict(B=8, H=32, Nq=1000, Nk=1000, d=96, causal=True, window=(-1, -1), alibi=False, p=0.1, splits=0),
    "cfg5": dict(B=16, H=32, Nq=1, Nk=16384, d=128, causal=False, window=(-1, -1), alibi=False, p=0.0, splits=16),
}
# diagnostic shapes (not part of the contract; selectable with --workload, never in the default line)
DIAG = {
    "diag_noncausal": dict(B=4, H=16, Nq=2048, Nk=2048, d=128, causal=False, window=(-1, -1), alibi=False, p=0.0, splits=0),
    "diag_d64": dict(B=4, H=16, Nq=2048, Nk=2048, d=64, causal=True, window=(-1, -1), alibi=False, p=0.0, splits=0),
    "diag_long": dict(B=1, H=16, Nq=8192, Nk=8192, d=128, causal=True, window=(-1, -1), alibi=False, p=0.0, splits=0),
    "diag_window": dict(B=2, H=16, Nq=4096, Nk=4096, d=64, causal=False, window=(256, 0), alibi=False, p=0.0, splits=0),
    "diag_many_slices": dict(B=16, H=32, Nq=1024, Nk=1024, d=128, causal=True, window=(-1, -1), alibi=False, p=0.0, splits=0),
    "diag_many_slices_d64": dict(B=8, H=32, Nq=2048, Nk=2048, d=64, causal=True, window=(-1, -1), alibi=False, p=0.0, splits=0),
    "diag_many_slices_long": dict(B=8, H=32, Nq=4096, Nk=4096, d=128, causal=True, window=(-1, -1), alibi=False, p=0.0, splits=0),
    "diag_short": dict(B=32, H=32, Nq=512, Nk=512, d=64, causal=False, window=(-1, -1), alibi=False, p=0.0, splits=0),
    "diag_gqa_decode": dict(B=16, H=32, Hk=4, Nq=1, Nk=16384, d=128, causal=False, window=(-1, -1), alibi=False, p=0.0,
                            splits=16),
    # split-KV with more than one query row and the library's own split count (splits = -1): long keys, small batch
    "diag_split_long_keys": dict(B=1, H=8, Nq=512, Nk=32768, d=128, causal=False, window=(-1, -1), alibi=False, p=0.0, splits=-1),
    "diag_split_causal": dict(B=1, H=32, Nq=128, Nk=16384, d=128, causal=True, window=(-1, -1), alibi=False, p=0.0, splits=-1),
    "diag_split_ref_default": dict(B=2, H=8, Nq=1021, Nk=1021, d=31, causal=False, window=(-1, -1), alibi=False, p=0.0, splits=-1),
    # the reference's own run (src/main.cu:39-49) with the library's split count: one launch of 32-row work-groups
    "diag_ref_default": dict(B=1, H=8, Nq=1021, Nk=1021, d=31, causal=False, window=(-1, -1), alibi=False, p=0.0, splits=-1),
    # grouped-query prefill: the query heads of a K/V head read the same K and V
    "diag_gqa_prefill": dict(B=4, H=32, Hk=4, Nq=4096, Nk=4096, d=128, causal=True, window=(-1, -1), alibi=False, p=0.0, splits=0),
}
DESCR = {
    "cfg1": "plain fwd B=1 H=2 Nq=Nk=128 d=64",
    "cfg2": "causal prefill fwd B=4 H=16 Nq=Nk=2048 d=128",
    "cfg3": "local(256,0)+ALiBi fwd B=2 H=16 Nq=Nk=4096 d=64",
    "cfg4": "causal+dropout(0.1) fwd B=8 H=32 Nq=Nk=1000 d=96",
    "cfg5": "split-KV decode B=16 H=32 Nq=1 Nk=16384 d=128 num_splits=16",
    "diag_noncausal": "non-causal fwd B=4 H=16 Nq=Nk=2048 d=128 (diagnostic)",
    "diag_d64": "causal fwd B=4 H=16 Nq=Nk=2048 d=64 (diagnostic)",
    "diag_long": "causal fwd B=1 H=16 Nq=Nk=8192 d=128 (diagnostic)",
    "diag_many_slices": "causal fwd B=16 H=32 Nq=Nk=1024 d=128 (diagnostic)",
    "diag_many_slices_d64": "causal fwd B=8 H=32 Nq=Nk=2048 d=64 (diagnostic)",
    "diag_many_slices_long": "causal fwd B=8 H=32 Nq=Nk=4096 d=128 (diagnostic)",
    "diag_short": "plain fwd B=32 H=32 Nq=Nk=512 d=64 (diagnostic)",
    "diag_window": "local(256,0) fwd without ALiBi B=2 H=16 Nq=Nk=4096 d=64 (diagnostic)",
    "diag_gqa_decode": "split-KV decode, 8 query heads per K/V head, B=16 H=32 H_kv=4 Nq=1 Nk=16384 d=128 (diagnostic)",
    "diag_split_long_keys": "split-KV fwd, automatic split count, B=1 H=8 Nq=512 Nk=32768 d=128 (diagnostic)",
    "diag_split_causal": "split-KV causal fwd, automatic split count, B=1 H=32 Nq=128 Nk=16384 d=128 (diagnostic)",
    "diag_split_ref_default": "split-KV fwd, automatic split count, B=2 H=8 Nq=Nk=1021 d=31 (diagnostic)",
    "diag_ref_default": "split-KV fwd, automatic split count, B=1 H=8 Nq=Nk=1021 d=31: the reference's own run (diagnostic)",
    "diag_gqa_prefill": "causal fwd, 8 query heads per K/V head, B=4 H=32 H_kv=4 Nq=Nk=4096 d=128 (diagnostic)",
}


PROFILE_OF = {"cfg2": "fwd_kernel_d128_causal_prefill.md", "cfg3": "fwd_kernel_d64_local_alibi.md",
              "cfg4": "fwd_kernel_d96_causal_dropout.md", "cfg5": "decode_split_kernel_d128_splitkv_decode.md"}


def measured_traffic(name):
    """HBM bytes per launch from the committed rocprofv3 FETCH_SIZE / WRITE_SIZE summary of this workload (the line
    `traffic_bytes_per_launch: N` of the file under profiles/), or None when no summary exists."""
    f = PROFILE_OF.get(name)
    path = os.path.join(ROOT, "profiles", f) if f else None
    if not path or not os.path.exists(path):
        return None
    for line in open(path):
        if line.startswith("traffic_bytes_per_launch:"):
            return float(line.split(":")[1])
    return None


def flops_of(c):
    P = unmasked_pairs(c["Nq"], c["Nk"], c["causal"], *c["window"])
    return 4.0 * c["d"] * c["B"] * c["H"] * P


def decode_bytes(c):
    kv = 2 * c["B"] * c.get("Hk", c["H"]) * c["Nk"] * c["d"] * 2
    q = c["B"] * c["H"] * c["Nq"] * c["d"] * 2
    o = c["B"] * c["H"] * c["Nq"] * c["d"] * 2
    lse = c["B"] * c["H"] * c["Nq"] * 4
    return kv + q + o + lse


def make_inputs(c, seed=0):
    """Q, K, V = RN_fp16(N(0,1)) from the portable counter-based generator (oracle/: Philox4x32-10 + Box-Muller, a pure
    function of seed and element index), seeds 1, 2, 3 (+ 3 * seed); filled on the host, resident in HBM afterwards."""
    import torch
    from oracle import cpu_oracle as co

    out = []
    for n, s, heads in ((c["Nq"], 1, c["H"]), (c["Nk"], 2, c.get("Hk", c["H"])), (c["Nk"], 3, c.get("Hk", c["H"]))):
        out.append(torch.from_numpy(co.normal_f16((c["B"], heads, n, c["d"]), 3 * seed + s)).cuda())
    return out


def make_step(fa, c, q, k, v):
    """Returns a zero-argument callable that enqueues one pass (no allocation inside)."""
    import ctypes as C
    import torch
    from flash_attn_amd import binding

    B, H, Nq, Nk, d = c["B"], c["H"], c["Nq"], c["Nk"], c["d"]
    o = torch.empty((B, H, Nq, d), dtype=torch.float16, device="cuda")
    lse = torch.empty((B, H, Nq), dtype=torch.float32, device="cuda")
    slopes = None
    if c["alibi"]:
        slopes = torch.tensor([2.0 ** (-8.0 * (h + 1) / H) for h in range(H)], dtype=torch.float32, device="cuda")
    ws = (None, None)
    if c["splits"]:  # > 0: that many splits; < 0: split entry point with the library's own count
        S = fa.resolve_splits(B, H, Nq, Nk, d, max(0, c["splits"]), causal=c["causal"], window=c["window"],
                              H_kv=c.get("Hk", 0))
        if S > 1:
            ws = (torch.empty((B, H, S, Nq, d), dtype=torch.float32, device="cuda"),
                  torch.empty((B, H, S, Nq), dtype=torch.float32, device="cuda"))
    p = binding.make_params(q, k, v, o, lse, None, c["causal"], c["window"], slopes, c["p"], 1234, 0,
                            max(0, c["splits"]) if c["splits"] else 1, ws[0], ws[1])
    lib = fa.lib()
    fn = lib.flash_forward_splitkv if c["splits"] else lib.flash_forward
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    keep = (q, k, v, o, lse, slopes, ws)

    def step():
        rc = fn(C.byref(p), stream)
        if rc != 0:
            raise RuntimeError(f"launch failed: {rc} {keep is None}")

    return step, (o, lse)


def time_steps(step, steps, warmup):
    """(host ms per step, event ms per step) over `steps` back-to-back launches."""
    import torch

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        step()
    e1.record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    return (t1 - t0) * 1e3 / steps, e0.elapsed_time(e1) / steps


def stage_timeline(fa, c, q, k, v):
    """Per-work-group time stamps of the instrumented kernel instance (flash_params.stage_stamps_out, a debug output of
    the library): where a work-group of this workload spends its time, in microseconds of the 100 MHz device counter."""
    import numpy as np
    import torch

    slopes = None
    if c["alibi"]:
        slopes = torch.tensor([2.0 ** (-8.0 * (h + 1) / c["H"]) for h in range(c["H"])], dtype=torch.float32, device="cuda")
    kw = dict(causal=c["causal"], window=c["window"], alibi_slopes=slopes, dropout_p=c["p"], seed=1234, offset=0)
    for _ in range(300):  # long enough for the clocks to settle (a GPU fresh out of idle runs slower for some 50 ms)
        fa.flash_forward(q, k, v, **kw)
    st = fa.flash_forward(q, k, v, return_stage_stamps=True, **kw)[-1]
    torch.cuda.synchronize()
    t = st.cpu().numpy().astype(np.int64)
    t0 = t[:, 0].min()
    names = fa.stage_stamp_names()
    rel = (t[:, 1:7] - t[:, :1]) / 100.0
    tiles = t[:, 7] >> 32
    loop = (t[:, 5] - t[:, 4]) / 100.0
    out = {"work_groups": int(t.shape[0]), "first_entry_to_last_exit_us": float((t[:, 6].max() - t0) / 100.0),
           "mean_lifetime_us": float(rel[:, 5].mean()),
           "us_after_entry": {names[i + 1]: {"mean": float(rel[:, i].mean()), "min": float(rel[:, i].min()),
                                             "max": float(rel[:, i].max())} for i in range(6)},
           "tiles_per_group": {"mean": float(tiles.mean()), "max": int(tiles.max())},
           "us_per_tile_in_loop": float(loop.sum() / max(1, int((tiles - 1).clip(min=0).sum()))),
           "epilogue_us": float((rel[:, 5] - rel[:, 4]).mean())}
    # word 8: shader-clock cycles between the first barrier and the end of the loop -> the clock the CUs ran at there
    span = (t[:, 5] - t[:, 3]) / 100.0
    ok = span >= 3.0
    if ok.any():
        mhz = t[ok, 8] / span[ok]
        out["loop_clock_mhz"] = {"mean": float(mhz.mean()), "min": float(mhz.min()), "max": float(mhz.max())}
        out["shader_cycles_per_tile_in_loop"] = float(t[ok, 8].sum() / max(1, int(tiles[ok].sum())))
    xcc = (t[:, 7] >> 16) & 0xf
    cu_se = (t[:, 7] & 0xffff) >> 8  # CU, SH and SE fields of HW_ID
    out["distinct_cus"] = int(len(set(zip(xcc.tolist(), cu_se.tolist()))))
    return out


def shape_grid(fa):
    """Forward rate over the customary grid of attention benchmarks: 16384 tokens per launch, sequence lengths
    512 ... 16384, head dim 128 with 16 heads and 64 with 32, plain and causal.  Diagnostic only."""
    out = {}
    for d, H in ((128, 16), (64, 32)):
        for causal in (False, True):
            row = {}
            for N in (512, 1024, 2048, 4096, 8192, 16384):
                c = dict(B=16384 // N, H=H, Nq=N, Nk=N, d=d, causal=causal, window=(-1, -1), alibi=False, p=0.0, splits=0)
                q, k, v = make_inputs(c)
                step, _ = make_step(fa, c, q, k, v)
                fl = flops_of(c)
                _, ev_ms = time_steps(step, max(10, min(300, int(3e12 / fl))), 3)
                row[f"N={N}"] = round(fl / (ev_ms * 1e-3) / 1e12, 1)
                del q, k, v, step
            out[f"d={d} H={H} {'causal' if causal else 'plain'}"] = row
    return out


def mfma_sustained():
    """Sustained 32x32x16 fp16 MFMA rate of this GPU for zero / constant / random operands, and for random operands
    with the companion instructions of an attention loop beside every MFMA, measured by the stand-alone probe
    tests/driver/mfma_rate (a child process; about a second).  None when the probe is not built."""
    exe = os.path.join(ROOT, "tests", "driver", "mfma_rate")
    if not os.path.exists(exe):
        return None
    try:
        out = subprocess.run([exe], capture_output=True, text=True, timeout=120)
        return json.loads(out.stdout.strip().splitlines()[-1]) if out.returncode == 0 else None
    except (OSError, ValueError, IndexError, subprocess.TimeoutExpired):
        return None


# (b,h) slices of the 1-core sample per workload: about 2-12 s of CPU work each (cfg1 and cfg5 are small enough to run whole)
CPU_SLICES = {"cfg1": 2, "cfg2": 16, "cfg3": 8, "cfg4": 128, "cfg5": 512}


def cpu_baseline(c, q, k, v, budget_slices):
    """The reference's CPU path on a bounded sample of (b,h) slices of the workload, with the workload's own options.

    One core, as in the reference (src/main.cu:299-385 is single-threaded): the reference's own attention_forward_cpu
    (oracle/_ref, compiled from the reference checkout; kind "reference") where it can express the workload -- Nq == Nk,
    no dropout, and a window that is symmetric or (left, 0), which it computes as causal + symmetric window (the same
    visible set, src/main.cu:330-349) -- and the restatement (oracle/, kind "port") otherwise: explicit keep-mask,
    Nq != Nk.  Beside it, under "all_cores", the restatement spread over the host cores with OpenMP (rows in parallel, no
    masked-work skipping, like the reference).  Rates are algorithmic work of the sample over its time."""
    import numpy as np
    from oracle import cpu_oracle as co

    B, H, Nq, Nk, d = c["B"], c["H"], c["Nq"], c["Nk"], c["d"]
    wl, wr = c["window"]
    scale = 1.0 / math.sqrt(d)
    slopes_h = np.array([2.0 ** (-8.0 * (h + 1) / H) for h in range(H)], dtype=np.float32) if c["alibi"] else None
    decode = Nq == 1

    def sample(n):
        """First n slices in (b, h) order as a batch of one: [1, n, N, d] arrays, per-slice slopes, keep-mask."""
        qs = q.reshape(B * H, Nq, d)[:n].float().cpu().numpy()[None]
        g = H // k.shape[1]  # query heads per K/V head
        idx = [(i // H) * k.shape[1] + (i % H) // g for i in range(n)]
        ks = k.reshape(-1, Nk, d)[idx].float().cpu().numpy()[None]
        vs = v.reshape(-1, Nk, d)[idx].float().cpu().numpy()[None]
        sl = None if slopes_h is None else np.array([slopes_h[i % H] for i in range(n)], dtype=np.float32)
        keep = None
        if c["p"] > 0.0:  # the mask the kernel applies (seed 1234, offset 0 as in make_step), materialised on the CPU
            nb = (n + H - 1) // H
            keep = co.dropout_keep_mask(1234, 0, c["p"], nb, H, Nq, Nk).reshape(1, nb * H, Nq, Nk)[:, :n]
        return qs, ks, vs, sl, keep

    def work(n):
        if decode:
            return decode_bytes(dict(c, B=1, H=n, Hk=n)), "GB/s", 1e9
        return 4.0 * d * n * unmasked_pairs(Nq, Nk, c["causal"], wl, wr), "TFLOP/s", 1e12

    n = max(1, min(budget_slices, B * H))
    qs, ks, vs, sl, keep = sample(n)
    as_reference = (co.ref_lib() is not None and Nq == Nk and keep is None
                    and (wl == wr or (wl >= 0 and wr == 0)))
    reps = 20 if n * Nq * Nk * d < 5e7 else 1  # a sub-millisecond sample is repeated, best run kept
    best = float("inf")
    for _ in range(reps):
        t0 = time.perf_counter()
        if as_reference:
            co.ref_attention_forward_cpu(qs, ks, vs, scale, causal=c["causal"] or (wl >= 0 and wr == 0 and wl != wr),
                                         window_size=wl, slopes=sl)
        else:
            co.attention_forward(qs, ks, vs, scale, causal=c["causal"], window=c["window"], slopes=sl, keep_mask=keep,
                                 p_drop=c["p"], nthreads=1, skip_masked=False)
        best = min(best, time.perf_counter() - t0)
    w, unit, div = work(n)
    out = {"value": w / best / div, "unit": unit, "cores": 1, "kind": "reference" if as_reference else "port",
           "sample": f"{n} of {B * H} (b,h) slices of the same workload with its mask / slopes / keep-mask, {best:.3f} s"
                     + (f" (best of {reps})" if reps > 1 else "") + ", algorithmic work of the sample / time"}
    # all host cores: four times the slices, rows in parallel
    threads = co.default_threads()
    na = max(1, min(4 * n, B * H))
    if na != n:
        qs, ks, vs, sl, keep = sample(na)
    best = float("inf")
    for _ in range(reps):
        t0 = time.perf_counter()
        co.attention_forward(qs, ks, vs, scale, causal=c["causal"], window=c["window"], slopes=sl, keep_mask=keep,
                             p_drop=c["p"], nthreads=threads, skip_masked=False)
        best = min(best, time.perf_counter() - t0)
    w, unit, div = work(na)
    out["all_cores"] = {"value": w / best / div, "unit": unit, "cores": threads, "kind": "port",
                        "sample": f"{na} of {B * H} (b,h) slices, OpenMP over rows, {best:.3f} s"}
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU-baseline leg")
    ap.add_argument("--only-main", action="store_true", help="time only the headline workload (for profiling)")
    ap.add_argument("--workload", default="cfg2", choices=sorted(CONFIGS) + sorted(DIAG), help="headline workload")
    ap.add_argument("--cpu-slices", type=int, default=0,
                    help="(b,h) slices of the one-core CPU sample of every workload (0: a default per workload, "
                         "2-12 s of CPU work each)")
    ap.add_argument("--steady-launches", type=int, default=1000,
                    help="launches of the steady-state leg (the reference times 1000, src/main.cu:187-213); 0 = skip")
    ap.add_argument("--stage-timeline", action="store_true",
                    help="print the per-stage timeline of the headline workload (instrumented kernel instance) and exit")
    ap.add_argument("--zero-inputs", action="store_true",
                    help="diagnostic: all-zero Q, K, V instead of N(0,1) (same instruction stream; the power management "
                         "then leaves the clock high -- compare loop_clock_mhz of --stage-timeline); never a valid rate")
    ap.add_argument("--grid", action="store_true",
                    help="print a table of forward rates over sequence lengths 512 ... 16384 at 16384 tokens per launch "
                         "(d = 128 with 16 heads, d = 64 with 32; plain and causal) and exit")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also launch one plain elementwise kernel reading and writing 256 MiB each, so that a "
                         "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE run can be scaled against a known transfer")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no multi-GPU path exists); use --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    import flash_attn_amd as fa

    fa.lib()  # fails loudly when the HIP library is missing
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(2)

    if args.copy_calibration:
        src = torch.zeros(64 * 1024 * 1024, dtype=torch.float32, device="cuda")  # 256 MiB
        dst = torch.empty_like(src)
        torch.add(src, 1.0, out=dst)  # reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst

    if args.grid:
        print(json.dumps({"grid": shape_grid(fa), "unit": "TFLOP/s", "tokens_per_launch": 16384}))
        return

    name = args.workload
    c = CONFIGS[name] if name in CONFIGS else DIAG[name]
    q, k, v = make_inputs(c)
    if args.zero_inputs:
        for t in (q, k, v):
            t.zero_()
    if args.stage_timeline:
        print(json.dumps({"workload": f"{name}: {DESCR[name]}", "stage_timeline": stage_timeline(fa, c, q, k, v)}))
        return
    step, _ = make_step(fa, c, q, k, v)
    st_ms = None
    if args.steady_launches > 0 and not args.only_main:
        # The reference's own protocol comes first: one warm-up launch, then 1000 back-to-back launches between two
        # events (src/main.cu:187-213).  A GPU that comes out of idle runs its first tens of milliseconds at lower
        # clocks (the same launch takes 85-100 us there and 79 us from then on), so a timed region of 20 launches
        # taken first would measure the power management's ramp; taken after this leg it measures the rate the part
        # sustains, which is also what this leg reports.
        _, st_ms = time_steps(step, args.steady_launches, 1)
    host_ms, ev_ms = time_steps(step, args.steps, args.warmup)
    if c["Nq"] == 1:
        by = decode_bytes(c)
        value, unit = by / (host_ms * 1e-3) / 1e9, "GB/s"
        roof = {"bound": "hbm", "achieved": by / (ev_ms * 1e-3) / 1e9, "peak": PEAK_HBM_GBPS, "unit": "GB/s"}
    else:
        fl = flops_of(c)
        value, unit = fl / (host_ms * 1e-3) / 1e12, "TFLOP/s"
        roof = {"bound": "mfma", "achieved": fl / (ev_ms * 1e-3) / 1e12, "peak": PEAK_F16_TFLOPS, "unit": "TFLOP/s"}
    roof["frac"] = roof["achieved"] / roof["peak"]
    roof["kernel_ms"] = ev_ms
    roof["timed_over"] = f"{args.steps} launches (--steps) between two events on the launch stream"
    if st_ms is not None:
        # the steadier figure is the headline fraction: the 1000-launch leg; the --steps leg stays beside it
        ach = (by / (st_ms * 1e-3) / 1e9) if c["Nq"] == 1 else (flops_of(c) / (st_ms * 1e-3) / 1e12)
        roof["timed_steps"] = {"launches": args.steps, "ms": ev_ms, "achieved": roof["achieved"], "frac": roof["frac"]}
        roof.update(achieved=ach, frac=ach / roof["peak"], kernel_ms=st_ms,
                    timed_over=f"1 warm-up + {args.steady_launches} launches between two events on the launch stream "
                               f"(the reference's protocol), run before the --steps leg")
        roof["steady_state"] = {"launches": args.steady_launches, "ms": st_ms, "achieved": ach, "unit": roof["unit"],
                                "frac": ach / roof["peak"]}
    roof["traffic"] = measured_traffic(name)
    roof["traffic_source"] = (f"profiles/{PROFILE_OF[name]} (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of a committed run, "
                              f"not measured by this run)") if roof["traffic"] is not None else None
    if roof["bound"] == "mfma" and not args.only_main:
        # `peak` is the published figure: 256 CUs x 4 SIMDs x 1024 flop per cycle x 2.4 GHz.  The clock the kernel is
        # allowed on this data is read from inside it (stage stamps of one instrumented launch, taken while the GPU
        # is still warm from the timed legs): shader cycles of the work-groups' loops over the time they took.
        roof["peak_basis"] = {"cus": 256, "simds_per_cu": 4, "flop_per_simd_cycle": 1024, "clock_ghz": 2.4}
        try:
            tl = stage_timeline(fa, c, q, k, v)
            if "loop_clock_mhz" in tl:
                clk = tl["loop_clock_mhz"]["mean"]
                roof["loop_clock_mhz"] = clk
                roof["frac_of_peak_at_loop_clock"] = roof["achieved"] / (PEAK_F16_TFLOPS * clk / 2400.0)
        except Exception as e:  # a diagnostic: the line is valid without it
            roof["loop_clock_mhz"] = None
            print(f"bench.py: stage stamps unavailable ({e})", file=sys.stderr)
        # what the MFMA pipe of this GPU sustains on changing random operands (with no
        # other work at all) is measured beside it, since the power management makes it data dependent
        sus = mfma_sustained()
        if sus:
            roof["mfma_sustained"] = sus
            roof["frac_of_sustained_random"] = roof["achieved"] / sus["random"]
            if sus.get("random_attention_mix"):
                # MFMAs on random operands with one LDS fragment read, four fma and one exp issued beside each
                roof["frac_of_attention_mix_ceiling"] = roof["achieved"] / sus["random_attention_mix"]

    result = {
        "metric": METRIC, "value": value, "unit": unit, "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": host_ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16",
        "data": "synthetic", "config": {"workload": f"{name}: {DESCR[name]}", "inputs": ("ALL ZERO (diagnostic run, not a valid rate)" if args.zero_inputs
                                                   else "fp16 RN(N(0,1)) from the portable generator (Philox4x32-10 + Box-Muller), seeds Q=1 K=2 V=3, resident in HBM"),
                                        "accumulate": "fp32", "outputs": "fp16 O + fp32 LSE"},
        "roofline": roof,
    }

    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(c, q, k, v, args.cpu_slices or CPU_SLICES.get(name, 16))
    del q, k, v, step

    if not args.only_main:
        others = {}
        for n2, c2 in CONFIGS.items():
            if n2 == name:
                continue
            q, k, v = make_inputs(c2)
            st, _ = make_step(fa, c2, q, k, v)
            # the reference's protocol is 1000 launches (src/main.cu:187-213); fewer where a launch takes long
            steps2 = {"cfg4": 500, "cfg5": 100}.get(n2, 1000)
            _, ev = time_steps(st, steps2, 10)
            if n2 == "cfg5":
                by = decode_bytes(c2)
                others[n2] = {"workload": DESCR[n2], "ms": ev, "GB/s": by / (ev * 1e-3) / 1e9,
                              "frac_hbm_peak": by / (ev * 1e-3) / 1e9 / PEAK_HBM_GBPS, "algorithmic_bytes": by}
            else:
                fl = flops_of(c2)
                others[n2] = {"workload": DESCR[n2], "ms": ev, "TFLOP/s": fl / (ev * 1e-3) / 1e12,
                              "frac_mfma_peak": fl / (ev * 1e-3) / 1e12 / PEAK_F16_TFLOPS, "algorithmic_flops": fl}
            if n2 == "cfg5":
                # the same launch with the library's own split count (num_splits = 0) instead of the 16 the configuration names
                c3 = dict(c2, splits=-1)
                st3, _ = make_step(fa, c3, q, k, v)
                _, ev3 = time_steps(st3, steps2, 10)
                others[n2]["automatic_split_count"] = {
                    "splits": fa.resolve_splits(c2["B"], c2["H"], c2["Nq"], c2["Nk"], c2["d"], 0), "ms": ev3,
                    "GB/s": by / (ev3 * 1e-3) / 1e9, "frac_hbm_peak": by / (ev3 * 1e-3) / 1e9 / PEAK_HBM_GBPS}
                del st3
            if not args.no_cpu:
                others[n2]["cpu_baseline"] = cpu_baseline(c2, q, k, v, args.cpu_slices or CPU_SLICES[n2])
            del q, k, v, st
        result["other_workloads"] = others
        if "cfg5" in others:
            result["roofline_decode"] = {"bound": "hbm", "achieved": others["cfg5"]["GB/s"], "peak": PEAK_HBM_GBPS,
                                         "unit": "GB/s", "frac": others["cfg5"]["frac_hbm_peak"],
                                         "traffic": measured_traffic("cfg5"),
                                         "traffic_source": f"profiles/{PROFILE_OF['cfg5']}",
                                         "automatic_split_count": others["cfg5"]["automatic_split_count"]}
            if "cpu_baseline" in others["cfg5"]:
                result["roofline_decode"]["cpu_baseline"] = others["cfg5"]["cpu_baseline"]
    print(json.dumps(result))


if __name__ == "__main__":
    main()
