"""CPU tests of the boundary: the shared library loads, exports every symbol the public header declares, its struct
matches the header, argument checking returns codes without touching a GPU, and the host-side logic (split
heuristic, split resolution, workspace sizing, dropout threshold) agrees with the oracle / golden tables."""
import ctypes as C
import json
import os
import re
import subprocess
import tempfile

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
HEADER = os.path.join(ROOT, "include", "flash_attn_mi355.h")

E_INVAL, E_HEADDIM, E_ALIGN, E_WORKSPACE, E_SPLITS = -1, -2, -3, -4, -5


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(flash_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol(fa):
    names = declared_functions()
    assert {"flash_forward", "flash_forward_splitkv", "flash_splitkv_workspace_bytes",
            "flash_num_splits_heuristic", "flash_dropout_keep_mask"} <= set(names)
    L = C.CDLL(fa.library_path())
    for n in names:
        assert hasattr(L, n), f"{n} declared in the header but not exported"


def test_ctypes_struct_matches_header(fa):
    """sizeof / offsetof from the C compiler against the ctypes mirror."""
    fields = [f[0] for f in fa.FlashParams._fields_]
    prog = "#include <stdio.h>\n#include <stddef.h>\n#include \"flash_attn_mi355.h\"\nint main(){printf(\"%zu\\n\",sizeof(flash_params));\n"
    for f in fields:
        prog += f'printf("%zu\\n", offsetof(flash_params, {f}));\n'
    prog += "return 0;}\n"
    with tempfile.TemporaryDirectory() as td:
        src, exe = os.path.join(td, "t.c"), os.path.join(td, "t")
        open(src, "w").write(prog)
        subprocess.check_call(["gcc", "-std=c99", "-I", os.path.join(ROOT, "include"), src, "-o", exe])
        out = [int(x) for x in subprocess.check_output([exe]).split()]
    assert out[0] == C.sizeof(fa.FlashParams)
    for f, off in zip(fields, out[1:]):
        assert getattr(fa.FlashParams, f).offset == off, f


def _params(fa, **kw):
    p = fa.FlashParams()
    p.B, p.H, p.Nq, p.Nk, p.d = 1, 1, 16, 16, 64
    p.softmax_scale = 0.125
    p.window_left = p.window_right = -1
    p.num_splits = 1
    # fake but well-aligned device addresses: validation must reject before anything is dereferenced or launched
    p.Q, p.K, p.V, p.O, p.LSE = 0x1000, 0x2000, 0x3000, 0x4000, 0x5000
    for k, v in kw.items():
        setattr(p, k, v)
    return p


def test_argument_errors_are_codes_not_aborts(fa):
    L = fa.lib()
    assert L.flash_forward(None, None) == E_INVAL
    assert L.flash_forward_splitkv(None, None) == E_INVAL
    for entry in (L.flash_forward, L.flash_forward_splitkv):
        assert entry(C.byref(_params(fa, d=0)), None) == E_INVAL
        assert entry(C.byref(_params(fa, d=-4)), None) == E_INVAL
        assert entry(C.byref(_params(fa, Nq=-1)), None) == E_INVAL
        assert entry(C.byref(_params(fa, d=129)), None) == E_HEADDIM  # reference: "Please reduce the value of head_dim"
        assert entry(C.byref(_params(fa, d=256)), None) == E_HEADDIM
        assert entry(C.byref(_params(fa, Q=None)), None) == E_INVAL
        assert entry(C.byref(_params(fa, O=None)), None) == E_INVAL
        assert entry(C.byref(_params(fa, LSE=None)), None) == E_INVAL
        assert entry(C.byref(_params(fa, K=None)), None) == E_INVAL
        assert entry(C.byref(_params(fa, Q=0x1008)), None) == E_ALIGN
        assert entry(C.byref(_params(fa, V=0x3002)), None) == E_ALIGN
        assert entry(C.byref(_params(fa, dropout_p=1.0)), None) == E_INVAL
        assert entry(C.byref(_params(fa, dropout_p=-0.1)), None) == E_INVAL
        assert entry(C.byref(_params(fa, dropout_p=float("nan"))), None) == E_INVAL
        assert entry(C.byref(_params(fa, softmax_scale=float("inf"))), None) == E_INVAL
        assert entry(C.byref(_params(fa, num_splits=129)), None) == E_SPLITS
        assert entry(C.byref(_params(fa, Nk=1 << 25, d=64)), None) == E_INVAL  # a K/V slice of 4 GiB
        assert entry(C.byref(_params(fa, H=6, H_kv=4)), None) == E_INVAL  # query heads must be a multiple of K/V heads
        assert entry(C.byref(_params(fa, H=2, H_kv=4)), None) == E_INVAL
        assert entry(C.byref(_params(fa, H=2, H_kv=-1)), None) == E_INVAL
        assert entry(C.byref(_params(fa, kernel_hint=3)), None) == E_INVAL
        assert entry(C.byref(_params(fa, kernel_hint=-1)), None) == E_INVAL
        assert entry(C.byref(_params(fa, stage_stamps_out=0x6004)), None) == E_ALIGN
        assert entry(C.byref(_params(fa, Nq=2 ** 30, Nk=2 ** 30, d=1)), None) == E_INVAL
        # empty problems are a no-op
        assert entry(C.byref(_params(fa, B=0)), None) == 0
        assert entry(C.byref(_params(fa, Nq=0, Q=None, O=None, LSE=None)), None) == 0
    # a split run without its workspace
    assert L.flash_forward_splitkv(C.byref(_params(fa, Nk=1024, num_splits=4)), None) == E_WORKSPACE
    # odd head dims only need element alignment
    assert L.flash_forward(C.byref(_params(fa, d=31, Q=0x1001)), None) == E_ALIGN
    # the entry point that brings its own scratch: same checks, and a size limit instead of the workspace check
    assert L.flash_forward_splitkv_static(None, None) == E_INVAL
    assert L.flash_forward_splitkv_static(C.byref(_params(fa, d=129)), None) == E_HEADDIM
    assert L.flash_forward_splitkv_static(C.byref(_params(fa, B=0)), None) == 0
    big = _params(fa, B=64, H=64, Nq=1, Nk=16384, d=128, num_splits=128)  # 270 MB of partials
    assert L.flash_forward_splitkv_static(C.byref(big), None) == -8
    for code in (0, -1, -2, -3, -4, -5, -6, -7, -8):
        assert L.flash_strerror(code)
    assert b"head_dim" in L.flash_strerror(E_HEADDIM)


def test_heuristic_matches_reference_table(fa, oracle):
    t = json.load(open(os.path.join(HERE, "golden", "heuristic_table.json")))
    for *args, want in t["rows"]:
        assert fa.num_splits_heuristic(*args) == want, args
    rng = np.random.default_rng(0)
    for _ in range(2000):
        nblk = int(rng.integers(1, 200))
        args = (int(rng.integers(1, 3000)), int(rng.choice([108, 256, 64])), nblk, int(rng.integers(1, 200)),
                nblk * 128 if rng.random() < 0.8 else int(rng.integers(1, 30000)))
        assert fa.num_splits_heuristic(*args) == oracle.num_splits_heuristic(*args), args


def test_split_resolution_and_workspace(fa):
    # decode configuration: caller pins 16 splits
    assert fa.resolve_splits(16, 32, 1, 16384, 128, 16) == 16
    assert fa.workspace_bytes(16, 32, 1, 16384, 128, 16) == (16 * 32 * 16 * 1 * 128 * 4, 16 * 32 * 16 * 4)
    # never more splits than 128-key blocks; one split needs no workspace
    assert fa.resolve_splits(1, 1, 1, 300, 64, 16) == 3
    assert fa.resolve_splits(1, 1, 128, 128, 64, 8) == 1
    assert fa.workspace_bytes(1, 1, 128, 128, 64, 8) == (0, 0)
    # automatic choice (num_splits <= 0) for Nq > 1: the count with the lowest estimated time (work-groups on the fullest
    # CU, prologue / epilogue per work-group, partial results per split).  The reference's checked-in shape
    # B=1,H=8,N=1021,d=31 stays whole (64 work-groups of 16 short tiles: measured 14.4 us, 4 splits 16.3), and so does
    # twice that batch (14.4 us, 4 splits 22.0); so do half as many slices of twice the length at d = 63, where work-groups
    # of 32 rows whose waves share out the key tiles serve the unsplit launch (with the 128-row instances it would split 4
    # ways); at d = 100 those work-groups have one LDS stage per wave and wait for much of every tile request, and four
    # splits win; few rows in front of long keys split as before; the prefill benchmark shapes stay unsplit
    assert fa.resolve_splits(1, 8, 1021, 1021, 31, 0) == 1
    assert fa.resolve_splits(2, 8, 1021, 1021, 31, 0) == 1
    assert fa.resolve_splits(1, 4, 2048, 2048, 63, 0) == 1
    assert fa.resolve_splits(1, 4, 2048, 2048, 63, 0, kernel_hint=fa.KERNEL_4WAVE) == 4
    assert fa.resolve_splits(1, 4, 2048, 2048, 100, 0) == 4
    assert fa.resolve_splits(1, 8, 200, 8000, 100, 0) == 16
    assert fa.resolve_splits(4, 16, 2048, 2048, 128, 0) == 1
    assert fa.resolve_splits(4, 16, 2048, 2048, 128, 0, causal=True) == 1
    assert fa.resolve_splits(8, 32, 1000, 1000, 96, 0, causal=True) == 1
    # long keys, few rows: one work-group per CU; two where a split stays long enough to pay for them
    assert fa.resolve_splits(1, 8, 512, 32768, 128, 0) == 16
    assert fa.resolve_splits(1, 32, 128, 16384, 128, 0, causal=True) == 8
    assert fa.resolve_splits(1, 16, 256, 8192, 64, 0) == 8
    assert fa.resolve_splits(1, 4, 1024, 65536, 64, 0) == 16
    assert fa.resolve_splits(1, 40, 128, 8192, 128, 0) == 6      # 240 work-groups, not five rounds of short ones
    assert fa.resolve_splits(2, 4, 300, 20000, 96, 0) == 10
    # 10 key blocks, 52 work-groups: 4 splits of 3 blocks fill 208 of 256 CUs (the reference's rule only looks at counts
    # with 1280 % (128 s) == 0 and would take 10 splits of one block)
    assert fa.resolve_splits(1, 52, 100, 1280, 64, 0, kernel_hint=fa.KERNEL_4WAVE) == 4
    # (left to itself the library serves this launch unsplit with work-groups of 32 rows whose waves share out the key
    # tiles: measured 11.3 us against 15.1 us in 4 splits)
    assert fa.resolve_splits(1, 52, 100, 1280, 64, 0) == 1
    assert fa.num_splits_heuristic(52, 256, 10, 128, 1280) == 10
    # causal with one work-group per CU at most: split along the keys when the heaviest row block is long enough to
    # pay for the partial results
    assert fa.resolve_splits(1, 16, 2048, 2048, 128, 0, causal=True) == 1
    assert fa.resolve_splits(1, 2, 16384, 16384, 64, 0, causal=True) == 5
    # a narrow window leaves a row block two or three key blocks: nothing to split
    assert fa.resolve_splits(1, 4, 4096, 4096, 64, 0, window=(256, 0)) == 1
    # one query row (decode, bandwidth-bound), one-row kernel: about one work-group per CU, at most sqrt(Nk / 3) splits
    assert fa.resolve_splits(16, 32, 1, 16384, 128, 0) == 1
    assert fa.resolve_splits(1, 32, 1, 16384, 128, 0) == 8
    assert fa.resolve_splits(1, 32, 1, 2048, 128, 0) == 8
    assert fa.resolve_splits(4, 8, 1, 65536, 128, 0) == 8
    assert fa.resolve_splits(1, 8, 1, 1 << 20, 128, 0) == 32
    assert fa.resolve_splits(512, 32, 1, 16384, 128, 0) == 1
    assert fa.resolve_splits(64, 32, 1, 4096, 128, 0) == 1
    assert fa.resolve_splits(2, 1, 1, 16384, 64, 0) == 64         # few heads: bounded by sqrt(Nk / 3)
    assert fa.resolve_splits(2, 16, 1, 32768, 128, 0, H_kv=8) == 16   # two query heads per work-group: 16 work-groups per split
    assert fa.resolve_splits(1, 1, 1, 300, 64, 0) == 3
    # grouped heads as the rows of the tiled kernel, and requests the one-row kernel cannot serve: the tiled estimate
    assert fa.resolve_splits(16, 32, 1, 16384, 128, 0, H_kv=8) == 4
    assert fa.resolve_splits(16, 32, 1, 16384, 128, 0, H_kv=4) == 8
    assert fa.resolve_splits(1, 16, 1, 8192, 31, 0) == 16
    with pytest.raises(fa.FlashError):
        fa.resolve_splits(1, 1, 1, 128, 64, 1000)


def test_automatic_split_count_stays_in_range_on_random_shapes(fa):
    """2000 random shapes and masks through the host-side resolution (no GPU): the count is at least 1, at most
    FLASH_MAX_SPLITS and at most the number of 128-key blocks, an explicit count is honoured up to those limits, and the
    workspace sizes are those of the count.  (tests/test_sanitizers.py runs this file against the instrumented build.)"""
    rng = np.random.default_rng(5)
    for it in range(2000):
        d = int(rng.choice([8, 31, 32, 40, 64, 72, 96, 100, 128]))
        B, H = int(rng.integers(1, 9)), int(rng.choice([1, 2, 3, 8, 16, 40, 64]))
        Nq = int(rng.choice([1, 2, 16, 100, 128, 129, 512, 1000, 4096, 20000]))
        Nk = int(rng.choice([1, 64, 127, 128, 129, 1000, 4096, 30000, 131072, 1 << 20]))
        if 2 * Nk * d >= 1 << 32 or 2 * Nq * d >= 1 << 32:
            continue
        causal = bool(rng.integers(0, 2))
        window = (int(rng.choice([-1, 0, 5, 256, 5000, 2 ** 31 - 1])), int(rng.choice([-1, 0, 7, 1024, 2 ** 31 - 1])))
        Hk = int(rng.choice([h for h in (1, 2, 4, 8, H) if H % h == 0]))
        n_blocks = (Nk + 127) // 128
        s = fa.resolve_splits(B, H, Nq, Nk, d, 0, causal=causal, window=window, H_kv=Hk)
        assert 1 <= s <= min(fa.FLASH_MAX_SPLITS, max(1, n_blocks)), (B, H, Nq, Nk, d, causal, window, Hk, s)
        want = int(rng.integers(1, fa.FLASH_MAX_SPLITS + 1))
        got = fa.resolve_splits(B, H, Nq, Nk, d, want, causal=causal, window=window, H_kv=Hk)
        assert got == min(want, max(1, n_blocks))
        ob, lb = fa.workspace_bytes(B, H, Nq, Nk, d, want, causal=causal, window=window, H_kv=Hk)
        rows = B * H * got * Nq if got > 1 else 0
        assert (ob, lb) == (rows * d * 4, rows * 4)


def test_automatic_split_count_is_remembered_per_request(fa):
    """The library remembers the answers of a thread's last four distinct automatic requests.  Ten requests that differ
    in one field each (shape, mask, window, K/V heads, kernel hint), asked in turn three times over -- so that every one
    is evicted before it comes round again -- and twice in a row: always the first answer."""
    import threading
    base = dict(B=1, H=8, Nq=4096, Nk=4096, d=128, causal=True, window=(-1, -1), H_kv=8, kernel_hint=0)
    variants = [dict(), dict(B=2), dict(H=4, H_kv=4), dict(Nq=2048), dict(Nk=16384), dict(d=64), dict(causal=False),
                dict(window=(1024, -1)), dict(H_kv=2), dict(kernel_hint=fa.KERNEL_4WAVE)]

    def ask(v):
        c = dict(base, **v)
        return fa.resolve_splits(c["B"], c["H"], c["Nq"], c["Nk"], c["d"], 0, causal=c["causal"], window=c["window"],
                                 H_kv=c["H_kv"], kernel_hint=c["kernel_hint"])

    first = [ask(v) for v in variants]
    assert len(set(first)) > 1, "the variants should not all resolve to the same count"
    for _ in range(3):
        assert [ask(v) for v in variants] == first
    for v, want in zip(variants, first):
        assert ask(v) == want and ask(v) == want
    # another thread has a memory of its own
    got = []
    t = threading.Thread(target=lambda: got.extend(ask(v) for v in variants))
    t.start()
    t.join()
    assert got == first


def test_stage_stamp_buffer_size(fa):
    L = fa.lib()
    nb = C.c_size_t(99)
    words = 8 * fa.FLASH_STAMP_WORDS
    # causal prefill benchmark shape: 8-wave kernel, 256 rows per work-group; 128 with the 4-wave kernel
    p = _params(fa, B=4, H=16, Nq=2048, Nk=2048, d=128, is_causal=1)
    assert L.flash_stage_stamps_bytes(C.byref(p), 0, C.byref(nb)) == 0 and nb.value == 64 * 8 * words
    p.kernel_hint = 1
    assert L.flash_stage_stamps_bytes(C.byref(p), 0, C.byref(nb)) == 0 and nb.value == 64 * 16 * words
    # split entry point: one row per work-group of the split launch; the decode stream is not stamped
    p = _params(fa, B=1, H=4, Nq=1021, Nk=1021, d=31, num_splits=3)
    assert L.flash_stage_stamps_bytes(C.byref(p), 1, C.byref(nb)) == 0 and nb.value == 4 * 8 * 3 * words
    p = _params(fa, B=16, H=32, Nq=1, Nk=16384, d=128, num_splits=16)
    assert L.flash_stage_stamps_bytes(C.byref(p), 1, C.byref(nb)) == 0 and nb.value == 0
    # eight query heads per K/V head decoding together: heads become rows of the tiled kernel
    p = _params(fa, B=16, H=32, H_kv=4, Nq=1, Nk=16384, d=128, num_splits=16)
    assert L.flash_stage_stamps_bytes(C.byref(p), 1, C.byref(nb)) == 0 and nb.value == 16 * 4 * 16 * words
    assert L.flash_stage_stamps_bytes(C.byref(_params(fa, B=0)), 0, C.byref(nb)) == 0 and nb.value == 0
    assert L.flash_stage_stamps_bytes(C.byref(p), 1, None) == E_INVAL


def test_no_environment_lookups_in_the_dispatch():
    csrc = os.path.join(ROOT, "flash_attn_amd", "csrc")
    for f in os.listdir(csrc):
        if f.endswith((".hip", ".h")):
            assert "getenv" not in open(os.path.join(csrc, f)).read(), f


def test_dropout_threshold_matches_oracle(fa, oracle):
    for p in (0.0, 0.1, 0.25, 0.5, 0.3333, 0.9, 0.999999):
        assert fa.dropout_threshold(p) == oracle.dropout_threshold(p)


def test_product_does_not_reach_into_the_oracle():
    pkg = os.path.join(ROOT, "flash_attn_amd")
    for dirpath, _, files in os.walk(pkg):
        if "build" in dirpath:
            continue
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp", "Makefile")):
                text = open(os.path.join(dirpath, f), errors="ignore").read()
                assert "oracle" not in text, f"{f} mentions the oracle"
    out = subprocess.check_output(["nm", "-D", os.path.join(pkg, "lib", "libflash_attn_mi355.so")]).decode()
    assert "oracle_" not in out
