"""GPU parity on the edge cases of the path: ragged sizes, odd head dims, Nq != Nk, window / ALiBi / causal combinations,
fully masked rows, dropout determinism, general split-KV (Nq > 1) with every mask, empty problems, and size-independent
properties at full size.  Everything goes through the C ABI; the checker is the CPU oracle."""
import numpy as np
import pytest

from helpers import check_o_lse, oracle_forward_batched, randn_f16_gpu, to_f32_np

pytestmark = pytest.mark.gpu


def _qkv(B, H, Nq, Nk, d, seed=0):
    return (randn_f16_gpu((B, H, Nq, d), 3 * seed + 1), randn_f16_gpu((B, H, Nk, d), 3 * seed + 2),
            randn_f16_gpu((B, H, Nk, d), 3 * seed + 3))


def _slopes(oracle, H):
    import torch
    s = oracle.alibi_slopes(H)
    return s, torch.from_numpy(s).cuda()


# head dims: every bucket edge, multiples of 8 that are not bucket widths, values that are not multiples of 8 (rows at
# any 2-byte alignment: every length of the partial last chunk, 1 ... 7 elements, in every bucket; below 8, where a row
# is shorter than a chunk, served by the any-alignment instance that serves every request); 31 is the reference's
# checked-in head_dim (src/main.cu:42).  With ALiBi the ALiBi instance of the any-alignment path runs.
@pytest.mark.parametrize("d", [1, 2, 3, 5, 7, 8, 9, 10, 11, 12, 13, 14, 15, 16, 24, 31, 32, 33, 40, 41, 47, 60, 63, 64,
                               65, 72, 77, 90, 95, 96, 97, 100, 106, 119, 125, 127, 128])
def test_head_dims(fa, oracle, d):
    q, k, v = _qkv(2, 3, 150, 150, d, seed=d)
    sl, sl_t = _slopes(oracle, 3)
    for kw, okw in ((dict(), dict()), (dict(causal=True), dict(causal=True)),
                    (dict(causal=True, alibi_slopes=sl_t), dict(causal=True, slopes=sl))):
        if "alibi_slopes" in kw and d % 8 == 0 and d not in (8, 128):
            continue
        o, lse = fa.flash_forward(q, k, v, **kw)
        O, L = oracle_forward_batched(oracle, q, k, v, **okw)
        check_o_lse(o, lse, O, L, f"d={d} {sorted(kw)}")


# Rows at any alignment have four kernel instances per bucket: plain, ALiBi, dropout, and the one that serves every other
# request (both features at once, dropout thresholds of 0, non-positive scales).  Each is run on every length of the
# partial last chunk, unsplit (O leaves as the row's whole chunks plus its last 16 bytes) and in three splits (fp32
# partial rows, 4-byte aligned), with the keep decisions dumped where dropout is on; a threshold of 1 is the smallest the
# dropout instance's packed decisions see.
@pytest.mark.parametrize("d", [9, 12, 15, 17, 27, 31, 34, 45, 62, 63, 67, 76, 93, 99, 100, 105, 110, 123, 127])
def test_any_alignment_instances(fa, oracle, d):
    import torch
    B, H, Nq, Nk = 1, 3, 135, 203
    q, k, v = _qkv(B, H, Nq, Nk, d, seed=1000 + d)
    sl, sl_t = _slopes(oracle, H)
    p_of = {"dropout": 0.3, "dropout_thr1": 2.0 ** -16, "dropout_thr0": 1e-6}
    for feat in ("plain", "alibi", "dropout", "dropout_thr1", "both", "dropout_thr0", "negative_scale"):
        kw, okw = dict(causal=True), dict(causal=True)
        if feat in ("alibi", "both"):
            kw["alibi_slopes"], okw["slopes"] = sl_t, sl
        if feat == "negative_scale":
            kw["softmax_scale"], okw["scale"] = -0.2, -0.2
        p = p_of.get(feat, 0.3 if feat == "both" else 0.0)
        if p > 0.0:
            keep = oracle.dropout_keep_mask(77, d, p, B, H, Nq, Nk)
            kw.update(dropout_p=p, seed=77, offset=d)
            okw.update(keep_mask=torch.from_numpy(keep), p_drop=p)
        O, L = oracle_forward_batched(oracle, q, k, v, **okw)
        if p > 0.0:
            o, lse, km = fa.flash_forward(q, k, v, return_keep_mask=True, **kw)
            vis = np.tril(np.ones((Nq, Nk), dtype=bool), k=Nk - Nq)
            assert np.array_equal(km.cpu().numpy()[..., vis], keep[..., vis]), f"d={d} {feat}"
        else:
            o, lse = fa.flash_forward(q, k, v, **kw)
        check_o_lse(o, lse, O, L, f"d={d} {feat}")
        o3, lse3 = fa.flash_forward_splitkv(q, k, v, num_splits=3, **kw)
        check_o_lse(o3, lse3, O, L, f"d={d} {feat} three splits")


# The 8-wave kernel on rows shorter than its 128-element bucket, in whole chunks (104, 112, 120) and at any alignment
# (every length of the partial last chunk): plain, causal + ALiBi, window + dropout with the keep decisions dumped, ragged
# Nq and Nk, unsplit and in three splits (fp32 partial rows with the same column mapping).
@pytest.mark.parametrize("d", [97, 98, 99, 100, 101, 102, 103, 104, 110, 112, 119, 120, 127])
def test_8wave_kernel_on_shorter_rows(fa, oracle, d):
    import torch
    B, H, Nq, Nk = 1, 2, 333, 471
    q, k, v = _qkv(B, H, Nq, Nk, d, seed=3000 + d)
    sl, sl_t = _slopes(oracle, H)
    keep = oracle.dropout_keep_mask(11, d, 0.25, B, H, Nq, Nk)
    cases = ((dict(), dict(), False),
             (dict(causal=True, alibi_slopes=sl_t), dict(causal=True, slopes=sl), False),
             (dict(window=(200, 50), dropout_p=0.25, seed=11, offset=d),
              dict(window=(200, 50), keep_mask=torch.from_numpy(keep), p_drop=0.25), True))
    for kw, okw, drop in cases:
        O, L = oracle_forward_batched(oracle, q, k, v, **okw)
        for S in (1, 3):
            o, lse = fa.flash_forward_splitkv(q, k, v, num_splits=S, kernel_hint=fa.KERNEL_8WAVE, **kw)
            check_o_lse(o, lse, O, L, f"8-wave d={d} S={S} {sorted(kw)}")
            o4, lse4 = fa.flash_forward_splitkv(q, k, v, num_splits=S, kernel_hint=fa.KERNEL_4WAVE, **kw)
            check_o_lse(o4, lse4, O, L, f"4-wave d={d} S={S} {sorted(kw)}")
        if drop:
            _, _, km = fa.flash_forward(q, k, v, return_keep_mask=True, kernel_hint=fa.KERNEL_8WAVE, **kw)
            i, j = np.arange(Nq)[:, None] + (Nk - Nq), np.arange(Nk)[None, :]
            vis = (j >= i - 200) & (j <= i + 50)
            assert np.array_equal(km.cpu().numpy()[..., vis], keep[..., vis]), f"d={d}"


# Small unsplit problems (the reference's own run among them) take work-groups of 32 rows whose four waves
# walk every fourth key tile each and merge their results through LDS.  Ragged row and key counts (rows that are not a
# multiple of 32, a last tile of one key), causal rows whose upper waves get no tile at all, Nq != Nk in both directions
# (leading row blocks without a visible key), wide windows, grouped K/V heads, head dims in both buckets: whole chunks,
# the bucket width, every alignment.  kernel_hint = KERNEL_4WAVE runs the 128-row instances on the same request.
@pytest.mark.parametrize("B,H,Hk,Nq,Nk,d,kw", [
    (1, 8, 8, 1021, 1021, 31, dict()),                      # the reference's checked-in run (src/main.cu:39-49)
    (1, 8, 8, 1021, 1021, 31, dict(causal=True)),
    (1, 4, 4, 1000, 1025, 64, dict(causal=True)),
    (2, 4, 2, 777, 777, 64, dict()),
    (1, 6, 3, 300, 2000, 40, dict(window=(700, 100))),
    (1, 3, 3, 900, 600, 63, dict(causal=True)),             # rows 0 ... 299 see nothing
    (1, 2, 1, 33, 4097, 17, dict()),
    (2, 2, 2, 515, 515, 56, dict(causal=True, window=(600, -1))),
    (1, 5, 5, 640, 640, 32, dict(window=(-1, 64))),
    (1, 4, 4, 1, 3000, 20, dict(dropout_p=0.0)),            # one row: the decode kernel, not these instances
    # above d = 64 a wave has one LDS stage and requests K and V of its next tile separately (rows of the bucket's
    # width only: the shorter rows in this list run the 128-row instances)
    (1, 8, 8, 1024, 1024, 128, dict(causal=True)),
    (1, 4, 2, 777, 1100, 96, dict(window=(1000, 20))),
    (1, 2, 2, 600, 700, 128, dict(causal=True, dropout_p=0.3, seed=9, offset=2)),
    (1, 3, 1, 70, 2100, 128, dict(alibi=True)),
    (1, 4, 2, 777, 1100, 100, dict(window=(1000, 20))),
    (2, 2, 2, 515, 515, 96, dict(alibi=True)),
    (1, 3, 3, 900, 600, 127, dict(causal=True)),
    (1, 2, 2, 600, 700, 120, dict(causal=True, dropout_p=0.3, seed=9, offset=2)),
    (1, 2, 1, 40, 5000, 72, dict()),
    (1, 4, 2, 700, 700, 64, dict(causal=True, alibi=True)),
    (1, 3, 3, 500, 1100, 31, dict(alibi=True)),
    (1, 2, 2, 600, 600, 48, dict(causal=True, dropout_p=0.2, seed=5, offset=77)),
    (2, 2, 1, 333, 900, 27, dict(window=(800, 30), alibi=True, dropout_p=0.5, seed=2 ** 35, offset=1)),
])
def test_narrow_instances(fa, oracle, B, H, Hk, Nq, Nk, d, kw):
    import torch
    q = randn_f16_gpu((B, H, Nq, d), 41)
    k = randn_f16_gpu((B, Hk, Nk, d), 42)
    v = randn_f16_gpu((B, Hk, Nk, d), 43)
    kr, vr = (t.repeat_interleave(H // Hk, dim=1).contiguous() for t in (k, v))
    kw = dict(kw)
    okw = {x: kw[x] for x in ("causal", "window") if x in kw}
    if kw.pop("alibi", False):
        sl, sl_t = _slopes(oracle, H)
        kw["alibi_slopes"], okw["slopes"] = sl_t, sl
    p = kw.get("dropout_p", 0.0)
    if p > 0.0:
        keep = oracle.dropout_keep_mask(kw["seed"], kw["offset"], p, B, H, Nq, Nk)
        okw.update(keep_mask=torch.from_numpy(keep), p_drop=p)
        _, _, km = fa.flash_forward(q, k, v, return_keep_mask=True, **kw)
        i, j = np.arange(Nq)[:, None] + (Nk - Nq), np.arange(Nk)[None, :]
        wl, wr = kw.get("window", (-1, -1))
        vis = np.ones((Nq, Nk), dtype=bool)
        if kw.get("causal"):
            vis &= j <= i
        if wl >= 0:
            vis &= j >= i - wl
        if wr >= 0:
            vis &= j <= i + wr
        assert np.array_equal(km.cpu().numpy()[..., vis], keep[..., vis])
    O, L = oracle_forward_batched(oracle, q, kr, vr, **okw)
    o = torch.full((B, H, Nq, d), float("nan"), dtype=torch.float16, device="cuda")
    lse = torch.full((B, H, Nq), float("nan"), dtype=torch.float32, device="cuda")
    fa.flash_forward(q, k, v, out=o, lse=lse, **kw)
    check_o_lse(o, lse, O, L, f"32-row work-groups {(B, H, Hk, Nq, Nk, d)} {sorted(kw)}")
    o1, lse1 = fa.flash_forward_splitkv(q, k, v, num_splits=1, **kw)
    assert torch.equal(o, o1) and torch.equal(lse, lse1)
    o4, lse4 = fa.flash_forward(q, k, v, kernel_hint=fa.KERNEL_4WAVE, **kw)
    check_o_lse(o4, lse4, O, L, f"128-row work-groups {(B, H, Hk, Nq, Nk, d)} {sorted(kw)}")
    assert torch.allclose(o.float(), o4.float(), atol=2e-3, rtol=1e-2)


# sequence lengths around the tile sizes (64-key tiles, 128-row groups); 1021 is the reference's checked-in seq_len
@pytest.mark.parametrize("N", [1, 2, 31, 63, 64, 65, 127, 128, 129, 191, 257, 1000, 1021])
def test_ragged_lengths(fa, oracle, N):
    q, k, v = _qkv(1, 2, N, N, 64, seed=N)
    sl, sl_t = _slopes(oracle, 2)
    for kw, okw in ((dict(), dict()), (dict(causal=True), dict(causal=True)),
                    (dict(window=(37, 5), alibi_slopes=sl_t), dict(window=(37, 5), slopes=sl))):
        o, lse = fa.flash_forward(q, k, v, **kw)
        O, L = oracle_forward_batched(oracle, q, k, v, **okw)
        check_o_lse(o, lse, O, L, f"N={N} {list(kw)}")


@pytest.mark.parametrize("Nq,Nk", [(1, 700), (5, 333), (64, 1000), (200, 77), (130, 131), (300, 64)])
def test_nq_differs_from_nk(fa, oracle, Nq, Nk):
    """Mask and bias row index is i + Nk - Nq.  Nk < Nq with a causal mask leaves leading rows with nothing to attend
    to: O = 0 and LSE = -inf there."""
    q, k, v = _qkv(2, 2, Nq, Nk, 64, seed=Nq + Nk)
    sl, sl_t = _slopes(oracle, 2)
    for kw, okw in ((dict(), dict()), (dict(causal=True), dict(causal=True)),
                    (dict(window=(50, 10)), dict(window=(50, 10))),
                    (dict(causal=True, alibi_slopes=sl_t), dict(causal=True, slopes=sl))):
        o, lse = fa.flash_forward(q, k, v, **kw)
        O, L = oracle_forward_batched(oracle, q, k, v, **okw)
        check_o_lse(o, lse, O, L, f"Nq={Nq} Nk={Nk} {list(kw)}")


@pytest.mark.parametrize("d", [128, 72, 31, 9, 3])
def test_row_blocks_without_visible_keys(fa, oracle, d):
    """Nq > Nk under a causal mask: whole row blocks see no key and are filled with O = 0, LSE = -inf by work-groups that
    request nothing (one contiguous piece of memory per block, at the alignment the head dim leaves it: 16-byte stores,
    the last one ending with the piece; pieces shorter than 16 bytes element by element).  Unsplit in both tiled kernels,
    and in three splits, where the empty work-groups fill their partial results."""
    import torch
    B, H, Nq, Nk = 1, 3, 700, 150
    q, k, v = _qkv(B, H, Nq, Nk, d, seed=300 + d)
    O, L = oracle_forward_batched(oracle, q, k, v, causal=True)
    assert np.isneginf(L[..., :Nq - Nk]).all() and not np.isneginf(L[..., Nq - Nk:]).any()
    for hint in ((fa.KERNEL_4WAVE, fa.KERNEL_8WAVE) if d == 128 else (0,)):
        o = torch.full((B, H, Nq, d), float("nan"), dtype=torch.float16, device="cuda")
        lse = torch.full((B, H, Nq), float("nan"), dtype=torch.float32, device="cuda")
        fa.flash_forward_splitkv(q, k, v, num_splits=1, causal=True, out=o, lse=lse, kernel_hint=hint)
        check_o_lse(o, lse, O, L, f"d={d} hint={hint}")
        assert (o[..., :Nq - Nk, :] == 0).all()
    o3, lse3, ws = fa.flash_forward_splitkv(q, k, v, num_splits=3, causal=True, return_partials=True)
    check_o_lse(o3, lse3, O, L, f"d={d} three splits")
    # a single row shorter than 16 bytes per head slice, nothing visible
    q1, k1, v1 = _qkv(1, 2, 2, 1, d, seed=d)
    o1, l1 = fa.flash_forward(q1, k1, v1, causal=True)
    O1, L1 = oracle_forward_batched(oracle, q1, k1, v1, causal=True)
    check_o_lse(o1, l1, O1, L1, f"d={d} two rows, one key")


@pytest.mark.parametrize("B,H,Nq,Nk,d,S,kw", [
    (1, 8, 1021, 1021, 31, 1, dict()),                                   # 32-row work-groups
    (2, 8, 640, 640, 128, 1, dict(causal=True, kernel_hint=2)),          # 8-wave kernel
    (2, 4, 300, 5000, 64, 6, dict(causal=True)),                         # tiled split kernel + combine
    (4, 8, 1, 7000, 128, 5, dict()),                                     # decode kernel + combine
])
def test_graph_replay_of_the_entry_points(fa, B, H, Nq, Nk, d, S, kw):
    """flash_forward / flash_forward_splitkv with caller-owned outputs and workspace captured into a HIP graph: three
    replays with new inputs and cleared outputs in between, each bit-identical to an eager call on the same inputs (the
    library records kernel launches only: no memset node, no allocation)."""
    import torch
    q, k, v = _qkv(B, H, Nq, Nk, d, seed=77)
    o = torch.empty((B, H, Nq, d), dtype=torch.float16, device="cuda")
    lse = torch.empty((B, H, Nq), dtype=torch.float32, device="cuda")
    ws = (torch.empty((B, H, S, Nq, d), dtype=torch.float32, device="cuda"),
          torch.empty((B, H, S, Nq), dtype=torch.float32, device="cuda")) if S > 1 else None

    def call(out, out_lse, workspace):
        if S == 1:
            fa.flash_forward(q, k, v, out=out, lse=out_lse, **kw)
        else:
            fa.flash_forward_splitkv(q, k, v, num_splits=S, out=out, lse=out_lse, workspace=workspace, **kw)

    call(o, lse, ws)  # first call of this kernel instance: its attributes are set outside the capture
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        call(o, lse, ws)
    for rep in range(3):
        q.copy_(randn_f16_gpu((B, H, Nq, d), 500 + rep))
        v.copy_(randn_f16_gpu((B, H, Nk, d), 600 + rep))
        o.fill_(float("nan"))
        lse.fill_(float("nan"))
        if ws is not None:
            ws[0].fill_(float("nan"))
            ws[1].fill_(float("nan"))
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        o_e, lse_e = torch.empty_like(o), torch.empty_like(lse)
        ws_e = (torch.empty_like(ws[0]), torch.empty_like(ws[1])) if ws is not None else None
        call(o_e, lse_e, ws_e)
        torch.cuda.synchronize()
        assert torch.equal(o, o_e) and torch.equal(lse, lse_e), f"replay {rep} differs from the eager call"


def test_concurrent_callers_on_their_own_streams(fa):
    """Four host threads, each with a stream of its own, call the library at the same time (ctypes releases the
    interpreter lock for the duration of a call) on different shapes -- both tiled kernels, 32-row work-groups, decode,
    split + combine with the automatic count, whose answers each thread remembers for itself.  Results must be bit-identical
    to the same calls made one after the other."""
    import threading
    import torch
    shapes = [(1, 8, 1021, 1021, 31, dict()), (2, 16, 512, 512, 128, dict(causal=True)), (4, 16, 1, 4096, 64, dict()),
              (1, 4, 300, 9000, 96, dict(causal=True)), (2, 8, 700, 700, 128, dict(kernel_hint=fa.KERNEL_8WAVE)),
              (1, 2, 2048, 2048, 64, dict(causal=True)), (1, 6, 100, 3000, 40, dict(window=(500, 20))),
              (8, 8, 256, 256, 80, dict())]
    inputs = [tuple(randn_f16_gpu(sz, 900 + 3 * n + j) for j, sz in enumerate(((B, H, Nq, d), (B, H, Nk, d), (B, H, Nk, d))))
              for n, (B, H, Nq, Nk, d, kw) in enumerate(shapes)]
    want = [fa.flash_forward_splitkv(*qkv, num_splits=0, **sh[5]) for qkv, sh in zip(inputs, shapes)]
    torch.cuda.synchronize()
    errors = []

    def worker(t):
        try:
            st = torch.cuda.Stream()
            with torch.cuda.stream(st):
                for rep in range(6):
                    for n in range(len(shapes)):
                        m = (n + 2 * t + rep) % len(shapes)
                        o, lse = fa.flash_forward_splitkv(*inputs[m], num_splits=0, stream=st, **shapes[m][5])
                        st.synchronize()
                        if not (torch.equal(o, want[m][0]) and torch.equal(lse, want[m][1])):
                            errors.append((t, rep, m))
        except Exception as e:  # noqa: BLE001 -- reported by the assertion below
            errors.append((t, repr(e)))

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(4)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not errors, errors


@pytest.mark.parametrize("causal", [False, True])
def test_many_head_slices_in_chunks(fa, oracle, causal):
    """With far more work-groups than the GPU holds at once the kernels deal the head slices out in chunks (here 256
    slices in two chunks of 128, in both tiled kernels): every (slice, row block) must still be served exactly once."""
    B, H, N, d = 8, 32, 1024, 128
    q, k, v = _qkv(B, H, N, N, d, seed=31)
    o4, l4 = fa.flash_forward(q, k, v, causal=causal, kernel_hint=fa.KERNEL_4WAVE)
    o8, l8 = fa.flash_forward(q, k, v, causal=causal, kernel_hint=fa.KERNEL_8WAVE)
    assert (o4.float() - o8.float()).abs().max().item() <= 4e-3
    assert (l4 - l8).abs().max().item() <= 2e-4
    for b, h in ((0, 0), (3, 31), (4, 0), (7, 31), (5, 17)):  # first / last slice of each chunk and one inside
        sl = (slice(b, b + 1), slice(h, h + 1))
        O, L = oracle_forward_batched(oracle, q[sl], k[sl], v[sl], causal=causal)
        check_o_lse(o4[sl], l4[sl], O, L, f"4-wave slice ({b},{h}) causal={causal}")
        check_o_lse(o8[sl], l8[sl], O, L, f"8-wave slice ({b},{h}) causal={causal}")


@pytest.mark.parametrize("d", [64, 128])
@pytest.mark.parametrize("Nq,Nk", [(520, 520), (480, 544), (500, 520), (96, 544)])
def test_mask_bounds_along_block_diagonals(fa, oracle, Nq, Nk, d):
    """Causal masks and windows whose offsets are multiples of 32 put the bounds of a wave's 32 rows on the diagonals of
    32 x 32 score blocks, which the kernels mask with lane-mask constants; ragged ends, a shift Nk - Nq that is no
    multiple of 32 and split boundaries send the same requests down the per-score comparison instead."""
    q, k, v = _qkv(1, 2, Nq, Nk, d, seed=23)
    for window in ((0, 0), (32, 0), (0, 32), (32, 32), (64, 96), (256, 0), (-1, 0), (-1, 64), (96, -1)):
        for causal in (False, True):
            O, L = oracle_forward_batched(oracle, q, k, v, window=window, causal=causal)
            o, lse = fa.flash_forward(q, k, v, window=window, causal=causal)
            check_o_lse(o, lse, O, L, f"Nq={Nq} Nk={Nk} d={d} window={window} causal={causal}")
            o, lse = fa.flash_forward_splitkv(q, k, v, num_splits=3, window=window, causal=causal)
            check_o_lse(o, lse, O, L, f"3 splits Nq={Nq} Nk={Nk} d={d} window={window} causal={causal}")
            if d == 128 and Nq > 128:
                o, lse = fa.flash_forward(q, k, v, window=window, causal=causal, kernel_hint=fa.KERNEL_8WAVE)
                check_o_lse(o, lse, O, L, f"8-wave Nq={Nq} Nk={Nk} window={window} causal={causal}")


@pytest.mark.parametrize("window", [(0, 0), (1, 0), (0, 3), (100, 100), (128, 128), (256, 0), (5, 300), (-1, 7), (9, -1)])
def test_windows(fa, oracle, window):
    """window (128,128) is the reference's own window_attention setting (src/main.cu:57-60)."""
    q, k, v = _qkv(1, 2, 520, 520, 64, seed=11)
    o, lse = fa.flash_forward(q, k, v, window=window)
    O, L = oracle_forward_batched(oracle, q, k, v, window=window)
    check_o_lse(o, lse, O, L, f"window={window}")
    o, lse = fa.flash_forward(q, k, v, window=window, causal=True)
    O, L = oracle_forward_batched(oracle, q, k, v, window=window, causal=True)
    check_o_lse(o, lse, O, L, f"window={window} causal")


def test_alibi_all_buckets(fa, oracle):
    for d in (32, 64, 96, 128, 48):
        H = 4
        q, k, v = _qkv(1, H, 300, 300, d, seed=d + 1)
        sl, sl_t = _slopes(oracle, H)
        o, lse = fa.flash_forward(q, k, v, alibi_slopes=sl_t, causal=True)
        O, L = oracle_forward_batched(oracle, q, k, v, slopes=sl, causal=True)
        check_o_lse(o, lse, O, L, f"alibi d={d}")


def test_scale_values(fa, oracle):
    """A non-positive scale takes the kernel variant that scales before the row maximum."""
    q, k, v = _qkv(1, 2, 200, 200, 64, seed=5)
    for scale in (1.0, 0.02, -0.125, 0.0):
        o, lse = fa.flash_forward(q, k, v, softmax_scale=scale, causal=True)
        O, L = oracle_forward_batched(oracle, q, k, v, scale=scale, causal=True)
        check_o_lse(o, lse, O, L, f"scale={scale}")


@pytest.mark.parametrize("shape", [(2, 3, 200, 200, 64), (1, 2, 100, 333, 96), (1, 2, 129, 129, 31), (1, 1, 300, 300, 128)])
def test_dropout_mask_bit_exact_and_output(fa, oracle, shape):
    import torch
    B, H, Nq, Nk, d = shape
    q, k, v = _qkv(B, H, Nq, Nk, d, seed=sum(shape))
    for p, seed, off in ((0.1, 1234, 0), (0.5, 2 ** 40 + 17, 3), (0.9, 7, 2 ** 33 + 5)):
        o, lse, km = fa.flash_forward(q, k, v, dropout_p=p, seed=seed, offset=off, return_keep_mask=True)
        keep = oracle.dropout_keep_mask(seed, off, p, B, H, Nq, Nk)
        assert np.array_equal(km.cpu().numpy(), keep), "fused kernel's keep decisions differ from the CPU Philox replica"
        assert np.array_equal(fa.dropout_keep_mask(B, H, Nq, Nk, p, seed, off).cpu().numpy(), keep)
        O, L = oracle_forward_batched(oracle, q, k, v, keep_mask=torch.from_numpy(keep), p_drop=p)
        check_o_lse(o, lse, O, L, f"dropout p={p} {shape}")
        # same seed, same result; the mask does not depend on whether it is dumped
        o2, _ = fa.flash_forward(q, k, v, dropout_p=p, seed=seed, offset=off)
        assert torch.equal(o, o2)


@pytest.mark.parametrize("shape", [(1, 2, 300, 300, 128), (1, 2, 150, 150, 64)])
def test_dropout_threshold_edges(fa, oracle, shape):
    """The smallest thresholds: p below 2^-16 has threshold 0 (every element kept, survivors still scaled by 1/(1-p)) and
    is served by the any-alignment instance that serves every request; p = 2^-16 has threshold 1, the smallest one the vector instances' packed
    keep decisions (saturating subtraction of threshold - 1) see; p close to 1 the largest."""
    import torch
    B, H, Nq, Nk, d = shape
    q, k, v = _qkv(B, H, Nq, Nk, d, seed=sum(shape) + 1)
    for p in (1e-6, 2.0 ** -16, 3.0 * 2.0 ** -16, 1.0 - 2.0 ** -15):
        o, lse, km = fa.flash_forward(q, k, v, causal=True, dropout_p=p, seed=5, offset=9, return_keep_mask=True)
        keep = oracle.dropout_keep_mask(5, 9, p, B, H, Nq, Nk)
        vis = np.tril(np.ones((Nq, Nk), dtype=bool))  # the dump covers the pairs the mask leaves visible
        assert np.array_equal(km.cpu().numpy()[..., vis], keep[..., vis]), f"p={p}"
        if p == 1e-6:
            assert keep.all()
        O, L = oracle_forward_batched(oracle, q, k, v, causal=True, keep_mask=torch.from_numpy(keep), p_drop=p)
        if p < 0.5:
            check_o_lse(o, lse, O, L, f"dropout p={p} {shape}")
        else:  # survivors are scaled by 32768: compare relative to that
            assert np.allclose(lse.cpu().numpy(), L, atol=1e-4)
            assert np.allclose(o.float().cpu().numpy() * (1 - p), O * (1 - p), atol=2e-3, rtol=1e-2)


@pytest.mark.parametrize("S", [1, 2, 3, 5, 8])
def test_general_splitkv_matches_unsplit(fa, oracle, S):
    """The reference's split path for Nq > 1 (its checked-in run: N=1021, d=31, src/main.cu:39-49) with every mask;
    result must not depend on the split count, and the partials must match the oracle's restatement."""
    B, H, N, d = 1, 4, 1021, 31
    q, k, v = _qkv(B, H, N, N, d, seed=S)
    sl, sl_t = _slopes(oracle, H)
    for kw, okw in ((dict(), dict()), (dict(causal=True), dict(causal=True)),
                    (dict(window=(300, 40), alibi_slopes=sl_t), dict(window=(300, 40), slopes=sl))):
        o, lse, ws = fa.flash_forward_splitkv(q, k, v, num_splits=S, return_partials=True, **kw)
        O, L = oracle_forward_batched(oracle, q, k, v, **okw)
        check_o_lse(o, lse, O, L, f"split S={S} {list(kw)}")
        if S > 1:
            Ot, Ls, Ms, LSEp = oracle.splitkv_partials(to_f32_np(q), to_f32_np(k), to_f32_np(v), S, **okw)
            op, lp = to_f32_np(ws[0]), to_f32_np(ws[1])
            assert np.array_equal(np.isneginf(lp), np.isneginf(LSEp))
            fin = np.isfinite(LSEp)
            assert np.abs(lp[fin] - LSEp[fin]).max() <= 1e-4
            assert np.abs(op - Ot).max() <= 2e-3


@pytest.mark.parametrize("H", [1, 2, 4, 8, 3])
@pytest.mark.parametrize("S", [2, 4, 6])
def test_split_index_rotation(fa, oracle, H, S):
    """1, 2 or 4 head slices with an even split count: the kernels deal the splits to the XCDs by rotating the split
    index with the row block.  Every partial must still be the one the oracle computes for that split index (same
    layout [B,H,S,Nq,d]); 8 and 3 slices take the plain order."""
    B, N, d = 1, 777, 64
    q, k, v = _qkv(B, H, N, N, d, seed=40 + H + S)
    o, lse, ws = fa.flash_forward_splitkv(q, k, v, num_splits=S, causal=True, return_partials=True)
    O, L = oracle_forward_batched(oracle, q, k, v, causal=True)
    check_o_lse(o, lse, O, L, f"H={H} S={S}")
    Ot, Ls, Ms, LSEp = oracle.splitkv_partials(to_f32_np(q), to_f32_np(k), to_f32_np(v), S, causal=True)
    op, lp = to_f32_np(ws[0]), to_f32_np(ws[1])
    assert np.array_equal(np.isneginf(lp), np.isneginf(LSEp))
    fin = np.isfinite(LSEp)
    assert np.abs(lp[fin] - LSEp[fin]).max() <= 1e-4
    assert np.abs(op - Ot).max() <= 2e-3


@pytest.mark.parametrize("B,H,Nq,Nk,d,causal,want", [
    (1, 8, 512, 32768, 128, False, 16),   # long keys, small batch: two work-groups per CU
    (1, 32, 128, 16384, 128, True, 8),    # causal with Nq < Nk: every split holds visible keys
    (1, 8, 200, 8000, 100, False, 16),    # rows at any alignment
    (1, 1, 16384, 16384, 64, True, None), # causal, one work-group per CU at most: split for the heaviest row block
    (1, 40, 128, 8192, 128, False, 6),
])
def test_automatic_split_count_shapes(fa, oracle, B, H, Nq, Nk, d, causal, want):
    """num_splits <= 0 for Nq > 1: the library's own count (more than one on these shapes) gives the unsplit result; the
    first and the last head slice are checked against the oracle."""
    q, k, v = _qkv(B, H, Nq, Nk, d, seed=B + H + d)
    S = fa.resolve_splits(B, H, Nq, Nk, d, 0, causal=causal)
    assert S > 1 and (want is None or S == want)
    o, lse, ws = fa.flash_forward_splitkv(q, k, v, num_splits=0, causal=causal, return_partials=True)
    assert ws[0].shape == (B, H, S, Nq, d)
    o1, lse1 = fa.flash_forward(q, k, v, causal=causal)
    assert (o.float() - o1.float()).abs().max().item() <= 2e-3
    assert (lse - lse1).abs().max().item() <= 1e-4
    for b, h in ((0, 0), (B - 1, H - 1)):
        sl = (slice(b, b + 1), slice(h, h + 1))
        O, L = oracle_forward_batched(oracle, q[sl], k[sl], v[sl], causal=causal)
        check_o_lse(o[sl], lse[sl], O, L, f"auto split S={S} slice ({b},{h})")


@pytest.mark.parametrize("B,H,N,d", [(1, 32, 2048, 128), (1, 48, 2048, 64), (1, 30, 1200, 96), (3, 33, 700, 128)])
def test_resident_work_groups_in_snake_order(fa, oracle, B, H, N, d):
    """Launches whose work-groups all sit on the GPU at once (here 350-770 of them at two or three per CU) run every
    second block of 256 work-groups in reverse order; every (slice, row block) must still be served exactly once --
    also where the resident part ends inside a block of 256 or is no multiple of 8."""
    import torch
    q, k, v = _qkv(B, H, N, N, d, seed=N + d)
    o, lse = fa.flash_forward(q, k, v, causal=True, kernel_hint=fa.KERNEL_4WAVE)
    for b, h in ((0, 0), (B - 1, H - 1), (B // 2, H // 2), (0, H - 1)):
        sl = (slice(b, b + 1), slice(h, h + 1))
        O, L = oracle_forward_batched(oracle, q[sl], k[sl], v[sl], causal=True)
        check_o_lse(o[sl], lse[sl], O, L, f"slice ({b},{h})")
    # every row written: compare all slices with a launch that is far beyond the resident part (chunks of slices)
    o2, lse2 = fa.flash_forward(torch.cat([q] * 4), torch.cat([k] * 4), torch.cat([v] * 4), causal=True,
                                kernel_hint=fa.KERNEL_4WAVE)
    for r in range(4):
        assert torch.equal(o2[r * B:(r + 1) * B], o) and torch.equal(lse2[r * B:(r + 1) * B], lse)


def test_splitkv_heuristic_and_decode_variants(fa, oracle):
    # num_splits <= 0: the library's heuristic (4 splits for this shape on 256 CUs)
    q, k, v = _qkv(1, 8, 1021, 1021, 32, seed=3)
    o, lse = fa.flash_forward_splitkv(q, k, v, num_splits=0)
    O, L = oracle_forward_batched(oracle, q, k, v)
    check_o_lse(o, lse, O, L, "heuristic split")
    # decode kernel: head-dim buckets, ragged Nk, window, ALiBi, one split and many
    for d, Nk, S in ((128, 5000, 7), (64, 777, 3), (32, 130, 2), (96, 4096, 16), (128, 300, 1), (40, 1000, 4)):
        H = 4
        q, k, v = _qkv(2, H, 1, Nk, d, seed=d + Nk)
        sl, sl_t = _slopes(oracle, H)
        for kw, okw in ((dict(), dict()), (dict(window=(200, 0), alibi_slopes=sl_t), dict(window=(200, 0), slopes=sl)),
                        (dict(causal=True), dict(causal=True))):
            o, lse = fa.flash_forward_splitkv(q, k, v, num_splits=S, **kw)
            O, L = oracle_forward_batched(oracle, q, k, v, **okw)
            check_o_lse(o, lse, O, L, f"decode d={d} Nk={Nk} S={S} {list(kw)}")
    # Nq == 1 with rows shorter than a chunk falls back to the tiled kernel
    q, k, v = _qkv(1, 2, 1, 900, 5, seed=9)
    o, lse = fa.flash_forward_splitkv(q, k, v, num_splits=4)
    O, L = oracle_forward_batched(oracle, q, k, v)
    check_o_lse(o, lse, O, L, "decode d < 8")


# The decode kernel on rows at any alignment: every length of the partial last chunk in every bucket of its lane mapping
# (4, 8 or 16 lanes per key), plain / window + ALiBi, two query heads per K/V head, unsplit and split (where the partial
# rows take the same column mapping); d = 8 ... 15 are rows of a single, partial or whole, chunk.
@pytest.mark.parametrize("d", [8, 9, 11, 14, 15, 17, 23, 26, 31, 33, 37, 44, 50, 63, 65, 71, 78, 92, 100, 109, 121, 127])
def test_decode_rows_at_any_alignment(fa, oracle, d):
    B, H, Hk, Nk = 2, 4, 2, 700 + d
    q = randn_f16_gpu((B, H, 1, d), 7000 + d)
    k, v = randn_f16_gpu((B, Hk, Nk, d), 7100 + d), randn_f16_gpu((B, Hk, Nk, d), 7200 + d)
    sl, sl_t = _slopes(oracle, H)
    kr, vr = k.repeat_interleave(H // Hk, dim=1), v.repeat_interleave(H // Hk, dim=1)
    for kw, okw in ((dict(), dict()), (dict(window=(300, 0), alibi_slopes=sl_t), dict(window=(300, 0), slopes=sl))):
        O, L = oracle_forward_batched(oracle, q, kr, vr, **okw)
        for S in (1, 3):
            o, lse = fa.flash_forward_splitkv(q, k, v, num_splits=S, **kw)
            check_o_lse(o, lse, O, L, f"decode d={d} S={S} {sorted(kw)}")


# grouped-query / multi-query attention: K, V carry H_kv heads and query head h reads K/V head h // (H // H_kv); the
# oracle sees the K/V heads repeated (the reference has one K/V head per query head, src/flash_forward.h:57-59)
@pytest.mark.parametrize("H,Hk,Nq,Nk,d,kw", [
    (8, 2, 300, 300, 128, dict(causal=True)),       # 8-wave kernel
    (6, 3, 200, 333, 64, dict()),                    # 4-wave kernel, Nq != Nk
    (4, 1, 129, 129, 31, dict(window=(40, 10))),     # multi-query, head dim at any alignment
    (8, 4, 64, 500, 96, dict(causal=True)),
    # slice counts that are multiples of 8 x (query heads per K/V head): the slice order keeps the heads of a K/V head
    # on one XCD (a permutation of the slices inside a chunk, in both tiled kernels and in split mode)
    (16, 4, 300, 300, 128, dict(causal=True)),
    (64, 8, 140, 200, 64, dict()),
    (32, 16, 333, 333, 128, dict(causal=True, kernel_hint=2)),
    (48, 2, 70, 130, 32, dict(window=(50, 20))),
])
def test_grouped_query_heads(fa, oracle, H, Hk, Nq, Nk, d, kw):
    B = 2
    hint = dict(kernel_hint=kw.pop("kernel_hint")) if "kernel_hint" in kw else {}
    q = randn_f16_gpu((B, H, Nq, d), 11)
    k = randn_f16_gpu((B, Hk, Nk, d), 12)
    v = randn_f16_gpu((B, Hk, Nk, d), 13)
    kr, vr = (t.repeat_interleave(H // Hk, dim=1).contiguous() for t in (k, v))
    O, L = oracle_forward_batched(oracle, q, kr, vr, **kw)
    kw.update(hint)
    o, lse = fa.flash_forward(q, k, v, **kw)
    check_o_lse(o, lse, O, L, f"GQA H={H} Hk={Hk} tiled")
    # the same through split-KV (tiled split kernel + combine)
    o, lse = fa.flash_forward_splitkv(q, k, v, num_splits=3, **kw)
    check_o_lse(o, lse, O, L, f"GQA H={H} Hk={Hk} split")
    # identical to the library's own result on the repeated heads, bit for bit
    o2, lse2 = fa.flash_forward(q, kr, vr, **kw)
    assert (o2 == fa.flash_forward(q, k, v, **kw)[0]).all()


@pytest.mark.parametrize("H,Hk,d,Nk,kw", [
    (16, 2, 128, 3000, dict()),                      # 8 query heads per K/V head: one work-group serves all 8
    (8, 2, 64, 1500, dict(window=(700, 0))),          # 4 per group
    (6, 3, 32, 900, dict()),                          # 2 per group
    (6, 2, 128, 777, dict()),                         # 3 per group: falls back to one query head per work-group
    (32, 2, 96, 2100, dict(alibi=True)),              # 16 per group: two work-groups of 8
    (4, 1, 128, 5000, dict(causal=True)),             # multi-query
    (32, 2, 128, 2500, dict()),                       # 16 per group, no row-dependent mask: tiled kernel, heads as rows
    (32, 1, 64, 1111, dict()),                        # 32 per group
    (8, 2, 72, 900, dict()),                          # head dim not a bucket width
    (12, 2, 31, 700, dict()),                         # 6 per group, odd head dim
    (32, 2, 128, 2500, dict(window=(-1, 0))),         # "causal" written as a right window of 0: must not cut a head's keys
    (32, 2, 128, 2500, dict(window=(-1, 3))),
])
def test_grouped_query_decode(fa, oracle, H, Hk, d, Nk, kw):
    B = 2
    q = randn_f16_gpu((B, H, 1, d), 21)
    k = randn_f16_gpu((B, Hk, Nk, d), 22)
    v = randn_f16_gpu((B, Hk, Nk, d), 23)
    kr, vr = (t.repeat_interleave(H // Hk, dim=1).contiguous() for t in (k, v))
    okw, gkw = dict(kw), dict(kw)
    if kw.get("alibi"):
        sl, sl_t = _slopes(oracle, H)
        okw.pop("alibi"), gkw.pop("alibi")
        okw["slopes"], gkw["alibi_slopes"] = sl, sl_t
    O, L = oracle_forward_batched(oracle, q, kr, vr, **okw)
    for S in (1, 6):
        o, lse = fa.flash_forward_splitkv(q, k, v, num_splits=S, **gkw)
        check_o_lse(o, lse, O, L, f"GQA decode H={H} Hk={Hk} S={S}")


# One query row under grouped heads: the three routes of the split entry point (heads as rows of the tiled kernel,
# streaming kernel with G heads per work-group, tiled fallback) each see every mask family.
@pytest.mark.parametrize("G", [1, 3, 4, 8, 16])
@pytest.mark.parametrize("window", [(-1, -1), (-1, 0), (-1, 5), (700, 0), (700, -1)])
@pytest.mark.parametrize("causal", [False, True])
def test_decode_routes_times_masks(fa, oracle, G, window, causal):
    B, Hk, d, Nk = 2, 2, 128, 1300
    H = Hk * G
    q = randn_f16_gpu((B, H, 1, d), 41)
    k = randn_f16_gpu((B, Hk, Nk, d), 42)
    v = randn_f16_gpu((B, Hk, Nk, d), 43)
    kr, vr = (t.repeat_interleave(G, dim=1).contiguous() for t in (k, v))
    O, L = oracle_forward_batched(oracle, q, kr, vr, window=window, causal=causal)
    for extra in (dict(), dict(dropout_p=0.0, softmax_scale=d ** -0.5)):
        o, lse = fa.flash_forward_splitkv(q, k, v, num_splits=4, window=window, causal=causal, **extra)
        check_o_lse(o, lse, O, L, f"decode G={G} window={window} causal={causal}")
    # the tiled fallback for rows at any alignment (odd head dim) under the same masks
    q2, k2, v2 = q[..., :31].contiguous(), k[..., :31].contiguous(), v[..., :31].contiguous()
    O2, L2 = oracle_forward_batched(oracle, q2, k2.repeat_interleave(G, dim=1), v2.repeat_interleave(G, dim=1),
                                    window=window, causal=causal)
    o, lse = fa.flash_forward_splitkv(q2, k2, v2, num_splits=3, window=window, causal=causal)
    check_o_lse(o, lse, O2, L2, f"decode odd d G={G} window={window} causal={causal}")


def test_unbounded_windows_written_as_large_numbers(fa):
    """A window bound that cannot cut (INT_MAX is a common spelling of "off") equals no bound, bit for bit."""
    import torch
    big = 2 ** 31 - 1
    q, k, v = _qkv(1, 2, 300, 333, 64, seed=3)
    for causal in (False, True):
        o0, l0 = fa.flash_forward(q, k, v, causal=causal)
        for w in ((big, big), (big, -1), (-1, big), (333, 300), (10 ** 9, 5)):
            ref = (o0, l0) if w[1] != 5 else fa.flash_forward(q, k, v, causal=causal, window=(-1, 5))
            o, l = fa.flash_forward(q, k, v, causal=causal, window=w)
            assert torch.equal(o, ref[0]) and torch.equal(l, ref[1]), (w, causal)
    q1 = q[:, :, :1].contiguous()
    o0, l0 = fa.flash_forward_splitkv(q1, k, v, num_splits=2)
    o, l = fa.flash_forward_splitkv(q1, k, v, num_splits=2, window=(big, big))
    assert torch.equal(o, o0) and torch.equal(l, l0)


@pytest.mark.parametrize("hint,N,d,kw", [
    (2, 600, 128, dict(causal=True)),                 # 8-wave kernel
    (1, 600, 128, dict(causal=True)),                 # 4-wave kernel, tiles fetched straight into LDS
    (0, 300, 64, dict(window=(100, 0))),              # 4-wave kernel, register-staged tiles
    (0, 150, 31, dict()),                             # any-alignment instance
])
def test_stage_stamps(fa, oracle, hint, N, d, kw):
    """Debug output: per work-group stamps of the constant 100 MHz counter are non-decreasing from stage to stage, the
    last word carries the tile count, and the instrumented instance returns what the plain one returns."""
    import torch
    B, H = 2, 3
    q, k, v = _qkv(B, H, N, N, d, seed=hint + N)
    o0, l0 = fa.flash_forward(q, k, v, kernel_hint=hint, **kw)
    o, l, st = fa.flash_forward(q, k, v, kernel_hint=hint, return_stage_stamps=True, **kw)
    assert torch.equal(o, o0) and torch.equal(l, l0)
    O, L = oracle_forward_batched(oracle, q, k, v, **kw)
    check_o_lse(o, l, O, L, "instrumented instance")
    rows = 256 if hint == 2 else 128
    assert st.shape == (B * H * ((N + rows - 1) // rows), fa.FLASH_STAMP_WORDS)
    t = st.cpu().numpy()
    assert (t[:, 0] > 0).all()
    assert (np.diff(t[:, :7], axis=1) >= 0).all(), "stamps must not run backwards"
    assert ((t[:, 6] - t[:, 0]) < 100_000_000).all()  # less than a second
    tiles = t[:, 7] >> 32
    assert tiles.min() >= 1 and tiles.max() <= (N + 63) // 64
    # word 8: shader-clock cycles between stamps 3 and 5; over their distance in time a plausible clock (the 100 MHz
    # counter resolves 10 ns, so only work-groups that spent a few microseconds there are judged)
    dt = (t[:, 5] - t[:, 3]) / 100.0
    long_enough = dt >= 3.0
    if long_enough.any():
        mhz = t[long_enough, 8] / dt[long_enough]
        assert mhz.min() > 300 and mhz.max() < 3500, mhz
    # split entry point: one stamp row per work-group of the split launch
    o, l, st2 = fa.flash_forward_splitkv(q, k, v, num_splits=2, kernel_hint=hint, return_stage_stamps=True, **kw)
    check_o_lse(o, l, O, L, "instrumented split instance")
    assert st2.shape[0] == 2 * st.shape[0]
    assert (np.diff(st2.cpu().numpy()[:, :7], axis=1) >= 0).all()


def test_grouped_query_head_counts_must_divide(fa):
    with pytest.raises(ValueError):
        fa.flash_forward(randn_f16_gpu((1, 6, 8, 64), 1), randn_f16_gpu((1, 4, 8, 64), 2), randn_f16_gpu((1, 4, 8, 64), 3))


def test_empty_and_degenerate(fa):
    import torch
    z = lambda *s: torch.zeros(s, dtype=torch.float16, device="cuda")
    o, lse = fa.flash_forward(z(0, 2, 16, 64), z(0, 2, 16, 64), z(0, 2, 16, 64))
    assert o.shape == (0, 2, 16, 64)
    o, lse = fa.flash_forward(z(1, 2, 0, 64), z(1, 2, 16, 64), z(1, 2, 16, 64))
    assert o.shape == (1, 2, 0, 64)
    # no keys at all: every row is fully masked
    o, lse = fa.flash_forward(randn_f16_gpu((1, 2, 10, 64), 1), z(1, 2, 0, 64), z(1, 2, 0, 64))
    assert torch.all(o == 0) and torch.all(torch.isneginf(lse))
    o, lse = fa.flash_forward_splitkv(randn_f16_gpu((1, 2, 1, 64), 1), z(1, 2, 0, 64), z(1, 2, 0, 64), num_splits=4)
    assert torch.all(o == 0) and torch.all(torch.isneginf(lse))


def test_head_dim_limit_is_an_error(fa):
    import torch
    t = torch.zeros((1, 1, 16, 136), dtype=torch.float16, device="cuda")
    with pytest.raises(fa.FlashError) as e:
        fa.flash_forward(t, t, t)
    assert e.value.code == -2


def test_full_size_properties_causal_prefill(fa):
    """Size-independent checks at the full benchmark shape (B=4,H=16,N=2048,d=128): V = const gives O = const;
    permuting the heads permutes the result; LSE of row 0 is the single score it sees."""
    import torch
    B, H, N, d = 4, 16, 2048, 128
    q, k, v = _qkv(B, H, N, N, d, seed=77)
    ones = torch.ones_like(v)
    o, lse = fa.flash_forward(q, k, ones, causal=True)
    assert torch.allclose(o.float(), torch.ones_like(o, dtype=torch.float32), atol=2e-3)
    o1, l1 = fa.flash_forward(q, k, v, causal=True)
    perm = torch.randperm(H, device="cuda")
    o2, l2 = fa.flash_forward(q[:, perm].contiguous(), k[:, perm].contiguous(), v[:, perm].contiguous(), causal=True)
    assert torch.equal(o1[:, perm], o2) and torch.equal(l1[:, perm], l2)
    s00 = (q[:, :, 0].float() * k[:, :, 0].float()).sum(-1) * d ** -0.5
    assert torch.allclose(l1[:, :, 0], s00, atol=1e-4)
    assert torch.allclose(o1[:, :, 0].float(), v[:, :, 0].float(), atol=2e-3, rtol=1e-2)


def test_full_size_properties_decode(fa):
    """Decode shape (B=16,H=32,Nk=16384,d=128): independence of the split count and the V = const identity."""
    import torch
    B, H, Nk, d = 16, 32, 16384, 128
    q, k, v = _qkv(B, H, 1, Nk, d, seed=78)
    o16, l16 = fa.flash_forward_splitkv(q, k, v, num_splits=16)
    for S in (1, 4, 128):
        oS, lS = fa.flash_forward_splitkv(q, k, v, num_splits=S)
        assert torch.allclose(oS.float(), o16.float(), atol=1e-3)
        assert torch.allclose(lS, l16, atol=2e-5)
    o, _ = fa.flash_forward_splitkv(q, k, torch.full_like(v, 0.5), num_splits=16)
    assert torch.allclose(o.float(), torch.full_like(o, 0.5, dtype=torch.float32), atol=1e-3)


def _torch_reference_long_keys(q, k, v, lo, hi):
    """softmax(q k^T / sqrt(d)) v over the keys lo[i] <= j <= hi[i] of one head slice, fp32 on the GPU, keys in chunks
    (running maximum / sum), for shapes far too long for the CPU oracle.  q [Nq,d], k, v [Nk,d]; returns (O, LSE)."""
    import torch
    Nq, d = q.shape
    Nk = k.shape[0]
    qf = q.float() * d ** -0.5
    m = torch.full((Nq,), float("-inf"), device=q.device, dtype=torch.float64)
    l = torch.zeros((Nq,), device=q.device, dtype=torch.float64)
    o = torch.zeros((Nq, d), device=q.device, dtype=torch.float64)
    step = 1 << 20
    for j0 in range(0, Nk, step):
        j1 = min(Nk, j0 + step)
        if int(hi.max()) < j0 or int(lo.min()) >= j1:
            continue
        sc = (qf @ k[j0:j1].float().T).double()
        j = torch.arange(j0, j1, device=q.device)
        sc = sc.masked_fill((j[None, :] < lo[:, None]) | (j[None, :] > hi[:, None]), float("-inf"))
        m_new = torch.maximum(m, sc.max(1).values)
        safe = torch.where(torch.isinf(m_new), torch.zeros_like(m_new), m_new)
        p = torch.exp(sc - safe[:, None])
        alpha = torch.where(torch.isinf(m), torch.zeros_like(m), torch.exp(m - safe))
        l = l * alpha + p.sum(1)
        o = o * alpha[:, None] + p @ v[j0:j1].double()
        m = m_new
    return (o / l[:, None]).float(), (m + torch.log(l)).float()


def test_largest_key_count(fa):
    """The longest K / V the C ABI accepts at d = 128 (a head slice just short of 4 GiB: the kernels address it with
    32-bit byte offsets), two head slices, so that the second one lies beyond 4 GiB from the tensor's start.  Keys at the
    start, around the 2 GiB mark and at the very end share a direction with every query (scores around 17 against 0 +- 0.7
    elsewhere) and carry nearly all of the softmax mass in three equal parts, so that a wrong address there moves O and LSE.
    Checked against an fp32/fp64 torch evaluation on the GPU (inputs from torch's generator: at this size neither the
    portable generator nor the CPU oracle finishes in test time): decode, both tiled kernels in split mode, and a
    causal sliding window at the far end, whose work-groups start at the last tiles."""
    import torch
    d, H = 128, 2
    Nk = (1 << 24) - 128
    assert 2 * Nk * d < 1 << 32 <= 2 * (Nk + 128) * d
    g = torch.Generator(device="cuda").manual_seed(5)
    k = torch.randn((1, H, Nk, d), generator=g, device="cuda", dtype=torch.float16) * 0.5
    v = torch.randn((1, H, Nk, d), generator=g, device="cuda", dtype=torch.float16)
    u = torch.where(torch.rand(d, generator=g, device="cuda") < 0.5, -1.0, 1.0).half()  # |u|^2 = d
    for a, b in ((0, 256), ((1 << 23) - 128, (1 << 23) + 128), (Nk - 256, Nk)):
        k[:, :, a:b] += 1.5 * u
    with pytest.raises(fa.FlashError):  # one 128-key block more is refused
        fa.resolve_splits(1, H, 1, Nk + 128, d)

    def check(o, lse, q, lo, hi, what):
        for h in range(H):
            o_ref, l_ref = _torch_reference_long_keys(q[0, h], k[0, h], v[0, h], lo, hi)
            check_o_lse(o[0, h], lse[0, h], to_f32_np(o_ref), to_f32_np(l_ref), f"{what} head {h}")

    # decode
    q1 = torch.randn((1, H, 1, d), generator=g, device="cuda", dtype=torch.float16) + u
    full = (torch.zeros(1, device="cuda", dtype=torch.long), torch.full((1,), Nk - 1, device="cuda", dtype=torch.long))
    o, lse = fa.flash_forward_splitkv(q1, k, v, num_splits=0)
    check(o, lse, q1, *full, "decode")
    # tiled kernels, split over the keys
    Nq = 300
    q = torch.randn((1, H, Nq, d), generator=g, device="cuda", dtype=torch.float16) + u
    lo = torch.zeros(Nq, device="cuda", dtype=torch.long)
    hi = torch.full((Nq,), Nk - 1, device="cuda", dtype=torch.long)
    for hint in (fa.KERNEL_4WAVE, fa.KERNEL_8WAVE):
        o, lse = fa.flash_forward_splitkv(q, k, v, num_splits=64, kernel_hint=hint)
        check(o, lse, q, lo, hi, f"split, kernel hint {hint}")
    # causal + left window at the far end (rows are aligned to the end of the keys), unsplit
    i = torch.arange(Nq, device="cuda") + (Nk - Nq)
    for hint in (fa.KERNEL_4WAVE, fa.KERNEL_8WAVE):
        o, lse = fa.flash_forward(q, k, v, causal=True, window=(1000, -1), kernel_hint=hint)
        check(o, lse, q, i - 1000, i, f"window at the end, kernel hint {hint}")


def test_largest_query_count(fa):
    """The longest Q / O the C ABI accepts at d = 128 (2^24 - 128 rows: a head slice just short of 4 GiB) over 200 keys,
    two head slices, both tiled kernels, plain and causal (rows are aligned to the end of the keys: all but the last 200
    rows see no key and must come back as O = 0, LSE = -inf), against torch fp32 on the GPU."""
    import torch
    d, H, Nk = 128, 2, 200
    Nq = (1 << 24) - 128
    g = torch.Generator(device="cuda").manual_seed(6)
    q = torch.randn((1, H, Nq, d), generator=g, device="cuda", dtype=torch.float16)
    k = torch.randn((1, H, Nk, d), generator=g, device="cuda", dtype=torch.float16)
    v = torch.randn((1, H, Nk, d), generator=g, device="cuda", dtype=torch.float16)
    with pytest.raises(fa.FlashError):
        fa.resolve_splits(1, H, Nq + 128, Nk, d)
    tail = 4096  # rows compared in full: the first and the last `tail` of every slice (the last ones lie beyond 4 GiB - 1 MiB)
    for hint in (fa.KERNEL_4WAVE, fa.KERNEL_8WAVE):
        o, lse = fa.flash_forward(q, k, v, kernel_hint=hint)
        oc, lsec = fa.flash_forward(q, k, v, causal=True, kernel_hint=hint)
        for h in range(H):
            for rows in (slice(0, tail), slice(Nq - tail, Nq)):
                sc = (q[0, h, rows].float() @ k[0, h].float().T) * d ** -0.5
                o_ref = torch.softmax(sc, -1) @ v[0, h].float()
                check_o_lse(o[0, h, rows], lse[0, h, rows], to_f32_np(o_ref), to_f32_np(torch.logsumexp(sc, -1)),
                            f"hint {hint} head {h} rows {rows}")
            # every row at once, cheaply: the row sums of O and the LSE against fp32 torch in chunks
            for r0 in range(0, Nq, 1 << 21):
                r1 = min(Nq, r0 + (1 << 21))
                sc = (q[0, h, r0:r1].float() @ k[0, h].float().T) * d ** -0.5
                assert torch.allclose(lse[0, h, r0:r1], torch.logsumexp(sc, -1), atol=1e-4)
                osum = (torch.softmax(sc, -1) @ v[0, h].float().sum(-1, keepdim=True))[:, 0]
                assert torch.allclose(o[0, h, r0:r1].float().sum(-1), osum, atol=2e-2)
            # causal: rows before Nq - Nk see nothing
            assert torch.isneginf(lsec[0, h, :Nq - Nk]).all() and not o[0, h, :0].any()
            assert not oc[0, h, :Nq - Nk].any()
            i = torch.arange(Nq - Nk, Nq, device="cuda")
            sc = (q[0, h, Nq - Nk:].float() @ k[0, h].float().T) * d ** -0.5
            sc = sc.masked_fill(torch.arange(Nk, device="cuda")[None, :] > (i - (Nq - Nk))[:, None], float("-inf"))
            check_o_lse(oc[0, h, Nq - Nk:], lsec[0, h, Nq - Nk:], to_f32_np(torch.softmax(sc, -1) @ v[0, h].float()),
                        to_f32_np(torch.logsumexp(sc, -1)), f"causal hint {hint} head {h}")


# The 8-wave kernel (d = 128; by preference only large grids of long rows, forced here through kernel_hint):
# ragged lengths, Nq != Nk in both directions, every mask incl. narrow windows, grouped heads, dropout, split mode.
@pytest.mark.parametrize("Nq,Nk,Hk,kw", [
    (1100, 1100, 2, dict(causal=True)),
    (1100, 1333, 2, dict(causal=True)),
    (1333, 1100, 2, dict(causal=True)),                       # leading rows see no key: O = 0, LSE = -inf
    (1100, 1100, 1, dict(causal=True)),                       # two query heads per K/V head
    (1100, 1100, 2, dict(causal=True, window=(600, -1))),
    (1100, 1100, 2, dict(causal=True, alibi=True)),
    (1061, 1061, 2, dict(causal=True, dropout_p=0.2, seed=99, offset=5)),
    (300, 1500, 2, dict(window=(700, 900))),
    (300, 300, 2, dict(causal=True)),
    (513, 700, 2, dict(window=(40, 3))),
    (129, 129, 2, dict()),
])
def test_eight_wave_kernel_cases(fa, oracle, Nq, Nk, Hk, kw):
    import torch
    B, H, d = 1, 2, 128
    q = randn_f16_gpu((B, H, Nq, d), 21)
    k = randn_f16_gpu((B, Hk, Nk, d), 22)
    v = randn_f16_gpu((B, Hk, Nk, d), 23)
    kr, vr = (t.repeat_interleave(H // Hk, dim=1).contiguous() for t in (k, v))
    kw = dict(kw, kernel_hint=fa.KERNEL_8WAVE)
    okw = {x: kw[x] for x in ("causal", "window") if x in kw}
    if kw.pop("alibi", False):
        sl, sl_t = _slopes(oracle, H)
        kw["alibi_slopes"], okw["slopes"] = sl_t, sl
    p = kw.get("dropout_p", 0.0)
    if p > 0.0:
        keep = oracle.dropout_keep_mask(kw["seed"], kw["offset"], p, B, H, Nq, Nk)
        okw.update(keep_mask=torch.from_numpy(keep), p_drop=p)
        o, lse, km = fa.flash_forward(q, k, v, return_keep_mask=True, **kw)
        vis = np.tril(np.ones((Nq, Nk), dtype=bool), Nk - Nq)
        assert np.array_equal(km.cpu().numpy()[..., vis], keep[..., vis])
    else:
        o, lse = fa.flash_forward(q, k, v, **kw)
    O, L = oracle_forward_batched(oracle, q, kr, vr, **okw)
    check_o_lse(o, lse, O, L, f"8-wave Nq={Nq} Nk={Nk} {sorted(kw)}")
    if p == 0.0:
        for S in (3, 4):  # (an even count over two slices: the split index is rotated by the row block)
            o, lse = fa.flash_forward_splitkv(q, k, v, num_splits=S, **kw)
            check_o_lse(o, lse, O, L, f"8-wave split S={S} Nq={Nq} Nk={Nk} {sorted(kw)}")


@pytest.mark.parametrize("Nq,Nk,d,Hk,kw", [
    (200, 200, 64, 2, dict(causal=True)),
    (130, 333, 128, 1, dict(window=(50, 20), alibi=True)),
    (1, 700, 128, 1, dict()),                                  # decode with 8 query heads per K/V head
    (300, 300, 31, 2, dict(causal=True, window=(100, -1), softmax_scale=-0.2)),
])
def test_score_dump(fa, oracle, Nq, Nk, d, Hk, kw):
    """The optional score matrix is the one the result was computed from: its -inf pattern is the mask, its row-wise
    log-sum-exp is the LSE output, and softmax(scores) V is O -- for the plain and for the split entry point."""
    import torch
    B, H = 2, 8 if Nq == 1 else 2
    q = randn_f16_gpu((B, H, Nq, d), 31)
    k = randn_f16_gpu((B, Hk, Nk, d), 32)
    v = randn_f16_gpu((B, Hk, Nk, d), 33)
    kw = dict(kw)
    okw = {x: kw[x] for x in ("causal", "window") if x in kw}
    if "softmax_scale" in kw:
        okw["scale"] = kw["softmax_scale"]
    if kw.pop("alibi", False):
        sl, sl_t = _slopes(oracle, H)
        kw["alibi_slopes"], okw["slopes"] = sl_t, sl
    kr, vr = (t.repeat_interleave(H // Hk, dim=1).contiguous() for t in (k, v))
    O, L = oracle_forward_batched(oracle, q, kr, vr, **okw)
    ii = np.arange(Nq)[:, None] + (Nk - Nq)
    jj = np.arange(Nk)[None, :]
    wl, wr = kw.get("window", (-1, -1))
    vis = np.ones((Nq, Nk), dtype=bool)
    if kw.get("causal"):
        vis &= jj <= ii
    if wl >= 0:
        vis &= jj >= ii - wl
    if wr >= 0:
        vis &= jj <= ii + wr
    for entry, extra in ((fa.flash_forward, {}), (fa.flash_forward_splitkv, dict(num_splits=3))):
        sc = torch.full((B, H, Nq, Nk), float("-inf"), dtype=torch.float32, device="cuda")
        o, lse = entry(q, k, v, scores_out=sc, **extra, **kw)
        check_o_lse(o, lse, O, L, f"score dump {entry.__name__}")
        S = sc.cpu().numpy().astype(np.float64)
        assert np.array_equal(np.isfinite(S), np.broadcast_to(vis, S.shape)), "-inf pattern is not the mask"
        m = np.where(vis.any(1), np.max(np.where(vis, S, -np.inf), axis=-1), 0.0)
        P = np.where(vis, np.exp(S - m[..., None]), 0.0)
        l = P.sum(-1)
        rows = vis.any(1)
        assert np.abs((m + np.log(np.where(l > 0, l, 1.0)))[..., rows] - L[..., rows]).max() <= 1e-4
        Oref = np.einsum("bhij,bhjd->bhid", P / np.where(l > 0, l, 1.0)[..., None], to_f32_np(vr).astype(np.float64))
        assert np.abs(Oref - O).max() <= 2e-3
