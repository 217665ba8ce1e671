"""ctypes/numpy front end of the CPU oracle (oracle/liboracle.so) and, when built, of the reference's own CPU
functions (oracle/_ref/libref_cpu.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the benchmark's CPU-baseline leg.  The
shipped package never imports this module.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
# FLASH_ORACLE_LIB: another build of the same source (the sanitizer build of tests/test_sanitizers.py)
_LIB_PATH = os.environ.get("FLASH_ORACLE_LIB") or os.path.join(_HERE, "liboracle.so")
_REF_PATH = os.path.join(_HERE, "_ref", "libref_cpu.so")

_f32p = C.POINTER(C.c_float)
_u8p = C.POINTER(C.c_uint8)
_u32p = C.POINTER(C.c_uint32)
_i32p = C.POINTER(C.c_int)


def _fp(a):
    return None if a is None else a.ctypes.data_as(_f32p)


def _bp(a):
    return None if a is None else a.ctypes.data_as(_u8p)


def _f32c(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.float32)


_lib = None
_ref = None


def lib():
    """liboracle.so, built on demand with `make -C oracle liboracle.so` if missing."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            import subprocess

            subprocess.check_call(["make", "-C", _HERE, "liboracle.so"])
        L = C.CDLL(_LIB_PATH)
        L.oracle_attention_forward_slices.restype = C.c_int
        L.oracle_attention_forward_slices.argtypes = [_f32p, _f32p, _f32p] + [C.c_int] * 5 + [C.c_float] + [C.c_int] * 3 + [
            _f32p, _u8p, C.c_float, _f32p, _f32p, C.c_int, C.c_int, C.c_int, C.c_int]
        L.oracle_splitkv_partials.restype = C.c_int
        L.oracle_splitkv_partials.argtypes = [_f32p, _f32p, _f32p] + [C.c_int] * 5 + [C.c_float] + [C.c_int] * 3 + [
            _f32p, C.c_int, _f32p, _f32p, _f32p, _f32p, C.c_int]
        L.oracle_splitkv_combine.restype = None
        L.oracle_splitkv_combine.argtypes = [_f32p, _f32p, _f32p] + [C.c_int] * 5 + [_f32p, _f32p]
        L.oracle_split_key_range.restype = None
        L.oracle_split_key_range.argtypes = [C.c_int, C.c_int, C.c_int, _i32p, _i32p]
        L.oracle_num_splits_heuristic.restype = C.c_int
        L.oracle_num_splits_heuristic.argtypes = [C.c_int] * 5
        L.oracle_verify_count.restype = C.c_longlong
        L.oracle_verify_count.argtypes = [_f32p, _f32p, C.c_longlong, C.c_float]
        L.oracle_alibi_slopes.restype = None
        L.oracle_alibi_slopes.argtypes = [C.c_int, _f32p]
        L.oracle_philox4x32_10.restype = None
        L.oracle_philox4x32_10.argtypes = [_u32p, _u32p, _u32p]
        L.oracle_dropout_threshold.restype = C.c_uint32
        L.oracle_dropout_threshold.argtypes = [C.c_float]
        L.oracle_dropout_keep_mask.restype = None
        L.oracle_dropout_keep_mask.argtypes = [C.c_uint64, C.c_uint64, C.c_float] + [C.c_int] * 4 + [_u8p, C.c_int]
        L.oracle_max_threads.restype = C.c_int
        L.oracle_f32_to_f16.restype = None
        L.oracle_f32_to_f16.argtypes = [_f32p, C.c_void_p, C.c_uint64]
        L.oracle_fill_normal_f16.restype = None
        L.oracle_fill_normal_f16.argtypes = [C.c_void_p, C.c_uint64, C.c_uint64, C.c_uint64, C.c_int]
        _lib = L
    return _lib


def ref_lib():
    """The reference's compiled CPU functions, or None when oracle/_ref has not been built."""
    global _ref
    if _ref is None and os.path.exists(_REF_PATH):
        R = C.CDLL(_REF_PATH)
        R.ref_attention_forward_cpu.restype = None
        R.ref_attention_forward_cpu.argtypes = [_f32p, _f32p, _f32p, C.c_float] + [C.c_int] * 4 + [_f32p, C.c_int,
                                                                                                  C.c_int, _f32p]
        R.ref_num_splits_heuristic.restype = C.c_int
        R.ref_num_splits_heuristic.argtypes = [C.c_int] * 5
        _ref = R
    return _ref


def default_threads():
    return max(1, min(16, os.cpu_count() or 1))


def attention_forward(q, k, v, scale=None, causal=False, window=(-1, -1), slopes=None, keep_mask=None, p_drop=0.0,
                      nthreads=None, skip_masked=True, slices=None):
    """q [B,H,Nq,d], k,v [B,H,Nk,d] (any float dtype; widened to fp32).  Returns (O fp32 [B,H,Nq,d], LSE fp32 [B,H,Nq]).
    `slices=(begin,end)` restricts the computation to a range of b*H+h slices (other rows are left zero)."""
    q, k, v = _f32c(q), _f32c(k), _f32c(v)
    B, H, Nq, d = q.shape
    Nk = k.shape[2]
    assert k.shape == (B, H, Nk, d) and v.shape == (B, H, Nk, d)
    if scale is None:
        scale = 1.0 / np.sqrt(d)
    slopes = _f32c(slopes)
    if keep_mask is not None:
        keep_mask = np.ascontiguousarray(keep_mask, dtype=np.uint8)
        assert keep_mask.shape == (B, H, Nq, Nk)
    O = np.zeros((B, H, Nq, d), dtype=np.float32)
    LSE = np.zeros((B, H, Nq), dtype=np.float32)
    s0, s1 = (0, B * H) if slices is None else slices
    rc = lib().oracle_attention_forward_slices(_fp(q), _fp(k), _fp(v), B, H, Nq, Nk, d, float(scale), int(bool(causal)),
                                               int(window[0]), int(window[1]), _fp(slopes), _bp(keep_mask),
                                               float(p_drop), _fp(O), _fp(LSE), int(nthreads or default_threads()),
                                               int(bool(skip_masked)), int(s0), int(s1))
    if rc != 0:
        raise MemoryError("oracle_attention_forward failed")
    return O, LSE


def split_key_range(Nk, num_splits, s):
    b, e = C.c_int(), C.c_int()
    lib().oracle_split_key_range(Nk, num_splits, s, C.byref(b), C.byref(e))
    return b.value, e.value


def splitkv_partials(q, k, v, num_splits, scale=None, causal=False, window=(-1, -1), slopes=None, nthreads=None):
    """Returns (O_tmp [B,H,S,Nq,d], L [B,H,S,Nq], M [B,H,S,Nq], LSE_partial [B,H,S,Nq]), all fp32."""
    q, k, v = _f32c(q), _f32c(k), _f32c(v)
    B, H, Nq, d = q.shape
    Nk = k.shape[2]
    if scale is None:
        scale = 1.0 / np.sqrt(d)
    slopes = _f32c(slopes)
    S = num_splits
    O_tmp = np.zeros((B, H, S, Nq, d), dtype=np.float32)
    L = np.zeros((B, H, S, Nq), dtype=np.float32)
    M = np.zeros((B, H, S, Nq), dtype=np.float32)
    LSEp = np.zeros((B, H, S, Nq), dtype=np.float32)
    lib().oracle_splitkv_partials(_fp(q), _fp(k), _fp(v), B, H, Nq, Nk, d, float(scale), int(bool(causal)),
                                  int(window[0]), int(window[1]), _fp(slopes), S, _fp(O_tmp), _fp(L), _fp(M), _fp(LSEp),
                                  int(nthreads or default_threads()))
    return O_tmp, L, M, LSEp


def splitkv_combine(O_tmp, L, M):
    O_tmp, L, M = _f32c(O_tmp), _f32c(L), _f32c(M)
    B, H, S, Nq, d = O_tmp.shape
    O = np.zeros((B, H, Nq, d), dtype=np.float32)
    LSE = np.zeros((B, H, Nq), dtype=np.float32)
    lib().oracle_splitkv_combine(_fp(O_tmp), _fp(L), _fp(M), B, H, Nq, d, S, _fp(O), _fp(LSE))
    return O, LSE


def num_splits_heuristic(batch_nheads_mblocks, num_sms, num_n_blocks, max_splits, seq_len):
    return lib().oracle_num_splits_heuristic(batch_nheads_mblocks, num_sms, num_n_blocks, max_splits, seq_len)


def verify_count(o_cpu, o_dev, tol):
    o_cpu, o_dev = _f32c(o_cpu).ravel(), _f32c(o_dev).ravel()
    return lib().oracle_verify_count(_fp(o_cpu), _fp(o_dev), o_cpu.size, float(tol))


def alibi_slopes(H):
    s = np.zeros(H, dtype=np.float32)
    lib().oracle_alibi_slopes(H, _fp(s))
    return s


def philox4x32_10(ctr, key):
    c = (C.c_uint32 * 4)(*[int(x) & 0xFFFFFFFF for x in ctr])
    k = (C.c_uint32 * 2)(*[int(x) & 0xFFFFFFFF for x in key])
    o = (C.c_uint32 * 4)()
    lib().oracle_philox4x32_10(c, k, o)
    return [int(x) for x in o]


def normal_f16(shape, seed, first=0, nthreads=None):
    """RN_fp16(N(0,1)) of the portable generator: element e of the flattened array is a function of (seed, first + e)."""
    n = int(np.prod(shape, dtype=np.int64))
    out = np.empty(n, dtype=np.uint16)
    lib().oracle_fill_normal_f16(out.ctypes.data_as(C.c_void_p), int(first), n, int(seed),
                                 int(nthreads or default_threads()))
    return out.view(np.float16).reshape(shape)


def f32_to_f16_bits(x):
    """fp16 bit patterns of the generator's own round-to-nearest-even conversion (for tests)."""
    x = np.ascontiguousarray(x, dtype=np.float32).ravel()
    out = np.empty(x.size, dtype=np.uint16)
    lib().oracle_f32_to_f16(_fp(x), out.ctypes.data_as(C.c_void_p), x.size)
    return out


def dropout_threshold(p):
    return int(lib().oracle_dropout_threshold(float(p)))


def dropout_keep_mask(seed, offset, p, B, H, Nq, Nk, nthreads=None):
    m = np.zeros((B, H, Nq, Nk), dtype=np.uint8)
    lib().oracle_dropout_keep_mask(int(seed), int(offset), float(p), B, H, Nq, Nk, _bp(m),
                                   int(nthreads or default_threads()))
    return m


# ---------------------------------------------------------------------------------------------------------------
# The reference's own functions (only where oracle/_ref/libref_cpu.so was built from the reference checkout).

def ref_attention_forward_cpu(q, k, v, scale, causal=False, window_size=-1, slopes=None):
    """attention_forward_cpu of the reference (src/main.cu:279-388): Nq == Nk, symmetric window, fp32 O only."""
    R = ref_lib()
    if R is None:
        raise RuntimeError("oracle/_ref/libref_cpu.so is not built")
    q, k, v = _f32c(q), _f32c(k), _f32c(v)
    B, H, N, d = q.shape
    slopes = _f32c(slopes)
    O = np.zeros((B, H, N, d), dtype=np.float32)
    R.ref_attention_forward_cpu(_fp(q), _fp(k), _fp(v), float(scale), B, H, N, d, _fp(O), int(bool(causal)),
                                int(window_size), _fp(slopes))
    return O


def ref_num_splits_heuristic(batch_nheads_mblocks, num_sms, num_n_blocks, max_splits, seq_len):
    R = ref_lib()
    if R is None:
        raise RuntimeError("oracle/_ref/libref_cpu.so is not built")
    return R.ref_num_splits_heuristic(batch_nheads_mblocks, num_sms, num_n_blocks, max_splits, seq_len)
