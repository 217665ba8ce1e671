"""ctypes binding of include/flash_attn_mi355.h.

The functions mirror the launch path of the reference's main() (src/main.cu:109-192): fill the parameter struct
from [B,H,N,d] fp16 tensors, call flash_forward / flash_forward_splitkv on the current stream, return fp16 O and
fp32 LSE.  Error behaviour: a non-zero return code of the library becomes FlashError (the reference prints and
exits, src/main.cu:18-25,182-185).
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "lib", "libflash_attn_mi355.so")

FLASH_OK = 0
FLASH_MAX_HEAD_DIM = 128
FLASH_MAX_SPLITS = 128
FLASH_STAMP_WORDS = 9
FLASH_STATIC_SCRATCH_BYTES = 32 << 20
KERNEL_AUTO, KERNEL_4WAVE, KERNEL_8WAVE = 0, 1, 2


class FlashError(RuntimeError):
    def __init__(self, code, where):
        self.code = code
        detail = lib().flash_strerror(code).decode()
        hip = lib().flash_last_hip_error().decode()
        super().__init__(f"{where}: {detail} (code {code})" + (f" [{hip}]" if hip else ""))


class FlashParams(C.Structure):
    """struct flash_params, field for field."""
    _fields_ = [
        ("Q", C.c_void_p), ("K", C.c_void_p), ("V", C.c_void_p), ("O", C.c_void_p),
        ("LSE", C.c_void_p), ("O_partial", C.c_void_p), ("LSE_partial", C.c_void_p),
        ("B", C.c_int), ("H", C.c_int), ("Nq", C.c_int), ("Nk", C.c_int), ("d", C.c_int),
        ("softmax_scale", C.c_float),
        ("is_causal", C.c_int), ("window_left", C.c_int), ("window_right", C.c_int),
        ("alibi_slopes", C.c_void_p),
        ("dropout_p", C.c_float),
        ("seed", C.c_uint64), ("offset", C.c_uint64),
        ("num_splits", C.c_int),
        ("keep_mask_out", C.c_void_p),
        ("H_kv", C.c_int),
        ("scores_out", C.c_void_p),
        ("kernel_hint", C.c_int),
        ("stage_stamps_out", C.c_void_p),
    ]


_lib = None


def library_path():
    return _LIB_PATH


def lib():
    """The loaded shared library.  Raises if it has not been built (no fallback exists)."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise ImportError(
                f"{_LIB_PATH} is missing: build it with `make -C flash_attn_amd/csrc` "
                "(or __graft_entry__.build()); this package has no fallback path")
        # PyTorch carries its own copy of the HIP runtime (same soname).  Import it first so that the dynamic
        # loader binds this library to that copy: two HIP runtimes in one process do not share a device context.
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
        L = C.CDLL(_LIB_PATH)
        pp = C.POINTER(FlashParams)
        L.flash_forward.restype = C.c_int
        L.flash_forward.argtypes = [pp, C.c_void_p]
        L.flash_forward_splitkv.restype = C.c_int
        L.flash_forward_splitkv.argtypes = [pp, C.c_void_p]
        L.flash_forward_splitkv_static.restype = C.c_int
        L.flash_forward_splitkv_static.argtypes = [pp, C.c_void_p]
        L.flash_splitkv_workspace_bytes.restype = C.c_int
        L.flash_splitkv_workspace_bytes.argtypes = [pp, C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]
        L.flash_splitkv_resolve_splits.restype = C.c_int
        L.flash_splitkv_resolve_splits.argtypes = [pp]
        L.flash_stage_stamps_bytes.restype = C.c_int
        L.flash_stage_stamps_bytes.argtypes = [pp, C.c_int, C.POINTER(C.c_size_t)]
        L.flash_num_splits_heuristic.restype = C.c_int
        L.flash_num_splits_heuristic.argtypes = [C.c_int] * 5
        L.flash_dropout_keep_mask.restype = C.c_int
        L.flash_dropout_keep_mask.argtypes = [pp, C.c_void_p, C.c_void_p]
        L.flash_dropout_threshold.restype = C.c_uint32
        L.flash_dropout_threshold.argtypes = [C.c_float]
        L.flash_last_hip_error.restype = C.c_char_p
        L.flash_strerror.restype = C.c_char_p
        L.flash_strerror.argtypes = [C.c_int]
        L.flash_params_init.restype = None
        L.flash_params_init.argtypes = [pp]
        L.flash_params_size.restype = C.c_size_t
        if L.flash_params_size() != C.sizeof(FlashParams):
            raise ImportError(f"{_LIB_PATH} was built with another flash_params ({L.flash_params_size()} bytes, this "
                              f"binding: {C.sizeof(FlashParams)}): rebuild the library")
        _lib = L
    return _lib


def _ptr(t):
    return None if t is None else t.data_ptr()


def _stream_handle(stream):
    import torch

    s = stream if stream is not None else torch.cuda.current_stream()
    return C.c_void_p(s.cuda_stream)


def _check_qkv(q, k, v):
    import torch

    if q.dim() != 4 or k.dim() != 4 or v.dim() != 4:
        raise ValueError("Q, K, V must be [B,H,N,d]")
    for t in (q, k, v):
        if t.dtype != torch.float16 or not t.is_cuda or not t.is_contiguous():
            raise ValueError("Q, K, V must be contiguous fp16 device tensors")
    B, H, Nq, d = q.shape
    Hk = k.shape[1]
    if k.shape[0] != B or Hk < 1 or H % Hk != 0 or k.shape[3] != d or v.shape != k.shape:
        raise ValueError("K, V must be [B,H_kv,Nk,d] matching Q, with H a multiple of H_kv")
    return B, H, Nq, k.shape[2], d


def make_params(q, k, v, o, lse, softmax_scale=None, causal=False, window=(-1, -1), alibi_slopes=None,
                dropout_p=0.0, seed=0, offset=0, num_splits=1, o_partial=None, lse_partial=None, keep_mask_out=None,
                scores_out=None, kernel_hint=KERNEL_AUTO):
    B, H, Nq, Nk, d = _check_qkv(q, k, v)
    p = FlashParams()
    lib().flash_params_init(C.byref(p))
    p.Q, p.K, p.V, p.O, p.LSE = _ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(lse)
    p.O_partial, p.LSE_partial = _ptr(o_partial), _ptr(lse_partial)
    p.B, p.H, p.Nq, p.Nk, p.d = B, H, Nq, Nk, d
    p.softmax_scale = float(softmax_scale) if softmax_scale is not None else d ** -0.5
    p.is_causal = int(bool(causal))
    p.window_left, p.window_right = int(window[0]), int(window[1])
    p.alibi_slopes = _ptr(alibi_slopes)
    p.dropout_p = float(dropout_p)
    p.seed, p.offset = int(seed), int(offset)
    p.num_splits = int(num_splits)
    p.keep_mask_out = _ptr(keep_mask_out)
    p.H_kv = int(k.shape[1])
    p.scores_out = _ptr(scores_out)
    p.kernel_hint = int(kernel_hint)
    return p


def _attach_stamps(p, split, device):
    """Allocates the stage-stamp buffer of the call described by p ([work-groups, FLASH_STAMP_WORDS] int64) and points
    p at it; None when the call runs no tiled kernel."""
    import torch

    nb = C.c_size_t()
    rc = lib().flash_stage_stamps_bytes(C.byref(p), int(split), C.byref(nb))
    if rc != FLASH_OK:
        raise FlashError(rc, "flash_stage_stamps_bytes")
    if nb.value == 0:
        return None
    st = torch.zeros((nb.value // (8 * FLASH_STAMP_WORDS), FLASH_STAMP_WORDS), dtype=torch.int64, device=device)
    p.stage_stamps_out = st.data_ptr()
    return st


def flash_forward(q, k, v, softmax_scale=None, causal=False, window=(-1, -1), alibi_slopes=None, dropout_p=0.0,
                  seed=0, offset=0, return_keep_mask=False, stream=None, out=None, lse=None, scores_out=None,
                  kernel_hint=KERNEL_AUTO, return_stage_stamps=False):
    """O = softmax(mask(Q K^T * scale - slope * |i - j|)) V over the whole key range.
    q [B,H,Nq,d], k,v [B,H,Nk,d] fp16 on the GPU.  Returns (O fp16 [B,H,Nq,d], LSE fp32 [B,H,Nq]) and, when
    return_keep_mask, the uint8 keep decisions [B,H,Nq,Nk] the kernel applied.  scores_out: optional fp32
    [B,H,Nq,Nk] tensor (pre-filled with -inf) that receives the visible scores (debug; slow kernel instance).
    kernel_hint: KERNEL_AUTO / KERNEL_4WAVE / KERNEL_8WAVE.  return_stage_stamps: also return the per-work-group
    time stamps [groups, FLASH_STAMP_WORDS] int64 of the instrumented kernel instance (debug), as the last element."""
    import torch

    B, H, Nq, Nk, d = _check_qkv(q, k, v)
    o = out if out is not None else torch.empty((B, H, Nq, d), dtype=torch.float16, device=q.device)
    l = lse if lse is not None else torch.empty((B, H, Nq), dtype=torch.float32, device=q.device)
    km = torch.zeros((B, H, Nq, Nk), dtype=torch.uint8, device=q.device) if return_keep_mask else None
    p = make_params(q, k, v, o, l, softmax_scale, causal, window, alibi_slopes, dropout_p, seed, offset, 1,
                    keep_mask_out=km, scores_out=scores_out, kernel_hint=kernel_hint)
    stamps = _attach_stamps(p, 0, q.device) if return_stage_stamps else None
    rc = lib().flash_forward(C.byref(p), _stream_handle(stream))
    if rc != FLASH_OK:
        raise FlashError(rc, "flash_forward")
    res = (o, l, km) if return_keep_mask else (o, l)
    return res + (stamps,) if return_stage_stamps else res


def flash_forward_splitkv(q, k, v, num_splits=0, softmax_scale=None, causal=False, window=(-1, -1),
                          alibi_slopes=None, dropout_p=0.0, seed=0, offset=0, stream=None, workspace=None,
                          return_partials=False, out=None, lse=None, scores_out=None, kernel_hint=KERNEL_AUTO,
                          return_stage_stamps=False):
    """Split-KV forward + combine.  num_splits <= 0 asks the library's heuristic; a larger request than there are
    128-key blocks is clamped by the library (flash_splitkv_resolve_splits tells the count used).  `workspace` may
    carry a pre-allocated (O_partial, LSE_partial) pair with at least the bytes flash_splitkv_workspace_bytes
    reports; otherwise it is allocated here (the caller owns the workspace, as in src/main.cu:160-162).
    return_partials hands back views of the workspace in the layout the library wrote, for the resolved split count
    S: [B,H,S,Nq,d] / [B,H,S,Nq], or -- one query row with four or more query heads per K/V head, no ALiBi, left
    window or dropout -- [B,H_kv,S,G,d] / [B,H_kv,S,G] with G = H / H_kv; (None, None) when S == 1."""
    import torch

    B, H, Nq, Nk, d = _check_qkv(q, k, v)
    o = out if out is not None else torch.empty((B, H, Nq, d), dtype=torch.float16, device=q.device)
    l = lse if lse is not None else torch.empty((B, H, Nq), dtype=torch.float32, device=q.device)
    p = make_params(q, k, v, o, l, softmax_scale, causal, window, alibi_slopes, dropout_p, seed, offset, num_splits,
                    scores_out=scores_out, kernel_hint=kernel_hint)
    S = lib().flash_splitkv_resolve_splits(C.byref(p))
    if S < 0:
        raise FlashError(S, "flash_splitkv_resolve_splits")
    rows = B * H * S * Nq if S > 1 else 0
    if workspace is None and rows:
        workspace = (torch.empty(rows * d, dtype=torch.float32, device=q.device),
                     torch.empty(rows, dtype=torch.float32, device=q.device))
    if workspace is not None:
        if workspace[0].numel() < rows * d or workspace[1].numel() < rows:
            raise ValueError(f"workspace too small for {S} splits: need {rows * d} and {rows} fp32 elements")
        for t in workspace:
            if t.dtype != torch.float32 or not t.is_cuda or not t.is_contiguous():
                raise ValueError("workspace tensors must be contiguous fp32 device tensors")
        p.O_partial, p.LSE_partial = _ptr(workspace[0]), _ptr(workspace[1])
    stamps = _attach_stamps(p, 1, q.device) if return_stage_stamps else None
    rc = lib().flash_forward_splitkv(C.byref(p), _stream_handle(stream))
    if rc != FLASH_OK:
        raise FlashError(rc, "flash_forward_splitkv")
    res = (o, l)
    if return_partials:
        if rows:
            Hk = k.shape[1]
            G = H // Hk
            grouped = (Nq == 1 and G >= 4 and alibi_slopes is None and not (0 <= window[0] < Nk) and dropout_p == 0.0
                       and scores_out is None)
            shp = (B, Hk, S, G) if grouped else (B, H, S, Nq)
            res += ((workspace[0].reshape(-1)[:rows * d].view(*shp, d), workspace[1].reshape(-1)[:rows].view(*shp)),)
        else:
            res += ((None, None),)
    return res + (stamps,) if return_stage_stamps else res


def dropout_keep_mask(B, H, Nq, Nk, dropout_p, seed, offset=0, device="cuda", stream=None):
    """uint8 [B,H,Nq,Nk] keep-mask of the dropout contract, generated on the GPU."""
    import torch

    m = torch.empty((B, H, Nq, Nk), dtype=torch.uint8, device=device)
    p = FlashParams()
    p.B, p.H, p.Nq, p.Nk, p.d = B, H, Nq, Nk, 8
    p.dropout_p, p.seed, p.offset = float(dropout_p), int(seed), int(offset)
    rc = lib().flash_dropout_keep_mask(C.byref(p), C.c_void_p(m.data_ptr()), _stream_handle(stream))
    if rc != FLASH_OK:
        raise FlashError(rc, "flash_dropout_keep_mask")
    return m


def dropout_threshold(p):
    return int(lib().flash_dropout_threshold(float(p)))


def num_splits_heuristic(batch_nheads_mblocks, num_cus, num_n_blocks, max_splits, seq_len):
    return lib().flash_num_splits_heuristic(batch_nheads_mblocks, num_cus, num_n_blocks, max_splits, seq_len)


def stage_stamp_names():
    """Meaning of the nine words of a stage-stamp row (see stage_stamps_out in the header)."""
    return ("entry", "requests_issued", "requests_landed", "first_barrier", "first_scores", "loop_done", "stored",
            "tiles<<32|xcc<<16|hw_id", "shader_cycles_first_barrier_to_loop_done")


def _shape_params(B, H, Nq, Nk, d, num_splits, causal=False, window=(-1, -1), H_kv=0, kernel_hint=KERNEL_AUTO):
    p = FlashParams()
    lib().flash_params_init(C.byref(p))
    p.B, p.H, p.Nq, p.Nk, p.d = B, H, Nq, Nk, d
    p.softmax_scale = 1.0
    p.num_splits = num_splits
    p.is_causal = int(bool(causal))
    p.window_left, p.window_right = int(window[0]), int(window[1])
    p.H_kv = int(H_kv)
    p.kernel_hint = int(kernel_hint)
    return p


def resolve_splits(B, H, Nq, Nk, d, num_splits=0, causal=False, window=(-1, -1), H_kv=0, kernel_hint=KERNEL_AUTO):
    """The split count flash_forward_splitkv will use for such a call (num_splits <= 0: the library's choice)."""
    rc = lib().flash_splitkv_resolve_splits(C.byref(_shape_params(B, H, Nq, Nk, d, num_splits, causal, window, H_kv,
                                                                kernel_hint)))
    if rc < 0:
        raise FlashError(rc, "flash_splitkv_resolve_splits")
    return rc


def workspace_bytes(B, H, Nq, Nk, d, num_splits=0, causal=False, window=(-1, -1), H_kv=0, kernel_hint=KERNEL_AUTO):
    ob, lb = C.c_size_t(), C.c_size_t()
    rc = lib().flash_splitkv_workspace_bytes(C.byref(_shape_params(B, H, Nq, Nk, d, num_splits, causal, window, H_kv,
                                                                kernel_hint)),
                                             C.byref(ob), C.byref(lb))
    if rc != FLASH_OK:
        raise FlashError(rc, "flash_splitkv_workspace_bytes")
    return ob.value, lb.value
