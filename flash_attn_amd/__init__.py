"""MI355X (gfx950) FlashAttention forward: thin host-side front end over the C ABI of
flash_attn_amd/lib/libflash_attn_mi355.so (declared in include/flash_attn_mi355.h).

PyTorch is used only to own device memory and to name the current HIP stream; every computation goes through the
C entry points.  There is no CPU or PyTorch fallback: if the library is missing, importing the binding raises.
"""
from .binding import (  # noqa: F401
    FlashError,
    FlashParams,
    flash_forward,
    flash_forward_splitkv,
    dropout_keep_mask,
    dropout_threshold,
    num_splits_heuristic,
    resolve_splits,
    workspace_bytes,
    library_path,
    stage_stamp_names,
    KERNEL_AUTO,
    KERNEL_4WAVE,
    KERNEL_8WAVE,
    FLASH_STAMP_WORDS,
    FLASH_STATIC_SCRATCH_BYTES,
    FLASH_MAX_SPLITS,
    lib,
)
