// Host-side launchers of the decode / combine / keep-mask kernels (decode_kernels.hip).
#pragma once
#include "common.h"

#define FLASH_MAX_SPLITS_K 128  // must equal FLASH_MAX_SPLITS of the public header

namespace fa {
// each returns the hipError_t of the launch as int
int launch_decode_split(const FwdArgs& a, hipStream_t st);
int launch_combine(const FwdArgs& a, hipStream_t st);
int launch_keep_mask(uint8_t* mask, int B, int H, int Nq, int Nk, uint32_t thr, uint64_t seed, uint64_t offset,
                     hipStream_t st);
}  // namespace fa
