// Instances of the tiled forward kernels for the head-dim bucket d <= 128.
#include <cstdlib>

#include "fwd_pp_kernel.h"
namespace fa {
bool fwd_uses_pingpong(int d, bool vec, int Nq, int causal, int wl, int wr)
{
    // d == 128, more than one 128-row block of queries and no narrow window: the 8-wave ping-pong kernel (measured
    // 3-18 % faster than the 4-wave kernel there; slower for d = 64 and for windows much smaller than its 256-row
    // block, which make it compute mostly masked tiles).  Short causal problems stay with the 4-wave kernel: up to
    // 1024 rows the diagonal, where the waves of a 256-row block run out of keys one after the other, is too large a
    // share of the work (measured 4-9 % slower over B*H = 8 ... 1024 at N = 512 and 1024).
    // FLASH_ATTN_NO_PINGPONG=1 forces the 4-wave kernel (A/B runs).
    static const bool no_pp = std::getenv("FLASH_ATTN_NO_PINGPONG") != nullptr;
    const bool narrow_window = (wl >= 0 && wl < 512) || (wr >= 0 && wr < 512 && !causal);
    const bool short_causal = causal && Nq <= 1024;
    return vec && d == 128 && Nq > 128 && !narrow_window && !short_causal && !no_pp;
}

int launch_fwd_d128(const FwdArgs& a, int variant, int nb, hipStream_t st)
{
    (void)nb;
    if (fwd_uses_pingpong(a.d, (variant & kVarVec) != 0, a.Nq, a.causal, a.wl, a.wr))
        return launch_fwd_pp_bucket<128>(a, variant, st);
    return launch_fwd_bucket<128, 1>(a, variant, st);
}
}  // namespace fa
