// Instances of the tiled forward kernel for the head-dim bucket d <= 64.
#include "fwd_kernel.h"
namespace fa {
int launch_fwd_d64(const FwdArgs& a, int variant, int nb, hipStream_t st)
{
    (void)nb;
    return launch_fwd_bucket<64, 1>(a, variant, st);
}
}  // namespace fa
