// Instances of the tiled forward kernel for the head-dim bucket d <= 128.
#include "fwd_kernel.h"
namespace fa {
int launch_fwd_d128(const FwdArgs& a, int variant, int nb, hipStream_t st)
{
    (void)nb;
    return launch_fwd_bucket<128, 1>(a, variant, st);
}
}  // namespace fa
