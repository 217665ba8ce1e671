// Instances of the tiled forward kernels for the head-dim bucket d <= 128.
#include "fwd_pp_kernel.h"
namespace fa {
bool fwd_uses_pingpong(int d, bool direct, int Nq, int Nk, int causal, int wl, int wr, long long slices, int hint)
{
    // 96 < d <= 128, more than one 128-row block of queries and no narrow window: the 8-wave ping-pong kernel (measured
    // 3-18 % faster than the 4-wave kernel there; slower for d = 64 and for windows much smaller than its 256-row
    // block, which make it compute mostly masked tiles; a causal window of 1024 keys still measured 0-19 % slower on
    // ten shapes of twelve).  Short causal problems stay with the 4-wave kernel: where a row sees 512 keys or fewer on
    // average (Nq = Nk <= 1024) the diagonal, where the waves of a 256-row block run out of keys one after the other,
    // is too large a share of the work (measured 4-9 % slower over B*H = 8 ... 1024 at N = 512 and 1024; few rows in
    // front of many keys are another matter: Nq 256 Nk 4096 23 % faster with the 8-wave kernel).  And with one 8-wave
    // work-group per CU its grid should make at least two full rounds of the 256 CUs: below that the 4-wave kernel
    // (two work-groups of half the rows per CU) fills the chip better (measured +4 ... +13 %, one shape -8 %) -- except
    // where an unmasked launch is one round that fills three quarters of the CUs or more (192 ... 256 work-groups:
    // measured 3-13 % faster with the 8-wave kernel on eleven random shapes of twelve, 128 and fewer 15-35 % slower).
    // The caller's hint (flash_params::kernel_hint: 1 = 4-wave, 2 = 8-wave) overrides these preferences for A/B runs
    // and tests; the 8-wave kernel still needs 96 < d <= 128, more than 128 query rows and a request that the instances
    // with tiles straight into LDS serve (direct: not one for the instance that serves every request).
    const bool able = direct && d > 96 && d <= 128 && Nq > 128;
    if (hint == 1) return false;
    if (hint == 2) return able;
    const bool narrow_window = (wl >= 0 && wl < 512) || (wr >= 0 && wr < 512 && !causal) ||
                               (wl >= 0 && wl < 1536 && (causal || (wr >= 0 && wl + wr < 1536)));
    const bool short_causal = causal && Nk - Nq / 2 <= 512;
    const long long groups = slices * ((Nq + 255) / 256);
    const bool one_full_round = !causal && wl < 0 && wr < 0 && groups >= 192 && groups <= 256;
    return able && !narrow_window && !short_causal && (groups >= 512 || one_full_round);
}

int launch_fwd_d128(const FwdArgs& a, int variant, int nb, hipStream_t st)
{
    (void)nb;
    if (fwd_uses_pingpong(a.d, !fwd_needs_every_instance(a, variant), a.Nq, a.Nk, a.causal, a.wl, a.wr, (long long)a.B * a.H * a.num_splits,
                          a.kernel_hint))
        return launch_fwd_pp_bucket<128>(a, variant, st);
    return launch_fwd_bucket<128, 1>(a, variant, st);
}
}  // namespace fa
