// C ABI of the library (include/flash_attn_mi355.h): argument checking, split resolution and kernel dispatch.
// Host counterpart of the launch logic in the reference's main() (src/main.cu:109-192): fill the launch
// arguments, pick the kernel, size the grid, enqueue (+ combine when the key range is split).
#include "flash_attn_mi355.h"

#include <atomic>
#include <cmath>
#include <cstdio>
#include <cstring>

#include "common.h"
#include "decode_kernels.h"
#include "fwd_kernel.h"

static_assert(FLASH_MAX_SPLITS == FLASH_MAX_SPLITS_K, "split limits out of sync");

namespace {

thread_local char g_hip_error[256] = "";

int record_hip(int e)
{
    if (e == (int)hipSuccess) return FLASH_OK;
    std::snprintf(g_hip_error, sizeof(g_hip_error), "%s", hipGetErrorString((hipError_t)e));
    return FLASH_ELAUNCH;
}

constexpr int kNumCU = 256;  // MI355X

// The library carries gfx950 code only: on any other device the first launch would fail with a HIP error that says
// little.  Checked once per device (0 = not yet, 1 = gfx950, 2 = something else).
int device_usable()
{
    static std::atomic<int> state[fa::kMaxDevices];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return FLASH_ENODEVICE;
    const bool cached = dev >= 0 && dev < fa::kMaxDevices;
    int st = cached ? state[dev].load(std::memory_order_relaxed) : 0;
    if (st == 0) {
        hipDeviceProp_t prop;
        if (hipGetDeviceProperties(&prop, dev) != hipSuccess) return FLASH_ENODEVICE;
        st = std::strncmp(prop.gcnArchName, "gfx950", 6) == 0 ? 1 : 2;
        if (cached) state[dev].store(st, std::memory_order_relaxed);
    }
    return st == 1 ? FLASH_OK : FLASH_ENODEVICE;
}

inline bool misaligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) != 0; }

// shape / scalar checks shared by every entry point; *empty is set when there is nothing to compute
int validate_shape(const flash_params* p, bool* empty)
{
    *empty = false;
    if (!p) return FLASH_EINVAL;
    if (p->B < 0 || p->H < 0 || p->Nq < 0 || p->Nk < 0 || p->d <= 0) return FLASH_EINVAL;
    if (p->d > FLASH_MAX_HEAD_DIM) return FLASH_EHEADDIM;
    if (!(p->softmax_scale == p->softmax_scale) || std::isinf(p->softmax_scale)) return FLASH_EINVAL;
    if (!(p->dropout_p >= 0.0f && p->dropout_p < 1.0f)) return FLASH_EINVAL;
    if (p->num_splits > FLASH_MAX_SPLITS) return FLASH_ESPLITS;
    if ((long long)p->B * p->H > 0x7fffffffLL / 2) return FLASH_EINVAL;
    // one-dimensional grids: slices x row blocks x splits must fit the 2^31 - 1 work-groups of a launch
    if ((long long)p->B * p->H * (((long long)p->Nq + 127) / 128) > 0x7fffffffLL / FLASH_MAX_SPLITS) return FLASH_EINVAL;
    if ((long long)p->Nq + p->Nk > 0x7fffffffLL) return FLASH_EINVAL;  // row + window arithmetic stays in int
    // the tile requests address a [N,d] slice with 32-bit byte offsets
    if (2LL * p->Nq * p->d >= (1LL << 32) || 2LL * p->Nk * p->d >= (1LL << 32)) return FLASH_EINVAL;
    if (p->H_kv < 0 || (p->H_kv > 0 && (p->H_kv > p->H || p->H % p->H_kv != 0))) return FLASH_EINVAL;
    if (p->kernel_hint < 0 || p->kernel_hint > 2) return FLASH_EINVAL;
    if (p->B == 0 || p->H == 0 || p->Nq == 0) *empty = true;
    return FLASH_OK;
}

// pointer checks of the two launching entry points
int validate(const flash_params* p, bool* empty)
{
    const int rc = validate_shape(p, empty);
    if (rc != FLASH_OK || *empty) return rc;
    if (!p->Q || !p->O || !p->LSE) return FLASH_EINVAL;
    if (p->Nk > 0 && (!p->K || !p->V)) return FLASH_EINVAL;
    // The vector path moves 16 bytes at a time, as the reference's cp.async does (include/utils.h:63).
    const size_t need = (p->d % 8 == 0) ? 16 : 2;
    if (misaligned(p->Q, need) || misaligned(p->O, need) || misaligned(p->LSE, 4)) return FLASH_EALIGN;
    if (p->Nk > 0 && (misaligned(p->K, need) || misaligned(p->V, need))) return FLASH_EALIGN;
    if (p->alibi_slopes && misaligned(p->alibi_slopes, 4)) return FLASH_EALIGN;
    if (p->scores_out && misaligned(p->scores_out, 4)) return FLASH_EALIGN;
    if (p->stage_stamps_out && misaligned(p->stage_stamps_out, 8)) return FLASH_EALIGN;
    return FLASH_OK;
}

constexpr int kRowsPerGroup = 128;  // FwdCfg<D, 1>::BR

// A window bound that can never cut (i' - j <= Nk - 1, j - i' <= Nq - 1 for the row index i' = i + Nk - Nq) is the same
// as no bound; callers write "unbounded" as INT_MAX too, which the kernels' i' + right would overflow.  Everything
// that looks at the window (launch arguments, kernel choice, split count) looks at these.
inline int window_left_of(const flash_params* p) { return p->window_left >= p->Nk ? -1 : p->window_left; }
inline int window_right_of(const flash_params* p) { return p->window_right >= p->Nq ? -1 : p->window_right; }

void fill_args(const flash_params* p, int splits, fa::FwdArgs* a)
{
    std::memset(a, 0, sizeof(*a));
    a->Q = static_cast<const fa::half_t*>(p->Q);
    a->K = static_cast<const fa::half_t*>(p->K);
    a->V = static_cast<const fa::half_t*>(p->V);
    a->O = static_cast<fa::half_t*>(p->O);
    a->LSE = p->LSE;
    a->O_partial = p->O_partial;
    a->LSE_partial = p->LSE_partial;
    a->alibi = p->alibi_slopes;
    a->keep_out = p->dropout_p > 0.0f ? p->keep_mask_out : nullptr;
    a->scores_out = p->scores_out;
    a->stamps = p->stage_stamps_out;
    a->kernel_hint = p->kernel_hint;
    a->B = p->B;
    a->H = p->H;
    a->Nq = p->Nq;
    a->Nk = p->Nk;
    a->d = p->d;
    a->Hk = p->H_kv > 0 ? p->H_kv : (p->H > 0 ? p->H : 1);
    a->kv_group = p->H > 0 ? p->H / a->Hk : 1;
    a->causal = p->is_causal ? 1 : 0;
    a->wl = window_left_of(p);
    a->wr = window_right_of(p);
    a->alibi_left = (p->alibi_slopes && (a->causal || a->wr == 0)) ? 1 : 0;
    a->scale_log2 = p->softmax_scale * fa::kLog2e;
    a->drop_thr = flash_dropout_threshold(p->dropout_p);
    a->drop_sub2 = a->drop_thr > 0 ? (a->drop_thr - 1) * 0x00010001u : 0u;
    a->drop_rscale = 1.0f / (1.0f - p->dropout_p);
    a->seed_lo = (uint32_t)p->seed;
    a->seed_hi = (uint32_t)(p->seed >> 32);
    a->off_lo = (uint32_t)p->offset;
    a->num_splits = splits;
    const int blocks = (p->Nk + FLASH_SPLIT_KEY_GRANULE - 1) / FLASH_SPLIT_KEY_GRANULE;
    a->keys_per_split = ((blocks + splits - 1) / splits) * FLASH_SPLIT_KEY_GRANULE;  // splitkv.h:40-43
    a->Tr = (p->Nq + kRowsPerGroup - 1) / kRowsPerGroup;
}

// variant bits of the tiled kernel for p (kVarVec | kVarAlibi | kVarDropout of fwd_kernel.h)
// requests that only the tiled kernel's instance which serves every request takes (fa::fwd_needs_every_instance)
bool needs_every_instance(const flash_params* p)
{
    return p->softmax_scale <= 0.0f || p->scores_out || p->d < 8 ||
           (p->dropout_p > 0.0f && flash_dropout_threshold(p->dropout_p) == 0);
}

int tiled_variant(const flash_params* p)
{
    // A non-positive scale does not commute with the row maximum: only the any-alignment instance that serves every request scales first.
    int variant = (p->d % 8 == 0 && p->softmax_scale > 0.0f && !p->scores_out) ? 1 : 0;  // (the score dump lives there too)
    // A dropout probability below 2^-16 has threshold 0 (every element kept, survivors still scaled): the vector
    // instances apply the decisions with threshold - 1 and leave that case to the same instance.
    if (p->dropout_p > 0.0f && flash_dropout_threshold(p->dropout_p) == 0) variant = 0;
    if (p->alibi_slopes) variant |= 2;
    if (p->dropout_p > 0.0f) variant |= 4;
    return variant;
}

int launch_tiled(const flash_params* p, const fa::FwdArgs& a, hipStream_t st)
{
    const int variant = tiled_variant(p);
    int e;
    if (p->d <= 32) e = fa::launch_fwd_d32(a, variant, 1, st);
    else if (p->d <= 64) e = fa::launch_fwd_d64(a, variant, 1, st);
    else if (p->d <= 96) e = fa::launch_fwd_d96(a, variant, 1, st);
    else e = fa::launch_fwd_d128(a, variant, 1, st);
    return record_hip(e);
}

// work-groups of the tiled launch for the (final) arguments a
long long tiled_groups(const flash_params* p, const fa::FwdArgs& a)
{
    const bool pp = a.d > 96 && fa::fwd_uses_pingpong(a.d, !needs_every_instance(p), a.Nq, a.Nk, a.causal, a.wl, a.wr,
                                                      (long long)a.B * a.H * a.num_splits, a.kernel_hint);
    const int rows = pp ? 256 : kRowsPerGroup;
    return (long long)((a.Nq + rows - 1) / rows) * a.B * a.H * a.num_splits;
}

// Automatic split count of the tiled kernels (Nq > 1): the count with the lowest estimated time of split kernel +
// combine.  The reference's rule (src/main.cu:391-422, called at :125) only asks how full the last round of thread
// blocks over the SMs is, and only among counts with seq_len % (128 s) == 0, an artifact of its tiling (here the ranges
// are whole 128-key blocks whatever s is).  Sweeps of explicit counts on 256 CUs showed what else decides:
//  * work-groups i and i + 256 share a CU (the dispatcher deals them out round robin), so 320 work-groups take about as
//    long as 512: the unit is the number k of work-groups on the fullest CU
//    (B1 H8 Nq512 Nk32768 d128: 8 splits 87.6 us, 10: 100.5, 12: 91.9, 16: 84.2);
//  * k work-groups of a CU run side by side and finish in less than k times the time of one (1.3x faster in all where
//    the tiles come by LDS-DMA, 1.5-1.6x for the instances that are bound by load latency), but each pays a prologue
//    and an epilogue, and each split its partial results: 8 B H Nq d bytes written and read back, at about 3.5 TB/s;
//  * under a causal mask the launch takes as long as its heaviest work-group, the last row block's longest split, alone
//    on its CU for most of its life: with few head slices splitting shortens exactly that
//    (B1 H2 N16384 d64: 194 us unsplit, 124 us in 5 splits; B1 H16 N2048 d128 stays unsplit: 39 us against 44).
// The estimate for s splits: k a / rho + b t + [s > 1] (c0 + s * partials), k = work-groups on the fullest CU, t = their
// tiles (the heaviest one plus k - 1 average ones) taken in rounds of as many as the CU has places for, a round of n
// side by side costing the sum of its tiles over the gain of n, b = microseconds per 64-key tile of a work-group alone
// on its CU.  Over 21 swept shapes the count it picks is within 5 % of the best measured one on 19 (the others: 6 % and
// 9 %); the reference's rule with 256 CUs: 9 of 21, the worst 3.1 times slower than the best count.
int auto_splits_tiled_uncached(const flash_params* p, int n_blocks, bool decode);

// The estimate walks the row blocks once per candidate count (up to 0.26 ms on a causal sequence of 65536 rows), and
// callers in a loop ask for the same few shapes again and again: each thread remembers the answers to its last four
// distinct requests.  Everything the estimate reads is part of the key.
int auto_splits_tiled(const flash_params* p, int n_blocks, bool decode = false)
{
    struct Key {
        int B, H, H_kv, Nq, Nk, d, causal, wl, wr, hint, flags;
        bool operator==(const Key& o) const
        {
            return B == o.B && H == o.H && H_kv == o.H_kv && Nq == o.Nq && Nk == o.Nk && d == o.d && causal == o.causal &&
                   wl == o.wl && wr == o.wr && hint == o.hint && flags == o.flags;
        }
    };
    struct Entry { Key key; int splits; bool valid; };
    static thread_local Entry memo[4];
    static thread_local int next = 0;
    const Key key = {p->B, p->H, p->H_kv, p->Nq, p->Nk, p->d, p->is_causal, window_left_of(p), window_right_of(p), p->kernel_hint,
                     tiled_variant(p) | (p->softmax_scale > 0.0f ? 8 : 0) | (p->scores_out ? 16 : 0) | (decode ? 32 : 0) |
                         (p->dropout_p > 0.0f && flash_dropout_threshold(p->dropout_p) == 0 ? 64 : 0) |
                         (p->stage_stamps_out ? 128 : 0)};
    for (const Entry& e : memo)
        if (e.valid && e.key == key) return e.splits;
    const int splits = auto_splits_tiled_uncached(p, n_blocks, decode);
    memo[next] = Entry{key, splits, true};
    next = (next + 1) % 4;
    return splits;
}

int auto_splits_tiled_uncached(const flash_params* p, int n_blocks, bool decode)
{
    const int wl = window_left_of(p), wr = window_right_of(p);
    const bool every = needs_every_instance(p);
    const bool pp = fa::fwd_uses_pingpong(p->d, !every, p->Nq, p->Nk, p->is_causal, wl, wr, (long long)p->B * p->H, p->kernel_hint);
    const int rows = pp ? 256 : kRowsPerGroup;
    const int Tr = (p->Nq + rows - 1) / rows;
    const long long slices = (long long)p->B * p->H;
    if (slices * Tr >= 4LL * kNumCU) return 1;  // (the reference's early exit: four rounds of work-groups as they are)
    const int bucket = (p->d + 31) / 32;  // head-dim bucket of the kernel instance: 1 ... 4
    // microseconds per tile of a lone work-group, by bucket; x 1.5 for the instance that serves every request (tiles
    // staged through registers)
    static const float kTile[5] = {0.0f, 0.5f, 0.72f, 0.88f, 1.0f};
    const bool dma = !every && p->d == 32 * bucket;
    // (decode launches, whose tiles no other work-group has asked for before: twice that, and 0.04 us per split for
    // the combine of their few rows; fitted to 55 random decode shapes of the tiled routes)
    // (rows shorter than the bucket fetch and multiply past their end, but fewer bytes arrive: measured d = 72 at 0.86 of
    // d = 96 per tile, d = 100 at 0.9 of 128)
    const float shorter = (0.55f + 0.45f * (float)p->d / (float)(32 * bucket)) * ((p->d & 7) ? 1.05f : 1.0f);
    const float b = (pp ? 1.97f : kTile[bucket] * (dma ? 1.0f : every ? 1.5f : shorter)) * (decode ? 2.0f : 1.0f);
    const float rho2 = pp ? 1.0f : every ? 1.4f : 1.32f;
    const float rho3 = (!pp && !every && p->d <= 64) ? rho2 * 1.12f : rho2;  // three places per CU up to d = 64
    // a: prologue + epilogue of a work-group; c0 + c1 s: the combine launch and what every further split adds to it and to
    // the split launch; partials: 8 B H Nq d bytes written and read back per split at 4.2 TB/s.  (Fitted to sweeps of
    // explicit counts over 101 shapes, checked on 40 others.)
    const float a = 5.0f, c0 = 4.2f, c1 = decode ? 0.04f : 0.09f;
    const float partials = 8.0f * (float)slices * (float)p->Nq * (float)p->d / 4.2e6f;  // us per split
    const int shift = p->Nk - p->Nq;
    const bool masked = p->is_causal || wl >= 0 || wr >= 0;
    // An unsplit launch may take the narrow instances (fa::fwd_uses_narrow): four times the work-groups, each wave
    // walking a quarter of the tiles alone on its SIMD, two work-groups side by side per CU up to d = 32 and one in a
    // row above, 3 us for the launch and 4 us per work-group in a row on a CU (fitted to 12 shapes).
    bool narrow = false;
    if (!pp) {
        fa::FwdArgs unsplit;
        fill_args(p, 1, &unsplit);
        narrow = fa::fwd_uses_narrow(unsplit, tiled_variant(p), every);
    }
    int limit = FLASH_MAX_SPLITS;
    if (n_blocks < limit) limit = n_blocks;
    int best_s = 1, prev_per = -1;
    float best_t = 0.0f;
    for (int s = 1; s <= limit; ++s) {
        const int per = (n_blocks + s - 1) / s;
        if (per == prev_per) continue;  // the same ranges as s - 1 plus an empty split (src/main.cu:397-398)
        prev_per = per;
        const long long kps = (long long)per * FLASH_SPLIT_KEY_GRANULE;
        // work-groups with a visible key, their tiles, and the tiles of the heaviest one
        long long groups = 0, tiles = 0, tmax = 0;
        const int m_end = masked ? Tr : 1;  // without a mask every row block sees every key
        for (int m = 0; m < m_end; ++m) {
            long long lo = 0, hi = p->Nk;  // visible keys of the row block: [lo, hi)
            if (masked) {
                const long long first = (long long)m * rows + shift;
                const long long last = (long long)((m + 1) * rows < p->Nq ? (m + 1) * rows : p->Nq) - 1 + shift;
                if (wl >= 0 && first - wl > lo) lo = first - wl;
                if (p->is_causal && last + 1 < hi) hi = last + 1;
                if (wr >= 0 && last + wr + 1 < hi) hi = last + wr + 1;
                if (hi < 0) hi = 0;
                if (lo > hi) lo = hi;
            }
            if (hi <= lo) continue;
            const long long s_lo = lo / kps, s_hi = (hi - 1) / kps;
            groups += s_hi - s_lo + 1;
            tiles += (hi - lo + 63) / 64;
            const long long longest = s_hi > s_lo ? kps : hi - lo;
            if ((longest + 63) / 64 > tmax) tmax = (longest + 63) / 64;
        }
        if (!masked) {
            groups *= Tr;
            tiles *= Tr;
        }
        groups *= slices;
        tiles *= slices;
        if (groups == 0) return 1;
        const long long k = (groups + kNumCU - 1) / kNumCU;
        const float rho = k == 1 ? 1.0f : k == 2 ? rho2 : rho3;
        // The k work-groups of the fullest CU run `places` at a time: whole rounds side by side, and what is left over
        // in a last round with less company (three work-groups on two places take a round of two and a round of one).
        const int places = pp ? 1 : (!every && p->d <= 64) ? 3 : 2;
        const float avg = (float)tiles / (float)groups;
        const float gain[4] = {1.0f, 1.0f, rho2, rho3};
        float chain = 0.0f;  // tiles of the fullest CU, in units of a lone work-group's tile
        for (long long left = k; left > 0;) {
            const int n = left < places ? (int)left : places;
            chain += ((left == k ? (float)tmax + (float)(n - 1) * avg : (float)n * avg)) / gain[n];
            left -= n;
        }
        float t = (float)k * a / rho + b * chain;
        if (s == 1 && narrow) {
            // 32-row work-groups with a visible key, and the time per tile of a wave on its own, measured: x 1.15 with
            // two LDS stages per wave (d <= 64); with one, where the next tile's requests are only partly hidden, x 1.3 at
            // d = 96 and x 1.6 at d = 128 (rows shorter than those buckets do not take these instances), x 1.7 on top for
            // odd d (every second row off a 4-byte boundary: slower requests, which a wave on its own cannot hide); under
            // a causal mask with about as many rows as keys the work-groups that follow another on their CU are the
            // light ones of rows that found their tiles in L2 already, and take half of that
            const long long gn = (groups * ((p->Nq + 31) / 32) + Tr - 1) / Tr;
            const long long kn = (gn + kNumCU - 1) / kNumCU;
            const float rhon = kn >= 2 && p->d <= 32 ? rho2 : 1.0f;
            const float bn = (p->d <= 64 ? 1.15f : bucket == 3 ? 1.3f : 1.6f) * ((p->d & 1) ? 1.7f : 1.0f) * b;
            const float later = p->is_causal && 2 * p->Nq >= p->Nk ? 0.5f : 1.0f;
            t = (3.0f + (float)kn * (a - 1.0f) + bn * ((float)((tmax + 3) / 4) + later * (float)(kn - 1) * (float)tiles / (float)groups / 4.0f)) / rhon;
        }
        if (s > 1) t += c0 + (float)s * (c1 + partials);
        if (s == 1 || t < best_t) {
            best_t = t;
            best_s = s;
        }
    }
    return best_s;
}

int resolve_splits(const flash_params* p)
{
    const int n_blocks = (p->Nk + FLASH_SPLIT_KEY_GRANULE - 1) / FLASH_SPLIT_KEY_GRANULE;
    int s = p->num_splits;
    if (s <= 0 && p->Nq == 1) {
        // Decode.  The reference's rule (fill the SMs once) leaves most of the bandwidth unused here: a lone work-group
        // of the one-row kernel streams 13-16 GB/s, far fewer bytes in flight than a CU can keep.
        const int hk = p->H_kv > 0 ? p->H_kv : p->H;
        const int G = p->H / (hk > 0 ? hk : 1);
        const bool heads_as_rows = G >= 4 && !p->alibi_slopes && window_left_of(p) < 0 && p->dropout_p == 0.0f;
        const bool one_row_kernel = !heads_as_rows && p->d >= 8 && p->dropout_p == 0.0f && p->softmax_scale > 0.0f;
        if (one_row_kernel) {
            // Each wave keeps the 2 U loads of its next key block in flight while it works on the current one (64-128 KiB
            // per work-group), so one work-group per CU already covers the memory latency.  Measured over 61 random
            // shapes and 10 large ones on 256 CUs: the launch is fastest with about 256 work-groups whatever the batch,
            // heads and key count (B1 H32 Nk16384 d128: 1 / 4 / 6 / 8 / 16 / 32 splits 142 / 48 / 42 / 42 / 45 / 48 us;
            // B4 H8 Nk65536: best at 6; B16 H32 and B64 H32: unsplit); and every split adds to the combine, which
            // bounds the useful count by about sqrt(Nk / 3).
            const int per_group = G % 8 == 0 ? 8 : G % 4 == 0 ? 4 : G % 2 == 0 ? 2 : 1;  // query heads per work-group
            const long long groups = (long long)p->B * p->H / per_group;
            // (twice that where a work-group serves four or eight query heads, which only ALiBi or a window send here: it
            // then spends as long on arithmetic as on loads; B16 H32 H_kv8 Nk16384 with ALiBi 2 / 4 splits 185 / 171 us)
            const long long target = (per_group >= 4 ? 2LL : 1LL) * kNumCU;
            long long want = (2 * target + groups) / (2 * (groups > 0 ? groups : 1));  // round(target / groups)
            if (want < 1) want = 1;
            long long cap = FLASH_MAX_SPLITS;
            while (cap > 1 && cap * cap * 3 > (long long)p->Nk) --cap;  // cap <= sqrt(Nk / 3)
            if (want > cap) want = cap;
            s = (int)(want < n_blocks ? want : n_blocks);
        } else {
            // The tiled kernel serves four or more query heads of a K/V head together (heads as the rows of one problem per
            // K/V head) and every request the one-row kernel cannot (d < 8, dropout): the estimate of the tiled path
            // for that problem.
            flash_params r = *p;
            if (heads_as_rows) {
                r.H = hk;
                r.H_kv = 0;
                r.Nq = G;
                r.is_causal = 0;
                r.window_right = -1;
            }
            s = auto_splits_tiled(&r, n_blocks, true);
        }
        if (s >= 1) {  // the count whose splits are all non-empty (src/main.cu:397-398 skips the others too)
            const int per = (n_blocks + s - 1) / s;
            s = (n_blocks + per - 1) / per;
        }
    } else if (s <= 0) {
        s = auto_splits_tiled(p, n_blocks);
    }
    if (s > n_blocks) s = n_blocks;  // never more splits than key blocks
    if (s > FLASH_MAX_SPLITS) s = FLASH_MAX_SPLITS;
    if (s < 1) s = 1;
    return s;
}

// ---- built-in split workspace of flash_forward_splitkv_static (for callers that cannot allocate).
// A file-scope device array: every GPU the library runs on holds its own copy, at its own address, until the process
// ends.  In host code the array's name only stands for the symbol; the device address comes from hipGetSymbolAddress,
// looked up once per device with that device current, and only that address is ever handed to a kernel.
constexpr size_t kScratchBytes = FLASH_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

int scratch_of_current_device(unsigned char** out)
{
    static std::atomic<unsigned char*> addr[fa::kMaxDevices];
    int dev = 0;
    if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) return record_hip((int)e);
    if (dev < 0 || dev >= fa::kMaxDevices) return FLASH_ENODEVICE;
    unsigned char* p = addr[dev].load(std::memory_order_acquire);
    if (p == nullptr) {
        void* sym = nullptr;
        if (hipError_t e = hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch)); e != hipSuccess) return record_hip((int)e);
        if (sym == nullptr) return FLASH_ENODEVICE;
        p = static_cast<unsigned char*>(sym);
        addr[dev].store(p, std::memory_order_release);  // (a concurrent first call stores the same address)
    }
    *out = p;
    return FLASH_OK;
}

// Which kernel serves a split-KV call; may reshape the arguments (grouped decode).
constexpr int kRouteTiled = 0, kRouteStream = 1;
int splitkv_route(const flash_params* p, fa::FwdArgs* a)
{
    if (p->scores_out) return kRouteTiled;  // debug dump: the tiled kernel's instance that serves every request
    if (p->Nq == 1 && a->kv_group >= 4 && !p->alibi_slopes && a->wl < 0 && p->dropout_p == 0.0f) {
        // Decode with grouped K/V heads: the G query heads of one K/V head, one row each, are the G rows of one
        // attention problem over that K/V head -- Q [B,H,1,d] is [B,H_kv,G,d] in memory, and so are O, LSE and the
        // split workspace.  The tiled kernel then streams K/V once per K/V head and does the arithmetic on the MFMA
        // units (measured 1.4x - 4x faster than G dot products per key on the VALU for G = 8 ... 32, equal at G = 4).
        // The single query row sits at position Nk - 1 and sees every key whatever the causal flag or the right
        // window say; as rows of a G-row problem the heads must not get a mask that depends on the row.
        a->H = a->Hk;
        a->Nq = a->kv_group;
        a->kv_group = 1;
        a->causal = 0;
        a->wr = -1;
        a->Tr = (a->Nq + kRowsPerGroup - 1) / kRowsPerGroup;
        return kRouteTiled;
    }
    // one query row per head, rows of eight elements or more, no dropout: bandwidth-bound streaming kernel
    if (p->Nq == 1 && p->d >= 8 && p->dropout_p == 0.0f && p->softmax_scale > 0.0f) return kRouteStream;
    return kRouteTiled;
}

// split kernel (+ combine) for an already validated p and its resolved split count
int run_splitkv(const flash_params* p, int splits, hipStream_t st)
{
    if (splits > 1 && (!p->O_partial || !p->LSE_partial)) return FLASH_EWORKSPACE;
    if (splits > 1 && (misaligned(p->O_partial, 16) || misaligned(p->LSE_partial, 4))) return FLASH_EALIGN;
    if (const int rc = device_usable(); rc != FLASH_OK) return rc;
    fa::FwdArgs a;
    fill_args(p, splits, &a);
    const int route = splitkv_route(p, &a);
    const int e = route == kRouteStream ? record_hip(fa::launch_decode_split(a, st)) : launch_tiled(p, a, st);
    if (e != FLASH_OK || splits == 1) return e;
    return record_hip(fa::launch_combine(a, st));
}

}  // namespace

#define FLASH_EXPORT __attribute__((visibility("default")))

extern "C" {

FLASH_EXPORT int flash_forward(const flash_params* p, void* stream)
{
    bool empty;
    int rc = validate(p, &empty);
    if (rc != FLASH_OK || empty) return rc;
    // One query row per head takes the decode routes, unsplit: the streaming kernel, or the heads of a K/V head as the
    // rows of one problem (the tiled kernel as it stands would give each head a 128-row work-group of its own).
    if (p->Nq == 1) return run_splitkv(p, 1, static_cast<hipStream_t>(stream));
    if ((rc = device_usable()) != FLASH_OK) return rc;
    fa::FwdArgs a;
    fill_args(p, 1, &a);
    return launch_tiled(p, a, static_cast<hipStream_t>(stream));
}

FLASH_EXPORT int flash_forward_splitkv(const flash_params* p, void* stream)
{
    bool empty;
    const int rc = validate(p, &empty);
    if (rc != FLASH_OK || empty) return rc;
    return run_splitkv(p, resolve_splits(p), static_cast<hipStream_t>(stream));
}

FLASH_EXPORT int flash_forward_splitkv_static(const flash_params* p, void* stream)
{
    bool empty;
    int rc = validate(p, &empty);
    if (rc != FLASH_OK || empty) return rc;
    const int splits = resolve_splits(p);
    flash_params q = *p;
    q.O_partial = nullptr;
    q.LSE_partial = nullptr;
    if (splits > 1) {
        // O_partial at the start of the scratch array, LSE_partial behind it on the next 256-byte boundary.  Every
        // element the combine step reads is written by the split kernel of the same call, so nothing is cleared.
        const size_t rows = (size_t)p->B * p->H * splits * p->Nq;
        const size_t o_bytes = (rows * p->d * sizeof(float) + 255) & ~(size_t)255;
        if (o_bytes + rows * sizeof(float) > kScratchBytes) return FLASH_ESCRATCH;
        if ((rc = device_usable()) != FLASH_OK) return rc;
        unsigned char* base = nullptr;
        if ((rc = scratch_of_current_device(&base)) != FLASH_OK) return rc;
        q.O_partial = reinterpret_cast<float*>(base);
        q.LSE_partial = reinterpret_cast<float*>(base + o_bytes);
    }
    return run_splitkv(&q, splits, static_cast<hipStream_t>(stream));
}

FLASH_EXPORT int flash_stage_stamps_bytes(const flash_params* p, int split, size_t* bytes)
{
    if (!bytes) return FLASH_EINVAL;
    *bytes = 0;
    bool empty;
    const int rc = validate_shape(p, &empty);
    if (rc != FLASH_OK || empty) return rc;
    fa::FwdArgs a;
    fill_args(p, split ? resolve_splits(p) : 1, &a);
    if ((split || p->Nq == 1) && splitkv_route(p, &a) == kRouteStream) return FLASH_OK;  // (flash_forward routes Nq == 1 too)
    *bytes = (size_t)tiled_groups(p, a) * FLASH_STAMP_WORDS * sizeof(uint64_t);
    return FLASH_OK;
}

FLASH_EXPORT int flash_splitkv_resolve_splits(const flash_params* p)
{
    bool empty;
    const int rc = validate_shape(p, &empty);
    if (rc != FLASH_OK) return rc;
    return empty ? 1 : resolve_splits(p);
}

FLASH_EXPORT int flash_splitkv_workspace_bytes(const flash_params* p, size_t* o_partial_bytes, size_t* lse_partial_bytes)
{
    bool empty;
    const int rc = validate_shape(p, &empty);
    if (rc != FLASH_OK) return rc;
    const int splits = empty ? 1 : resolve_splits(p);
    const size_t rows = splits > 1 ? (size_t)p->B * p->H * splits * p->Nq : 0;
    if (o_partial_bytes) *o_partial_bytes = rows * p->d * sizeof(float);
    if (lse_partial_bytes) *lse_partial_bytes = rows * sizeof(float);
    return FLASH_OK;
}

FLASH_EXPORT int flash_num_splits_heuristic(int batch_nheads_mblocks, int num_SMs, int num_n_blocks, int max_splits, int seq_len)
{
    // Same decision procedure as src/main.cu:391-422: no split when the grid already fills four rounds of CUs;
    // otherwise the smallest eligible split count whose last-round occupancy reaches 85 % of the best one.
    if (num_SMs <= 0) return 1;
    if ((float)batch_nheads_mblocks >= 4.0f * (float)num_SMs) return 1;
    int limit = max_splits;
    if (num_SMs < limit) limit = num_SMs;
    if (num_n_blocks < limit) limit = num_n_blocks;
    auto per_split = [num_n_blocks](int s) { return (num_n_blocks + s - 1) / s; };
    auto eligible = [&](int s) {
        return (s == 1 || per_split(s) != per_split(s - 1)) && (seq_len % (FLASH_SPLIT_KEY_GRANULE * s) == 0);
    };
    auto occupancy = [&](int s) {
        const float rounds = (float)(batch_nheads_mblocks * s) / (float)num_SMs;
        return rounds / std::ceil(rounds);
    };
    float best = 0.0f;
    for (int s = 1; s <= limit; ++s)
        if (eligible(s)) best = std::fmax(best, occupancy(s));
    for (int s = 1; s <= limit; ++s)
        if (eligible(s) && occupancy(s) >= 0.85 * best) return s;
    return 1;
}

FLASH_EXPORT uint32_t flash_dropout_threshold(float dropout_p)
{
    double t = std::floor((double)dropout_p * 65536.0);
    if (!(t > 0.0)) t = 0.0;
    if (t > 65535.0) t = 65535.0;
    return (uint32_t)t;
}

FLASH_EXPORT int flash_dropout_keep_mask(const flash_params* p, uint8_t* mask_out, void* stream)
{
    if (!p || !mask_out) return FLASH_EINVAL;
    if (p->B < 0 || p->H < 0 || p->Nq < 0 || p->Nk < 0) return FLASH_EINVAL;
    if (!(p->dropout_p >= 0.0f && p->dropout_p < 1.0f)) return FLASH_EINVAL;
    if ((long long)p->B * p->H * p->Nq == 0 || p->Nk == 0) return FLASH_OK;
    return record_hip(fa::launch_keep_mask(mask_out, p->B, p->H, p->Nq, p->Nk, flash_dropout_threshold(p->dropout_p),
                                           p->seed, p->offset, static_cast<hipStream_t>(stream)));
}

FLASH_EXPORT void flash_params_init(flash_params* p)
{
    if (!p) return;
    std::memset(p, 0, sizeof(*p));
    p->window_left = -1;
    p->window_right = -1;
    p->num_splits = 1;
}

FLASH_EXPORT size_t flash_params_size(void) { return sizeof(flash_params); }

FLASH_EXPORT const char* flash_last_hip_error(void) { return g_hip_error; }

FLASH_EXPORT const char* flash_strerror(int code)
{
    switch (code) {
        case FLASH_OK: return "ok";
        case FLASH_EINVAL: return "invalid argument";
        case FLASH_EHEADDIM: return "Insufficient shared memory. Please reduce the value of head_dim (max 128)";
        case FLASH_EALIGN: return "pointer not aligned";
        case FLASH_EWORKSPACE: return "split workspace missing";
        case FLASH_ESPLITS: return "too many splits";
        case FLASH_ELAUNCH: return "HIP launch failed";
        case FLASH_ENODEVICE: return "the current device is not a gfx950";
        case FLASH_ESCRATCH: return "split workspace exceeds the built-in scratch (FLASH_STATIC_SCRATCH_BYTES)";
        default: return "unknown error";
    }
}

}  // extern "C"
