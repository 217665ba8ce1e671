// Tiled FlashAttention forward for gfx950 (wave64, MFMA 32x32x16 f16 -> f32).
//
// Replaces forward_kernel / forward_kernel_splitkv of the reference (src/flash_forward.h:13-306,
// src/flash_forward_splitkv.h:14-344); the math contract is the one of the reference's CPU verifier
// (src/main.cu:309-383).  The structure is specific to CDNA4:
//
//  * One work-group = 4 waves; wave w owns 32*NB query rows, the group 128*NB.  KV tiles hold 64 keys.
//  * Scores are computed transposed, S^T = K Q^T: the MFMA A operand is a K fragment read from LDS
//    (ds_read_b128), the B operand a Q fragment that stays in registers for the whole kernel.  In the 32x32
//    accumulator layout every lane then holds 16 keys of ONE query row (row = lane % 32), so the online-softmax
//    max / sum are in-lane reductions plus one v_permlane32_swap between lane l and l^32.
//  * The probabilities, rounded to fp16 where the reference rounds them (include/utils.h:47-55), already sit in
//    the B-operand layout of O^T += V^T P^T; no LDS round trip for P.  The V^T A operand needs four keys of one
//    head-dim column per lane: that is what ds_read_b64_tr_b16 delivers from the row-major V tile.
//  * O^T accumulates in registers (fp32) and is normalised once in the epilogue; the reference keeps O in shared
//    memory and renormalises it every tile (src/flash_forward.h:284-289).
//  * K and V tiles are double-buffered in LDS and requested straight into it (global_load_lds_dwordx4), tile t+1
//    while tile t is computed, one barrier per tile; only the instance that serves every request (rows of fewer than
//    eight elements among them) stages its tiles through registers.
//  * Small unsplit problems take the narrow instances: 32 query rows per work-group, held by all four waves, each of
//    which walks every fourth key tile with LDS stages of its own; the four results are merged through LDS.
//  * Every mask of the family (causal, sliding window, key bound for ragged Nk) is one per-row interval
//    [lo_i, hi_i] of allowed keys; tiles entirely inside the interval of every row of the wave skip the
//    element test.  The KV tile range of the group is pruned like src/flash_forward.h:39-48.
//  * Ragged Nq / Nk: row indices of loads are clamped, stores are predicated, keys >= Nk are masked (the
//    reference zero-fills them and leaves them unmasked).  Head dims that are not a multiple of 8 use the
//    instances for rows at any alignment (kVec = false).
#pragma once
#include <type_traits>

#include "common.h"

namespace fa {


template <int D, int NB>
struct FwdCfg {
    static constexpr int kWaves = 4;
    static constexpr int RW = 32 * NB;        // query rows per wave
    static constexpr int BR = kWaves * RW;    // query rows per work-group
    static constexpr int BC = 64;             // keys per tile
    static constexpr int KS = D / 16;         // k-steps of the QK^T contraction
    static constexpr int MB = D / 32;         // 32-wide head-dim blocks of O^T
    static constexpr int CH = D / 8;          // 16-byte chunks per row
    // LDS row strides in bytes.  K rows are read 16 bytes per lane by 32 consecutive rows: stride/16 odd spreads
    // them over all banks.  V rows are read by ds_read_b64_tr_b16, four consecutive rows of 64 bytes per half
    // wave: a stride of 64 (mod 128) puts the four rows on disjoint bank groups.
    static constexpr int SK = D * 2 + 16;
    static constexpr int SV = D * 2;
    // Where the row length is a multiple of 128 bytes, the two 64-byte halves of each 128 bytes are exchanged in rows
    // 2, 3 (mod 4), which has the same effect without padding.
    static constexpr bool VSWZ = (D * 2) % 128 == 0;
    static constexpr int KBUF = BC * SK;
    static constexpr int VBUF = BC * SV;
    static constexpr int SMEM = 2 * KBUF + 2 * VBUF;
    static constexpr int NSTG = 2;
    static constexpr int SMEM_DMA = NSTG * (KBUF + VBUF);
    static constexpr int NKX = (CH + 1 + 3) / 4;  // 1 KiB blocks of a K tile (CH + 1 of them) per wave, rounded up
    static constexpr int NVX = CH / 4;            // 1 KiB blocks of a V tile (CH of them) per wave
    static constexpr int NLD = BC * CH / 256;  // 16-byte chunks per thread per tile (K and V each)
    static_assert(D % 32 == 0 && D <= 128, "head-dim bucket");
    static_assert((BC * CH) % 256 == 0, "tile chunks must divide over the group");
};

// 8 fp16 of one row starting at column col (multiple of 8); columns >= d read as zero.
// kVec: rows are 16-byte aligned (d % 8 == 0); kFullD: d equals the bucket width, no column test at all.
template <bool kVec, bool kFullD>
__device__ __forceinline__ v4u load_chunk(const half_t* __restrict__ rowp, int col, int d)
{
    if constexpr (kFullD) {
        return *reinterpret_cast<const v4u*>(rowp + col);
    } else if constexpr (kVec) {
        const int cc = col < d ? col : d - 8;  // stay inside the row, discard below
        v4u v = *reinterpret_cast<const v4u*>(rowp + cc);
        const v4u z = {0u, 0u, 0u, 0u};
        return col < d ? v : z;
    } else {
        union { v8h h; v4u u; } r;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const int c = col + e;
            const half_t x = rowp[c < d ? c : d - 1];
            r.h[e] = c < d ? x : (half_t)0.0f;
        }
        return r.u;
    }
}

// Rows that start at any 2-byte boundary (d % 8 != 0), d >= 8: a chunk is still one 16-byte load -- the hardware runs in
// unaligned access mode -- taken at the chunk's own column, or, for the row's last, partial chunk and for chunks past the
// row, at column d - 8, so that no load ever leaves the row.  Nothing is moved into place afterwards: the last chunk
// position of a row simply stands for the columns d - 8 ... d - 1 instead of 8 (d / 8) ... 8 (d / 8) + 7.
//   Q   the columns that the chunk before has covered already (the first 8 - d % 8 of the partial chunk) are zeroed, and so
//       are chunks past the row (mask_q_chunk_anyalign): every product with them is 0 times finite data of the K row itself.
//   K   as loaded.
//   V   as loaded: the chunk position yields O's columns d - 8 ... d - 1, of which the epilogue stores the row's last 16
//       bytes; chunks past the row yield columns that are never stored.
// Element by element, a 64 x 32 tile took 16 two-byte loads per thread with an address computation each, where this takes
// two loads and no arithmetic on the data.
__device__ __forceinline__ v4u load_chunk_anyalign(const half_t* __restrict__ rowp, int col, int d)
{
    return *reinterpret_cast<const v4u_anyalign*>(rowp + (col + 8 <= d ? col : d - 8));
}

// Running maximum is only raised when some row of the wave outgrows it by more than this many powers of two;
// until then probabilities are taken relative to the stale maximum (bounded by 2^kLazyTau, exact in the end
// because numerator and denominator carry the same factor).  Saves the per-tile rescale of the O accumulators.
constexpr float kLazyTau = 8.0f;

// variant bits of the kernel template
// kVarStamp: debug time stamps.  kVarAlibiLeft (with kVarAlibi, kVarVec): every visible key lies at or left of its row
// (causal mask or a right window of 0), which lets the bias ride in the MFMA accumulator (see calib below).
// kVarKvOnce (with kVarVec, kVarFullD, no other feature): every K/V tile is requested by this work-group alone -- one row
// block per slice and one query head per K/V head, the shape of a decode launch -- and its requests are non-temporal.
// kVarEvery (with kVarAlibi and kVarDropout, without kVarVec): the instance that serves every request, see kEvery below.
// kVarNarrow (unsplit launches): the four waves of a work-group share 32 query rows and take every fourth key tile
// each, see kNarrow below.
constexpr int kVarVec = 1, kVarAlibi = 2, kVarDropout = 4, kVarFullD = 8, kVarStamp = 16, kVarAlibiLeft = 32, kVarKvOnce = 64,
              kVarEvery = 128, kVarNarrow = 256;

// work-groups per CU: three up to D = 64 (168 VGPRs), except for the instance that serves every request, which stages
// its tiles through registers
constexpr int fwd_groups_per_cu(int D, int NB, int VAR)
{
    if ((VAR & kVarNarrow) != 0) return 1;
    return NB == 1 ? (D <= 64 && (VAR & kVarEvery) == 0 ? 3 : 2) : 1;
}

template <int D, int NB, int VAR>
__global__ void __launch_bounds__(256, fwd_groups_per_cu(D, NB, VAR)) fwd_kernel(const FwdArgs a)
{
    constexpr bool kVec = (VAR & kVarVec) != 0, kAlibi = (VAR & kVarAlibi) != 0, kDropout = (VAR & kVarDropout) != 0,
                   kFullD = (VAR & kVarFullD) != 0, kStamp = (VAR & kVarStamp) != 0, kKvOnce = (VAR & kVarKvOnce) != 0;
    using C = FwdCfg<D, NB>;
    Stamps<kStamp> stamps;
    stamps.take(0);
    constexpr int BC = C::BC, KS = C::KS, MB = C::MB, CH = C::CH, SK = C::SK, SV = C::SV, NLD = C::NLD;
    // Tiles go from global memory straight into LDS (global_load_lds_dwordx4) instead of through registers: measured
    // +6-12 % at D = 128, +1-4 % at D = 64 and 96.  The request takes global addresses at any 2-byte boundary, so rows of
    // any length from eight elements on are served; only the instance that also serves shorter rows stages through
    // registers (kEvery, defined below).
    constexpr bool kDma = (VAR & kVarEvery) == 0;
    // Rows at any alignment (kVec false) have the same four instances as rows of whole chunks: plain, ALiBi, dropout, both.
    // They count on d >= 8, a positive scale, a slope table where ALiBi is compiled in and a dropout threshold of at least
    // 1 like the vector instances do.  One more instance, with both features compiled in, serves every request (kEvery:
    // slope 0 / threshold 0 make the features identities), a non-positive scale, rows of fewer than eight elements and
    // the score dump among them.
    constexpr bool kEvery = (VAR & kVarEvery) != 0;
    static_assert(!kEvery || (!kVec && kAlibi && kDropout), "the instance that serves every request");
    // Small problems -- fewer work-groups of 128 rows than half the CUs -- are bound by the chain of tiles that a
    // work-group walks through one after the other.  The narrow instances cut that chain to a quarter: a work-group owns
    // 32 query rows, all four waves hold those rows, and wave w takes the key tiles w, w + 4, w + 8, ... of the range on
    // its own: it requests them into LDS stages of its own (no work-group barrier inside the loop, every wave waits
    // for its own requests only), and the four partial results are merged through LDS at the end like the partial results
    // of a split -- in the same launch, where a split count of four would need the combine launch behind it.
    constexpr bool kNarrow = (VAR & kVarNarrow) != 0;
    static_assert(!kNarrow || (kDma && NB == 1 && !kStamp && !kKvOnce), "narrow instances");
    // (narrow: two stages per wave up to D = 64, one above: four waves' tiles of 26 / 33 KiB)
    constexpr int NSTG = kNarrow ? (D <= 64 ? 2 : 1) : kDma ? C::NSTG : 2;
    constexpr int BRW = kNarrow ? 32 : C::BR;  // query rows per work-group
    extern __shared__ __attribute__((aligned(16))) char smem[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = wave_uniform(tid >> 6);
    // tile buffers: of the work-group, or (narrow) of the wave
    constexpr int kWaveLds = NSTG * (C::KBUF + C::VBUF);
    const int lds_base = kNarrow ? wave * kWaveLds : 0;
    char* const Ks = smem + lds_base;
    char* const Vs = Ks + NSTG * C::KBUF;
    const int l32 = lane & 31;
    const int g = lane >> 5;

    // work-group -> (head slice, split, row block).  Slices vary fastest, so that with B*H a multiple of 8 a slice
    // always lands on the same XCD (and L2); the heaviest causal row blocks (largest m) are dispatched first.
    const int BH = a.B * a.H;
    // Slices are dealt out in chunks of a.slice_chunk (the launcher's choice: all of them unless the problem has far more
    // work-groups than the GPU holds at once): inside a chunk as above, chunk after chunk, so that the row blocks of a
    // slice run closer together in time and find its K and V in the caches.
    int bh, rest;
    {
        const int per_chunk = a.slice_chunk * a.Tr * a.num_splits;
        const int pos = work_position(blockIdx.x, a.snake_end);
        const int ch = pos / per_chunk, w = pos % per_chunk;
        bh = ch * a.slice_chunk + slice_of_position(w % a.slice_chunk, a.group_xcd);
        rest = w / a.slice_chunk;
    }
    int mi;
    const int split = split_of_rest(rest, a.num_splits, a.split_rotate, &mi);
    const int m_block = a.Tr - 1 - mi;
    const int h = bh % a.H;
    const int Nq = a.Nq, Nk = a.Nk, d = kFullD ? D : a.d;
    const int shift = Nk - Nq;
    const int q0 = m_block * BRW;
    const int wave_row0 = kNarrow ? 0 : wave * C::RW;  // first row of the wave inside the work-group's block

    // ---- key range of the work-group (block pruning, src/flash_forward.h:39-48; split range, splitkv.h:40-43)
    int kmin = 0, kmax = Nk;
    {
        const int last_row = (q0 + BRW - 1 < Nq ? q0 + BRW - 1 : Nq - 1) + shift;
        if (a.wl >= 0) kmin = max(0, q0 + shift - a.wl);
        if (a.causal) kmax = min(kmax, last_row + 1);
        if (a.wr >= 0) kmax = min(kmax, last_row + a.wr + 1);
        if (a.num_splits > 1) {
            const int s0 = split * a.keys_per_split;
            kmin = max(kmin, s0);
            kmax = min(kmax, s0 + a.keys_per_split);
        }
    }
    const int tile_begin = kmin / BC;
    const int ntiles = kmax > kmin ? (kmax + BC - 1) / BC - tile_begin : 0;
    if (!kStamp && ntiles == 0) {  // (the instrumented twins take the long way and report their stages)
        store_empty_rows(a, bh, split, q0, q0 + BRW < Nq ? q0 + BRW : Nq, tid, 256);
        return;
    }

    // ---- per-lane rows
    int row_i[NB], lo[NB], hi[NB];
    float iif[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
        const int i = q0 + wave_row0 + nb * 32 + l32;
        row_i[nb] = i;
        const int ii = (i < Nq ? i : Nq - 1) + shift;
        int l_ = 0, h_ = Nk - 1;
        if (a.wl >= 0) l_ = max(0, ii - a.wl);
        if (a.causal) h_ = min(h_, ii);
        if (a.wr >= 0) h_ = min(h_, ii + a.wr);
        if (a.num_splits > 1) {
            l_ = max(l_, kmin);
            h_ = min(h_, kmax - 1);
        }
        lo[nb] = l_;
        hi[nb] = h_;
        iif[nb] = (float)ii;
    }
    // wave-uniform bounds: [lo_max, hi_min] is visible to every row of the wave (a tile inside it needs no element
    // test), nothing outside [lo_min, hi_max] is visible to any of them (a tile outside it is skipped by the wave)
    int lo_max, hi_min, lo_min, hi_max;
    {
        const int first = q0 + wave_row0, last = first + C::RW - 1;
        const int iif_ = (first < Nq ? first : Nq - 1) + shift, iil_ = (last < Nq ? last : Nq - 1) + shift;
        lo_max = lo_min = 0;
        hi_min = hi_max = Nk - 1;
        if (a.wl >= 0) lo_max = max(0, iil_ - a.wl), lo_min = max(0, iif_ - a.wl);
        if (a.causal) hi_min = min(hi_min, iif_), hi_max = min(hi_max, iil_);
        if (a.wr >= 0) hi_min = min(hi_min, iif_ + a.wr), hi_max = min(hi_max, iil_ + a.wr);
        if (a.num_splits > 1) {
            lo_max = max(lo_max, kmin);
            lo_min = max(lo_min, kmin);
            hi_min = min(hi_min, kmax - 1);
            hi_max = min(hi_max, kmax - 1);
        }
    }

    const half_t* __restrict__ Qbh = a.Q + (size_t)bh * Nq * d;
    const int kvs = a.kv_slice(bh);
    const half_t* __restrict__ Kbh = a.K + (size_t)kvs * Nk * d;
    const half_t* __restrict__ Vbh = a.V + (size_t)kvs * Nk * d;

    // ---- Q fragments (B operand of S^T = K Q^T): lane holds row l32, columns 16*ks + 8*g .. +7
    v8h qf[NB][KS];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
        const int ic = row_i[nb] < Nq ? row_i[nb] : Nq - 1;
        const half_t* qrow = Qbh + (size_t)ic * d;
        if constexpr (kVec) {
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                union { v4u u; v8h h; } t;
                t.u = load_chunk<kVec, kFullD>(qrow, 16 * ks + 8 * g, d);
                qf[nb][ks] = t.h;
            }
        } else {
            // rows at any alignment: every load of the row block first, then the zero padding and the packing (written as
            // one chunk after the other, each 2-byte load was waited for before the next was issued)
            if (!kEvery || d >= 8) {
                v4u raw[KS];
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) raw[ks] = load_chunk_anyalign(qrow, 16 * ks + 8 * g, d);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    qf[nb][ks] = mask_q_chunk_anyalign(raw[ks], 16 * ks + 8 * g, d);
                }
            } else {
                half_t raw[KS][8];
#pragma unroll
                for (int ks = 0; ks < KS; ++ks)
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const int c = 16 * ks + 8 * g + e;
                        raw[ks][e] = qrow[c < d ? c : d - 1];
                    }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int ks = 0; ks < KS; ++ks)
#pragma unroll
                    for (int e = 0; e < 8; ++e) qf[nb][ks][e] = 16 * ks + 8 * g + e < d ? raw[ks][e] : (half_t)0.0f;
            }
        }
    }

    // ---- tile staging through registers (the instance that serves every request; all others request their tiles
    // straight into LDS, below): thread handles chunk ids tid + 256*x  ->  (row, chunk) of the 64 x CH tile.  The
    // loads of tile t+1 are issued in front of the arithmetic of tile t and waited for where their data is written to
    // LDS behind it: nothing is computed on what was loaded (a select on it would drag the wait for the whole tile in
    // front of the arithmetic).
    int ld_row[NLD], ld_col[NLD];
#pragma unroll
    for (int x = 0; x < NLD; ++x) {
        const int cid = tid + 256 * x;
        ld_row[x] = cid / CH;
        ld_col[x] = (cid % CH) * 8;
    }
    // A staged chunk: the 16 bytes as loaded (chunk positions past the row's whole chunks hold the row's last elements:
    // load_chunk_anyalign), except that rows of fewer than eight elements are fetched element by element and padded
    // with zeroes.
    v4u kreg[NLD], vreg[NLD];
    auto gload = [&](const half_t* __restrict__ base, int tile, v4u (&reg)[NLD]) {
        const int kb0 = tile * BC;
#pragma unroll
        for (int x = 0; x < NLD; ++x) {
            const int r = kb0 + ld_row[x];
            const half_t* __restrict__ rowp = base + (size_t)(r < Nk ? r : Nk - 1) * d;
            reg[x] = d >= 8 ? load_chunk_anyalign(rowp, ld_col[x], d) : load_chunk<false, false>(rowp, ld_col[x], d);
        }
    };
    auto put_k = [&](int buf) {
#pragma unroll
        for (int x = 0; x < NLD; ++x)
            *reinterpret_cast<v4u*>(Ks + buf * C::KBUF + ld_row[x] * SK + ld_col[x] * 2) = kreg[x];
    };
    auto put_v = [&](int buf) {
#pragma unroll
        for (int x = 0; x < NLD; ++x)
            *reinterpret_cast<v4u*>(Vs + buf * C::VBUF + ld_row[x] * SV +
                                    ((ld_col[x] * 2) ^ (C::VSWZ ? ((ld_row[x] >> 1) & 1) << 6 : 0))) = vreg[x];
    };

    // ---- direct global -> LDS path: the tile buffers keep their layout (K rows padded by one chunk, V rows with the
    // 64-byte halves exchanged in rows 2, 3 mod 4), and a request fills 64 consecutive 16-byte chunks of a buffer: lane l of
    // block x fetches whatever belongs into chunk 64 x + l (the pad chunk of a K row gets a copy of its neighbour).
    // Blocks go round the four waves; the odd K block goes to the waves that still have a block index left for it.
    // Rows shorter than the bucket: chunk positions past the row's whole chunks fetch the row's last 16 bytes (see
    // load_chunk_anyalign): for K they meet zero columns of Q, for V they only reach rows of O^T that are never stored.
    const int row_bytes = kFullD ? D * 2 : d * 2;
    auto chunk_offset = [&](int c) { return kFullD ? c * 16 : (c * 8 + 8 <= d ? c * 16 : (d - 8) * 2); };
    // (narrow: every block of a tile is the wave's own, and so is the buffer)
    constexpr int NKX = kNarrow ? CH + 1 : C::NKX, NVX = kNarrow ? CH : C::NVX;
    auto block_of = [&](int i) { return kNarrow ? i : wave + 4 * i; };
    uint32_t koff[NKX], voff[NVX];
    int krow[NKX], vrow[NVX];
    if constexpr (kDma) {
#pragma unroll
        for (int i = 0; i < NKX; ++i) {
            const int q = 64 * block_of(i) + lane;
            krow[i] = q / (CH + 1);
            const int col = q % (CH + 1);
            koff[i] = (uint32_t)(krow[i] * row_bytes + chunk_offset(col < CH ? col : CH - 1));
        }
#pragma unroll
        for (int i = 0; i < NVX; ++i) {
            const int q = 64 * block_of(i) + lane;
            vrow[i] = q / CH;
            const int c = q % CH;
            voff[i] = (uint32_t)(vrow[i] * row_bytes + chunk_offset(C::VSWZ ? c ^ (((vrow[i] >> 1) & 1) << 2) : c));
        }
    }
    const bool k_extra = kNarrow || wave + 4 * (NKX - 1) <= CH;  // the last round of K blocks exists for this wave
    auto dma_tile_parts = [&](int tile, int stage, auto k_part, auto v_part) {
        // The tile's offset joins the scalar base address, so that a request of a whole tile needs no vector
        // arithmetic at all; only the last tile of a ragged sequence adjusts rows: keys past Nk re-read key Nk - 1
        // (their scores are masked).
        const size_t tb = (size_t)tile * (size_t)(BC * row_bytes);
        const int rows_left = Nk - tile * BC;  // >= 1
        FA_LDS char* const kst = (FA_LDS char*)smem + lds_base + stage * C::KBUF;
        FA_LDS char* const vst = (FA_LDS char*)smem + lds_base + NSTG * C::KBUF + stage * C::VBUF;
        const char* const Kb = reinterpret_cast<const char*>(Kbh) + tb;
        const char* const Vb = reinterpret_cast<const char*>(Vbh) + tb;
        auto issue = [&](auto ragged_c) {
            constexpr bool kRagged = decltype(ragged_c)::value;
            // (laundered: the compiler otherwise carries one running vector offset per request through every tile
            // for the sake of this one)
            int rows_left = Nk - tile * BC;
            if constexpr (kRagged) asm volatile("" : "+s"(rows_left));
#pragma unroll
            for (int i = 0; i < NKX; ++i) {
                if (!decltype(k_part)::value || (i == NKX - 1 && !k_extra)) break;
                uint32_t o = koff[i];
                if (kRagged && krow[i] >= rows_left) o -= (uint32_t)((krow[i] - rows_left + 1) * row_bytes);
                if constexpr (kKvOnce) dma_kib_nt(Kb, o, kst + block_of(i) * 1024);
                else dma_kib(Kb, o, kst + block_of(i) * 1024);
            }
#pragma unroll
            for (int i = 0; i < NVX; ++i) {
                if (!decltype(v_part)::value) break;
                uint32_t o = voff[i];
                if (kRagged && vrow[i] >= rows_left) o -= (uint32_t)((vrow[i] - rows_left + 1) * row_bytes);
                if constexpr (kKvOnce) dma_kib_nt(Vb, o, vst + block_of(i) * 1024);
                else dma_kib(Vb, o, vst + block_of(i) * 1024);
            }
        };
        if (rows_left >= BC) issue(std::false_type{});
        else issue(std::true_type{});
    };
    auto dma_tile = [&](int tile, int stage) { dma_tile_parts(tile, stage, std::true_type{}, std::true_type{}); };
    // wait until at most the requests of one tile (the youngest) are still in flight / until none is
    auto dma_wait = [&](bool one_tile_in_flight) {
        if (!one_tile_in_flight) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        else if (k_extra) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NKX + NVX) : "memory");
        else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NKX + NVX - 1) : "memory");
    };

    // ---- accumulators
    v16f oacc[MB][NB];
    float m_ref[NB], l_run[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
        m_ref[nb] = -INFINITY;
        l_run[nb] = 0.0f;
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int r = 0; r < 16; ++r) oacc[mb][nb][r] = 0.0f;
    }

    // Scores leave the MFMA unscaled.  With a positive scale the scaling commutes with the row maximum and is folded
    // into the exponent (one fma per score): cs = scale, and the ALiBi bias is added beforehand divided by the scale.
    // A non-positive scale is served by the kEvery instance alone (the host sends it there): then the scores are
    // scaled first and cs = 1.
    const float c2 = a.scale_log2;
    const bool scale_late = !kEvery || c2 > 0.0f;
    const float cs = scale_late ? c2 : 1.0f;
    // The ALiBi slope of the head is read once the first tile requests are on their way (read_slope below): it is a
    // vector load, the wait for it counts every older request as well, and nothing before the first softmax needs it.
    float slope2 = 0.0f, nsig = 0.0f;

    // ALiBi where every visible key lies at or left of its row (causal mask, or a right window of 0: j <= i, keys right
    // of the row are masked anyway): |i - j| = i - j splits into a part that only depends on the accumulator register,
    // -nsig * (8 (r / 4) + r % 4), and a part per lane and 32-key block.  The first goes into the MFMA as the initial
    // accumulator value, the second into the addend of the exponent fma: no instruction per score is left.
    constexpr bool kFoldAlibi = kAlibi && kVec && (VAR & kVarAlibiLeft) != 0;
    v16f calib;
    auto read_slope = [&]() {
        if constexpr (kAlibi) {
            // (only the kEvery instance is launched without a slope table)
            slope2 = (!kEvery || a.alibi) ? a.alibi[h] * kLog2e : 0.0f;
            nsig = scale_late ? -slope2 / c2 : 0.0f;
            if constexpr (kFoldAlibi) {
#pragma unroll
                for (int r = 0; r < 16; ++r) calib[r] = -nsig * (float)(8 * (r >> 2) + (r & 3));
            }
        }
    };

    // LDS read offsets of this lane
    const int k_rd = l32 * SK + g * 16;                                          // + kb*32*SK + ks*32
    const int v_rd = (4 * g + ((lane & 15) >> 2)) * SV + (((lane >> 4) & 1) * 16 + (lane & 3) * 4) * 2;  // + row/col blocks
    const int v_sw = C::VSWZ ? ((lane >> 3) & 1) << 6 : 0;

    // S^T = K Q^T of the tile in K buffer `buf`
    auto qk = [&](int buf, v16f (&s)[2][NB]) {
        constexpr bool folded = kFoldAlibi;
        const char* kbase = Ks + buf * C::KBUF + k_rd;
        if constexpr (folded && NB == 1) {
            // The first k-step's MFMAs are inline asm here (below), which the issue-order groups at the end of this
            // function cannot name: with them in the stream the compiler fell back to waiting for every fragment right
            // behind its request.  So this instance is written out in issue order, fenced step by step: three fragments
            // ahead, then MFMA and read in turn.
            constexpr int n = 2 * KS, kAhead = 3;  // step i: k-step i / 2, key block i % 2
            v8h af[n];
#pragma unroll
            for (int i = 0; i < kAhead; ++i) af[i] = *reinterpret_cast<const v8h*>(kbase + (i & 1) * 32 * SK + (i >> 1) * 32);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < n; ++i) {
                const int ks = i >> 1, kb = i & 1;
                if (ks == 0) asm("v_mfma_f32_32x32x16_f16 %0, %1, %2, %3" : "=&v"(s[kb][0]) : "v"(af[i]), "v"(qf[0][ks]), "v"(calib));
                else s[kb][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], qf[0][ks], s[kb][0], 0, 0, 0);
                if (i + kAhead < n)
                    af[i + kAhead] = *reinterpret_cast<const v8h*>(kbase + ((i + kAhead) & 1) * 32 * SK + ((i + kAhead) >> 1) * 32);
                __builtin_amdgcn_sched_barrier(0);
            }
            return;
        }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
                const v8h af = *reinterpret_cast<const v8h*>(kbase + kb * 32 * SK + ks * 32);
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) {
                    if (ks == 0) {
                        // first k-step: the accumulator starts from zero (an inline constant) or, with the ALiBi bias
                        // folded in, from the per-register bias constants, which stay where they are
                        if constexpr (folded) {
                            // written out: the compiler only knows the form whose result overwrites the addend and would
                            // copy the sixteen constants for every tile.  Hazards of an MFMA the compiler cannot see as
                            // one: its operands are ready (the asm's inputs: af comes with the wait for its LDS read,
                            // qf and calib were written long before); its result is next read as the addend of the
                            // second k-step's MFMA on the same registers, a dependency the hardware interlocks -- hence
                            // at least two k-steps -- and by VALU code only after that one.
                            static_assert(!folded || KS >= 2, "the score accumulator is first read by a following MFMA");
                            asm("v_mfma_f32_32x32x16_f16 %0, %1, %2, %3" : "=&v"(s[kb][nb]) : "v"(af), "v"(qf[nb][ks]), "v"(calib));
                        } else {
                            const v16f z = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                            s[kb][nb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af, qf[nb][ks], z, 0, 0, 0);
                        }
                    } else {
                        s[kb][nb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af, qf[nb][ks], s[kb][nb], 0, 0, 0);
                    }
                }
            }
        }
        // issue order: kQkAhead fragment reads first, then read and MFMA in turn (left to itself the compiler waits
        // for each fragment right after requesting it)
        if constexpr (NB == 1) {
            constexpr int kQkAhead = 3, n = 2 * KS;
            __builtin_amdgcn_sched_group_barrier(0x100, kQkAhead, 0);
#pragma unroll
            for (int i = 0; i < n - kQkAhead; ++i) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            }
            __builtin_amdgcn_sched_group_barrier(0x008, kQkAhead, 0);
        }
    };

    // online softmax of one tile (per query row = per lane); leaves P^T packed to fp16 in pf
    // mask_sides: bit 0 = some row of the wave has its first allowed key inside or after this tile, bit 1 = some row
    // has its last allowed key inside or before it (both wave-uniform)
    auto softmax = [&](int mask_sides, int kb0, v16f (&s)[2][NB], v8h (&pf)[2][2][NB]) {
        constexpr bool folded = kFoldAlibi;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            // folded ALiBi: bias of 32-key block kb that is common to the lane's 16 scores there (score units)
            float abias[2] = {0.0f, 0.0f};
            if constexpr (folded) {
                abias[0] = nsig * (iif[nb] - (float)(kb0 + 4 * g));
                abias[1] = abias[0] - nsig * 32.0f;
            }
            if constexpr (kAlibi && !folded) {
                // score*scale - slope*|i - j|  (src/main.cu:315,324), in the log2 domain
                const float jb = (float)(kb0 + 4 * g) - iif[nb];
                if (scale_late) {
#pragma unroll
                    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                        for (int r = 0; r < 16; ++r)
                            s[kb][nb][r] = __builtin_fmaf(nsig, __builtin_fabsf(jb + (float)(32 * kb + 8 * (r >> 2) + (r & 3))), s[kb][nb][r]);
                } else {
#pragma unroll
                    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                        for (int r = 0; r < 16; ++r)
                            s[kb][nb][r] = s[kb][nb][r] * c2 - slope2 * __builtin_fabsf(jb + (float)(32 * kb + 8 * (r >> 2) + (r & 3)));
                }
            }
            if (mask_sides != 0) {
                // Wave-uniform and rare (boundary tiles only); the masking itself is inline asm (common.h), which keeps
                // these real branches.  The bounds of the wave's rows run along block diagonals when they move by one
                // key per row and start at a multiple of 32 (causal masks and windows whose offsets are multiples of 32,
                // rows not clipped by a sequence or split end): then lane-mask constants per 32-key block do the
                // masking; otherwise a tile takes one comparison per score and crossed end of the interval.
                const float ninf = -INFINITY;
                const bool hi_diag = NB == 1 && hi_max - hi_min == 31 && (hi_min & 31) == 0;
                const bool lo_diag = NB == 1 && lo_max - lo_min == 31 && (lo_min & 31) == 0;
                if (((mask_sides & 1) == 0 || lo_diag) && ((mask_sides & 2) == 0 || hi_diag)) {
#pragma unroll
                    for (int kb = 0; kb < 2; ++kb) {
                        // last / first visible key of the wave's first row relative to the block: multiples of 32
                        const int dh = (mask_sides & 2) ? hi_min - (kb0 + 32 * kb) : 64;
                        const int dl = (mask_sides & 1) ? lo_min - (kb0 + 32 * kb) : -64;
                        if (dh < 0 || dl >= 32) {
                            mask_whole_block(s[kb][nb], ninf);
                        } else {
                            if (dh == 0) mask_off_diagonal<true>(s[kb][nb], ninf);
                            if (dl == 0) mask_off_diagonal<false>(s[kb][nb], ninf);
                        }
                    }
                } else {
                    const int lo_rel = lo[nb] - kb0 - 4 * g, hi_rel = hi[nb] - kb0 - 4 * g;
#pragma unroll
                    for (int kb = 0; kb < 2; ++kb) {
                        if (mask_sides & 1) mask_beyond<false>(s[kb][nb], lo_rel - 32 * kb, ninf);
                        if (mask_sides & 2) mask_beyond<true>(s[kb][nb], hi_rel - 32 * kb, ninf);
                    }
                }
            }
            if constexpr (kEvery) {
                if (a.scores_out != nullptr && row_i[nb] < Nq) {  // debug dump of the visible scores, natural-log units
                    float* srow = a.scores_out + ((size_t)bh * Nq + row_i[nb]) * Nk;
                    const float unit = (scale_late ? cs : 1.0f) * kLn2;
#pragma unroll
                    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                        for (int r = 0; r < 16; ++r) {
                            const int j = kb0 + 4 * g + 32 * kb + 8 * (r >> 2) + (r & 3);
                            if (j >= lo[nb] && j <= hi[nb]) srow[j] = s[kb][nb][r] * unit;
                        }
                }
            }
            float mx = -INFINITY;
            if constexpr (folded) {
                float mk[2] = {-INFINITY, -INFINITY};
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int r = 0; r < 16; ++r) mk[kb] = fmaxf(mk[kb], s[kb][nb][r]);
                mx = fmaxf(mk[0] + abias[0], mk[1] + abias[1]);
            } else {
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[kb][nb][r]);
            }
            mx = xhalf_max(mx);
            mx *= cs;  // cs > 0
            if (__builtin_amdgcn_ballot_w64(mx > m_ref[nb] + kLazyTau) != 0ull) {
                const float m_new = fmaxf(m_ref[nb], mx);
                float alpha = (m_new == -INFINITY) ? 1.0f : fast_exp2(m_ref[nb] - m_new);
                asm volatile("; raise running max" : "+v"(alpha));  // keeps the rescale inside this rare branch
                m_ref[nb] = m_new;
                l_run[nb] *= alpha;
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                    for (int r = 0; r < 16; ++r) oacc[mb][nb][r] *= alpha;
            }
            const float m_use = (m_ref[nb] == -INFINITY) ? 0.0f : m_ref[nb];  // nothing seen yet: exp2(-inf - 0) = 0
            float rs = 0.0f;
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
                const float addend = folded ? __builtin_fmaf(abias[kb], cs, -m_use) : -m_use;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const float p = fast_exp2(__builtin_fmaf(s[kb][nb][r], cs, addend));
                    rs += p;
                    s[kb][nb][r] = p;
                }
            }
            l_run[nb] += rs;  // per-lane partial; the two half-waves are added in the epilogue
            if constexpr (kDropout) {
                // drop iff field < threshold, row sum left undropped (src/flash_forward.h:221-237); the survivors' factor
                // 1/(1-p) is common to the whole row and multiplies O once in the epilogue instead of every score here
                const uint32_t i_u = (uint32_t)row_i[nb];
                // first-round Philox product of the head-slice word: the same for the whole work-group, so a scalar multiply
                const uint64_t bh_prod = (uint64_t)0xCD9E8D57u * (uint64_t)(uint32_t)bh;
                const uint32_t bh_hi = (uint32_t)(bh_prod >> 32), bh_lo = (uint32_t)bh_prod;
                uint8_t* kout = a.keep_out ? a.keep_out + ((size_t)bh * Nq + row_i[nb]) * Nk : nullptr;
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int q = 0; q < 2; ++q) {
                        // the lane's eight keys among the 16 from jg on: field f belongs to key jg + 8*(f>>2) + 4*g + (f&3)
                        const int jg = kb0 + 32 * kb + 16 * q;
                        const v4u w = philox4x32_10_c2(dropout_call((uint32_t)(jg + 4 * g)), i_u, bh_hi, bh_lo, a.off_lo, a.seed_lo, a.seed_hi);
                        if constexpr (!kEvery) {
                            // registers 8q + 2k and 8q + 2k + 1 become one packed fp16 word, fields 2k and 2k + 1 are the
                            // halves of Philox word k: the decisions are applied to the packed word (keep_pair)
#pragma unroll
                            for (int k = 0; k < 4; ++k) {
                                union { v2h h; uint32_t u; } pk;
                                pk.h = pack_f16(s[kb][nb][8 * q + 2 * k], s[kb][nb][8 * q + 2 * k + 1]);
                                pk.u = keep_pair(pk.u, w[k], a.drop_sub2);
                                pf[kb][q][nb][2 * k] = pk.h[0];
                                pf[kb][q][nb][2 * k + 1] = pk.h[1];
                            }
                        } else {
#pragma unroll
                            for (int f = 0; f < 8; ++f) {
                                const int r = 8 * q + f;
                                s[kb][nb][r] = philox_field16(w, f) >= a.drop_thr ? s[kb][nb][r] : 0.0f;
                            }
                        }
                        if (a.keep_out != nullptr) {  // debug dump: one uniform branch per call, none per score
#pragma unroll
                            for (int f = 0; f < 8; ++f) {
                                const int j = jg + 8 * (f >> 2) + 4 * g + (f & 3);
                                if (row_i[nb] < Nq && j < Nk) kout[j] = philox_field16(w, f) >= a.drop_thr ? 1 : 0;
                            }
                        }
                    }
            }
            if constexpr (!(kDropout && !kEvery)) {  // (there the dropout step has packed them already)
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int tt = 0; tt < 2; ++tt)
#pragma unroll
                        for (int e = 0; e < 8; e += 2) {
                            const v2h h2 = pack_f16(s[kb][nb][8 * tt + e], s[kb][nb][8 * tt + e + 1]);
                            pf[kb][tt][nb][e] = h2[0];
                            pf[kb][tt][nb][e + 1] = h2[1];
                        }
            }
        }
    };

    // O^T += V^T P^T with the tile in V buffer `buf`
    auto pv = [&](int buf, v8h (&pf)[2][2][NB]) {
        // (a lane's rows all share bit 1 of the row index: the swizzle is one per-lane choice between two bases)
        const char* const vb[2] = {Vs + buf * C::VBUF + v_rd + v_sw, Vs + buf * C::VBUF + v_rd + (v_sw ^ (C::VSWZ ? 64 : 0))};
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
            for (int tt = 0; tt < 2; ++tt) {
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) {
                    const char* p0 = C::VSWZ ? vb[mb & 1] + (32 * kb + 16 * tt) * SV + (mb >> 1) * 128
                                             : vb[0] + (32 * kb + 16 * tt) * SV + mb * 64;
                    union { v4hp p[2]; v8h v; } af;
                    af.p[0] = __builtin_amdgcn_ds_read_tr16_b64_v4f16((FA_LDS v4hp*)(p0));
                    af.p[1] = __builtin_amdgcn_ds_read_tr16_b64_v4f16((FA_LDS v4hp*)(p0 + 8 * SV));
#pragma unroll
                    for (int nb = 0; nb < NB; ++nb)
                        oacc[mb][nb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af.v, pf[kb][tt][nb], oacc[mb][nb], 0, 0, 0);
                }
            }
        }
    };

    // The Q fragments must have landed before the loop starts: a load still counted as outstanding at the loop
    // header makes the compiler guard every use of qf inside the loop with a vmcnt wait, and since vmcnt counts in
    // order, that wait would also drain the K/V prefetch of the same iteration.
    auto pin_q = [&]() {
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) asm volatile("" : "+v"(qf[nb][ks]));
    };

    // ---- loop over the key tiles
    // A wave whose rows all lie past Nq (fewer than 128 query rows: short prompts, or the heads of one K/V head decoding
    // together) only helps to stage the tiles, and so does any wave for a tile that none of its rows can see (the far
    // end of the causal diagonal block, the near end of a sliding window).
    const bool wave_live = q0 + wave_row0 < Nq;
    auto tile_math = [&](int t, int buf) {
        const int kb0 = (tile_begin + t) * BC;
        if (wave_live && kb0 <= hi_max && kb0 + BC - 1 >= lo_min) {
            v16f s[2][NB];
            v8h pf[2][2][NB];
            const int mask_sides = (kb0 < lo_max ? 1 : 0) | (kb0 + BC - 1 > hi_min ? 2 : 0);
            qk(buf, s);
            softmax(mask_sides, kb0, s, pf);
            pv(buf, pf);
        }
    };
    if constexpr (kNarrow) {
        // Wave w walks the tiles w, w + 4, ... with two stages of its own: tile n + 2 is requested into the stage of
        // tile n as soon as that tile's fragments have been read, and before tile n + 1 is touched its requests (older
        // than those of tile n + 2) have been waited for.  No other wave reads or writes these buffers.
        const int nt = wave < ntiles ? (ntiles - wave + 3) / 4 : 0;
        static_assert(NKX + NVX <= 63, "vmcnt immediate");
#pragma unroll
        for (int u = 0; u < NSTG; ++u)
            if (u < nt) dma_tile(tile_begin + wave + 4 * u, u);
        read_slope();
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        pin_q();
        if constexpr (NSTG == 2) {
            int buf = 0;
            for (int n = 0; n < nt; ++n) {
                tile_math(wave + 4 * n, buf);
                if (n + 2 < nt) {
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the stage has been read
                    dma_tile(tile_begin + wave + 4 * (n + 2), buf);
                    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NKX + NVX) : "memory");
                } else {
                    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                }
                buf ^= 1;
            }
        } else {
            // One stage: K(n + 1) is requested as soon as the scores of tile n are out of the K buffer, V(n + 1) as soon
            // as the V buffer has been read; each is waited for right before its first use, the younger request of the
            // other tensor staying in flight.
            for (int n = 0; n < nt; ++n) {
                const int kb0 = (tile_begin + wave + 4 * n) * BC;
                const bool live = wave_live && kb0 <= hi_max && kb0 + BC - 1 >= lo_min;
                const bool more = n + 1 < nt;
                v16f s[2][NB];
                v8h pf[2][2][NB];
                if (live) qk(0, s);
                if (more) {
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                    dma_tile_parts(tile_begin + wave + 4 * (n + 1), 0, std::true_type{}, std::false_type{});
                }
                if (live) softmax((kb0 < lo_max ? 1 : 0) | (kb0 + BC - 1 > hi_min ? 2 : 0), kb0, s, pf);
                // V(n): older than the K request just issued
                if (more) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NKX) : "memory");
                else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                if (live) pv(0, pf);
                if (more) {
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                    dma_tile_parts(tile_begin + wave + 4 * (n + 1), 0, std::false_type{}, std::true_type{});
                    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NVX) : "memory");  // K(n + 1) is there
                }
            }
        }
    } else if constexpr (kDma) {
        // Tile t + PF is requested when tile t starts (its stage was read last during tile t - 1, behind a barrier);
        // before the barrier that ends tile t, the requests of tile t + 1 have landed, those of t + 2 may be in flight.
        // Before tile 0 every stage is free: the prologue requests one tile per stage, so that the request which
        // tile 0 would issue is already on its way (a work-group with few tiles otherwise pays the memory latency a
        // second time at the end of its first tile).
        constexpr int PF = NSTG - 1;
        static_assert(PF == 1 || PF == 2, "prefetch distance");
        static_assert(NKX + NVX <= 63, "vmcnt immediate");
#pragma unroll
        for (int u = 0; u < NSTG; ++u)
            if (u < ntiles) dma_tile(tile_begin + u, u);
        read_slope();
        stamps.take(1);
        dma_wait(false);
        pin_q();
        stamps.take(2);
        __syncthreads();
        stamps.take(3);
        int buf = 0, nbuf = PF % NSTG;  // stages of tile t and of tile t + PF
        for (int t = 0; t < ntiles; ++t) {
            const bool more = t + PF < ntiles;
            if (more && t > 0) dma_tile(tile_begin + t + PF, nbuf);
            tile_math(t, buf);
            if (kStamp && t == 0) stamps.take(4);
            dma_wait(PF == 2 && more);
            __syncthreads();
            buf = buf + 1 == NSTG ? 0 : buf + 1;
            nbuf = nbuf + 1 == NSTG ? 0 : nbuf + 1;
        }
    } else {
        // double-buffered through registers: tile t+1 is fetched from global memory while tile t is computed
        if (ntiles > 0) {
            gload(Kbh, tile_begin, kreg);
            gload(Vbh, tile_begin, vreg);
        }
        read_slope();
        if (ntiles > 0) {
            stamps.take(1);
            put_k(0);
            put_v(0);
        }
        pin_q();
        stamps.take(2);
        __syncthreads();
        stamps.take(3);
        for (int t = 0; t < ntiles; ++t) {
            const int cur = t & 1;
            const bool has1 = t + 1 < ntiles;
            if (has1) {
                gload(Kbh, tile_begin + t + 1, kreg);
                gload(Vbh, tile_begin + t + 1, vreg);
            }
            tile_math(t, cur);
            if (kStamp && t == 0) stamps.take(4);
            if (has1) {
                put_k(cur ^ 1);
                put_v(cur ^ 1);
            }
            __syncthreads();
        }
    }

    if constexpr (kNarrow) {
        // ---------------- merge of the four waves' partial results (same rows, disjoint keys), then O and LSE.
        // Like the combine of split partials: weights 2^(m_w - M) on the row sums and on the unnormalised O.
        __syncthreads();  // every wave is done with its tile buffers
        float* const sm = reinterpret_cast<float*>(smem);  // [4][32] running maxima (log2 units)
        float* const sl = sm + 4 * 32;                      // [4][32] row sums
        float* const so = sl + 4 * 32;                      // [4][32][D] unnormalised O, by chunk position
        static_assert((2 * 4 * 32 + 4 * 32 * D) * 4 <= 4 * kWaveLds, "merge buffers fit the tile buffers");
        const float l = xhalf_sum(l_run[0]);
        if (g == 0) {
            sm[wave * 32 + l32] = m_ref[0];
            sl[wave * 32 + l32] = l;
        }
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int rg = 0; rg < 4; ++rg) {
                const v4f o = {oacc[mb][0][4 * rg], oacc[mb][0][4 * rg + 1], oacc[mb][0][4 * rg + 2], oacc[mb][0][4 * rg + 3]};
                *reinterpret_cast<v4f*>(so + (wave * 32 + l32) * D + 32 * mb + 8 * rg + 4 * g) = o;
            }
        __syncthreads();
        // thread -> one row and D / 8 consecutive chunk positions of it
        constexpr int CPT = D / 8;
        const int row = tid >> 3, cp0 = (tid & 7) * CPT;
        float M = -INFINITY;
#pragma unroll
        for (int w = 0; w < 4; ++w) M = fmaxf(M, sm[w * 32 + row]);
        const float Mu = (M == -INFINITY) ? 0.0f : M;
        float L = 0.0f, wgt[4];
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            wgt[w] = fast_exp2(sm[w * 32 + row] - Mu);
            L += wgt[w] * sl[w * 32 + row];
        }
        const float inv = L > 0.0f ? (kDropout ? a.drop_rscale : 1.0f) / L : 0.0f;
        const int gi = q0 + row;
        if (gi < Nq) {
            half_t* const op = a.O + ((size_t)bh * Nq + gi) * d;
            const int cfull = d & ~7, rem = d & 7;
#pragma unroll
            for (int c = 0; c < CPT; ++c) {
                const int cc = cp0 + c;
                float o = 0.0f;
#pragma unroll
                for (int w = 0; w < 4; ++w) o = __builtin_fmaf(wgt[w], so[(w * 32 + row) * D + cc], o);
                // column of chunk position cc: behind the row's whole chunks sit the columns d - 8 ... d - 1, of which
                // the first 8 - d % 8 belong to the positions before
                const int col = kFullD || cc < cfull ? cc : cc - (8 - rem);
                const bool ok = kFullD || cc < cfull || (rem != 0 && cc < cfull + 8 && col >= cfull);
                if (ok) op[col] = (half_t)(o * inv);
            }
            if ((tid & 7) == 0)
                a.LSE[(size_t)bh * Nq + gi] = L > 0.0f ? __builtin_fmaf(M, kLn2, fast_log2(L) * kLn2) : -INFINITY;
        }
        return;
    }

    // ---------------- epilogue: normalise once, store O (fp16) + LSE, or the fp32 split partials
    stamps.take(5);
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
        const float l = xhalf_sum(l_run[nb]);
        const float inv = l > 0.0f ? (kDropout ? a.drop_rscale : 1.0f) / l : 0.0f;
        const float lse = l > 0.0f ? __builtin_fmaf(m_ref[nb], kLn2, fast_log2(l) * kLn2) : -INFINITY;  // (one rounding at the size of m)
        const int i = row_i[nb];
        if (i >= Nq) continue;
        if (a.num_splits > 1) {
            const size_t prow = ((size_t)bh * a.num_splits + split) * Nq + i;
            if (g == 0) a.LSE_partial[prow] = lse;
            float* op = a.O_partial + prow * d;
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int rg = 0; rg < 4; ++rg) {
                    const int dc = 32 * mb + 8 * rg + 4 * g;
                    if (kVec) {
                        if (kFullD || dc < d) {
                            v4f o = {oacc[mb][nb][4 * rg] * inv, oacc[mb][nb][4 * rg + 1] * inv,
                                     oacc[mb][nb][4 * rg + 2] * inv, oacc[mb][nb][4 * rg + 3] * inv};
                            *reinterpret_cast<v4f*>(op + dc) = o;
                        }
                    } else if (!kEvery || d >= 8) {
                        // rows at any alignment: the chunk position behind the row's whole chunks holds columns d - 8 ... d - 1
                        const int c0 = d & ~7, rem = d & 7;
                        if (dc < c0 || (rem != 0 && dc < c0 + 8)) {
                            v4f o = {oacc[mb][nb][4 * rg] * inv, oacc[mb][nb][4 * rg + 1] * inv,
                                     oacc[mb][nb][4 * rg + 2] * inv, oacc[mb][nb][4 * rg + 3] * inv};
                            *reinterpret_cast<v4f_anyalign*>(op + (dc < c0 ? dc : dc - (8 - rem))) = o;
                        }
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            if (dc + e < d) op[dc + e] = oacc[mb][nb][4 * rg + e] * inv;
                    }
                }
        } else {
            if (g == 0) a.LSE[(size_t)bh * Nq + i] = lse;
            if (kEvery && d < 8) {
                half_t* op = a.O + ((size_t)bh * Nq + i) * d;
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                    for (int rg = 0; rg < 4; ++rg) {
                        const int dc = 32 * mb + 8 * rg + 4 * g;
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            if (dc + e < d) op[dc + e] = (half_t)(oacc[mb][nb][4 * rg + e] * inv);
                    }
            }
        }
    }
    if (!kEvery || d >= 8) {
        if (a.num_splits == 1) {
            // A lane holds 4 consecutive head-dim columns of one row at a time, which as a direct
            // store would be 32 rows x 8 bytes per instruction.  The wave's 32 x d block goes through LDS instead (the tile
            // buffers are free behind the last barrier; rows padded by 16 bytes) and leaves in consecutive 16-byte pieces
            // of whole rows.  The stores are non-temporal: O is not read again by this launch, and lines left dirty in L2
            // would only be written back when the kernel ends.
            constexpr int SO = 2 * D + 16;
            static_assert(4 * NB * 32 * SO <= C::SMEM, "O staging fits the tile buffers");
            char* const ost = smem + wave * (NB * 32 * SO);
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                const float l = xhalf_sum(l_run[nb]);
                const float inv = l > 0.0f ? (kDropout ? a.drop_rscale : 1.0f) / l : 0.0f;
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                    for (int rg = 0; rg < 4; ++rg) {
                        v4h o = {(half_t)(oacc[mb][nb][4 * rg] * inv), (half_t)(oacc[mb][nb][4 * rg + 1] * inv),
                                 (half_t)(oacc[mb][nb][4 * rg + 2] * inv), (half_t)(oacc[mb][nb][4 * rg + 3] * inv)};
                        *reinterpret_cast<v4h*>(ost + (nb * 32 + l32) * SO + (32 * mb + 8 * rg + 4 * g) * 2) = o;
                    }
            }
            char* const Ob = reinterpret_cast<char*>(a.O + (size_t)bh * Nq * d);
            constexpr int NP = NB * 32 * CH;  // 16-byte pieces of the wave's block, CH per row
#pragma unroll
            for (int p0 = 0; p0 < NP; p0 += 64) {
                const int p = p0 + lane;
                const int rl = p / CH, ch = p % CH;
                const int gi = q0 + wave * C::RW + rl;
                if (p < NP && gi < Nq && (kFullD || ch * 8 < d)) {
                    const v4u piece = *reinterpret_cast<const v4u*>(ost + rl * SO + ch * 16);
                    if constexpr (kVec)
                        __builtin_nontemporal_store(piece, reinterpret_cast<v4u*>(Ob + (size_t)gi * d * 2 + ch * 16));
                    else  // rows at any alignment: the last chunk position holds the row's last 16 bytes
                        __builtin_nontemporal_store(piece, reinterpret_cast<v4u_anyalign*>(Ob + (size_t)gi * d * 2 + (ch * 8 + 8 <= d ? ch * 16 : (d - 8) * 2)));
                }
            }
        }
    }
    if constexpr (kStamp) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the result stores of this wave have left
        stamps.take(6);
        stamps.store(a.stamps, ntiles);
    }
}

// Launcher of one head-dim bucket, defined in fwd_d{32,64,96,128}.hip.
// variant bits: kVarVec (d % 8 == 0), kVarAlibi, kVarDropout; kVarFullD is derived here (d == bucket width).
int launch_fwd_d32(const FwdArgs& a, int variant, int nb, hipStream_t st);
int launch_fwd_d64(const FwdArgs& a, int variant, int nb, hipStream_t st);
int launch_fwd_d96(const FwdArgs& a, int variant, int nb, hipStream_t st);
int launch_fwd_d128(const FwdArgs& a, int variant, int nb, hipStream_t st);
// whether launch_fwd_d128 takes the 8-wave kernel (256 query rows per work-group instead of 128)
// (slices = B * H * num_splits; hint = flash_params::kernel_hint)
bool fwd_uses_pingpong(int d, bool direct, int Nq, int Nk, int causal, int wl, int wr, long long slices, int hint);

// Head slices per chunk of the work-group order: the smallest divisor of the slice count (a multiple of 8, which keeps a
// slice on one XCD) whose chunk still holds twice the work-groups that run at once -- enough for "heaviest row blocks
// first" to balance the tail of a chunk; all slices when there is no such divisor below the slice count.
// Measured on causal + dropout B8 H32 N1000 d96 (256 slices, 8 row blocks, 512 work-groups at once): chunks of 128
// slices +3-5 %; 64: +-0; 32: -2 %; 16: -9 %; 96 and 192 (a ragged last chunk): -1 %.  With this rule, against all
// slices in one chunk: causal B16 H32 N1024 d128 +5 %, B8 H32 N2048 d64 +4 %, B8 H32 N4096 d128 (8-wave kernel) +16 %;
// once or four times the resident work-groups per chunk instead of twice: 0 ... -4 %.
constexpr int kNumCus = 256;  // MI355X
inline int slice_chunk_for(int slices, int groups_per_slice, int resident, int step = 8)
{
    if (slices <= 0 || groups_per_slice <= 0) return 1;
    const long long want = (2LL * resident + groups_per_slice - 1) / groups_per_slice;
    for (long long c = (want + step - 1) / step * step; c < slices; c += step)
        if (slices % c == 0) return (int)c;
    return slices;
}

// slice_chunk and group_xcd of a launch: with grouped K/V heads the chunks are multiples of 8 G slices where the slice
// count allows, so that the heads of a K/V head can share an XCD (slice_of_position)
inline void set_slice_order(FwdArgs& b, int groups_per_slice, int resident)
{
    const int slices = b.B * b.H;
    b.group_xcd = 0;
    if (b.kv_group > 1 && slices % (8 * b.kv_group) == 0) {
        b.slice_chunk = slice_chunk_for(slices, groups_per_slice, resident, 8 * b.kv_group);
        if (b.slice_chunk % (8 * b.kv_group) == 0) b.group_xcd = b.kv_group;
    } else {
        b.slice_chunk = slice_chunk_for(slices, groups_per_slice, resident);
    }
}

template <int D, int NB, int VAR>
inline hipError_t launch_fwd_instance(const FwdArgs& a, hipStream_t st)
{
    using C = FwdCfg<D, NB>;
    auto kern = fwd_kernel<D, NB, VAR>;
    static DeviceFlags attr_done;  // per instantiation and device
    constexpr int smem = C::SMEM_DMA > C::SMEM ? C::SMEM_DMA : C::SMEM;  // (equal: both paths use two stages)
    if (hipError_t e = ensure_dynamic_lds(reinterpret_cast<const void*>(kern), smem, attr_done); e != hipSuccess) return e;
    const long long groups = (long long)a.Tr * a.B * a.H * a.num_splits;
    FwdArgs b = a;
    constexpr int kResident = (NB == 1 ? fwd_groups_per_cu(D, NB, VAR) : 2) * kNumCus;
    set_slice_order(b, a.Tr * a.num_splits, kResident);
    b.split_rotate = split_rotate_for(b.num_splits, b.slice_chunk);
    b.snake_end = snake_end_for(groups, kResident);
    return launch_kernel(kern, dim3((unsigned)groups), dim3(256), smem, st, b);
}

// The instances of a bucket: {d == bucket, d % 8 == 0} x {plain, ALiBi, ALiBi with every visible key at or left of its
// row, dropout, both}, for rows at any alignment (d % 8 != 0) {plain, ALiBi, dropout, both}, and the one that serves
// every other request.  ST = kVarStamp selects their instrumented twins (debug time stamps).
// The narrow instances (kNarrow in fwd_kernel): unsplit launches that would
// occupy at most half the CUs with work-groups of 128 rows, each of them with 16 key tiles or more ahead of it (8 where
// they occupy a quarter of the CUs).  Measured against the 128-row instances, same box: B1 H8 N1021 d31 (the reference's
// own run) 14.2 -> 11.8 us, B1 H8 N1024 d64 15.0 -> 10.2, B1 H8 N2048 d64 causal 27.3 -> 17.8, B1 H1 N2048 d32 causal
// 22.2 -> 10.5, B1 H4 N4096 d64 50.1 -> 38.0, B1 H8 N1024 d128 20.9 -> 14.3; with 128 work-groups of 8 tiles (B1 H32
// N512 d64) 10.3 -> 11.8, hence the limit.
inline bool fwd_uses_narrow(const FwdArgs& a, int variant, bool every)
{
    if (every || a.num_splits != 1 || a.stamps != nullptr || a.kernel_hint != 0) return false;
    const long long groups = (long long)a.B * a.H * ((a.Nq + 127) / 128);
    if (2 * groups > kNumCus) return false;
    // (above d = 64 a wave has one LDS stage and waits for most of every tile request: rows shorter than the bucket,
    // whose requests take longer, measured slower than the 128-row instances there, and so did launches of more 32-row
    // work-groups than CUs unless causal -- B2 H2 Nq4096 Nk1024 d128 25.6 against 20.9 us, the same causal shapes 39.5
    // against 69.0 us)
    if (a.d > 64 && (a.d % 32 != 0 || (!a.causal && (long long)a.B * a.H * ((a.Nq + 31) / 32) > kNumCus))) return false;
    const int keys = 4 * groups <= kNumCus ? 512 : 1024;  // visible keys per row that make the chain worth cutting
    return a.Nk >= keys && (a.wl < 0 || a.wl >= keys - 64);
}

template <int D, int VAR>
inline hipError_t launch_fwd_narrow_instance(const FwdArgs& a, hipStream_t st)
{
    using C = FwdCfg<D, 1>;
    auto kern = fwd_kernel<D, 1, VAR | kVarNarrow>;
    static DeviceFlags attr_done;  // per instantiation and device
    constexpr int smem = 4 * (D <= 64 ? 2 : 1) * (C::KBUF + C::VBUF);  // two stages per wave up to D = 64, one above
    if (hipError_t e = ensure_dynamic_lds(reinterpret_cast<const void*>(kern), smem, attr_done); e != hipSuccess) return e;
    FwdArgs b = a;
    b.Tr = (a.Nq + 31) / 32;
    const long long groups = (long long)b.Tr * a.B * a.H;
    set_slice_order(b, b.Tr, kNumCus);
    b.split_rotate = 0;
    b.snake_end = snake_end_for(groups, kNumCus);
    return launch_kernel(kern, dim3((unsigned)groups), dim3(256), smem, st, b);
}

// requests that only the instance which serves every request takes (kEvery in fwd_kernel)
inline bool fwd_needs_every_instance(const FwdArgs& a, int variant)
{
    return a.scale_log2 <= 0.0f || a.scores_out != nullptr || a.d < 8 || ((variant & kVarDropout) && a.drop_thr == 0);
}

template <int D, int NB, int ST>
inline int launch_fwd_bucket_st(const FwdArgs& a, int variant, hipStream_t st)
{
    hipError_t e;
    const int feat = variant & (kVarAlibi | kVarDropout);
    constexpr int AL = kVarAlibi | kVarAlibiLeft;  // ALiBi with no visible key right of its row
    if constexpr (ST == 0) {
        if (fwd_uses_narrow(a, variant, fwd_needs_every_instance(a, variant))) {
            // plain: by row length like the others; with ALiBi or dropout: up to d = 64 the instances for rows at any
            // alignment, which serve every row length from eight elements on, above the ones for rows of the bucket's
            // width (the only rows that come here)
            constexpr int F = D <= 64 ? 0 : kVarVec | kVarFullD;
            if (feat == kVarAlibi) return (int)launch_fwd_narrow_instance<D, F | kVarAlibi>(a, st);
            if (feat == kVarDropout) return (int)launch_fwd_narrow_instance<D, F | kVarDropout>(a, st);
            if (feat != 0) return (int)launch_fwd_narrow_instance<D, F | kVarAlibi | kVarDropout>(a, st);
            if (a.d == D) return (int)launch_fwd_narrow_instance<D, kVarVec | kVarFullD>(a, st);
            if constexpr (D <= 64) {  // (above, only rows of the bucket's width come here)
                if (!(variant & kVarVec)) return (int)launch_fwd_narrow_instance<D, 0>(a, st);
                return (int)launch_fwd_narrow_instance<D, kVarVec>(a, st);
            }
        }
    }
    if (!(variant & kVarVec)) {
        // rows at any alignment: plain, ALiBi, dropout, both, and one more with both features compiled in (slope 0 /
        // threshold 0 make them identities) for every other request: a non-positive scale (its ALiBi step is where the
        // scores are scaled ahead of the row maximum), the score dump, rows of fewer than eight elements, a dropout
        // threshold of 0
        if (fwd_needs_every_instance(a, variant)) e = launch_fwd_instance<D, NB, ST | kVarAlibi | kVarDropout | kVarEvery>(a, st);
        else if (feat == 0) e = launch_fwd_instance<D, NB, ST>(a, st);
        else if (feat == kVarAlibi) e = launch_fwd_instance<D, NB, ST | kVarAlibi>(a, st);
        else if (feat == kVarDropout) e = launch_fwd_instance<D, NB, ST | kVarDropout>(a, st);
        else e = launch_fwd_instance<D, NB, ST | kVarAlibi | kVarDropout>(a, st);
    } else if (a.d == D) {
        constexpr int V = ST | kVarVec | kVarFullD;
        const bool kv_once = ST == 0 && a.Tr == 1 && a.kv_group == 1;
        if (feat == 0) e = kv_once ? launch_fwd_instance<D, NB, V | (ST == 0 ? kVarKvOnce : 0)>(a, st) : launch_fwd_instance<D, NB, V>(a, st);
        else if (feat == kVarAlibi) e = a.alibi_left ? launch_fwd_instance<D, NB, V | AL>(a, st) : launch_fwd_instance<D, NB, V | kVarAlibi>(a, st);
        else if (feat == kVarDropout) e = launch_fwd_instance<D, NB, V | kVarDropout>(a, st);
        else e = a.alibi_left ? launch_fwd_instance<D, NB, V | AL | kVarDropout>(a, st) : launch_fwd_instance<D, NB, V | kVarAlibi | kVarDropout>(a, st);
    } else {
        constexpr int V = ST | kVarVec;
        if (feat == 0) e = launch_fwd_instance<D, NB, V>(a, st);
        else if (feat == kVarAlibi) e = a.alibi_left ? launch_fwd_instance<D, NB, V | AL>(a, st) : launch_fwd_instance<D, NB, V | kVarAlibi>(a, st);
        else if (feat == kVarDropout) e = launch_fwd_instance<D, NB, V | kVarDropout>(a, st);
        else e = a.alibi_left ? launch_fwd_instance<D, NB, V | AL | kVarDropout>(a, st) : launch_fwd_instance<D, NB, V | kVarAlibi | kVarDropout>(a, st);
    }
    return (int)e;
}

template <int D, int NB>
inline int launch_fwd_bucket(const FwdArgs& a, int variant, hipStream_t st)
{
    return a.stamps ? launch_fwd_bucket_st<D, NB, kVarStamp>(a, variant, st) : launch_fwd_bucket_st<D, NB, 0>(a, variant, st);
}

}  // namespace fa
