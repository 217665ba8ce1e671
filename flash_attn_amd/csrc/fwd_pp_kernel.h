// Ping-pong variant of the tiled forward kernel for the head-dim bucket 128 (96 < d <= 128; rows shorter than 128 elements
// and rows at any 2-byte alignment as in fwd_kernel.h: chunk positions behind a row's whole chunks hold its last 16 bytes).
//
// Same math as fwd_kernel.h (S^T = K Q^T and O^T += V^T P^T on MFMA 32x32x16, Q in registers, online softmax per
// lane, 64-key tiles).  What changes is the schedule and the way tiles reach LDS:
//
//  * One work-group = 8 waves = 256 query rows and fills a CU: every SIMD hosts two of its waves (w and w+4).
//  * Each wave alternates between a VALU phase, softmax(S(t)) -> P(t), and an MFMA phase, O += P(t) V(t) followed by
//    S(t+1) = K(t+1) Q^T.  Waves 0-3 and waves 4-7 run half an iteration apart: the second group passes one extra
//    barrier before the loop, and every phase ends in a work-group barrier.  So on every SIMD one wave is in its MFMA
//    phase while the other is in its VALU phase.  (Two independent 4-wave groups per CU do not interleave this way
//    by themselves: measured MFMA / VALU co-execution was 11 % of the time.)
//  * Tiles go from global memory straight into LDS (global_load_lds_dwordx4: 64 lanes write one contiguous KiB, each
//    lane fetching 16 bytes from its own global address): no staging registers, no ds_write.  A stage holds its tile
//    row-major with the 16-byte chunks of every row permuted (exclusive-or with low bits of the row number), so that
//    a request covers four whole rows of global memory and the fragment reads (ds_read_b128 for K, ds_read_b64_tr_b16
//    for V) are free of bank conflicts; a fragment address is one base register ^ constant plus an immediate.
//    Q and O go through 8 KiB of wave-private LDS in the same layout, for the same reason (whole rows per request).
//  * Four LDS stages per tensor: V(t+2) is requested at the start of the VALU phase of iteration t and waited for (vmcnt)
//    at the end of its MFMA phase; K(t+3) is requested at the end of that MFMA phase and waited for at the end of the next
//    one.  With the half-iteration offset of the wave groups their slots (K(t-1), V(t-2)) were last read at least two
//    barriers before the request, and the first reader comes at least one barrier after the wait of the later group.
//  * Barriers wait for LDS traffic only; the first V fragment reads of a phase are issued before its barrier.
#pragma once
#include "fwd_kernel.h"

namespace fa {

template <int D>
struct PPCfg {
    static constexpr int kWaves = 8;
    static constexpr int BR = 32 * kWaves;    // query rows per work-group
    static constexpr int BC = 64;             // keys per tile
    static constexpr int KS = D / 16;
    static constexpr int MB = D / 32;
    static constexpr int KBUF = BC * D * 2;   // bytes per K stage (row-major, permuted chunks, no padding)
    static constexpr int VBUF = BC * D * 2;
    static constexpr int NST = 4;             // LDS stages per tensor
    static constexpr int XBUF = 16 * 1024;    // with the stages that are empty at start: 8 KiB per wave for its Q rows
    static constexpr int SMEM = NST * (KBUF + VBUF) + XBUF;
    static constexpr int NKL = (2 * KS) / 8;  // 1 KiB K blocks loaded per wave per tile
    static constexpr int NVL = (4 * MB) / 8;  // 1 KiB V blocks loaded per wave per tile
    static_assert(D == 64 || D == 128, "ping-pong kernel: head dim 64 or 128");
};

// LDS-only barrier: global loads in flight are not waited for.
// The sched_barrier fences keep the compiler from moving ALU work of one phase across the barrier into the other.
__device__ __forceinline__ void lds_barrier()
{
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
}

// Barrier between the VALU and the MFMA phase: LDS writes of this wave are done (they were issued before the reads
// that may still be in flight: LDS operations of a wave complete in order, so waiting until at most `kReads` operations
// are outstanding covers every write), the first V fragment reads stay in flight across the barrier.
template <int kReads>
__device__ __forceinline__ void lds_barrier_keep(void)
{
    static_assert(kReads == 8 || kReads == 12 || kReads == 16 || kReads == 4, "");
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (kReads == 16) asm volatile("s_waitcnt lgkmcnt(15)\n\ts_barrier" ::: "memory");
    else if constexpr (kReads == 12) asm volatile("s_waitcnt lgkmcnt(12)\n\ts_barrier" ::: "memory");
    else if constexpr (kReads == 8) asm volatile("s_waitcnt lgkmcnt(8)\n\ts_barrier" ::: "memory");
    else asm volatile("s_waitcnt lgkmcnt(4)\n\ts_barrier" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
}

template <int D, int VAR>
__global__ void __launch_bounds__(512, 2) fwd_pp_kernel(const FwdArgs a)
{
    constexpr bool kAlibi = (VAR & kVarAlibi) != 0, kDropout = (VAR & kVarDropout) != 0, kStamp = (VAR & kVarStamp) != 0,
                   kFullD = (VAR & kVarFullD) != 0;
    using C = PPCfg<D>;
    Stamps<kStamp> stamps;
    stamps.take(0);
    constexpr int BC = C::BC, KS = C::KS, MB = C::MB, NKL = C::NKL, NVL = C::NVL, NST = C::NST;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    FA_LDS char* const Ks = (FA_LDS char*)smem;
    FA_LDS char* const Vs = Ks + NST * C::KBUF;
    FA_LDS char* const Xs = Vs + NST * C::VBUF;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = wave_uniform(tid >> 6);
    const int grp = wave >> 2;  // waves w and w+4 share a SIMD and run half an iteration apart
    const int l32 = lane & 31;
    const int g = lane >> 5;

    // work-group -> (head slice, split, row block) as in fwd_kernel: slices fastest inside a chunk of a.slice_chunk
    // slices, heaviest row blocks first, chunk after chunk
    int bh, rest;
    {
        const int per_chunk = a.slice_chunk * a.Tr * a.num_splits;
        const int pos = work_position(blockIdx.x, a.snake_end);  // (one work-group per CU: the identity)
        const int ch = pos / per_chunk, w = pos % per_chunk;
        bh = ch * a.slice_chunk + slice_of_position(w % a.slice_chunk, a.group_xcd);
        rest = w / a.slice_chunk;
    }
    int mi;
    const int split = split_of_rest(rest, a.num_splits, a.split_rotate, &mi);
    const int m_block = a.Tr - 1 - mi;
    const int h = bh % a.H;
    const int Nq = a.Nq, Nk = a.Nk;
    const int d = kFullD ? D : a.d;  // 8 <= d <= D
    // byte offset of chunk position c inside a row of global memory
    auto chunk_offset = [&](int c) { return kFullD ? c * 16 : (c * 8 + 8 <= d ? c * 16 : (d - 8) * 2); };
    const int shift = Nk - Nq;
    const int q0 = m_block * C::BR;

    // ---- key range of the work-group (same pruning as fwd_kernel)
    int kmin = 0, kmax = Nk;
    {
        const int last_row = (q0 + C::BR - 1 < Nq ? q0 + C::BR - 1 : Nq - 1) + shift;
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
        store_empty_rows(a, bh, split, q0, q0 + C::BR < Nq ? q0 + C::BR : Nq, tid, 512);
        return;
    }

    // ---- this lane's query row and its interval of allowed keys
    // Row block of this wave: SIMD s hosts waves s and s + 4; giving them row blocks s and 7 - s evens out how long
    // each SIMD stays busy in the causal diagonal, where upper row blocks run out of visible keys first.
    const int rblk = wave < 4 ? wave : 11 - wave;
    const int row_i = q0 + rblk * 32 + l32;
    int lo, hi;
    float iif;
    {
        const int ii = (row_i < Nq ? row_i : Nq - 1) + shift;
        lo = 0;
        hi = Nk - 1;
        if (a.wl >= 0) lo = max(0, ii - a.wl);
        if (a.causal) hi = min(hi, ii);
        if (a.wr >= 0) hi = min(hi, ii + a.wr);
        if (a.num_splits > 1) {
            lo = max(lo, kmin);
            hi = min(hi, kmax - 1);
        }
        iif = (float)ii;
    }
    int lo_max, hi_min;  // wave-uniform: does a tile need the element test at all
    int lo_min, hi_max;  // wave-uniform: can a tile hold any visible key for this wave
    {
        const int first = q0 + rblk * 32, last = first + 31;
        const int iif_ = (first < Nq ? first : Nq - 1) + shift, iil_ = (last < Nq ? last : Nq - 1) + shift;
        lo_max = 0;
        hi_min = Nk - 1;
        if (a.wl >= 0) lo_max = max(0, iil_ - a.wl);
        if (a.causal) hi_min = min(hi_min, iif_);
        if (a.wr >= 0) hi_min = min(hi_min, iif_ + a.wr);
        if (a.num_splits > 1) {
            lo_max = max(lo_max, kmin);
            hi_min = min(hi_min, kmax - 1);
        }
        lo_min = 0;
        hi_max = Nk - 1;
        if (a.wl >= 0) lo_min = max(0, iif_ - a.wl);
        if (a.causal) hi_max = min(hi_max, iil_);
        if (a.wr >= 0) hi_max = min(hi_max, iil_ + a.wr);
    }

    const half_t* __restrict__ Qbh = a.Q + (size_t)bh * Nq * d;
    const int kvs = a.kv_slice(bh);
    const half_t* __restrict__ Kbh = a.K + (size_t)kvs * Nk * d;
    const half_t* __restrict__ Vbh = a.V + (size_t)kvs * Nk * d;

    // ---- Q fragments: fetched through LDS in the prologue below
    v8h qf[KS];

    // ---- direct global -> LDS tile loads.  A stage holds its 64-key tile row-major (256 bytes per key) with the
    // 16-byte chunks of a row permuted, so that the requests of a wave are whole consecutive rows (four per KiB: the
    // memory pipeline serves those 2.4x faster than 16-byte pieces of 32 different rows) and the fragment reads stay
    // free of bank conflicts:
    //   K: chunk c of key r sits in slot c ^ (r % 16)   -> ds_read_b128 of 16 keys x one chunk covers all 64 banks
    //   V: 32-byte chunk c of key r sits in slot c ^ sigma(r), sigma(r) = 2 (r % 4) + (r / 4) % 2
    //                                                  -> a transpose read of 4 keys x 2 chunks x 2 lane groups does
    // KiB block x of a stage = keys 4x .. 4x+3; wave w requests blocks w and w + 8, lane i the 16 bytes of slot i % 16
    // of key 4x + i / 16.  Offsets are bytes from the slice base for the first tile of the group.
    static_assert(D == 128, "tile layout below: 16 chunks of 16 bytes per key");
    const int dkey = 4 * wave + (lane >> 4);  // key of this lane in block w; + 32 in block w + 8
    uint32_t kgo, vgo;
    {
        const int slot = lane & 15;
        const int sigma = 2 * (dkey & 3) + ((dkey >> 2) & 1);
        // (unsigned: a slice may be just short of 4 GiB)
        const uint32_t row0 = (uint32_t)(tile_begin * BC + dkey) * (uint32_t)(d * 2);
        kgo = row0 + (uint32_t)chunk_offset(slot ^ (dkey & 15));
        vgo = row0 + (uint32_t)chunk_offset((((slot >> 1) ^ sigma) << 1) | (slot & 1));
    }
    const char* const Kb = reinterpret_cast<const char*>(Kbh);
    const char* const Vb = reinterpret_cast<const char*>(Vbh);
    // tile index t counts from tile_begin; keys past Nk re-read key Nk - 1 (their scores are masked).  The tile's
    // offset joins the scalar base address: a whole tile is requested without any vector arithmetic, only the last
    // tile of a ragged sequence adjusts rows.
    auto load_tile = [&](const char* base, uint32_t go, int t, FA_LDS char* stage) {
        const char* const tbase = base + (size_t)t * (size_t)(BC * d * 2);
        auto issue = [&](auto ragged_c) {
            constexpr bool kRagged = decltype(ragged_c)::value;
            int rows_left = Nk - (tile_begin + t) * BC;  // >= 1
            if constexpr (kRagged) asm volatile("" : "+s"(rows_left));  // (no running vector offsets for this case)
#pragma unroll
            for (int x = 0; x < NKL; ++x) {
                const int key = dkey + 32 * x;
                uint32_t o = go + (uint32_t)(32 * x * d * 2);
                if (kRagged && key >= rows_left) o -= (uint32_t)((key - rows_left + 1) * d * 2);
                dma_kib(tbase, o, stage + (wave + 8 * x) * 1024);
            }
        };
        if (Nk - (tile_begin + t) * BC >= BC) issue(std::false_type{});
        else issue(std::true_type{});
    };
    static_assert(NKL == NVL, "K and V tiles have the same shape");
    auto load_k = [&](int t, FA_LDS char* stage) { load_tile(Kb, kgo, t, stage); };
    auto load_v = [&](int t, FA_LDS char* stage) { load_tile(Vb, vgo, t, stage); };

    // ---- accumulators
    v16f oacc[MB];
    float m_ref = -INFINITY, l_run = 0.0f;
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[mb][r] = 0.0f;

    // Scores leave the MFMA unscaled.  With a positive scale the scaling commutes with the row maximum and is folded
    // into the exponent (one fma per score): cs = scale, and the ALiBi bias is added beforehand divided by the scale.
    // (The host sends a non-positive scale to the element-wise instance of the 4-wave kernel.)
    const float c2 = a.scale_log2, cs = c2;
    float nsig = 0.0f;  // ALiBi slope / scale, negated: read behind the prologue requests (below)

    // Lane parts of the fragment addresses (layout above).  K fragment (ks, kb): key 32 kb + l32, chunk 2 ks + g
    // -> k_rd ^ (32 ks) + 8192 kb.  V transpose read (st, mb, half h) of lane (G = lane / 16, e = lane / 4 % 4,
    // j = lane % 4): key 16 st + 8 h + 4 (G / 2) + e, 32-byte chunk 2 mb + G % 2, bytes 8 j .. 8 j + 7
    // -> v_rd ^ (64 mb) + 4096 st + 2048 h.
    const int k_rd = l32 * 256 + ((g ^ (l32 & 1)) << 4) + (((l32 & 15) >> 1) << 5);
    int v_rd;
    {
        const int G = lane >> 4, e = (lane >> 2) & 3, j = lane & 3;
        v_rd = (4 * (G >> 1) + e) * 256 + (((G & 1) ^ (G >> 1)) << 5) + 8 * j + (e << 6);
    }

    v16f s[2];
    v8h pf[2][2];

    // Fragment registers of the MFMA phase.  The phase is one software-pipelined stream of LDS reads and MFMAs:
    //   before the barrier : V fragments of key steps 0 and 1 (the tile has been in LDS for a whole iteration)
    //   PV step st         : MFMAs of step st, reads of step st+2; the last two steps read the first K fragments
    //   QK step ks         : MFMAs of step ks, reads of step ks+KPD
    // so that no MFMA waits for a read issued less than ~8 MFMAs earlier.
    union VF { v4hp p[2]; v8h v; };
    VF vf[4][MB];
    constexpr int KPD = KS < 3 ? KS : 3;  // K k-steps in flight
    v8h kf[KS][2];
    // vbase / kbase: stage address + lane part, as an integer (the stage bases are multiples of 16 KiB, so the
    // exclusive-or only touches the lane part)
    auto lds_ptr = [](uint32_t addr) { return reinterpret_cast<FA_LDS const char*>(static_cast<uintptr_t>(addr)); };
    auto v_read = [&](uint32_t vbase, int st) {
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            FA_LDS const char* p0 = lds_ptr(vbase ^ (uint32_t)(mb << 6)) + st * 4096;
            vf[st][mb].p[0] = __builtin_amdgcn_ds_read_tr16_b64_v4f16((FA_LDS v4hp*)(p0));
            vf[st][mb].p[1] = __builtin_amdgcn_ds_read_tr16_b64_v4f16((FA_LDS v4hp*)(p0 + 2048));
        }
    };
    auto k_read = [&](uint32_t kbase, int ks) {
        FA_LDS const char* p0 = lds_ptr(kbase ^ (uint32_t)(ks << 5));
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) kf[ks][kb] = *reinterpret_cast<FA_LDS const v8h*>(p0 + kb * 8192);
    };
    // Stage address + lane part of a fragment address.  The sum is laundered through an empty asm once per phase: the
    // compiler would otherwise precompute every per-fragment address across iterations and keep one register per read.
    auto frag_base = [&](FA_LDS const char* stage, int lane_part) {
        uint32_t v = (uint32_t)(uintptr_t)stage + (uint32_t)lane_part;
        asm volatile("" : "+v"(v));
        return v;
    };
    auto pv_mfma = [&](int st) {
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
            oacc[mb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf[st][mb].v, pf[st >> 1][st & 1], oacc[mb], 0, 0, 0);
    };
    auto qk_mfma = [&](int ks) {
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) s[kb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[ks][kb], qf[ks], s[kb], 0, 0, 0);
    };
    auto s_clear = [&]() {
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int r = 0; r < 16; ++r) s[kb][r] = 0.0f;
    };
    // stand-alone S^T = K Q^T (prologue only)
    auto qk = [&](FA_LDS const char* __restrict__ rdk) {
        const uint32_t kbase = frag_base(rdk, k_rd);
#pragma unroll
        for (int ks = 0; ks < KPD; ++ks) k_read(kbase, ks);
        s_clear();
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            if (ks + KPD < KS) k_read(kbase, ks + KPD);
            qk_mfma(ks);
        }
    };
    // MFMA phase body after the barrier: O += P V(t) with the first K(t+1) fragments fetched under its last MFMAs,
    // then S = K(t+1) Q^T.  One basic block, so that the read / MFMA interleaving below can be pinned.  The wave's last
    // tile has no successor whose scores it could use: its phase (last_c true) is the PV part alone.
    auto mfma_phase = [&](auto last_c, uint32_t vbase, uint32_t kbase) __attribute__((always_inline)) {
        constexpr bool kLast = decltype(last_c)::value;
        pv_mfma(0);
        __builtin_amdgcn_sched_barrier(0);  // step 0 first: its fragments were requested first
        v_read(vbase, 2);
        pv_mfma(1);
        v_read(vbase, 3);
        pv_mfma(2);
        if constexpr (!kLast) {
#pragma unroll
            for (int ks = 0; ks < KPD; ++ks) k_read(kbase, ks);
        }
        pv_mfma(3);
        if constexpr (!kLast) {
            s_clear();
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                if (ks + KPD < KS) k_read(kbase, ks + KPD);
                qk_mfma(ks);
            }
        }
        // pin the order: [2MB reads][MB MFMA][2MB reads][MB MFMA][2*KPD reads][MB MFMA]{[2 reads][2 MFMA]}...
        __builtin_amdgcn_sched_group_barrier(0x100, 2 * MB, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, MB, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 2 * MB, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, MB, 0);
        if constexpr (!kLast) __builtin_amdgcn_sched_group_barrier(0x100, 2 * KPD, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, MB, 0);
        if constexpr (!kLast) {
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                if (ks + KPD < KS) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
                __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
            }
        }
    };

    // online softmax of the tile whose scores sit in s; leaves P^T packed to fp16 in pf
    // mask_sides: bit 0 = some row of the wave has its first allowed key inside or after this tile, bit 1 = some row has
    // its last allowed key inside or before it (both wave-uniform)
    auto softmax = [&](int mask_sides, int kb0) __attribute__((always_inline)) {
        if constexpr (kAlibi) {
            // score*scale - slope*|i - j|  (src/main.cu:315,324), in the log2 domain
            const float jb = (float)(kb0 + 4 * g) - iif;
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    s[kb][r] = __builtin_fmaf(nsig, __builtin_fabsf(jb + (float)(32 * kb + 8 * (r >> 2) + (r & 3))), s[kb][r]);
        }
        if (mask_sides != 0) {
            // Wave-uniform and rare (boundary tiles only); the masking itself is inline asm (common.h), which keeps these
            // real branches.  Where the bounds of the wave's rows run along block diagonals (one key per row, from a
            // multiple of 32: causal masks and windows whose offsets are multiples of 32, rows not clipped by a sequence
            // or split end), lane-mask constants per 32-key block do the masking; otherwise a tile takes one
            // comparison per score and crossed end of the interval.
            const float ninf = -INFINITY;
            const int hi_f = __builtin_amdgcn_readlane(hi, 0), hi_l = __builtin_amdgcn_readlane(hi, 31);
            const int lo_f = __builtin_amdgcn_readlane(lo, 0), lo_l = __builtin_amdgcn_readlane(lo, 31);
            const bool hi_diag = hi_l - hi_f == 31 && (hi_f & 31) == 0;
            const bool lo_diag = lo_l - lo_f == 31 && (lo_f & 31) == 0;
            if (((mask_sides & 1) == 0 || lo_diag) && ((mask_sides & 2) == 0 || hi_diag)) {
#pragma unroll
                for (int kb = 0; kb < 2; ++kb) {
                    // last / first visible key of the wave's first row relative to the block: multiples of 32
                    const int dh = (mask_sides & 2) ? hi_f - (kb0 + 32 * kb) : 64;
                    const int dl = (mask_sides & 1) ? lo_f - (kb0 + 32 * kb) : -64;
                    if (dh < 0 || dl >= 32) {
                        mask_whole_block(s[kb], ninf);
                    } else {
                        if (dh == 0) mask_off_diagonal<true>(s[kb], ninf);
                        if (dl == 0) mask_off_diagonal<false>(s[kb], ninf);
                    }
                }
            } else {
                const int lo_rel = lo - kb0 - 4 * g, hi_rel = hi - kb0 - 4 * g;
#pragma unroll
                for (int kb = 0; kb < 2; ++kb) {
                    if (mask_sides & 1) mask_beyond<false>(s[kb], lo_rel - 32 * kb, ninf);
                    if (mask_sides & 2) mask_beyond<true>(s[kb], hi_rel - 32 * kb, ninf);
                }
            }
        }
        float mx = -INFINITY;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[kb][r]);
        mx = xhalf_max(mx);
        mx *= cs;  // cs > 0
        if (__builtin_amdgcn_ballot_w64(mx > m_ref + kLazyTau) != 0ull) {
            const float m_new = fmaxf(m_ref, mx);
            float alpha = (m_new == -INFINITY) ? 1.0f : fast_exp2(m_ref - m_new);
            asm volatile("; raise running max" : "+v"(alpha));
            m_ref = m_new;
            l_run *= alpha;
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int r = 0; r < 16; ++r) oacc[mb][r] *= alpha;
        }
        const float m_use = (m_ref == -INFINITY) ? 0.0f : m_ref;
        float rs = 0.0f;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float p = fast_exp2(__builtin_fmaf(s[kb][r], cs, -m_use));
                rs += p;
                s[kb][r] = p;
            }
        l_run += rs;
        if constexpr (kDropout) {
            const uint32_t i_u = (uint32_t)row_i;
            // first-round Philox product of the head-slice word: the same for the whole work-group, so a scalar multiply
            const uint64_t bh_prod = (uint64_t)0xCD9E8D57u * (uint64_t)(uint32_t)bh;
            const uint32_t bh_hi = (uint32_t)(bh_prod >> 32), bh_lo = (uint32_t)bh_prod;
            uint8_t* kout = a.keep_out ? a.keep_out + ((size_t)bh * Nq + row_i) * Nk : nullptr;
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int q = 0; q < 2; ++q) {
                    // the lane's eight keys among the 16 from jg on: field f belongs to key jg + 8*(f>>2) + 4*g + (f&3)
                    const int jg = kb0 + 32 * kb + 16 * q;
                    const v4u w = philox4x32_10_c2(dropout_call((uint32_t)(jg + 4 * g)), i_u, bh_hi, bh_lo, a.off_lo, a.seed_lo, a.seed_hi);
                    // the decisions are applied to the packed fp16 words (keep_pair); the 1/(1-p) waits for the epilogue
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        union { v2h h; uint32_t u; } pk;
                        pk.h = pack_f16(s[kb][8 * q + 2 * k], s[kb][8 * q + 2 * k + 1]);
                        pk.u = keep_pair(pk.u, w[k], a.drop_sub2);
                        pf[kb][q][2 * k] = pk.h[0];
                        pf[kb][q][2 * k + 1] = pk.h[1];
                    }
                    if (a.keep_out != nullptr) {  // debug dump: one uniform branch per call, none per score
#pragma unroll
                        for (int f = 0; f < 8; ++f) {
                            const int j = jg + 8 * (f >> 2) + 4 * g + (f & 3);
                            if (row_i < Nq && j < Nk) kout[j] = philox_field16(w, f) >= a.drop_thr ? 1 : 0;
                        }
                    }
                }
        }
        if constexpr (!kDropout) {  // (there the dropout step has packed them already)
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int tt = 0; tt < 2; ++tt)
#pragma unroll
                    for (int e = 0; e < 8; e += 2) {
                        const v2h h2 = pack_f16(s[kb][8 * tt + e], s[kb][8 * tt + e + 1]);
                        pf[kb][tt][e] = h2[0];
                        pf[kb][tt][e + 1] = h2[1];
                    }
        }
    };

    // One iteration.  The four stage pointers are distinct LDS regions; declaring them restrict is what lets the
    // compiler issue the fragment reads without first waiting (vmcnt) for the LDS-DMA writes into the other stages.
    auto iteration = [&](auto last_c, FA_LDS const char* __restrict__ rdv, FA_LDS const char* __restrict__ rdk,
                         FA_LDS char* __restrict__ wrk, FA_LDS char* __restrict__ wrv, int t) __attribute__((always_inline)) {
        const int kb0 = (tile_begin + t) * BC;
        // ---------------- VALU phase: request the V tile to come, softmax of tile t
        if (t + 2 < ntiles) load_v(t + 2, wrv);
        const int mask_sides = (kb0 < lo_max ? 1 : 0) | (kb0 + BC - 1 > hi_min ? 2 : 0);
        softmax(mask_sides, kb0);
        __builtin_amdgcn_sched_barrier(0);
        const uint32_t vbase = frag_base(rdv, v_rd);
        const uint32_t kbase = frag_base(rdk, k_rd);
        v_read(vbase, 0);
        __builtin_amdgcn_sched_barrier(0);  // keep the request order: step 0 is consumed first
        v_read(vbase, 1);
        lds_barrier_keep<4 * MB>();
        // ---------------- MFMA phase: O += P(t) V(t), then S(t+1) = K(t+1) Q^T
        __builtin_amdgcn_s_setprio(1);
        mfma_phase(last_c, vbase, kbase);
        __builtin_amdgcn_s_setprio(0);
        // K(t+3) is requested here, behind the wave's last MFMA of the phase (the four waves of a group reach the start
        // of their VALU phase together: requests issued there queue up in front of the softmax), and waited for one
        // iteration later: what must have landed now is K(t+2), requested an iteration ago, and V(t+2).
        if (t + 3 < ntiles) {
            load_k(t + 3, wrk);
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NKL) : "memory");
        } else {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
        lds_barrier();
    };

    // ---- prologue: Q, K(0..2), V(0..1) requested; everything landed before the first barrier.
    // Q takes the same route as the tiles (whole rows per request, chunk c of row r in slot c ^ (r % 16)): each wave
    // stages its own 32 rows in 8 KiB of LDS that no tile uses before the first loop iteration, and reads its eight
    // B-operand fragments back from there.  Private to the wave: only its own vmcnt wait stands between the two.
    {
        FA_LDS char* const qst = wave < 2   ? Xs + wave * 8192
                                 : wave < 4 ? Vs + 2 * C::VBUF + (wave - 2) * 8192
                                 : wave < 6 ? Ks + 3 * C::KBUF + (wave - 4) * 8192
                                            : Vs + 3 * C::VBUF + (wave - 6) * 8192;
        static_assert(C::XBUF == 2 * 8192 && C::KBUF == 2 * 8192 && C::VBUF == 2 * 8192 && C::NST == 4, "Q staging map");
        const char* const Qb = reinterpret_cast<const char*>(Qbh);
#pragma unroll
        for (int x = 0; x < 8; ++x) {
            const int rl = 4 * x + (lane >> 4);  // row of the wave's 32
            const int gi = q0 + rblk * 32 + rl;
            const uint32_t off = (uint32_t)(gi < Nq ? gi : Nq - 1) * (uint32_t)(d * 2) + (uint32_t)chunk_offset((lane & 15) ^ (rl & 15));
            dma_kib(Qb, off, qst + x * 1024);
        }
        if (ntiles > 0) {
            load_k(0, Ks);
            load_v(0, Vs);
            if (ntiles > 1) {
                load_k(1, Ks + C::KBUF);
                load_v(1, Vs + C::VBUF);
            }
            if (ntiles > 2) load_k(2, Ks + 2 * C::KBUF);
        }
        // (a vector load: the wait for it counts every older request too, so it goes last; only launched with a table)
        if constexpr (kAlibi) nsig = -(a.alibi[h] * kLog2e) / c2;
        stamps.take(1);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // (a memory clobber: the reads below stay below)
        stamps.take(2);
        const uint32_t qbase = (uint32_t)(uintptr_t)qst + (uint32_t)k_rd;  // same lane part as a K fragment
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
            qf[ks] = *reinterpret_cast<FA_LDS const v8h*>(
                reinterpret_cast<FA_LDS const char*>(static_cast<uintptr_t>(qbase ^ (uint32_t)(ks << 5))));
        if constexpr (!kFullD) {  // zeroes where the chunk before has covered a column already, and past the row
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                union { v8h h; v4u u; } t;
                t.h = qf[ks];
                qf[ks] = mask_q_chunk_anyalign(t.u, 16 * ks + 8 * g, d);
            }
        }
    }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) asm volatile("" : "+v"(qf[ks]));  // Q is in registers before the loop
    lds_barrier();  // tiles visible to all waves; every wave has read its Q rows (their LDS is reused by the loop)
    stamps.take(3);
    if (ntiles > 0) {
        qk(Ks);
        if constexpr (kStamp) {
            // reading a score back makes the wave wait for the last MFMA before the stamp is taken
            const int done = __builtin_amdgcn_readfirstlane(__float_as_int(s[1][15]));
            asm volatile("; first scores are there" ::"s"(done));
            stamps.take(4);
        }
    }
    if (grp == 1) lds_barrier();  // second wave group runs half an iteration behind

    // Tiles whose keys (and whose successor's keys) are all invisible to this wave contribute nothing: there the wave
    // only serves its share of the loads and the barriers.  Live tiles form one contiguous range [t_lo, t_hi).
    auto idle_iteration = [&](int t) {
        if (t + 2 < ntiles) load_v(t + 2, Vs + ((t + 2) % NST) * C::VBUF);
        lds_barrier();
        if (t + 3 < ntiles) {
            load_k(t + 3, Ks + ((t + 3) % NST) * C::KBUF);
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NKL) : "memory");
        } else {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
        lds_barrier();
    };
    // The full loop starts one tile before the first visible one: that tile is masked entirely (whatever stale scores
    // the wave holds for it), and its iteration produces the scores of the first visible tile.
    int t_lo = lo_min / BC - tile_begin - 1;
    int t_hi = hi_max >= 0 ? hi_max / BC - tile_begin + 1 : 0;  // one past the last tile with a visible key
    t_lo = t_lo < 0 ? 0 : t_lo;
    t_hi = t_hi > ntiles ? ntiles : t_hi;
    if (t_lo > t_hi) t_lo = t_hi;
    int t = 0;
    for (; t < t_lo; ++t) idle_iteration(t);
    for (; t < t_hi - 1; ++t)
        iteration(std::false_type{}, Vs + (t % NST) * C::VBUF, Ks + ((t + 1) % NST) * C::KBUF,
                  Ks + ((t + 3) % NST) * C::KBUF, Vs + ((t + 2) % NST) * C::VBUF, t);
    if (t < t_hi) {  // the wave's last tile: no scores of a successor to compute
        iteration(std::true_type{}, Vs + (t % NST) * C::VBUF, Ks + ((t + 1) % NST) * C::KBUF,
                  Ks + ((t + 3) % NST) * C::KBUF, Vs + ((t + 2) % NST) * C::VBUF, t);
        ++t;
    }
    for (; t < ntiles; ++t) idle_iteration(t);
    if (grp == 0) lds_barrier();  // both groups pass the same number of barriers
    stamps.take(5);

    // ---------------- epilogue
    {
        const float l = xhalf_sum(l_run);
        const float inv = l > 0.0f ? (kDropout ? a.drop_rscale : 1.0f) / l : 0.0f;
        const float lse = l > 0.0f ? __builtin_fmaf(m_ref, kLn2, fast_log2(l) * kLn2) : -INFINITY;
        if (a.num_splits > 1) {
            if (row_i < Nq) {
                const size_t prow = ((size_t)bh * a.num_splits + split) * Nq + row_i;
                if (g == 0) a.LSE_partial[prow] = lse;
                float* op = a.O_partial + prow * d;
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                    for (int rg = 0; rg < 4; ++rg) {
                        const int dc = 32 * mb + 8 * rg + 4 * g;
                        v4f o = {oacc[mb][4 * rg] * inv, oacc[mb][4 * rg + 1] * inv, oacc[mb][4 * rg + 2] * inv,
                                 oacc[mb][4 * rg + 3] * inv};
                        if constexpr (kFullD) {
                            *reinterpret_cast<v4f*>(op + dc) = o;
                        } else {
                            // the chunk position behind the row's whole chunks holds columns d - 8 ... d - 1
                            const int c0 = d & ~7, rem = d & 7;
                            if (dc < c0 || (rem != 0 && dc < c0 + 8))
                                *reinterpret_cast<v4f_anyalign*>(op + (dc < c0 ? dc : dc - (8 - rem))) = o;
                        }
                    }
            }
        } else {
            if (row_i < Nq && g == 0) a.LSE[(size_t)bh * Nq + row_i] = lse;
            // O: a lane holds 4 consecutive head-dim columns of one row at a time; written like that, a wave store
            // would touch 32 rows x 8 bytes.  The wave's 32 x 128 fp16 block is turned round in 8 KiB of LDS instead
            // (all tile reads of the work-group are behind the last barrier; chunk c of row r in slot c ^ (r % 16), as
            // for the tiles), and leaves as four whole rows per store instruction (non-temporal: O is not read again by this
            // launch, and lines left dirty in L2 would only be written back when the kernel ends).
            FA_LDS char* const ost = Ks + wave * 8192;
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int rg = 0; rg < 4; ++rg) {
                    v4h o = {(half_t)(oacc[mb][4 * rg] * inv), (half_t)(oacc[mb][4 * rg + 1] * inv),
                             (half_t)(oacc[mb][4 * rg + 2] * inv), (half_t)(oacc[mb][4 * rg + 3] * inv)};
                    const int slot = (4 * mb + rg) ^ (l32 & 15);
                    *reinterpret_cast<FA_LDS v4h*>(ost + l32 * 256 + slot * 16 + g * 8) = o;
                }
            char* const Ob = reinterpret_cast<char*>(a.O + (size_t)bh * Nq * d);
#pragma unroll
            for (int x = 0; x < 8; ++x) {
                const int rl = 4 * x + (lane >> 4);
                const int gi = q0 + rblk * 32 + rl;
                const v4u val = *reinterpret_cast<FA_LDS const v4u*>(ost + x * 1024 + lane * 16);
                const int c = (lane & 15) ^ (rl & 15);
                if constexpr (kFullD) {
                    if (gi < Nq) __builtin_nontemporal_store(val, reinterpret_cast<v4u*>(Ob + (size_t)gi * d * 2 + (c << 4)));
                } else {
                    if (gi < Nq && c * 8 < d)
                        __builtin_nontemporal_store(val, reinterpret_cast<v4u_anyalign*>(Ob + (size_t)gi * d * 2 + chunk_offset(c)));
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

template <int D, int VAR>
inline hipError_t launch_fwd_pp_instance(const FwdArgs& a, hipStream_t st)
{
    using C = PPCfg<D>;
    auto kern = fwd_pp_kernel<D, VAR>;
    static DeviceFlags attr_done;  // per instantiation and device
    if (hipError_t e = ensure_dynamic_lds(reinterpret_cast<const void*>(kern), C::SMEM, attr_done); e != hipSuccess) return e;
    FwdArgs b = a;
    b.Tr = (a.Nq + C::BR - 1) / C::BR;
    const long long groups = (long long)b.Tr * a.B * a.H * a.num_splits;
    set_slice_order(b, b.Tr * a.num_splits, kNumCus);  // one work-group per CU at a time
    b.split_rotate = split_rotate_for(b.num_splits, b.slice_chunk);
    b.snake_end = snake_end_for(groups, kNumCus);
    return launch_kernel(kern, dim3((unsigned)groups), dim3(512), C::SMEM, st, b);
}

// {d == D, shorter rows} x {plain, ALiBi, dropout, both}; ST = kVarStamp: their instrumented twins
template <int D, int ST>
inline int launch_fwd_pp_bucket_st(const FwdArgs& a, int variant, hipStream_t st)
{
    const int feat = variant & (kVarAlibi | kVarDropout);
    hipError_t e;
    if (a.d == D) {
        constexpr int V = ST | kVarFullD;
        if (feat == 0) e = launch_fwd_pp_instance<D, V>(a, st);
        else if (feat == kVarAlibi) e = launch_fwd_pp_instance<D, V | kVarAlibi>(a, st);
        else if (feat == kVarDropout) e = launch_fwd_pp_instance<D, V | kVarDropout>(a, st);
        else e = launch_fwd_pp_instance<D, V | kVarAlibi | kVarDropout>(a, st);
    } else {
        if (feat == 0) e = launch_fwd_pp_instance<D, ST>(a, st);
        else if (feat == kVarAlibi) e = launch_fwd_pp_instance<D, ST | kVarAlibi>(a, st);
        else if (feat == kVarDropout) e = launch_fwd_pp_instance<D, ST | kVarDropout>(a, st);
        else e = launch_fwd_pp_instance<D, ST | kVarAlibi | kVarDropout>(a, st);
    }
    return (int)e;
}

template <int D>
inline int launch_fwd_pp_bucket(const FwdArgs& a, int variant, hipStream_t st)
{
    return a.stamps ? launch_fwd_pp_bucket_st<D, kVarStamp>(a, variant, st) : launch_fwd_pp_bucket_st<D, 0>(a, variant, st);
}

}  // namespace fa
