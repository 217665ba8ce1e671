// Shared definitions for the gfx950 FlashAttention-forward kernels: launch-argument structs, vector types,
// wave64 helpers and the counter-based Philox used for dropout.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

namespace fa {

typedef _Float16 half_t;
typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef _Float16 v4h __attribute__((ext_vector_type(4)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef float v2f __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef uint32_t v4u __attribute__((ext_vector_type(4)));
// 16 bytes at any 2-byte / 4-byte boundary (the hardware runs in unaligned access mode): rows of d % 8 != 0 elements
typedef v4u __attribute__((aligned(2))) v4u_anyalign;
typedef v4f __attribute__((aligned(4))) v4f_anyalign;
// operand type of the ds_read_b64_tr_b16 builtin
typedef __fp16 v4hp __attribute__((__vector_size__(4 * sizeof(__fp16))));

#define FA_LDS __attribute__((address_space(3)))

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// Arguments of the tiled forward kernel and of the decode/combine kernels, filled by the host from flash_params
// (which is itself the superset of the reference's mykernelParamType, include/utils.h:21-44).
struct FwdArgs {
    const half_t* Q;
    const half_t* K;
    const half_t* V;
    half_t* O;
    float* LSE;
    float* O_partial;    // [B,H,S,Nq,d] fp32, normalised per split (reference O_tmp)
    float* LSE_partial;  // [B,H,S,Nq]   fp32, m_s + log l_s   (reference M, L)
    const float* alibi;  // [H] or nullptr
    uint8_t* keep_out;   // [B,H,Nq,Nk] or nullptr
    float* scores_out;   // [B,H,Nq,Nk] or nullptr (element-wise instance of the 4-wave kernel only)
    uint64_t* stamps;    // [work-groups][kStampWords] or nullptr (instrumented instances only)
    int B, H, Nq, Nk, d;
    int Hk, kv_group;    // K/V heads and query heads per K/V head (H = Hk * kv_group)
    int causal, wl, wr;  // wl / wr < 0: unbounded
    float scale_log2;    // softmax_scale * log2(e)
    uint32_t drop_thr;   // keep iff 16-bit philox field >= drop_thr
    uint32_t drop_sub2;  // drop_thr - 1 in both 16-bit halves (vector instances; they are launched with drop_thr >= 1)
    float drop_rscale;   // 1 / (1 - p)
    uint32_t seed_lo, seed_hi, off_lo;
    int num_splits;      // 1: write O/LSE; > 1: write the partial workspace
    int keys_per_split;  // multiple of 128
    int Tr;              // number of query row blocks
    int kernel_hint;     // 0: by shape, 1: 4-wave kernel, 2: 8-wave kernel where it can serve the call
    int alibi_left;      // ALiBi and no visible key lies right of its row (causal, or right window 0)
    int slice_chunk;     // head slices per chunk of the work-group order (set by the kernel's launcher)
    int snake_end;       // work-groups below this index sit on the GPU together; odd 256-blocks of them run reversed (launcher)
    int group_xcd;       // > 1: query heads per K/V head, and the slice order keeps the heads of a K/V head on one XCD (launcher)
    int split_rotate;    // 1: the split index of a work-group is rotated by its row block (launcher; split_of_rest)

    // index of the K/V slice [Nk,d] read by query slice bh = b * H + h
    __device__ __forceinline__ int kv_slice(int bh) const { return (bh / H) * Hk + (bh % H) / kv_group; }
};

__device__ __forceinline__ int wave_uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }

// Q chunk for the chunk position at column col (a multiple of 8) of a row of d >= 8 elements at any alignment, where the
// position behind the row's whole chunks stands for columns d - 8 ... d - 1 and v holds what was loaded from there (see
// fwd_kernel.h): the columns that the chunk before has covered already are zeroed, and so are positions past the row.
__device__ __forceinline__ v8h mask_q_chunk_anyalign(v4u v, int col, int d)
{
    union { v4u u; v8h h; } t;
    t.u = v;
    const int covered = col + 8 <= d ? 0 : col < d ? 8 - (d & 7) : 8;  // leading elements that must not count
#pragma unroll
    for (int e = 0; e < 8; ++e) t.h[e] = e >= covered ? t.h[e] : (half_t)0.0f;
    return t.h;
}

// A work-group whose rows see no key at all (rows above a causal diagonal that starts below them, a split of the key
// range beyond their mask): O = 0 and LSE = -inf for rows [r0, r1) of head slice bh, or the same in the slice's partial
// results of split `split`.  The rows are one contiguous piece of memory; it is filled with 16-byte stores at whatever
// alignment the piece has, the last one ending with the piece.  Called by every thread of the group, before anything else
// is requested: such a group is done in the time of its stores.
__device__ __forceinline__ void store_empty_rows(const FwdArgs& a, int bh, int split, int r0, int r1, int tid, int nthreads)
{
    char* base;
    float* lse;
    size_t bytes;
    if (a.num_splits > 1) {
        const size_t prow = ((size_t)bh * a.num_splits + split) * a.Nq + r0;
        base = reinterpret_cast<char*>(a.O_partial + prow * a.d);
        lse = a.LSE_partial + prow;
        bytes = (size_t)(r1 - r0) * a.d * sizeof(float);
    } else {
        const size_t row = (size_t)bh * a.Nq + r0;
        base = reinterpret_cast<char*>(a.O + row * a.d);
        lse = a.LSE + row;
        bytes = (size_t)(r1 - r0) * a.d * sizeof(half_t);
    }
    const v4u z = {0u, 0u, 0u, 0u};
    const size_t whole = bytes / 16;
    for (size_t i = tid; i < whole; i += nthreads) __builtin_nontemporal_store(z, reinterpret_cast<v4u_anyalign*>(base + 16 * i));
    if (tid == 0 && (bytes & 15) != 0) {
        if (whole > 0) {
            *reinterpret_cast<v4u_anyalign*>(base + bytes - 16) = z;
        } else {
            for (size_t i = 0; i < bytes; i += 2) *reinterpret_cast<uint16_t*>(base + i) = 0;
        }
    }
    for (int i = tid; i < r1 - r0; i += nthreads) lse[i] = -INFINITY;
}

// Position of a work-group in the launch's work order.  The order is "heaviest first", which balances a launch that
// makes several rounds: whichever place frees up takes the heaviest work-group left.  But the work-groups of the first
// round are not placed by load: the dispatcher deals work-group i to XCD i % 8 and there to CU (i / 8) % 32, so that with
// r places per CU work-groups i, i + 256, ..., i + 256 (r - 1) share a CU whatever they weigh (measured: a causal launch
// of 512 work-groups at two per CU left the CUs with 2 ... 32 key tiles each).  Inside that resident part (indices below
// snake_end = min(work-groups, places), a multiple of 8) every second block of 256 therefore takes its items in reverse
// CU order -- the CU with the heaviest item of one block gets the lightest of the next -- while i % 8, the XCD and with it
// the L2 that a head slice's K and V sit in, stays as it is.
__device__ __forceinline__ int work_position(int block, int snake_end)
{
    if (block < snake_end && (block & 256)) {
        const int base = block & ~255;
        const int size = snake_end - base < 256 ? snake_end - base : 256;  // a multiple of 8
        const int pos = block - base;
        return base + ((size >> 3) - 1 - (pos >> 3)) * 8 + (pos & 7);
    }
    return block;
}

// Head slice of position `local` in a chunk of the slice order.  Position p runs on XCD p % 8 (slices vary fastest over
// the work-groups).  With grouped K/V heads the G = group_xcd query heads of a K/V head are G consecutive slices and would
// land on G different XCDs, each pulling the same K and V into its own L2 (measured on B4 H32 H_kv4 N4096 d128 causal:
// 3.7 times the K/V/Q bytes fetched).  Instead position (x, y) = (p % 8, p / 8) takes query head y % G of K/V slice
// 8 (y / G) + x: the heads of a K/V head share an XCD and follow each other there.  A bijection on chunks whose size is
// a multiple of 8 G (the launcher sets group_xcd only then).
// Split index and row-block index of the position `rest` inside a slice (splits fastest).  Where the slices of a chunk
// are not a multiple of 8, the XCD of a work-group depends on its split: with 4 slices and 2 splits, XCDs 0-3 get
// every first split and XCDs 4-7 every second one, and under a causal mask, whose first splits are the long ones, half the
// chip then carries three quarters of the work (measured B1 H4 N16384 d32 causal, 2 splits: 201 us, against 160 us
// unsplit and 158 us with 5 splits).  Rotating the split index by the row-block index deals every split to every XCD.
// The launcher asks for it exactly where the plain order aliases: work-group x + 8 n of XCD x has split
// (x / c + (8 / c) n) % S for c = 1, 2 or 4 slices per chunk, which reaches every split only if S is odd; other chunk
// sizes mix by themselves, and rotating an order that already mixes measured 0 ... -14 %.
__device__ __forceinline__ int split_of_rest(int rest, int num_splits, int rotate, int* row_block_index)
{
    const int mi = rest / num_splits, s0 = rest % num_splits;
    *row_block_index = mi;
    return rotate ? (s0 + mi) % num_splits : s0;
}
inline int split_rotate_for(int num_splits, int slice_chunk)
{
    return num_splits > 1 && num_splits % 2 == 0 && (slice_chunk == 1 || slice_chunk == 2 || slice_chunk == 4) ? 1 : 0;
}

__device__ __forceinline__ int slice_of_position(int local, int group_xcd)
{
    if (group_xcd > 1) {
        const int x = local & 7, y = local >> 3;
        return ((y / group_xcd) * 8 + x) * group_xcd + y % group_xcd;
    }
    return local;
}

// snake_end for a launch of `groups` work-groups with `resident` places on the GPU
inline int snake_end_for(long long groups, int resident)
{
    const long long n = groups < resident ? groups : resident;
    return (int)(n & ~7LL);
}

// Exchange between lane l and lane l^32 (v_permlane32_swap): result[0] holds the low half's value in both halves,
// result[1] the high half's.
__device__ __forceinline__ float xhalf_max(float v)
{
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float xhalf_sum(float v)
{
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// Debug time stamps of the instrumented kernel instances: readings of the constant 100 MHz counter, taken by every wave
// (they are scalar) and stored by the first lane of the work-group in the epilogue with an ordinary vector store.
// Beside stages 3 and 5 the shader-clock counter is read as well: their difference over the time between the two stages
// is the clock the work-group ran at in its key-tile loop.
constexpr int kStampTimes = 7;
constexpr int kStampWords = 9;  // FLASH_STAMP_WORDS of the public header
template <bool kOn>
struct Stamps {
    uint64_t t[kOn ? kStampTimes : 1];
    uint64_t cyc[kOn ? 2 : 1];
    // stage 0 also presets the later stages: one that a work-group never reaches (no key tile) is stored as the time
    // of the stage before it
    __device__ __forceinline__ void take(int i)
    {
        if constexpr (kOn) {
            const uint64_t now = __builtin_amdgcn_s_memrealtime();
            if (i == 0) {
#pragma unroll
                for (int k = 0; k < kStampTimes; ++k) t[k] = now;
                cyc[0] = cyc[1] = 0;
            } else {
                t[i] = now;
                if (i == 3) cyc[0] = __builtin_amdgcn_s_memtime();
                if (i == 5) cyc[1] = __builtin_amdgcn_s_memtime();
            }
        }
    }
    // word 7: tiles << 32 | XCC id << 16 | low half of HW_ID (wave, SIMD, pipe, CU, SH, SE); word 8: shader-clock cycles
    // between stages 3 and 5
    __device__ __forceinline__ void store(uint64_t* out, int ntiles) const
    {
        if constexpr (kOn) {
            if (out != nullptr && threadIdx.x == 0) {
                const uint32_t hw = __builtin_amdgcn_s_getreg((31 << 11) | 4);    // HW_REG_HW_ID
                const uint32_t xcc = __builtin_amdgcn_s_getreg((31 << 11) | 20);  // HW_REG_XCC_ID
                uint64_t* o = out + (size_t)blockIdx.x * kStampWords;
                uint64_t last = t[0];
#pragma unroll
                for (int i = 0; i < kStampTimes; ++i) {
                    last = t[i] > last ? t[i] : last;
                    o[i] = last;
                }
                o[kStampTimes] = ((uint64_t)(uint32_t)ntiles << 32) | ((uint64_t)(xcc & 0xfu) << 16) | (hw & 0xffffu);
                o[kStampTimes + 1] = cyc[1] > cyc[0] ? cyc[1] - cyc[0] : 0;
            }
        }
    }
};

// two fp32 -> packed fp16, round to nearest even, in one instruction (v_cvt_pk_f16_f32)
__device__ __forceinline__ v2h pack_f16(float a, float b)
{
    const v2f t = {a, b};
    return __builtin_convertvector(t, v2h);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

// Philox4x32-10.  Dropout contract: one call yields eight 16-bit fields (field f = bits 16*(f&1).. of output word f>>1)
// and serves eight keys of one query row: key = (lo32(seed), hi32(seed)), counter = (call(j), i, b*H + h, lo32(offset)),
// element (i, j) reads field(j) and is kept iff that field >= floor(p * 2^16).  Of every 16 consecutive keys the call
// with even index serves keys 0-3 and 8-11, the odd one keys 4-7 and 12-15: the eight keys whose scores one lane of the
// tiled kernels holds (32x32 MFMA accumulator layout), so that a lane uses every bit it computes.  Replaces the
// stateful curandStatePhilox4_32_10_t draw of the reference (src/flash_forward.h:50-54,227).
__host__ __device__ __forceinline__ uint32_t dropout_call(uint32_t j) { return 2u * (j >> 4) + ((j >> 2) & 1u); }
__host__ __device__ __forceinline__ uint32_t dropout_field(uint32_t j) { return 4u * ((j >> 3) & 1u) + (j & 3u); }
// 32 x 32 -> 64-bit product in one instruction (v_mad_u64_u32; integer multiplies run at a quarter of the VALU rate,
// and the compiler would issue two of them, v_mul_hi_u32 and v_mul_lo_u32, per product)
__device__ __forceinline__ void mul_wide_u32(uint32_t m, uint32_t x, uint32_t& hi, uint32_t& lo)
{
    uint64_t r;
    asm("v_mad_u64_u32 %0, vcc, %1, %2, 0" : "=v"(r) : "s"(m), "v"(x) : "vcc");
    hi = (uint32_t)(r >> 32);
    lo = (uint32_t)r;
}

// Element masks of a 32 x 32 score block whose boundary runs along its diagonal.  In the accumulator layout lane
// (l32 = lane % 32, g = lane / 32) holds in register r the score of query row l32 and key 8 (r / 4) + r % 4 + 4 g of the
// block, so "key right of the diagonal" (key > row) and "key left of it" (key < row) are fixed sets of lanes per register:
// sixteen 64-bit constants each, applied with one v_cndmask per register on a constant lane mask instead of a comparison
// and a select per score.
constexpr uint64_t diag_lane_mask(int r, bool right)
{
    uint64_t m = 0;
    for (int lane = 0; lane < 64; ++lane) {
        const int row = lane & 31, key = 8 * (r >> 2) + (r & 3) + 4 * (lane >> 5);
        if (right ? key > row : key < row) m |= 1ull << lane;
    }
    return m;
}
template <bool kRight, int R = 0>
__device__ __forceinline__ void mask_off_diagonal(v16f& s, float ninf)
{
    if constexpr (R < 16) {
        // (the constant goes into vcc inside the statement: as an operand the compiler would keep all thirty-two
        // constants in scalar registers across the key loop and spill them)
        constexpr uint64_t m = diag_lane_mask(R, kRight);
        asm("s_mov_b32 vcc_lo, %2\n\ts_mov_b32 vcc_hi, %3\n\tv_cndmask_b32_e32 %0, %0, %1, vcc"
            : "+v"(s[R])
            : "v"(ninf), "n"((uint32_t)m), "n"((uint32_t)(m >> 32))
            : "vcc");
        mask_off_diagonal<kRight, R + 1>(s, ninf);
    }
}

// The general case: the score in register R belongs to key 8 (R / 4) + R % 4 of the block (the caller folds the lane's
// 4 g and the block's position into the bound); scores of keys above (below) the lane's bound become -inf.  In place
// and as inline asm on purpose: written as selects the compiler copies the sixteen accumulator registers first, and
// turns a rare wave-uniform branch around them into selects that every tile executes.
template <bool kAbove, int R = 0>
__device__ __forceinline__ void mask_beyond(v16f& s, int bound, float ninf)
{
    if constexpr (R < 16) {
        constexpr int key = 8 * (R >> 2) + (R & 3);
        if constexpr (kAbove)
            asm("v_cmp_gt_i32_e32 vcc, %2, %1\n\tv_cndmask_b32_e32 %0, %0, %3, vcc" : "+v"(s[R]) : "v"(bound), "n"(key), "v"(ninf) : "vcc");
        else
            asm("v_cmp_lt_i32_e32 vcc, %2, %1\n\tv_cndmask_b32_e32 %0, %0, %3, vcc" : "+v"(s[R]) : "v"(bound), "n"(key), "v"(ninf) : "vcc");
        mask_beyond<kAbove, R + 1>(s, bound, ninf);
    }
}

__device__ __forceinline__ void mask_whole_block(v16f& s, float ninf)
{
#pragma unroll
    for (int r = 0; r < 16; ++r) asm("v_mov_b32 %0, %1" : "=v"(s[r]) : "v"(ninf));
}

// three-input exclusive or in one instruction (v_bitop3_b32, truth table 0x96)
__device__ __forceinline__ uint32_t xor3(uint32_t a, uint32_t b, uint32_t c) { return __builtin_amdgcn_bitop3_b32(a, b, c, 0x96); }

__device__ __forceinline__ v4u philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0, uint32_t k1)
{
#pragma unroll
    for (int r = 0; r < 10; ++r) {
        uint32_t hi0, lo0, hi1, lo1;
        mul_wide_u32(0xD2511F53u, c0, hi0, lo0);
        mul_wide_u32(0xCD9E8D57u, c2, hi1, lo1);
        c0 = xor3(hi1, c1, k0);
        c1 = lo1;
        c2 = xor3(hi0, c3, k1);
        c3 = lo0;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    v4u o = {c0, c1, c2, c3};
    return o;
}

// The same function for callers whose third counter word is the same in every lane (the head slice of a work-group):
// they pass its first-round product 0xCD9E8D57 * c2 as (c2_hi, c2_lo), computed once on the scalar unit, and the first
// round is left with one vector multiply; the exclusive-ors of uniform words fold into scalar ones as well.
__device__ __forceinline__ v4u philox4x32_10_c2(uint32_t c0, uint32_t c1, uint32_t c2_hi, uint32_t c2_lo, uint32_t c3, uint32_t k0,
                                                uint32_t k1)
{
    uint32_t hi0, lo0, hi1, lo1;
    // first Philox round
    mul_wide_u32(0xD2511F53u, c0, hi0, lo0);
    uint32_t n0 = c1 ^ (c2_hi ^ k0);
    const uint32_t u1 = c2_lo;  // uniform
    uint32_t n2 = hi0 ^ (c3 ^ k1);
    uint32_t n3 = lo0;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
    // second Philox round: its second word is still uniform
    mul_wide_u32(0xD2511F53u, n0, hi0, lo0);
    mul_wide_u32(0xCD9E8D57u, n2, hi1, lo1);
    c0 = hi1 ^ (u1 ^ k0);
    c1 = lo1;
    uint32_t c2 = xor3(hi0, n3, k1);
    c3 = lo0;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
#pragma unroll
    for (int r = 2; r < 10; ++r) {
        mul_wide_u32(0xD2511F53u, c0, hi0, lo0);
        mul_wide_u32(0xCD9E8D57u, c2, hi1, lo1);
        c0 = xor3(hi1, c1, k0);
        c1 = lo1;
        c2 = xor3(hi0, c3, k1);
        c3 = lo0;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    v4u o = {c0, c1, c2, c3};
    return o;
}

// Keep decisions of two scores at once: p2 holds their probabilities as packed fp16, w the two 16-bit Philox fields in the
// same halves, sub2 = threshold - 1 in both halves (threshold >= 1).  A saturating subtraction leaves a half non-zero
// iff field >= threshold; clipped to 1 it multiplies the fp16 bit pattern as an integer: the pattern, or zero.  Three
// packed instructions for two scores instead of a comparison and a select for each.
// (inline asm: from the same thing written with vector types the compiler recovers the comparison and emits a compare,
// a select and a byte permute per score)
__device__ __forceinline__ uint32_t keep_pair(uint32_t p2, uint32_t w, uint32_t sub2)
{
    uint32_t x;
    asm("v_pk_sub_u16 %0, %1, %2 clamp\n\tv_pk_min_u16 %0, %0, %3\n\tv_pk_mul_lo_u16 %0, %4, %0"
        : "=&v"(x)
        : "v"(w), "s"(sub2), "v"(0x00010001u), "v"(p2));
    return x;
}

// 16-bit field f (0..7) of a Philox output
__device__ __forceinline__ uint32_t philox_field16(const v4u& w, int f) { return (w[f >> 1] >> (16 * (f & 1))) & 0xffffu; }

// One KiB from global memory straight into LDS: lane l fetches 16 bytes at base + off (its own offset) and the wave
// writes them to lds_dst + 16 l.  Issued as inline asm on purpose: the compiler models the builtin form as a FLAT
// access that may touch LDS, and from then on degrades every LDS wait of the loop to "wait for everything".  The
// caller waits with s_waitcnt vmcnt(0) before the barrier that publishes the tile.
__device__ __forceinline__ void dma_kib(const char* base, uint32_t off, FA_LDS char* lds_dst)
{
    const uint32_t m0v = (uint32_t)(uintptr_t)lds_dst;
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(m0v), "v"(off), "s"(base)
                 : "memory", "m0");
}
// The same request marked non-temporal, for data that no other work-group will ask for (the K/V stream of a decode
// launch): measured 5.4 -> 6.3 TB/s on grouped-query decode with eight query heads per K/V head.
__device__ __forceinline__ void dma_kib_nt(const char* base, uint32_t off, FA_LDS char* lds_dst)
{
    const uint32_t m0v = (uint32_t)(uintptr_t)lds_dst;
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt"
                 :
                 : "s"(m0v), "v"(off), "s"(base)
                 : "memory", "m0");
}

// Launch with the error of THIS launch as the return value (hipGetLastError would also hand back whatever an
// unrelated earlier call of the process left behind).
template <typename T>
struct same_type { typedef T type; };
template <typename... P>
inline hipError_t launch_kernel(void (*kern)(P...), dim3 grid, dim3 block, size_t smem, hipStream_t st,
                                typename same_type<P>::type... args)
{
    void* argv[] = {static_cast<void*>(&args)...};
    return hipLaunchKernel(reinterpret_cast<const void*>(kern), grid, block, argv, smem, st);
}

// Raises the dynamic-LDS limit of a kernel once per device (the attribute belongs to the device's copy of the kernel).
// `done` is the caller's per-kernel flag array.  Concurrent first calls from several threads may both set the
// attribute, which is harmless; the flags are atomics so that such calls do not race in the language's sense either.
constexpr int kMaxDevices = 64;
typedef std::atomic<bool> DeviceFlags[kMaxDevices];
inline hipError_t ensure_dynamic_lds(const void* kern, int bytes, DeviceFlags& done)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= kMaxDevices) dev = kMaxDevices - 1;  // beyond the table: set it on every launch
    if (dev != kMaxDevices - 1 && done[dev].load(std::memory_order_acquire)) return hipSuccess;
    e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e == hipSuccess) done[dev].store(true, std::memory_order_release);
    return e;
}

}  // namespace fa
