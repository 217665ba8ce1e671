// Split-KV decode (one query row per head), split combine, and the stand-alone dropout keep-mask kernel.
//
// decode_split_kernel replaces forward_kernel_splitkv (src/flash_forward_splitkv.h:14-344) for Nq == 1, where the
// reference's 128-row MMA tile would waste 127 of 128 rows: the work is a pure stream over K and V, bound by HBM.
//   * one work-group per (head slice, split) -- per (G query heads of one K/V head, split) under grouped-query
//     attention, so that K and V are streamed once per K/V head; its 4 waves take blocks of the split's keys in turn
//   * a key row is spread over LPK lanes (16 bytes each), so one wave instruction reads 1 KiB of consecutive bytes
//   * q.k: v_dot2_f32_f16 per lane, then a DPP butterfly over the LPK lanes of the key (no LDS, no shuffles)
//   * online softmax per key group; p * V accumulated in fp32 per lane (8 head-dim columns per lane)
//   * key groups and waves are merged once at the end through LDS; partial O (normalised, fp32) and
//     LSE_s = m_s + log l_s go to the workspace (reference: O_tmp, M, L; src/flash_forward_splitkv.h:313-338)
// combine_kernel replaces forward_kernel_splitkv_combine (src/flash_forward_splitkv.h:347-399) with one wave per
// query row and coalesced reads of the partials (the reference uses one thread per row).
#include "common.h"
#include "decode_kernels.h"

namespace fa {

template <int CTRL>
__device__ __forceinline__ float dpp_mov(float v)
{
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}
// sum over the LPK consecutive lanes that share a key; every lane of the group ends with the total
template <int LPK>
__device__ __forceinline__ float group_sum(float v)
{
    v += dpp_mov<0xB1>(v);                          // quad_perm [1,0,3,2]
    v += dpp_mov<0x4E>(v);                          // quad_perm [2,3,0,1]
    if constexpr (LPK >= 8) v += dpp_mov<0x141>(v);   // row_half_mirror
    if constexpr (LPK >= 16) v += dpp_mov<0x140>(v);  // row_mirror
    return v;
}

// G = query heads served by one work-group: the G consecutive heads share one K/V head (grouped-query attention), so
// the K/V stream is read once for all of them.  G == 1 is the plain one-K/V-head-per-query-head case.
template <int LPK, bool kAlibi, int G>
__global__ void __launch_bounds__(256) decode_split_kernel(const FwdArgs a)
{
    constexpr int KPI = 64 / LPK;      // keys per wave instruction
    constexpr int U = G > 2 ? 4 : 8;   // load instructions in flight per tensor
    constexpr int KB = U * KPI;        // keys per wave block
    constexpr int NG = 4 * KPI;        // key groups per work-group
    constexpr int DB = LPK * 8;        // head-dim bucket
    __shared__ float s_acc[NG][DB];
    __shared__ float s_m[NG], s_l[NG];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = wave_uniform(tid >> 6);
    const int c = lane % LPK;
    const int kg = lane / LPK;
    const int BHG = a.B * a.H / G;
    const int bh0 = (blockIdx.x % BHG) * G;  // first of the G query slices of this work-group
    const int split = blockIdx.x / BHG;
    const int d = a.d, Nk = a.Nk;
    // Rows of any length from eight elements on, at any 2-byte alignment: a lane behind the row's whole chunks works
    // on the row's last 16 bytes, columns d - 8 ... d - 1 (no load leaves the row), with q zeroed where the lane before
    // has covered a column already; lanes past the row do the same with q = 0.
    const int col = 8 * c;
    const int colc = col + 8 <= d ? col : d - 8;

    union U8 { v4u u; v8h h; v2h p[4]; };
    U8 qv[G];
#pragma unroll
    for (int gq = 0; gq < G; ++gq)
        qv[gq].h = mask_q_chunk_anyalign(*reinterpret_cast<const v4u_anyalign*>(a.Q + (size_t)(bh0 + gq) * d + colc), col, d);

    // the single query row sits at position ii = Nk - 1 (row index i + Nk - Nq): causal / right window never cut
    const int ii = Nk - 1;
    int kstart = a.wl >= 0 ? max(0, ii - a.wl) : 0;
    int kend = Nk;
    if (a.num_splits > 1) {
        kstart = max(kstart, split * a.keys_per_split);
        kend = min(kend, (split + 1) * a.keys_per_split);
    }
    const int kvs = a.kv_slice(bh0);
    const half_t* __restrict__ Kbh = a.K + (size_t)kvs * Nk * d + colc;
    const half_t* __restrict__ Vbh = a.V + (size_t)kvs * Nk * d + colc;
    const float c2 = a.scale_log2;
    float slope2[G];
#pragma unroll
    for (int gq = 0; gq < G; ++gq) {
        slope2[gq] = 0.0f;
        if constexpr (kAlibi) slope2[gq] = a.alibi ? a.alibi[(bh0 + gq) % a.H] * kLog2e : 0.0f;
    }

    float m[G], l[G];
    float acc[G][8];
#pragma unroll
    for (int gq = 0; gq < G; ++gq) {
        m[gq] = -INFINITY;
        l[gq] = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[gq][e] = 0.0f;
    }

    // The key loop is double-buffered by hand: the 2 U loads of the wave's next block (16 bytes per lane each) are issued
    // before the current block is consumed, and a scheduling fence keeps them there.  Left to the compiler the loop
    // waited for every K row before requesting the next one (eight memory round trips in series per block: a lone
    // work-group streamed 13 GB/s).
    auto load_block = [&](int kb, U8 (&kr)[U], U8 (&vr)[U]) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < U; ++i) {
            const int j = kb + i * KPI + kg;
            const size_t off = (size_t)(j < kend ? j : kend - 1) * d;
            // (non-temporal: K and V are read once; as ordinary loads they measured 5.9 instead of 6.8 TB/s)
            kr[i].u = __builtin_nontemporal_load(reinterpret_cast<const v4u_anyalign*>(Kbh + off));
        }
#pragma unroll
        for (int i = 0; i < U; ++i) {
            const int j = kb + i * KPI + kg;
            const size_t off = (size_t)(j < kend ? j : kend - 1) * d;
            vr[i].u = __builtin_nontemporal_load(reinterpret_cast<const v4u_anyalign*>(Vbh + off));
        }
    };
    auto consume = [&](int kb, const U8 (&kr)[U], const U8 (&vr)[U]) __attribute__((always_inline)) {
#pragma unroll
        for (int gq = 0; gq < G; ++gq) {
            float t[U];
            float mb = -INFINITY;
#pragma unroll
            for (int i = 0; i < U; ++i) {
                float s = 0.0f;
#pragma unroll
                for (int e = 0; e < 4; ++e) s = __builtin_amdgcn_fdot2(qv[gq].p[e], kr[i].p[e], s, false);
                s = group_sum<LPK>(s);
                const int j = kb + i * KPI + kg;
                float tv = s * c2;
                if constexpr (kAlibi) tv -= slope2[gq] * (float)(ii - j);
                if (j >= kend) tv = -INFINITY;
                t[i] = tv;
                mb = fmaxf(mb, tv);
            }
            const float m_new = fmaxf(m[gq], mb);
            const float m_use = (m_new == -INFINITY) ? 0.0f : m_new;
            const float alpha = fast_exp2(m[gq] - m_use);
            m[gq] = m_new;
            float rs = 0.0f;
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[gq][e] *= alpha;
#pragma unroll
            for (int i = 0; i < U; ++i) {
                const float p = fast_exp2(t[i] - m_use);
                rs += p;
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[gq][e] = __builtin_fmaf(p, (float)vr[i].h[e], acc[gq][e]);
            }
            l[gq] = l[gq] * alpha + rs;
        }
    };
    {
        U8 k0[U], v0[U], k1[U], v1[U];
        int kb = kstart + wave * KB;  // wave-uniform
        if (kb < kend) load_block(kb, k0, v0);
        while (kb < kend) {
            const int kb1 = kb + 4 * KB;
            if (kb1 < kend) load_block(kb1, k1, v1);
            __builtin_amdgcn_sched_barrier(0);
            consume(kb, k0, v0);
            if (kb1 >= kend) break;
            const int kb2 = kb1 + 4 * KB;
            if (kb2 < kend) load_block(kb2, k0, v0);
            __builtin_amdgcn_sched_barrier(0);
            consume(kb1, k1, v1);
            kb = kb2;
        }
    }

    // ---- merge the NG key groups of the work-group, one query head after the other through the same LDS buffer
    const int grp = wave * KPI + kg;
#pragma unroll
    for (int gq = 0; gq < G; ++gq) {
        if (gq > 0) __syncthreads();
#pragma unroll
        for (int e = 0; e < 8; ++e) s_acc[grp][col + e] = acc[gq][e];
        if (c == 0) {
            s_m[grp] = m[gq];
            s_l[grp] = l[gq];
        }
        __syncthreads();
        if (tid < DB) {
            const int bh = bh0 + gq;
            float M = -INFINITY;
#pragma unroll
            for (int gI = 0; gI < NG; ++gI) M = fmaxf(M, s_m[gI]);
            const float Mu = (M == -INFINITY) ? 0.0f : M;
            float L = 0.0f, o = 0.0f;
#pragma unroll
            for (int gI = 0; gI < NG; ++gI) {
                const float w = fast_exp2(s_m[gI] - Mu);
                L += w * s_l[gI];
                o += w * s_acc[gI][tid];
            }
            const float inv = L > 0.0f ? 1.0f / L : 0.0f;
            const float lse = L > 0.0f ? __builtin_fmaf(M, kLn2, fast_log2(L) * kLn2) : -INFINITY;
            // column of position tid: the eight positions behind the row's whole chunks hold columns d - 8 ... d - 1, of
            // which the first 8 - d % 8 were written by the positions before
            const int c0 = d & ~7, rem = d & 7;
            const int tcol = tid < c0 ? tid : tid - (8 - rem);
            const bool ok = tid < c0 || (rem != 0 && tid < c0 + 8 && tcol >= c0);
            if (a.num_splits > 1) {
                const size_t prow = (size_t)bh * a.num_splits + split;  // Nq == 1
                if (ok) a.O_partial[prow * d + tcol] = o * inv;
                if (tid == 0) a.LSE_partial[prow] = lse;
            } else {
                if (ok) a.O[(size_t)bh * d + tcol] = (half_t)(o * inv);
                if (tid == 0) a.LSE[bh] = lse;
            }
        }
    }
}

// Reductions over the 64 lanes of a wave without LDS: DPP inside the rows of 16 lanes, v_permlane32_swap between the
// halves, v_readlane for the last two rows; the result is wave-uniform.
__device__ __forceinline__ float wave_sum(float v)
{
    v = xhalf_sum(group_sum<16>(v));  // lanes of rows r and r ^ 2 now hold the total of both rows
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0)) +
           __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
}
__device__ __forceinline__ float wave_max(float v)
{
    v = fmaxf(v, dpp_mov<0xB1>(v));
    v = fmaxf(v, dpp_mov<0x4E>(v));
    v = fmaxf(v, dpp_mov<0x141>(v));
    v = fmaxf(v, dpp_mov<0x140>(v));
    v = xhalf_max(v);
    return fmaxf(__int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0)),
                 __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16)));
}

// One wave per query row: LSE = logsumexp_s LSE_s, O = sum_s exp(LSE_s - LSE) O_s
// (same value as m = max M_s, l = sum e^{M_s-m} L_s, O = sum (L_s e^{M_s-m} / l) O_s of splitkv.h:359-397).
// The weights of a row live in LDS that only its wave touches, so no work-group barrier is needed.  With d % 8 == 0
// a lane holds four consecutive columns, the two halves of the wave take the even and the odd splits, and the first
// partial rows are requested before the log-sum-exp values they will be weighted with.
__global__ void __launch_bounds__(256) combine_kernel(const float* __restrict__ O_partial,
                                                      const float* __restrict__ LSE_partial, half_t* __restrict__ O,
                                                      float* __restrict__ LSE, int BH, int Nq, int d, int S)
{
    __shared__ float s_w[4][FLASH_MAX_SPLITS_K];
    const int lane = threadIdx.x & 63;
    const int wave = wave_uniform(threadIdx.x >> 6);
    const long long row = (long long)blockIdx.x * 4 + wave;
    if (row >= (long long)BH * Nq) return;
    const int bh = (int)(row / Nq), i = (int)(row % Nq);
    const float* lp = LSE_partial + (size_t)bh * S * Nq + i;  // stride Nq between splits
    const size_t sstride = (size_t)Nq * d;                     // floats between the partial rows of two splits
    const float* op = O_partial + ((size_t)bh * S * Nq + i) * d;
    const bool vec = (d & 7) == 0;  // rows of the partials and of O are 16-byte aligned (the host checks the bases)
    constexpr int U = 8;            // partial rows in flight per half-wave
    const int c4 = (lane & 31) * 4, grp = lane >> 5;
    const bool act = c4 < d;
    float4 pre[U];
    if (vec) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int s = grp + 2 * u;
            pre[u] = (act && s < S) ? *reinterpret_cast<const float4*>(op + s * sstride + c4) : float4{0.f, 0.f, 0.f, 0.f};
        }
    }
    float mx = -INFINITY;
    for (int s = lane; s < S; s += 64) mx = fmaxf(mx, lp[(size_t)s * Nq]);
    mx = wave_max(mx);
    const float mu = (mx == -INFINITY) ? 0.0f : mx;
    float sum = 0.0f;
    for (int s = lane; s < S; s += 64) {
        const float w = __expf(lp[(size_t)s * Nq] - mu);
        s_w[wave][s] = w;
        sum += w;
    }
    sum = wave_sum(sum);
    const float inv = sum > 0.0f ? 1.0f / sum : 0.0f;
    if (lane == 0) LSE[(size_t)bh * Nq + i] = sum > 0.0f ? mx + __logf(sum) : -INFINITY;
    if (vec) {
        float4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int s = grp + 2 * u;
            const float w = s < S ? s_w[wave][s] : 0.0f;
            acc.x += w * pre[u].x, acc.y += w * pre[u].y, acc.z += w * pre[u].z, acc.w += w * pre[u].w;
        }
        // the remaining partial rows, U at a time, requested together (one by one, every request waited for its
        // predecessor's arithmetic: with 64 splits and more the combine took longer than the split kernel)
        for (int s0 = grp + 2 * U; s0 < S; s0 += 2 * U) {  // (wave-uniform trip count: the first half-wave's)
            float4 nxt[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int s = s0 + 2 * u;
                nxt[u] = (act && s < S) ? *reinterpret_cast<const float4*>(op + s * sstride + c4) : float4{0.f, 0.f, 0.f, 0.f};
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int s = s0 + 2 * u;
                const float w = s < S ? s_w[wave][s] : 0.0f;
                acc.x += w * nxt[u].x, acc.y += w * nxt[u].y, acc.z += w * nxt[u].z, acc.w += w * nxt[u].w;
            }
        }
        acc.x = xhalf_sum(acc.x), acc.y = xhalf_sum(acc.y), acc.z = xhalf_sum(acc.z), acc.w = xhalf_sum(acc.w);
        if (act && grp == 0) {
            union { v2h h[2]; uint2 u; } r;
            r.h[0] = pack_f16(acc.x * inv, acc.y * inv);
            r.h[1] = pack_f16(acc.z * inv, acc.w * inv);
            *reinterpret_cast<uint2*>(O + ((size_t)bh * Nq + i) * d + c4) = r.u;
        }
    } else {
        for (int dc = lane; dc < d; dc += 64) {
            float o = 0.0f;
            for (int s = 0; s < S; ++s) o += s_w[wave][s] * op[s * sstride + dc];
            O[((size_t)bh * Nq + i) * d + dc] = (half_t)(o * inv);
        }
    }
}

// keep[b,h,i,j] = (16-bit field dropout_field(j) of the Philox call dropout_call(j) of row (b*H + h, i)) >= threshold;
// one thread per call, i.e. per eight keys: 16*(c >> 1) + 8*r2 + 4*(c & 1) + e
__global__ void __launch_bounds__(256) keep_mask_kernel(uint8_t* __restrict__ mask, long long rows, int Nq, int Nk,
                                                        uint32_t thr, uint32_t seed_lo, uint32_t seed_hi,
                                                        uint32_t off_lo)
{
    const int calls = 2 * ((Nk + 15) >> 4);
    const long long total = rows * calls;
    for (long long idx = (long long)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (long long)gridDim.x * 256) {
        const long long r = idx / calls;
        const int c = (int)(idx % calls);
        const uint32_t bh = (uint32_t)(r / Nq), i = (uint32_t)(r % Nq);
        const v4u w = philox4x32_10((uint32_t)c, i, bh, off_lo, seed_lo, seed_hi);
        uint8_t* mrow = mask + (size_t)r * Nk;
#pragma unroll
        for (int f = 0; f < 8; ++f) {
            const int j = 16 * (c >> 1) + 8 * (f >> 2) + 4 * (c & 1) + (f & 3);
            if (j < Nk) mrow[j] = philox_field16(w, f) >= thr ? 1 : 0;
        }
    }
}

template <int LPK, int G>
static hipError_t launch_decode_instance(const FwdArgs& a, hipStream_t st)
{
    const unsigned groups = (unsigned)((long long)a.B * a.H / G * a.num_splits);
    if (a.alibi != nullptr) return launch_kernel(decode_split_kernel<LPK, true, G>, dim3(groups), dim3(256), 0, st, a);
    return launch_kernel(decode_split_kernel<LPK, false, G>, dim3(groups), dim3(256), 0, st, a);
}

template <int LPK>
static hipError_t launch_decode_bucket(const FwdArgs& a, hipStream_t st)
{
    // as many of the query heads of a K/V head per work-group as divide the group (up to 8)
    if (a.kv_group % 8 == 0) return launch_decode_instance<LPK, 8>(a, st);
    if (a.kv_group % 4 == 0) return launch_decode_instance<LPK, 4>(a, st);
    if (a.kv_group % 2 == 0) return launch_decode_instance<LPK, 2>(a, st);
    return launch_decode_instance<LPK, 1>(a, st);
}

int launch_decode_split(const FwdArgs& a, hipStream_t st)
{
    if (a.d > 64) return (int)launch_decode_bucket<16>(a, st);
    if (a.d > 32) return (int)launch_decode_bucket<8>(a, st);
    return (int)launch_decode_bucket<4>(a, st);
}

int launch_combine(const FwdArgs& a, hipStream_t st)
{
    const long long rows = (long long)a.B * a.H * a.Nq;
    const unsigned groups = (unsigned)((rows + 3) / 4);
    return (int)launch_kernel(combine_kernel, dim3(groups), dim3(256), 0, st, a.O_partial, a.LSE_partial, a.O, a.LSE,
                              a.B * a.H, a.Nq, a.d, a.num_splits);
}

int launch_keep_mask(uint8_t* mask, int B, int H, int Nq, int Nk, uint32_t thr, uint64_t seed, uint64_t offset,
                     hipStream_t st)
{
    const long long rows = (long long)B * H * Nq;
    const long long total = rows * (2 * ((Nk + 15) / 16));  // one thread per Philox call
    long long groups = (total + 255) / 256;
    if (groups > 65536) groups = 65536;
    if (groups < 1) groups = 1;
    return (int)launch_kernel(keep_mask_kernel, dim3((unsigned)groups), dim3(256), 0, st, mask, rows, Nq, Nk, thr,
                              (uint32_t)seed, (uint32_t)(seed >> 32), (uint32_t)offset);
}

}  // namespace fa
