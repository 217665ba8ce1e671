/*
 * CPU oracle for the FlashAttention-forward hot path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is the checker, never the product: only the test-suite, the smoke
 * check and the CPU-baseline leg of the benchmark may load it.  The shipped
 * library (flash_attn_amd/csrc) neither links nor falls back to it.
 *
 * Every function restates, in plain C and fp32, what the reference computes on
 * its own CPU verification path, and cites the reference lines it follows
 * (paths relative to the reference checkout):
 *
 *   oracle_attention_forward   src/main.cu:279-388   attention_forward_cpu
 *   oracle_splitkv_partials    src/flash_forward_splitkv.h:40-52, 313-338
 *   oracle_splitkv_combine     src/flash_forward_splitkv.h:359-397
 *   oracle_num_splits_heuristic src/main.cu:391-422
 *   oracle_verify_count        src/main.cu:254-276   verfiy
 *   oracle_alibi_slopes        src/main.cu:61-67     (sign: positive, see below)
 *   oracle_philox4x32_10 / oracle_dropout_keep_mask
 *                              src/flash_forward.h:221-237 (drop rule), Philox
 *                              constants as in Random123 / cuRAND / rocRAND.
 *
 * How each function is pinned (tests/test_oracle*.py):
 *   attention (plain, causal, symmetric window, ALiBi): bit-exact against the
 *     reference's attention_forward_cpu compiled from the reference checkout
 *     (oracle/_ref, when present) and against golden vectors written from it;
 *     float64 brute force on small shapes.
 *   asymmetric window, Nq != Nk, LSE, explicit keep-mask: float64 brute force,
 *     closed forms (sum_j exp(s_ij - LSE_i) == 1, left=inf,right=0 == causal).
 *   split partials / combine: independence of the split count, equality with
 *     the unsplit result.
 *   heuristic: table generated from the compiled reference function.
 *   Philox: Random123 known-answer vectors.
 *   oracle_fill_normal_f16 (portable N(0,1) inputs; no counterpart in the reference, which fills U(0,10) from
 *     std::default_random_engine, src/main.cu:91-97): known bit patterns, moments, invariance under the first element.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORACLE_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------------- */
/* One query row.  Operation order follows src/main.cu:309-383 exactly:
 *   s = (sum_k q_k K_jk) * scale        (k ascending, fp32)          :311-315
 *   s -= slope * |i - j|                                             :320-327
 *   causal  j > i           -> -inf                                  :330-338
 *   window  |i - j| > w     -> -inf  (here: i-j > left || j-i > right) :340-349
 *   m = max_j s; e = expf(s - m); l = sum_j e (j ascending); p = e / l  :352-372
 *   O_k = sum_j p_j V_jk    (j ascending)                            :375-383
 * Extensions that the reference's CPU path lacks and the device contract has:
 *   ii = i + (Nk - Nq) replaces i in every mask/bias formula (equal when
 *   Nq == Nk, the only case the reference can express); LSE = m + logf(l);
 *   keep-mask dropout p_j <- keep_j ? p_j * (1/(1-p)) : 0 with the row sum l
 *   left undropped (src/flash_forward.h:191-237); a fully masked row yields
 *   O = 0 and LSE = -inf instead of the reference's NaN.
 * With skip_masked != 0 the dot products of masked columns are not evaluated;
 * they contribute exactly +0 to l and to O, so results are bit-identical.
 */
static void attention_row(const float *q, const float *K, const float *V, int i, int Nq, int Nk, int d,
                          float scale, int causal, int wl, int wr, int has_slope, float slope,
                          const uint8_t *keep_row, float p_drop, float *row, float *out, float *lse,
                          int skip_masked)
{
    const int ii = i + (Nk - Nq);
    int jlo = 0, jhi = Nk - 1; /* inclusive range of unmasked columns */
    if (causal && ii < jhi) jhi = ii;
    if (wr >= 0 && ii + wr < jhi) jhi = ii + wr;
    if (wl >= 0 && ii - wl > jlo) jlo = ii - wl;

    const int c0 = skip_masked ? jlo : 0;
    const int c1 = skip_masked ? jhi : Nk - 1;
    if (skip_masked) {
        for (int j = 0; j < Nk; ++j) row[j] = -INFINITY;
    }
    int j = c0;
    /* four independent k-ascending chains at a time: same per-element order */
    for (; j + 3 <= c1; j += 4) {
        const float *k0 = K + (size_t)j * d, *k1 = k0 + d, *k2 = k1 + d, *k3 = k2 + d;
        float s0 = 0.0f, s1 = 0.0f, s2 = 0.0f, s3 = 0.0f;
        for (int k = 0; k < d; ++k) {
            const float qk = q[k];
            s0 += qk * k0[k];
            s1 += qk * k1[k];
            s2 += qk * k2[k];
            s3 += qk * k3[k];
        }
        row[j] = s0 * scale;
        row[j + 1] = s1 * scale;
        row[j + 2] = s2 * scale;
        row[j + 3] = s3 * scale;
    }
    for (; j <= c1; ++j) {
        const float *kj = K + (size_t)j * d;
        float s = 0.0f;
        for (int k = 0; k < d; ++k) s += q[k] * kj[k];
        row[j] = s * scale;
    }
    if (has_slope) {
        for (j = c0; j <= c1; ++j) row[j] -= slope * abs(ii - j);
    }
    if (!skip_masked) {
        if (causal)
            for (j = 0; j < Nk; ++j)
                if (j > ii) row[j] = -INFINITY;
        for (j = 0; j < Nk; ++j)
            if ((wl >= 0 && ii - j > wl) || (wr >= 0 && j - ii > wr)) row[j] = -INFINITY;
    }

    float max_val = -INFINITY;
    for (j = 0; j < Nk; ++j) max_val = row[j] > max_val ? row[j] : max_val;
    if (max_val == -INFINITY) { /* nothing to attend to */
        for (int k = 0; k < d; ++k) out[k] = 0.0f;
        if (lse) *lse = -INFINITY;
        return;
    }
    float sum = 0.0f;
    for (j = 0; j < Nk; ++j) {
        row[j] = expf(row[j] - max_val);
        sum += row[j];
    }
    for (j = 0; j < Nk; ++j) row[j] /= sum;
    if (lse) *lse = max_val + logf(sum);
    if (keep_row) {
        const float rescale = 1.0f / (1.0f - p_drop);
        for (j = 0; j < Nk; ++j) row[j] = keep_row[j] ? row[j] * rescale : 0.0f;
    }
    for (int k = 0; k < d; ++k) out[k] = 0.0f;
    for (j = c0; j <= c1; ++j) {
        const float pj = row[j];
        const float *vj = V + (size_t)j * d;
        for (int k = 0; k < d; ++k) out[k] += pj * vj[k];
    }
}

/* Q [B,H,Nq,d], K,V [B,H,Nk,d], O [B,H,Nq,d], LSE [B,H,Nq] (may be NULL), all fp32, contiguous.
 * window_left / window_right < 0 mean unbounded on that side (reference: window_size = -1 is "off").
 * slopes [H] or NULL; keep_mask [B,H,Nq,Nk] bytes or NULL.  slice_begin/slice_end select a range of
 * (b*H + h) slices so that a bounded sample can be timed.  Returns 0, or -1 on allocation failure. */
ORACLE_API int oracle_attention_forward_slices(const float *Q, const float *K, const float *V, int B, int H, int Nq,
                                               int Nk, int d, float scale, int causal, int window_left,
                                               int window_right, const float *slopes, const uint8_t *keep_mask,
                                               float p_drop, float *O, float *LSE, int nthreads, int skip_masked,
                                               int slice_begin, int slice_end)
{
    (void)B;
    if (nthreads < 1) nthreads = 1;
    const long long rows = (long long)(slice_end - slice_begin) * Nq;
    int failed = 0;
#pragma omp parallel num_threads(nthreads)
    {
        float *row = (float *)malloc(sizeof(float) * (size_t)(Nk > 0 ? Nk : 1));
        if (!row) {
#pragma omp atomic write
            failed = 1;
        }
#pragma omp for schedule(dynamic, 16)
        for (long long r = 0; r < rows; ++r) {
            if (!row) continue;
            const int bh = slice_begin + (int)(r / Nq);
            const int i = (int)(r % Nq);
            const int h = bh % H;
            const float *q = Q + ((size_t)bh * Nq + i) * d;
            const float *Kp = K + (size_t)bh * Nk * d;
            const float *Vp = V + (size_t)bh * Nk * d;
            const uint8_t *kr = keep_mask ? keep_mask + ((size_t)bh * Nq + i) * Nk : NULL;
            attention_row(q, Kp, Vp, i, Nq, Nk, d, scale, causal, window_left, window_right, slopes != NULL,
                          slopes ? slopes[h] : 0.0f, kr, p_drop, row, O + ((size_t)bh * Nq + i) * d,
                          LSE ? LSE + (size_t)bh * Nq + i : NULL, skip_masked);
        }
        free(row);
    }
    return failed ? -1 : 0;
}

ORACLE_API int oracle_attention_forward(const float *Q, const float *K, const float *V, int B, int H, int Nq, int Nk,
                                        int d, float scale, int causal, int window_left, int window_right,
                                        const float *slopes, const uint8_t *keep_mask, float p_drop, float *O,
                                        float *LSE, int nthreads)
{
    return oracle_attention_forward_slices(Q, K, V, B, H, Nq, Nk, d, scale, causal, window_left, window_right, slopes,
                                           keep_mask, p_drop, O, LSE, nthreads, 1, 0, B * H);
}

/* ------------------------------------------------------------------------- */
/* Split-KV.  Key range of split s, at the reference's 128-key block granularity
 * (src/flash_forward_splitkv.h:40-43): blocks_per_split = ceil(ceil(Nk/128)/S),
 * split s owns key blocks [bps*s, min(bps*(s+1), Tc)). */
ORACLE_API void oracle_split_key_range(int Nk, int num_splits, int s, int *begin, int *end)
{
    const int total = (Nk + 127) / 128;
    const int bps = (total + num_splits - 1) / num_splits;
    int b0 = bps * s, b1 = b0 + bps;
    if (b1 > total) b1 = total;
    if (b0 > total) b0 = total;
    int k0 = b0 * 128, k1 = b1 * 128;
    if (k1 > Nk) k1 = Nk;
    if (k0 > Nk) k0 = Nk;
    *begin = k0;
    *end = k1;
}

/* Per-split partial results, as the reference's split kernel leaves them
 * (src/flash_forward_splitkv.h:313-338): O_tmp = (sum_{j in split} e^{s_ij - m_s} V_j) / l_s, the running sum l_s
 * and the running max m_s.  Layouts: O_tmp [B,H,S,Nq,d], Lsum / Mmax / LSE_partial [B,H,S,Nq].  LSE_partial
 * (= m_s + logf(l_s), -inf for an empty split) is the form the device workspace stores; any output may be NULL. */
ORACLE_API int oracle_splitkv_partials(const float *Q, const float *K, const float *V, int B, int H, int Nq, int Nk,
                                       int d, float scale, int causal, int window_left, int window_right,
                                       const float *slopes, int num_splits, float *O_tmp, float *Lsum, float *Mmax,
                                       float *LSE_partial, int nthreads)
{
    if (nthreads < 1) nthreads = 1;
    const long long rows = (long long)B * H * num_splits * Nq;
#pragma omp parallel for num_threads(nthreads) schedule(dynamic, 16)
    for (long long r = 0; r < rows; ++r) {
        const int i = (int)(r % Nq);
        const int s = (int)((r / Nq) % num_splits);
        const int bh = (int)(r / ((long long)Nq * num_splits));
        const int h = bh % H;
        int k0, k1;
        oracle_split_key_range(Nk, num_splits, s, &k0, &k1);
        const float *q = Q + ((size_t)bh * Nq + i) * d;
        const float *Kp = K + (size_t)bh * Nk * d;
        const float *Vp = V + (size_t)bh * Nk * d;
        const int ii = i + (Nk - Nq);
        float m = -INFINITY, l = 0.0f;
        float *acc = (float *)calloc((size_t)d, sizeof(float));
        float *sc = (float *)malloc(sizeof(float) * (size_t)(k1 > k0 ? k1 - k0 : 1));
        for (int j = k0; j < k1; ++j) {
            float sum = 0.0f;
            for (int k = 0; k < d; ++k) sum += q[k] * Kp[(size_t)j * d + k];
            float sv = sum * scale;
            if (slopes) sv -= slopes[h] * abs(ii - j);
            if (causal && j > ii) sv = -INFINITY;
            if ((window_left >= 0 && ii - j > window_left) || (window_right >= 0 && j - ii > window_right))
                sv = -INFINITY;
            sc[j - k0] = sv;
            m = sv > m ? sv : m;
        }
        if (m != -INFINITY) {
            for (int j = k0; j < k1; ++j) {
                const float e = expf(sc[j - k0] - m);
                l += e;
                for (int k = 0; k < d; ++k) acc[k] += e * Vp[(size_t)j * d + k];
            }
        }
        const size_t o = (((size_t)bh * num_splits + s) * Nq + i);
        if (O_tmp)
            for (int k = 0; k < d; ++k) O_tmp[o * d + k] = (l != 0.0f) ? acc[k] / l : 0.0f;
        if (Lsum) Lsum[o] = l;
        if (Mmax) Mmax[o] = m;
        if (LSE_partial) LSE_partial[o] = (l != 0.0f) ? m + logf(l) : -INFINITY;
        free(acc);
        free(sc);
    }
    return 0;
}

/* Combine, restating src/flash_forward_splitkv.h:359-397:
 *   m = max_s M_s ; l = sum_s expf(M_s - m) L_s ; O = sum_s (L_s expf(M_s - m) / l) O_tmp_s   (0 when l == 0)
 * plus LSE = m + logf(l) for the device contract.  Same layouts as above; O [B,H,Nq,d], LSE [B,H,Nq]. */
ORACLE_API void oracle_splitkv_combine(const float *O_tmp, const float *Lsum, const float *Mmax, int B, int H, int Nq,
                                       int d, int num_splits, float *O, float *LSE)
{
    for (long long bh = 0; bh < (long long)B * H; ++bh) {
        for (int i = 0; i < Nq; ++i) {
            float m = -INFINITY;
            for (int s = 0; s < num_splits; ++s) {
                const float ms = Mmax[((size_t)bh * num_splits + s) * Nq + i];
                m = ms > m ? ms : m;
            }
            float l = 0.0f;
            for (int s = 0; s < num_splits; ++s) {
                const size_t o = ((size_t)bh * num_splits + s) * Nq + i;
                if (Lsum[o] != 0.0f) l += expf(Mmax[o] - m) * Lsum[o];
            }
            float *out = O + ((size_t)bh * Nq + i) * d;
            for (int k = 0; k < d; ++k) out[k] = 0.0f;
            for (int s = 0; s < num_splits; ++s) {
                const size_t o = ((size_t)bh * num_splits + s) * Nq + i;
                if (Lsum[o] == 0.0f) continue;
                float factor = (l != 0.0f) ? (1.0f / l) : 0.0f;
                factor *= Lsum[o] * expf(Mmax[o] - m);
                for (int k = 0; k < d; ++k) out[k] += factor * O_tmp[o * d + k];
            }
            if (LSE) LSE[(size_t)bh * Nq + i] = (l != 0.0f) ? m + logf(l) : -INFINITY;
        }
    }
}

/* ------------------------------------------------------------------------- */
/* Split-count heuristic, restating src/main.cu:391-422 statement by statement. */
ORACLE_API int oracle_num_splits_heuristic(int batch_nheads_mblocks, int num_SMs, int num_n_blocks, int max_splits,
                                           int seq_len)
{
    if (batch_nheads_mblocks >= 4.0f * num_SMs) return 1;
    if (num_SMs < max_splits) max_splits = num_SMs;
    if (num_n_blocks < max_splits) max_splits = num_n_blocks;
    if (max_splits < 1) return 1;
    float max_efficiency = 0.f;
    float *efficiency = (float *)malloc(sizeof(float) * (size_t)max_splits);
    if (!efficiency) return 1;
#define CEILDIV(a, b) (((a) + (b)-1) / (b))
#define ELIGIBLE(s) \
    (((s) == 1 || CEILDIV(num_n_blocks, (s)) != CEILDIV(num_n_blocks, (s)-1)) && (seq_len % (128 * (s)) == 0))
    for (int s = 1; s <= max_splits; s++) {
        if (!ELIGIBLE(s)) {
            efficiency[s - 1] = 0.f;
        } else {
            float n_waves = (float)(batch_nheads_mblocks * s) / num_SMs;
            float eff = n_waves / ceilf(n_waves);
            if (eff > max_efficiency) max_efficiency = eff;
            efficiency[s - 1] = eff;
        }
    }
    int chosen = 1;
    for (int s = 1; s <= max_splits; s++) {
        if (!ELIGIBLE(s)) continue;
        if (efficiency[s - 1] >= 0.85 * max_efficiency) {
            chosen = s;
            break;
        }
    }
#undef ELIGIBLE
#undef CEILDIV
    free(efficiency);
    return chosen;
}

/* verfiy (src/main.cu:254-276): number of elements whose signed relative error exceeds the bound or whose device
 * value is NaN/Inf.  The denominator is the signed CPU value, as in the reference. */
ORACLE_API long long oracle_verify_count(const float *O_cpu, const float *O_dev, long long n, float range_of_error)
{
    long long error = 0;
    for (long long i = 0; i < n; i++) {
        float device_out = O_dev[i];
        if ((fabsf(O_dev[i] - O_cpu[i])) / O_cpu[i] > range_of_error || isnan(device_out) || isinf(device_out))
            error++;
    }
    return error;
}

/* Per-head ALiBi slopes 2^(-8 (h+1) / H), formula of src/main.cu:65-67 taken with a positive sign: the operator
 * subtracts slope * |i - j| (src/main.cu:324, src/flash_forward.h:173), so positive slopes give the usual penalty. */
ORACLE_API void oracle_alibi_slopes(int H, float *slopes)
{
    for (int i = 0; i < H; i++) slopes[i] = (float)pow(2, -8.0 / H * (i + 1));
}

/* ------------------------------------------------------------------------- */
/* Philox4x32-10 (Salmon et al., Random123; same constants as cuRAND's curandStatePhilox4_32_10_t, which the
 * reference draws from at src/flash_forward.h:227). */
ORACLE_API void oracle_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4])
{
    uint32_t c0 = ctr[0], c1 = ctr[1], c2 = ctr[2], c3 = ctr[3];
    uint32_t k0 = key[0], k1 = key[1];
    for (int r = 0; r < 10; ++r) {
        const uint64_t p0 = (uint64_t)0xD2511F53u * c0;
        const uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
        const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
        const uint32_t n1 = (uint32_t)p1;
        const uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
        const uint32_t n3 = (uint32_t)p0;
        c0 = n0; c1 = n1; c2 = n2; c3 = n3;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

/* Integer drop threshold: an element is kept iff its 16-bit random field >= floor(p * 2^16).  This is the reference's
 * rule "drop iff uniform < p" (src/flash_forward.h:227-234) stated on raw bits, so that no float rounding enters. */
ORACLE_API uint32_t oracle_dropout_threshold(float p)
{
    double t = floor((double)p * 65536.0);
    if (!(t > 0.0)) t = 0.0;
    if (t > 65535.0) t = 65535.0;
    return (uint32_t)t;
}

/* Keep-mask of the device contract.  One Philox call yields eight 16-bit fields (field f = bits 16*(f&1).. of output
 * word f>>1) and serves eight keys of one query row: key = (lo32(seed), hi32(seed)), counter =
 * (call(j), i, b*H + h, lo32(offset)) with call(j) = 2*(j >> 4) + ((j >> 2) & 1), and element (i, j) reads field
 * 4*((j >> 3) & 1) + (j & 3).  (Of every 16 consecutive keys, the call with odd index serves keys 4-7 and 12-15: the
 * eight keys whose scores one lane of the device kernel holds.)  mask [B,H,Nq,Nk] bytes, 1 = keep. */
ORACLE_API void oracle_dropout_keep_mask(uint64_t seed, uint64_t offset, float p, int B, int H, int Nq, int Nk,
                                         uint8_t *mask, int nthreads)
{
    const uint32_t thr = oracle_dropout_threshold(p);
    const uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
    if (nthreads < 1) nthreads = 1;
    const long long rows = (long long)B * H * Nq;
#pragma omp parallel for num_threads(nthreads) schedule(static)
    for (long long r = 0; r < rows; ++r) {
        const uint32_t bh = (uint32_t)(r / Nq), i = (uint32_t)(r % Nq);
        uint8_t *mrow = mask + (size_t)r * Nk;
        uint32_t have = 0xffffffffu, w[4] = {0, 0, 0, 0};
        for (int j = 0; j < Nk; ++j) {
            const uint32_t call = 2u * ((uint32_t)j >> 4) + (((uint32_t)j >> 2) & 1u);
            const uint32_t f = 4u * (((uint32_t)j >> 3) & 1u) + ((uint32_t)j & 3u);
            if (call != have) {
                const uint32_t ctr[4] = {call, i, bh, (uint32_t)offset};
                oracle_philox4x32_10(ctr, key, w);
                have = call;
            }
            mrow[j] = (uint8_t)(((w[f >> 1] >> (16u * (f & 1u))) & 0xffffu) >= thr);
        }
    }
}

/* ------------------------------------------------------------------------- */
/* Portable seeded inputs: out[e] = RN_fp16(z_e), z_e ~ N(0,1), a pure function of (seed, e) -- the same bits from any
 * program, thread count or starting element, unlike std::normal_distribution (src/main.cu:91-97 draws U(0,10) from
 * std::default_random_engine, whose sequence is fixed, but a normal distribution's algorithm is not) or a framework's
 * device generator.  Elements 4c .. 4c+3 come from one Philox4x32-10 call with key (lo32(seed), hi32(seed)) and
 * counter (lo32(c), hi32(c), 0x4e4f524d, 0): words (w0, w1) and (w2, w3) each give a Box-Muller pair
 *   u1 = (w + 1) / 2^32 in (0, 1],  u2 = w' / 2^32 in [0, 1),  r = sqrt(-2 ln u1),  z = r cos(2 pi u2), r sin(2 pi u2)
 * in double precision, rounded once to fp16 (round to nearest even).  Test infrastructure like everything here: the
 * bench + verify driver (--fill normal), the Python test harness and the benchmark draw their Q, K and V from it
 * (seeds 1, 2, 3 unless stated).  Pinned by known bit patterns, by its moments and by invariance under the starting
 * element. */
static uint16_t f32_to_f16_rne(float f)
{
    uint32_t x;
    memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    x &= 0x7fffffffu;
    if (x >= 0x7f800000u) return (uint16_t)(sign | 0x7c00u | (x > 0x7f800000u ? 0x200u : 0u)); /* inf / nan */
    if (x >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);                                   /* rounds to inf */
    if (x < 0x38800000u) {                                                                      /* subnormal half */
        if (x < 0x33000000u) return (uint16_t)sign;                                             /* below half the smallest */
        const int shift = 126 - (int)(x >> 23);                 /* 14 .. 24: mantissa bits to drop */
        const uint32_t m = (x & 0x7fffffu) | 0x800000u;
        uint32_t h = m >> shift;
        const uint32_t rem = m & ((1u << shift) - 1u), half = 1u << (shift - 1);
        if (rem > half || (rem == half && (h & 1u))) ++h;
        return (uint16_t)(sign | h);
    }
    uint32_t h = ((x >> 13) - (112u << 10));                    /* rebias the exponent 127 -> 15 */
    const uint32_t rem = x & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) ++h;     /* may carry into the exponent: still correct */
    return (uint16_t)(sign | h);
}

/* the conversion alone, so that tests can pin it against another implementation of IEEE round-to-nearest-even */
ORACLE_API void oracle_f32_to_f16(const float *in, uint16_t *out, uint64_t count)
{
    for (uint64_t i = 0; i < count; ++i) out[i] = f32_to_f16_rne(in[i]);
}

ORACLE_API void oracle_fill_normal_f16(uint16_t *out, uint64_t first, uint64_t count, uint64_t seed, int nthreads)
{
    const uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
    const uint64_t c_begin = first / 4, c_end = (first + count + 3) / 4;
    if (nthreads < 1) nthreads = 1;
#pragma omp parallel for num_threads(nthreads) schedule(static)
    for (uint64_t c = c_begin; c < c_end; ++c) {
        const uint32_t ctr[4] = {(uint32_t)c, (uint32_t)(c >> 32), 0x4e4f524du, 0u};
        uint32_t w[4];
        oracle_philox4x32_10(ctr, key, w);
        double z[4];
        for (int pair = 0; pair < 2; ++pair) {
            const double u1 = ((double)w[2 * pair] + 1.0) * (1.0 / 4294967296.0);
            const double u2 = (double)w[2 * pair + 1] * (1.0 / 4294967296.0);
            const double r = sqrt(-2.0 * log(u1)), a = 6.283185307179586476925286766559 * u2;
            z[2 * pair] = r * cos(a);
            z[2 * pair + 1] = r * sin(a);
        }
        for (int k = 0; k < 4; ++k) {
            const uint64_t e = 4 * c + (uint64_t)k;
            if (e >= first && e < first + count) out[e - first] = f32_to_f16_rne((float)z[k]);
        }
    }
}

ORACLE_API int oracle_max_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
