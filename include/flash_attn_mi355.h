/*
 * flash_attn_mi355.h -- C ABI of the MI355X (gfx950) FlashAttention forward library.
 *
 * The reference (Yhorm26/flash_attn) has no host library: its interface is the kernel launch
 *     kernel<<<dim3(Tr[*split], H, B), 256, smem>>>(mykernelParamType)
 * issued from main() (src/main.cu:141-192) with the by-value struct of include/utils.h:21-44.
 * The entry points below are what a binding for that path calls instead.  They take plain pointers and sizes
 * only; every pointer in flash_params is a DEVICE pointer owned by the caller (as in src/main.cu:84-87,160-162),
 * nothing is allocated or freed here, and work is enqueued asynchronously on the given HIP stream.
 */
#ifndef FLASH_ATTN_MI355_H
#define FLASH_ATTN_MI355_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Return codes.  The reference prints and exits (CUDA_CHECK, src/main.cu:18-25) or prints and returns
 * (src/main.cu:182-185); this library returns a code instead and never terminates the process. */
enum {
    FLASH_OK = 0,
    FLASH_EINVAL = -1,       /* NULL params / NULL required pointer / non-positive size / bad scalar          */
    FLASH_EHEADDIM = -2,     /* d > 128: "Insufficient shared memory. Please reduce the value of head_dim"   */
    FLASH_EALIGN = -3,       /* Q/K/V/O base not 16-byte aligned (reference's cp.async 16-B assumption)      */
    FLASH_EWORKSPACE = -4,   /* num_splits > 1 but O_partial / LSE_partial missing                           */
    FLASH_ESPLITS = -5,      /* num_splits larger than FLASH_MAX_SPLITS                                      */
    FLASH_ELAUNCH = -6,      /* the HIP runtime rejected a launch; see flash_last_hip_error()                */
    FLASH_ENODEVICE = -7,    /* the current device is not a gfx950 (the library carries code for nothing else) */
    FLASH_ESCRATCH = -8      /* flash_forward_splitkv_static: the split workspace would not fit the built-in scratch */
};

#define FLASH_MAX_HEAD_DIM 128
#define FLASH_MAX_SPLITS 128
#define FLASH_SPLIT_KEY_GRANULE 128 /* key-block size the split ranges are cut at (reference Bc, main.cu:117) */

/* Superset of mykernelParamType (include/utils.h:21-44).
 *   reference field            here
 *   Q,K,V (half*)              Q,K,V            fp16 [B,H,Nq|Nk,d] contiguous, same layout (K,V: [B,H_kv,Nk,d] if H_kv is set)
 *   O (float*)                 O                fp16 [B,H,Nq,d]  (the reference stores fp32)
 *   --                         LSE              fp32 [B,H,Nq]    natural-log sum-exp of the masked scaled scores
 *   O_tmp, L, M                O_partial, LSE_partial   fp32 [B,H,S,Nq,d] and [B,H,S,Nq]; LSE_s = M_s + log L_s
 *                                               (scratch of one call: with Nq == 1 and four or more query heads per
 *                                               K/V head the order inside is [B,H_kv,S,H/H_kv,d] and [B,H_kv,S,H/H_kv])
 *   N, d (+ gridDim.y/.z)      B, H, Nq, Nk, d
 *   Br,Bc,Tr,Tc                not part of the ABI (tiling is the library's business)
 *   softmax_scale              softmax_scale
 *   window_size_left/right     window_left/right   (< 0: unbounded on that side; reference uses -1 for "off")
 *   --                         is_causal           (template bool Is_causal in the reference)
 *   alibi_slopes_ptr           alibi_slopes        fp32 [H] or NULL; score -= slope[h] * |i - j|
 *   dropout_prob, seed, states dropout_p, seed, offset   counter-based Philox4x32-10 instead of curand states
 *   split_num                  num_splits          (<= 0: chosen by the library, see flash_forward_splitkv)
 * Row index used by masks and bias is i + (Nk - Nq), which is i whenever Nq == Nk (all the reference can express).
 *
 * EVERY field is read by the library: start from flash_params_init() (or from an all-zero struct with window_left =
 * window_right = -1) and set what the call needs.  A field left uninitialised is not detected -- a stray kernel_hint is
 * rejected with FLASH_EINVAL, a stray debug-output pointer is written through.  Fields are only ever appended to the
 * struct; flash_params_size() lets a caller built against another header notice before its first call.
 */
typedef struct flash_params {
    const void *Q;
    const void *K;
    const void *V;
    void *O;
    float *LSE;
    float *O_partial;
    float *LSE_partial;
    int B, H, Nq, Nk, d; /* one [N,d] slice of Q, K or V must stay below 4 GiB (N * d < 2^31) */
    float softmax_scale;
    int is_causal;
    int window_left;
    int window_right;
    const float *alibi_slopes;
    float dropout_p;
    uint64_t seed;
    uint64_t offset;
    int num_splits;
    /* Optional debug output: when non-NULL and dropout_p > 0, the forward kernel also stores the keep decision it
     * applied to (i, j) as one byte (1 = kept) into keep_mask_out [B,H,Nq,Nk], for every (i, j) that the masks leave
     * visible; the bytes of masked-out pairs may or may not be written.  No counterpart in the reference, whose
     * dropout is never verified (src/main.cu:44,222). */
    uint8_t *keep_mask_out;
    /* Number of K/V heads (grouped-query / multi-query attention): K and V are [B,H_kv,Nk,d] and query head h reads
     * K/V head h / (H / H_kv).  0 means H (one K/V head per query head, all the reference can express: it indexes
     * K and V with the query head, src/flash_forward.h:57-59).  H must be a multiple of H_kv. */
    int H_kv;
    /* Optional debug output: when non-NULL, the forward also stores the scores the softmax is taken over,
     * softmax_scale * q_i.k_j - slope_h * |i - j| in fp32, for every (i, j) that the masks leave visible, into
     * scores_out [B,H,Nq,Nk]; entries of masked pairs are not written (fill the buffer with -inf beforehand to read it
     * as the masked score matrix).  The call then takes the one kernel instance that serves every
     * feature and head dim, which is about 20 % slower.  No counterpart in the reference. */
    float *scores_out;
    /* Which tiled kernel serves the call, for A/B measurements and tests: 0 = the library chooses (by shape),
     * 1 = the 4-wave kernel with 128 query rows per work-group (left to itself the library gives small unsplit
     * problems work-groups of 32 rows whose waves share out the key tiles), 2 = the 8-wave ping-pong kernel (256 rows; needs
     * 96 < d <= 128, a positive scale and more than 128 query rows, and is ignored otherwise).  Any other value: FLASH_EINVAL.
     * The reference selects its kernel by template flags alone (src/main.cu:141-178) and has no such switch. */
    int kernel_hint;
    /* Optional debug output: when non-NULL, every work-group of the tiled kernel stores FLASH_STAMP_WORDS 64-bit words
     * at stage_stamps_out + FLASH_STAMP_WORDS * blockIdx (buffer size: flash_stage_stamps_bytes): words 0..6 are readings
     * of the constant 100 MHz device counter -- 0 entry, 1 all prologue requests issued, 2 own requests landed,
     * 3 first work-group barrier passed, 4 first score tile computed, 5 key-tile loop finished, 6 results stored --
     * word 7 packs (tiles of the work-group) << 32 | hardware id of the CU (bits 0-15 of HW_ID; bits 16-19 the
     * XCC), and word 8 is the number of shader-clock cycles (s_memtime) between readings 3 and 5: divided by their
     * distance in time it is the clock the CU ran at while the work-group was in its key-tile loop (the power
     * management lowers it when the MFMA operands change from instruction to instruction).  The call then runs instrumented instances of the same kernels (same arithmetic, same results).  With a
     * split count above 1 the combine step is not stamped.  The only instrumentation of the reference is the event
     * pair around its launches (src/main.cu:195-213). */
    uint64_t *stage_stamps_out;
} flash_params;

#define FLASH_STAMP_WORDS 9

/* Tiled forward over the whole key range: replaces
 *     forward_kernel<...><<<dim3(Tr,H,B),256,smem>>>(param)              (src/flash_forward.h:13-15, src/main.cu:189)
 * `stream` is a hipStream_t passed as void* (NULL = default stream, which is what the reference uses). */
int flash_forward(const flash_params *p, void *stream);

/* Split-KV forward plus combine on the same stream: replaces
 *     forward_kernel_splitkv<...><<<dim3(Tr*split,H,B),256,smem>>>(param);
 *     forward_kernel_splitkv_combine<<<dim3(Tr,H,B),Br>>>(param);          (src/flash_forward_splitkv.h:14-16,347-348,
 *                                                                          src/main.cu:189-192)
 * Uses p->num_splits; needs the workspace when the resulting split count is > 1.  With num_splits <= 0 the library
 * chooses: flash_num_splits_heuristic with 256 CUs (the reference's rule, src/main.cu:125) for Nq > 1; for Nq == 1,
 * which streams K and V once and is bound by memory bandwidth, enough splits of at least 512 keys to give every CU
 * several work-groups.  flash_splitkv_resolve_splits returns the count either way. */
int flash_forward_splitkv(const flash_params *p, void *stream);

/* flash_forward_splitkv for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference, whose main() allocates O_tmp, L and M
 * itself (src/main.cu:160-162).  Same arguments, same kernels and bit-identical results, but O_partial / LSE_partial of
 * p are ignored: the split partials go to a scratch array built into the library's device code, FLASH_STATIC_SCRATCH_BYTES
 * per GPU, held from the moment the library is loaded on that GPU until the process ends.  The call allocates and
 * frees nothing.  Its first call on a device looks up the array's address there (hipGetSymbolAddress) and, like every
 * entry point, the first launch of a kernel instance raises that kernel's dynamic-LDS limit: make one ordinary call
 * per device and shape class before capturing.  A problem whose partials need more than the scratch
 * (flash_splitkv_workspace_bytes: both sizes, the first rounded up to 256) returns FLASH_ESCRATCH and launches nothing.
 * All calls on one GPU share the array: calls that may overlap on that GPU (different streams, different threads)
 * race on it and must be serialised by the caller, or use flash_forward_splitkv with workspaces of their own. */
#define FLASH_STATIC_SCRATCH_BYTES (32u << 20)
int flash_forward_splitkv_static(const flash_params *p, void *stream);

/* Bytes of O_partial and of LSE_partial needed for p (the cudaMallocs of src/main.cu:160-162). Either may be NULL. */
int flash_splitkv_workspace_bytes(const flash_params *p, size_t *o_partial_bytes, size_t *lse_partial_bytes);

/* The split count flash_forward_splitkv will use for p (after the heuristic and clamping). */
int flash_splitkv_resolve_splits(const flash_params *p);

/* Bytes of the buffer stage_stamps_out must point to for p under the given entry point (split != 0: as launched by
 * flash_forward_splitkv, else by flash_forward): FLASH_STAMP_WORDS * 8 bytes per work-group of the tiled kernel that
 * the call launches; 0 when the call would not run a tiled kernel (Nq == 1 decode stream, empty problem). */
int flash_stage_stamps_bytes(const flash_params *p, int split, size_t *bytes);

/* num_splits_heuristic (src/main.cu:391-422), same arguments and return value; main() passes num_SMs = 108,
 * this library's callers pass the CU count (256). */
int flash_num_splits_heuristic(int batch_nheads_mblocks, int num_SMs, int num_n_blocks, int max_splits, int seq_len);

/* Keep-mask of the dropout contract alone, [B,H,Nq,Nk] bytes on the device (uses B,H,Nq,Nk,dropout_p,seed,offset of
 * p).  Stands where init_curand_states<<<...>>> (src/init_curand_states.h:7-14, src/main.cu:128-139) stood as the
 * separately launched RNG step; the counter-based generator needs no state, so this only materialises the mask. */
int flash_dropout_keep_mask(const flash_params *p, uint8_t *mask_out, void *stream);

/* Integer drop threshold floor(p * 2^16), at most 65535 (host helper).  The dropout contract, reproducible on a CPU:
 * Philox4x32-10 with key (lo32(seed), hi32(seed)) and counter (call(j), i, b*H + h, lo32(offset)), where
 * call(j) = 2*(j >> 4) + ((j >> 2) & 1); the 128 output bits are eight 16-bit fields (field f = bits 16*(f & 1) and
 * up of output word f >> 1), and element (i, j) is kept iff field 4*((j >> 3) & 1) + (j & 3) >= threshold.  Kept
 * probabilities are scaled by 1/(1 - dropout_p); the row sum of the softmax is taken before the drop. */
uint32_t flash_dropout_threshold(float dropout_p);

/* Defaults for every field: all pointers NULL, all sizes 0, no mask (is_causal 0, window_left = window_right = -1), no
 * bias, no dropout, num_splits 1 (unsplit), H_kv 0 (= H), kernel_hint 0, no debug outputs.  softmax_scale stays 0: the
 * caller sets it (the reference uses 1/sqrt(d), src/main.cu:112).  The reference fills its struct field by field and
 * leaves dropout_prob, states, split_num, O_tmp, L and M uninitialised on the paths that do not use them
 * (src/main.cu:109-123); this helper is what a binding calls first instead.  NULL is ignored. */
void flash_params_init(flash_params *p);

/* sizeof(flash_params) of the header the library was built with.  A caller compiled against another version of the
 * header would hand over a struct of another size (fields are only ever appended): compare before the first call. */
size_t flash_params_size(void);

/* Text of the last HIP error seen by this thread inside the library ("" if none). */
const char *flash_last_hip_error(void);

/* Human-readable name of a return code. */
const char *flash_strerror(int code);

#ifdef __cplusplus
}
#endif
#endif /* FLASH_ATTN_MI355_H */
