/*
 * C ABI of the MI355X (gfx950) FMHA forward library: split-KV forward + LSE combine, appendKV (rotary embedding +
 * paged-cache write), paged-KV attention and varlen batch prefill.
 *
 * Each entry point keeps the parameter order of the generated-library function FlashCK would dlsym for the same
 * operation (paths relative to the FlashCK tree), made C-clean:
 *   - `int` status instead of `void` + a message on std::cerr (fmha_common_jinja.h:5-12,58-60);
 *     0 = success, negative = FCK_ERR_*; fck_last_error() holds the text for the calling thread;
 *   - index arrays are int32 (FlashCK declares int64_t*, but the ck_tile kernels it instantiates read int32:
 *     ck_tile/ops/fmha/kernel/fmha_fwd_splitkv_kernel.hpp:263-264,491-492);
 *   - `std::array<int64_t,2> window_size` becomes two int64_t;
 *   - an explicit `dtype` (flashck::DataType id, core/utils/dtype.h:16-28) replaces the per-type instantiation.
 *
 * Conventions: every pointer is caller-owned device memory (workspaces included); launches are asynchronous on
 * `stream` (a hipStream_t passed as void*), nothing synchronises; no entry point allocates; the library keeps no
 * mutable state except the calling thread's last error text, so calls are re-entrant and stream-ordered.
 *
 * Tensor layouts (element strides; T = fp16 or bf16, 2 bytes):
 *   Q, O        batch mode [B, sq, Hq, D|Dv]; group mode (seqstart_q != NULL) [total_q, Hq, D|Dv]
 *   K, V        batch [B, sk, Hk, D|Dv]; group [total_k, Hk, D|Dv]; paged [num_pages, P, Hk, D|Dv]
 *               (fmha_fwd_split_kv_jinja.h:261-263,277-279,294-306,511-522)
 *   block_table int32 [B, max_num_page_blocks / B]        (fmha_fwd_split_kv_jinja.h:318,549-552)
 *   o_acc       fp32  [Bs, Hq, num_splits, Sq, Dv]        (fmha_fwd_split_kv_jinja.h:289,308,323,546-547)
 *   lse_acc     fp32  [Bs, Hq, num_splits, Sq]            (fmha_fwd_split_kv_combine_jinja.h:129,134,139)
 *               with (Bs, Sq) = (B, sq) in batch mode and (1, total_q) in group mode
 */
#ifndef FLASHCK_FMHA_C_API_H
#define FLASHCK_FMHA_C_API_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FCK_EXPORT __attribute__((visibility("default")))

/* flashck::DataType, core/utils/dtype.h:16-28 */
/* e4m3 (OCP, as ck_tile::fp8_t on gfx950).  As fck_fmha_attrs.kv_dtype: an fp8 K/V cache under 16-bit queries.  As the
 * `dtype` of fck_fmha_fwd / _pagedkv / _batch_prefill / _splitkv (+ _attrs) and _splitkv_combine: the all-fp8 roles of
 * FmhaFwdTypeConfig<fp8_t> (core/module/kernels/attention_kernels/fmha_common_jinja.h:157-171): Q, K, V and O are one
 * e4m3 byte per element, P is rounded to e4m3 before the second product (scale_p = 1, as the reference passes it:
 * fmha_fwd_jinja.h:327), LSE and the split-KV partial results stay fp32.  k = k_descale * stored, v = v_descale * stored
 * as for an fp8 cache (a query scale belongs into `scale`); O = saturate(o_scale * o).  Needs qk_head_dim = v_head_dim in
 * {64, 128, 256}; an elementwise bias holds fp32 for these roles (BiasDataType = float), strides in floats; not on
 * fck_fmha_fwd_splitkv_fused / _appendkv.  The products run on the bf16 matrix instructions (every e4m3 value is a bf16
 * value): the roles halve the memory traffic, they do not double the matrix rate. */
#define FCK_DTYPE_FP8 1
#define FCK_DTYPE_FP16 3
#define FCK_DTYPE_BF16 4

/* GenericAttentionMaskEnum, core/profiling/attention/fmha_library.h:81-87 */
#define FCK_MASK_NONE 0
#define FCK_MASK_TOP_LEFT 1
#define FCK_MASK_BOTTOM_RIGHT 2
#define FCK_MASK_GENERIC 3

/* RopeEnum, core/profiling/attention/fmha_library.h:195-200 */
#define FCK_ROPE_NONE 0
#define FCK_ROPE_INTERLEAVED 1
#define FCK_ROPE_HALF_ROTATED 2

/* BiasEnum, core/profiling/attention/fmha_library.h:121-126 */
#define FCK_BIAS_NONE 0
#define FCK_BIAS_ELEMENTWISE 1
#define FCK_BIAS_ALIBI 2

/*
 * What FlashCK fixes per generated kernel instance and this library takes per call: the bias kind and its rank
 * (core/profiling/attention/fmha_library.h:150-165, stride plumbing
 * core/module/kernels/attention_kernels/fmha_fwd_split_kv/fmha_fwd_split_kv_jinja.h:359-385) and the logits soft cap
 * (core/profiling/attention/fmha_fwd_split_kv/fmha_fwd_split_kv_problem.h:81).  Passed to the *_attrs entry points;
 * a NULL pointer (or the entry point without the suffix) means none of them.
 *
 * and static quantisation (is_static_quant, same file :79; fp8 type roles
 * core/module/kernels/attention_kernels/fmha_common_jinja.h:157-171).
 *
 * Scores: x = scale * q.k;  x = cap * tanh(x / cap) when logits_soft_cap > 0;  x += bias;  then the mask.
 *   ELEMENTWISE_BIAS  T elements (fp32 when dtype is FCK_DTYPE_FP8); (b, h, i, j) at bias[b * bias_batch_stride + h * bias_head_stride + i * bias_row_stride + j].
 *                     The reference's rank 0 (1*1*s*s) is head and batch stride 0, rank 1 (1*h*s*s) batch stride 0,
 *                     rank 2 (b*h*s*s) neither.  Group mode: i counts packed query rows (seqstart_q[b] + local row)
 *                     and bias_batch_stride is not used.
 *   ALIBI             fp32 slopes; (b, h) at bias[b * bias_batch_stride + h]: rank 0 (1*h) is batch stride 0, rank 1 (b*h)
 *                     is q_num_heads.  The term added is slope * j for a causal window (window_left < 0, window_right == 0,
 *                     mask_type != NONE), else -slope * |i - j| (top-left) or -slope * |i + sk - sq - j| (bottom-right,
 *                     and no mask).
 */
typedef struct fck_fmha_attrs {
    uint32_t size;             /* sizeof(fck_fmha_attrs) */
    int32_t bias_type;         /* FCK_BIAS_* */
    const void* bias;          /* used by the entry points without a bias argument (or when that argument is NULL) */
    int64_t bias_batch_stride; /* elements */
    int64_t bias_head_stride;
    int64_t bias_row_stride;
    float logits_soft_cap;     /* > 0: on; 0: off */
    /* K/V cache element type when it differs from `dtype`: 0 = same as Q, FCK_DTYPE_FP8 = one e4m3 byte per element
     * with static per-tensor scales (split-KV entry point only): k = k_descale * fp8 value, v = v_descale * fp8 value;
     * Q, the probabilities and the output keep `dtype`.  A descale of 0 means 1. */
    int32_t kv_dtype;
    float k_descale, v_descale;
    /* Split-KV kernel variant, the counterpart of the tile instance FlashCK's tuner picks per problem
     * (core/profiling/profiling_db.cc:64-71): 0 = the library chooses; 1 = one KV head per workgroup (32-key tiles);
     * 2 = two adjacent KV heads per workgroup (16-key tiles, 512-byte row pieces; needs an even kv_num_heads, at most
     * 16 packed query rows and head dim 64 or 128); 3 / 4 = as 1 / 2 with splits of equal size in keys instead of
     * num_splits equal parts of every sequence: split s of a sequence covers keys [s * chunk, (s + 1) * chunk) with
     * chunk = ceil(bound / num_splits) rounded up to 32, bound = max_seqlen_k below (the last split also takes whatever
     * lies beyond), so the work items of a ragged batch have one size and the splits a short sequence does not reach
     * are empty (lse_acc = -inf); the combine is unchanged.  3 / 4 need a block table with pages a multiple of 32 keys,
     * at most 16 packed query rows, head dim 64 or 128 and no bias / soft cap / fp8 cache.  A variant the problem
     * cannot take is an error. */
    int32_t decode_variant;
    /* Prefill tile variant, likewise: 0 = the library chooses; 1 = the default schedule of the kernel the call takes;
     * 2..4 = variants of the 8-wave ping-pong kernel (2: byte offsets of whole-tile requests computed once per
     * workgroup; 3: a tile's row maximum taken in the matrix phase that produced its scores; 4: both), which need head
     * dim 64 or 128, query runs longer than 128 rows, pages a multiple of 64 keys (or an unpaged cache) and no bias /
     * ALiBi / soft cap / fp8 cache.  A variant the problem cannot take is an error.  All variants give the same
     * results up to the rounding of the running maximum. */
    int32_t prefill_variant;
    /* ELEMENTWISE_BIAS: columns a bias row holds.  A key index is clamped to the last of them before the bias is read,
     * so a bias narrower than a sequence's key count is never read out of bounds (the scores of such keys then use
     * the last column).  0: not stated, only the sequence's own key count bounds the reads. */
    int64_t bias_cols;
    /* decode_variant 3 / 4: upper bound of the key counts of the batch (0 or anything above the block table's capacity:
     * that capacity).  A bound below a real key count costs balance, not correctness. */
    int64_t max_seqlen_k;
    /* dtype FCK_DTYPE_FP8 on fck_fmha_fwd / _pagedkv / _batch_prefill: the output is saturate(o_scale * o) in e4m3
     * (ck_tile's scale_o; the reference passes 1).  0 means 1.  The split-KV pair writes with scale 1. */
    float o_scale;
} fck_fmha_attrs;

#define FCK_OK 0
#define FCK_ERR_INVALID_ARGUMENT (-1) /* null pointer, non-positive size, Hq % Hk != 0 ... */
#define FCK_ERR_UNSUPPORTED (-2)      /* dtype / head_dim / feature this build has no kernel for */
/* Head dims: qk_head_dim and v_head_dim are independent multiples of 8 in [8, 256] (the reference pads them with its
 * is_pad_qk_head_dim / is_pad_v_head_dim traits, core/profiling/attention/fmha_fwd_split_kv/fmha_fwd_split_kv_codegen.h:106-107). */
#define FCK_ERR_LAUNCH (-3)           /* the HIP runtime refused the launch */

/* Text of the last error raised on the calling thread ("" when none). */
FCK_EXPORT const char* fck_last_error(void);

/* Library version string. */
FCK_EXPORT const char* fck_fmha_version(void);

/* Name of the kernel family (and addressing variant) the calling thread's last successful dispatch chose, "" before
 * the first one.  For tests and tuning records; FlashCK logs the same through its instance names
 * (core/profiling/attention/fmha_fwd_split_kv/fmha_fwd_split_kv_codegen.cc:60-94). */
FCK_EXPORT const char* fck_fmha_last_kernel(void);

/*
 * Dense / varlen forward.  Replaces `FmhaFwd`, fmha_fwd/fmha_fwd_jinja.h:124-147 (args :68-122, strides :186-304).
 * batch mode: seqstart_q = seqstart_k = NULL; seqlen_k_ptr optional per-batch key counts.
 * group mode: seqstart_q / seqstart_k are int32 [B+1] prefix sums; seqlen_q / seqlen_k are ignored.
 */
FCK_EXPORT int fck_fmha_fwd(const void* q, const void* k, const void* v, const void* bias, void* o,
                            const int32_t* seqstart_q, const int32_t* seqstart_k, const int32_t* seqlen_k_ptr,
                            int64_t batch, int64_t seqlen_q, int64_t seqlen_k, int64_t q_num_heads,
                            int64_t kv_num_heads, int64_t qk_head_dim, int64_t v_head_dim, int64_t q_max_seq_len,
                            float scale, int64_t window_left, int64_t window_right, uint32_t mask_type,
                            int32_t dtype, void* stream);
/* The same with bias / ALiBi / soft cap (`attrs` may be NULL): the instances FlashCK generates for
 * bias_str != "no" (fmha_fwd/fmha_fwd_jinja.h:124-147, BiasEnum fmha_library.h:121-126). */
FCK_EXPORT int fck_fmha_fwd_attrs(const void* q, const void* k, const void* v, const void* bias, void* o,
                                  const int32_t* seqstart_q, const int32_t* seqstart_k, const int32_t* seqlen_k_ptr,
                                  int64_t batch, int64_t seqlen_q, int64_t seqlen_k, int64_t q_num_heads,
                                  int64_t kv_num_heads, int64_t qk_head_dim, int64_t v_head_dim, int64_t q_max_seq_len,
                                  float scale, int64_t window_left, int64_t window_right, uint32_t mask_type,
                                  int32_t dtype, const fck_fmha_attrs* attrs, void* stream);

/*
 * Split-KV forward: per split s of num_splits, attention over keys [s*ceil(Lk/ns), min(Lk,(s+1)*ceil(Lk/ns)))
 * written as per-split normalised fp32 o_acc and lse_acc (= max + ln(sum), -inf for a split with no visible key).
 * Replaces `FmhaFwdSplitKV`, fmha_fwd_split_kv/fmha_fwd_split_kv_jinja.h:155-184 (args :76-151, strides :241-409).
 * K/V addressing: block_table != NULL -> paged cache with page_block_size tokens per page and per-sequence key
 * counts in seqlen_k_ptr; else seqstart_k != NULL -> group mode; else batch cache [*, seqlen_k, Hk, D] whose row
 * is cache_batch_idx[b] when that is given, with key counts seqlen_k_ptr[b] (or seqlen_k when NULL).
 */
FCK_EXPORT int fck_fmha_fwd_splitkv(const void* q, const void* k, const void* v, const void* bias, void* lse_acc,
                                    void* o_acc, const int32_t* seqstart_q, const int32_t* seqstart_k,
                                    const int32_t* seqlen_k_ptr, const int32_t* block_table,
                                    const int32_t* cache_batch_idx, int64_t batch, int64_t seqlen_q,
                                    int64_t seqlen_k, int64_t q_num_heads, int64_t kv_num_heads, int64_t qk_head_dim,
                                    int64_t v_head_dim, int64_t q_max_seq_len, int64_t num_splits,
                                    int64_t max_num_page_blocks, int64_t page_block_size, float scale,
                                    int64_t window_left, int64_t window_right, uint32_t mask_type, int32_t dtype,
                                    void* stream);
/* The same with bias / ALiBi / soft cap (`attrs` may be NULL): the instances FlashCK generates for
 * bias_str != "no" or has_logits_soft_cap (fmha_fwd_split_kv_jinja.h:359-385, fmha_fwd_split_kv_problem.h:81). */
FCK_EXPORT int fck_fmha_fwd_splitkv_attrs(const void* q, const void* k, const void* v, const void* bias, void* lse_acc,
                                          void* o_acc, const int32_t* seqstart_q, const int32_t* seqstart_k,
                                          const int32_t* seqlen_k_ptr, const int32_t* block_table,
                                          const int32_t* cache_batch_idx, int64_t batch, int64_t seqlen_q,
                                          int64_t seqlen_k, int64_t q_num_heads, int64_t kv_num_heads,
                                          int64_t qk_head_dim, int64_t v_head_dim, int64_t q_max_seq_len,
                                          int64_t num_splits, int64_t max_num_page_blocks, int64_t page_block_size,
                                          float scale, int64_t window_left, int64_t window_right, uint32_t mask_type,
                                          int32_t dtype, const fck_fmha_attrs* attrs, void* stream);

/*
 * Split-KV forward and LSE combine in ONE launch that allocates nothing: fck_fmha_fwd_splitkv with `o` in place of
 * the (lse_acc, o_acc) workspace.  It has no counterpart in the reference (whose callers always own the workspace and
 * launch FmhaFwdSplitKV and FmhaFwdSplitKVCombine separately); it is for callers that cannot allocate or want a single
 * launch: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
 *
 * The partial results go to a fixed device array inside the library (one copy per GPU, 4 slices of 16 MiB + 64 KiB,
 * held until the process ends) and the workgroup that delivers the last partial result of a (sequence, KV-head group)
 * merges the splits and writes `o`.  Limits: Bs * Hq * num_splits * Sq * (Dv + 1) <= 4 Mi floats and
 * B * Hk * row_tiles <= 16384, else FCK_ERR_UNSUPPORTED (nothing is launched).
 *
 * A stream owns one slice of the array on its GPU from its first fused call on, so calls on up to 4 different streams
 * of a GPU may overlap in time; a fifth stream is refused with FCK_ERR_UNSUPPORTED (nothing is launched) until
 * fck_fmha_fused_reset has forgotten the owners.  Calls on one stream are ordered by the stream, from whichever host
 * threads they come.  What still races: one captured graph replayed on two streams at once (its slice was fixed at
 * capture).
 *
 * num_splits > 0: that many equal key ranges, exactly as fck_fmha_fwd_splitkv.  num_splits == 0: the library takes
 * fck_fmha_num_splits_heuristic of the CU count and the longest possible KV length (the block table's capacity, else
 * seqlen_k).  The other arguments are those of fck_fmha_fwd_splitkv.
 */
FCK_EXPORT int fck_fmha_fwd_splitkv_fused(const void* q, const void* k, const void* v, const void* bias, void* o,
                                          const int32_t* seqstart_q, const int32_t* seqstart_k,
                                          const int32_t* seqlen_k_ptr, const int32_t* block_table,
                                          const int32_t* cache_batch_idx, int64_t batch, int64_t seqlen_q,
                                          int64_t seqlen_k, int64_t q_num_heads, int64_t kv_num_heads,
                                          int64_t qk_head_dim, int64_t v_head_dim, int64_t q_max_seq_len,
                                          int64_t num_splits, int64_t max_num_page_blocks, int64_t page_block_size,
                                          float scale, int64_t window_left, int64_t window_right, uint32_t mask_type,
                                          int32_t dtype, void* stream);

/*
 * Puts the arrival tickets of fck_fmha_fwd_splitkv_fused (of every slice) back to zero on the current device (one small
 * fill launch on `stream`, nothing allocated) and forgets which stream owns which slice.  The tickets reset themselves
 * at the end of every fused launch that runs to completion; after a launch that did not (a device error, a cancelled
 * graph launch) they may be left non-zero and every later fused call on that slice would merge at the wrong moment:
 * call this once before going on.  Also the way to hand the slices to other streams.  Call it only when no fused call
 * is in flight on the GPU, and order later fused calls after `stream`'s fill.  No counterpart in the reference.
 */
FCK_EXPORT int fck_fmha_fused_reset(void* stream);

/*
 * Debug aid: checks the paged-cache arguments that the attention kernels trust, on the GPU, without allocating and
 * without reading anything back (the reference's debug aid for tensors is the validator of
 * core/utils/debug_utils.cc:43-130; its FMHA glue has no such check).  Give either a block table
 * (block_table int32 [B, batch_stride_block_table] with seqlen_k int32 [B]; the page-list pointers NULL) or a page
 * list (kv_indptr int32 [B+1], kv_page_indices, optional kv_last_page_lens; block_table and seqlen_k NULL).
 * error_counts: int32[4] in device memory of the caller, overwritten by one single-workgroup launch on `stream`:
 *   [0] sequences whose key count is negative or larger than their table row / page list can address
 *   [1] page ids outside [0, num_total_pages) among the table entries the sequences use
 *   [2] malformed page lists (kv_indptr not monotone, kv_last_page_lens outside [1, page_block_size])
 *   [3] index of the first offending sequence, -1 when there is none
 * A kernel launched with arguments for which any of [0..2] is non-zero reads outside the cache.
 */
FCK_EXPORT int fck_fmha_validate_paged(const int32_t* seqlen_k, const int32_t* block_table,
                                       int64_t batch_stride_block_table, const int32_t* kv_indptr,
                                       const int32_t* kv_page_indices, const int32_t* kv_last_page_lens,
                                       int64_t batch, int64_t num_total_pages, int64_t page_block_size,
                                       int32_t* error_counts, void* stream);

/*
 * LSE combine: O = sum_s exp(lse_acc[s] - logsumexp_s lse_acc) * o_acc[s], stored as T.
 * Replaces `FmhaSplitKVCombine` / `FmhaFwdSplitKVCombine`, fmha_fwd_split_kv_combine_jinja.h:78-92
 * (args :37-76, strides :114-165), declared at fmha_fwd_split_kv_combine_call.h:26-36.
 * seqstart_q != NULL selects group mode (seqlen_q is then ignored; rows = seqstart_q[B]).
 */
FCK_EXPORT int fck_fmha_fwd_splitkv_combine(const void* lse_acc, const void* o_acc, void* o,
                                            const int32_t* seqstart_q, int64_t batch, int64_t seqlen_q,
                                            int64_t q_num_heads, int64_t v_head_dim, int64_t q_max_seq_len,
                                            int64_t num_splits, int32_t dtype, void* stream);

/*
 * AppendKV: rotate knew (and q, in place) and write knew / vnew behind the seqlen_k[b] tokens each sequence
 * already holds.  FlashCK only names this operation (FmhaKind::FwdAppendKV, fmha_library.h:19,41; config struct
 * core/utils/json_config.h:280-312); the argument list follows the ck_tile kernel it would instantiate
 * (ck_tile/ops/fmha/kernel/fmha_fwd_appendkv_kernel.hpp:146-231).
 *   q      [total_new, Hq, D] (cu_seqlens_knew given) or [B, seqlen_knew, Hq, D]; may be NULL
 *   knew   [total_new, Hk, D] or [B, seqlen_knew, Hk, D];  vnew likewise with Dv
 *   cu_seqlens_knew  int32 [B+1] or NULL (then every sequence appends seqlen_knew tokens, the ck_tile form)
 *   rotary_cos/sin   T [>= max position + 1, rotary_dim / 2]; row = absolute position
 *   has_mask         query i uses position seqlen_k[b] + i when non-zero, seqlen_k[b] otherwise
 *   block_table != NULL: paged cache; else batch cache with `seqlen_k_cache` rows per sequence, row chosen by
 *   cache_batch_idx[b] when given.
 */
FCK_EXPORT int fck_fmha_fwd_appendkv(void* q, void* k_cache, void* v_cache, const void* knew, const void* vnew,
                                     const int32_t* seqlen_k, const int32_t* cu_seqlens_knew, int64_t seqlen_knew,
                                     const void* rotary_cos, const void* rotary_sin, int64_t rotary_dim,
                                     int32_t rope_mode, int32_t has_mask, const int32_t* block_table,
                                     int64_t batch_stride_block_table, int64_t page_block_size,
                                     const int32_t* cache_batch_idx, int64_t seqlen_k_cache, int64_t batch,
                                     int64_t q_num_heads, int64_t kv_num_heads, int64_t qk_head_dim,
                                     int64_t v_head_dim, int32_t dtype, void* stream);

/* The same for a quantised cache: attrs->kv_dtype = FCK_DTYPE_FP8 makes k_cache / v_cache one e4m3 byte per element,
 * written as fp8(x / k_descale) resp. fp8(x / v_descale) with round-to-nearest-even and saturation at +-448, where x is
 * the element a cache of `dtype` would receive (the rotated K row rounded to `dtype`, the V row as given): the static
 * quantisation of the reference's fp8 type configuration (core/module/kernels/attention_kernels/fmha_common_jinja.h:157-171,
 * is_static_quant).  knew, vnew and q keep `dtype`.  The bias / soft cap fields of `attrs` must be unset. */
FCK_EXPORT int fck_fmha_fwd_appendkv_attrs(void* q, void* k_cache, void* v_cache, const void* knew, const void* vnew,
                                           const int32_t* seqlen_k, const int32_t* cu_seqlens_knew, int64_t seqlen_knew,
                                           const void* rotary_cos, const void* rotary_sin, int64_t rotary_dim,
                                           int32_t rope_mode, int32_t has_mask, const int32_t* block_table,
                                           int64_t batch_stride_block_table, int64_t page_block_size,
                                           const int32_t* cache_batch_idx, int64_t seqlen_k_cache, int64_t batch,
                                           int64_t q_num_heads, int64_t kv_num_heads, int64_t qk_head_dim,
                                           int64_t v_head_dim, int32_t dtype, const fck_fmha_attrs* attrs, void* stream);

/*
 * Varlen batch prefill over a page list.  FlashCK's problem definition:
 * core/profiling/attention/fmha_fwd_batch_prefill/fmha_fwd_batch_prefill_problem.h:35-100 (kv_indptr,
 * kv_page_indices, num_total_pages :98-99); kernel glue files are empty there.
 *   q, o  [total_q, Hq, D|Dv] packed by seqstart_q (int32 [B+1])
 *   sequence b owns pages kv_page_indices[kv_indptr[b] .. kv_indptr[b+1]) and
 *   (n_pages - 1) * page_block_size + kv_last_page_lens[b] keys (full last page when kv_last_page_lens is NULL).
 */
FCK_EXPORT int fck_fmha_batch_prefill(const void* q, const void* k_cache, const void* v_cache, void* o,
                                      const int32_t* seqstart_q, const int32_t* kv_indptr,
                                      const int32_t* kv_page_indices, const int32_t* kv_last_page_lens,
                                      int64_t num_total_pages, int64_t page_block_size, int64_t batch,
                                      int64_t q_num_heads, int64_t kv_num_heads, int64_t qk_head_dim,
                                      int64_t v_head_dim, int64_t q_max_seq_len, float scale, int64_t window_left,
                                      int64_t window_right, uint32_t mask_type, int32_t dtype, void* stream);
/* The same with bias / ALiBi / soft cap; the bias pointer travels in `attrs` (BiasEnum and has_logits_soft_cap of
 * core/profiling/attention/fmha_fwd_batch_prefill/fmha_fwd_batch_prefill_problem.h:35-100). */
FCK_EXPORT int fck_fmha_batch_prefill_attrs(const void* q, const void* k_cache, const void* v_cache, void* o,
                                            const int32_t* seqstart_q, const int32_t* kv_indptr,
                                            const int32_t* kv_page_indices, const int32_t* kv_last_page_lens,
                                            int64_t num_total_pages, int64_t page_block_size, int64_t batch,
                                            int64_t q_num_heads, int64_t kv_num_heads, int64_t qk_head_dim,
                                            int64_t v_head_dim, int64_t q_max_seq_len, float scale,
                                            int64_t window_left, int64_t window_right, uint32_t mask_type,
                                            int32_t dtype, const fck_fmha_attrs* attrs, void* stream);

/*
 * Prefill over a vLLM-style block table (no splits).  FlashCK's problem definition:
 * core/profiling/attention/fmha_fwd_paged_kv_prefill/fmha_fwd_paged_kv_prefill_problem.h:35-97.
 * seqstart_q NULL -> batch mode q [B, seqlen_q, Hq, D].
 */
FCK_EXPORT int fck_fmha_fwd_pagedkv(const void* q, const void* k_cache, const void* v_cache, void* o,
                                    const int32_t* seqstart_q, const int32_t* seqlen_k_ptr,
                                    const int32_t* block_table, int64_t batch_stride_block_table,
                                    int64_t page_block_size, int64_t batch, int64_t seqlen_q, int64_t q_num_heads,
                                    int64_t kv_num_heads, int64_t qk_head_dim, int64_t v_head_dim,
                                    int64_t q_max_seq_len, float scale, int64_t window_left, int64_t window_right,
                                    uint32_t mask_type, int32_t dtype, void* stream);
/* The same with bias / ALiBi / soft cap; the bias pointer travels in `attrs`
 * (core/profiling/attention/fmha_fwd_paged_kv_prefill/fmha_fwd_paged_kv_prefill_problem.h:35-97). */
FCK_EXPORT int fck_fmha_fwd_pagedkv_attrs(const void* q, const void* k_cache, const void* v_cache, void* o,
                                          const int32_t* seqstart_q, const int32_t* seqlen_k_ptr,
                                          const int32_t* block_table, int64_t batch_stride_block_table,
                                          int64_t page_block_size, int64_t batch, int64_t seqlen_q,
                                          int64_t q_num_heads, int64_t kv_num_heads, int64_t qk_head_dim,
                                          int64_t v_head_dim, int64_t q_max_seq_len, float scale,
                                          int64_t window_left, int64_t window_right, uint32_t mask_type,
                                          int32_t dtype, const fck_fmha_attrs* attrs, void* stream);

/*
 * Split count from the CU count and the KV length.  FlashCK's command line promises "0 = heuristic"
 * (fmha_fwd_split_kv_jinja.h:28-30) without implementing one; num_cu <= 0 asks the current device.
 * Returns a value in [1, 128].
 */
FCK_EXPORT int fck_fmha_num_splits_heuristic(int64_t batch, int64_t q_num_heads, int64_t kv_num_heads,
                                             int64_t seqlen_q, int64_t max_seqlen_k, int64_t head_dim,
                                             int64_t num_cu);

/* Bytes of o_acc followed by lse_acc for the shapes above (fmha_fwd_split_kv_jinja.h:543-547). */
FCK_EXPORT size_t fck_fmha_splitkv_workspace_bytes(int64_t shape_batch, int64_t q_num_heads, int64_t shape_seqlen_q,
                                                   int64_t v_head_dim, int64_t num_splits);

#ifdef __cplusplus
}
#endif
#endif
