/*
 * TEST INFRASTRUCTURE - NOT PART OF THE PRODUCT.
 *
 * CPU restatement (plain C, fp32 accumulation) of the attention arithmetic that
 * FlashCK's FMHA operators delegate to ck_tile.  Only tests, the smoke check and the
 * benchmark's cpu_baseline leg may link or load this; the shipped library never does.
 *
 * Every function names the reference text it follows.  "ck_tile" paths are relative to
 * /opt/rocm/include (third-party dependency of the reference, absent from its tree:
 * .gitmodules:1-4); other paths are relative to the FlashCK source tree.
 */
#ifndef FCK_FMHA_ORACLE_H
#define FCK_FMHA_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* flashck::DataType ids, core/utils/dtype.h:16-28 */
enum { FCK_ORC_FP8 = 1, FCK_ORC_FP16 = 3, FCK_ORC_BF16 = 4 };

/* GenericAttentionMaskEnum, core/profiling/attention/fmha_library.h:81-87 */
enum { FCK_ORC_NO_MASK = 0, FCK_ORC_MASK_TOP_LEFT = 1, FCK_ORC_MASK_BOTTOM_RIGHT = 2, FCK_ORC_MASK_GENERIC = 3 };

/* RopeEnum, core/profiling/attention/fmha_library.h:195-200 */
enum { FCK_ORC_ROPE_NONE = 0, FCK_ORC_ROPE_INTERLEAVED = 1, FCK_ORC_ROPE_HALF_ROTATED = 2 };

/* How K/V rows are found. */
enum {
    FCK_ORC_KV_BATCH = 0,       /* [B, sk, Hk, D] contiguous (fmha_fwd_jinja.h:186-304); optional cache_batch_idx */
    FCK_ORC_KV_GROUP = 1,       /* [total_k, Hk, D] packed by seqstart_k */
    FCK_ORC_KV_BLOCK_TABLE = 2, /* [num_pages, P, Hk, D] + block_table[B, stride] + seqlen_k[B]
                                   (fmha_fwd_split_kv_jinja.h:295-306,318,549-552) */
    FCK_ORC_KV_PAGE_LIST = 3    /* [num_pages, P, Hk, D] + kv_indptr[B+1] + kv_page_indices[] + kv_last_page_lens[B]
                                   (fmha_fwd_batch_prefill_problem.h:98-99) */
};

typedef struct {
    int32_t dtype;
    int32_t batch, hq, hk, d, dv;
    /* Q / O rows: group mode when seqstart_q != NULL ([total_q, Hq, D]), else [B, sq, Hq, D]. */
    const int32_t* seqstart_q;
    int32_t sq;
    /* K / V */
    int32_t kv_mode;
    int32_t sk;                 /* FCK_ORC_KV_BATCH without seqlen_k: key count; also the cache row length */
    const int32_t* seqstart_k;  /* FCK_ORC_KV_GROUP */
    const int32_t* seqlen_k;    /* per-sequence key count (BLOCK_TABLE; optional for BATCH) */
    const int32_t* block_table;
    int32_t block_table_stride;
    int32_t page_size;
    const int32_t* kv_indptr;
    const int32_t* kv_page_indices;
    const int32_t* kv_last_page_lens;
    const int32_t* cache_batch_idx;
    float scale;
    int32_t mask_type;
    int64_t window_left, window_right;
    /* Score modifiers, applied in this order before the mask (ck_tile/ops/fmha/pipeline/
       block_fmha_pipeline_qr_ks_vs.hpp:391-449): soft cap, then bias.
       BiasEnum: core/profiling/attention/fmha_library.h:121-126 (rank rule :150-165).
         1 elementwise: data dtype, (b, h, i, j) at bias[b*bias_batch_stride + h*bias_head_stride + i*bias_row_stride + j];
           group mode: i counts packed query rows, no batch stride (ck_tile/ops/fmha/kernel/fmha_fwd_splitkv_kernel.hpp:608-688)
         2 ALiBi: fp32 slopes, (b, h) at bias[b*bias_batch_stride + h]; term and mode:
           ck_tile/ops/fmha/block/block_position_encoding.hpp:19-121,138-152, ck_tile/ops/fmha/kernel/fmha_fwd_kernel.hpp:1482-1507
       logits_soft_cap > 0: s = cap * tanh(scale * qk / cap), ck_tile/ops/fmha/block/variants.hpp:208-209 */
    int32_t bias_type;
    const void* bias;
    int64_t bias_batch_stride, bias_head_stride, bias_row_stride;
    float logits_soft_cap;
    /* K/V element type when it is not `dtype`: FCK_ORC_FP8 = one e4m3 byte per element (the OCP format ck_tile::fp8_t
       is on gfx950, ck_tile/core/numeric/float8.hpp) with static per-tensor scales: k = k_descale * value,
       v = v_descale * value (0 means 1).  Type roles: core/module/kernels/attention_kernels/fmha_common_jinja.h:157-171;
       is_static_quant: core/profiling/attention/fmha_fwd_split_kv/fmha_fwd_split_kv_problem.h:79. */
    int32_t kv_dtype;
    float k_descale, v_descale;
    /* dtype FCK_ORC_FP8: the all-fp8 roles of FmhaFwdTypeConfig<fp8_t> (fmha_common_jinja.h:157-171): Q, K, V, P and O are
       e4m3 (K/V as with kv_dtype FCK_ORC_FP8, the descales apply).  P is cast to e4m3 before the second product
       (p_compute_element_func = scales{scale_p}, scale_p = 1 in the reference) and O = saturate(o_scale * o) (0 means 1;
       the reference passes scale_o = 1).  An elementwise bias holds fp32 (BiasDataType = float), strides in floats.  ck_tile/ops/fmha/kernel/fmha_fwd_kernel.hpp:1529-1553. */
    float o_scale;
} fck_orc_problem;

/* 1 when key j is visible to query i. */
int fck_orc_visible(int mask_type, int64_t wl, int64_t wr, int sq, int sk, int i, int j);

/* o: same row layout as q with Dv; lse (optional): fp32 [B, Hq, sq] or [Hq, total_q] in group mode. */
int fck_orc_fmha_fwd(const fck_orc_problem* p, const void* q, const void* k, const void* v, void* o, float* lse);

/* o_acc fp32 [Bs, Hq, ns, Sq, Dv], lse_acc fp32 [Bs, Hq, ns, Sq];
   (Bs, Sq) = (B, sq) in batch mode and (1, total_q) in group mode. */
int fck_orc_fmha_splitkv(const fck_orc_problem* p, const void* q, const void* k, const void* v,
                         int num_splits, float* o_acc, float* lse_acc);

int fck_orc_splitkv_combine(const float* lse_acc, const float* o_acc, void* o, float* lse,
                            const int32_t* seqstart_q, int batch, int sq, int hq, int dv,
                            int num_splits, int dtype, float o_scale);

/* x: [rows, heads, d] in place; row r uses table row pos[r]; cos/sin: [*, rotary_dim/2] in the data dtype. */
int fck_orc_rope(void* x, int rows, int heads, int d, const int32_t* pos, const void* cos_tab,
                 const void* sin_tab, int rotary_dim, int rope_mode, int dtype);

/* Append knew/vnew (packed by cu_seqlens_knew, [total_new, Hk, D|Dv]) behind seqlen_k[b] existing tokens,
   rotate knew and (in place, optional) q ([total_new, Hq, D], same packing). */
int fck_orc_appendkv(void* q, void* k_cache, void* v_cache, const void* knew, const void* vnew,
                     const int32_t* seqlen_k, const int32_t* cu_seqlens_knew, const void* cos_tab,
                     const void* sin_tab, int rotary_dim, int rope_mode, int has_mask,
                     const int32_t* block_table, int block_table_stride, int page_size,
                     const int32_t* cache_batch_idx, int64_t cache_batch_stride_rows, int batch, int hq,
                     int hk, int d, int dv, int dtype, int kv_dtype, float k_descale, float v_descale);
/* kv_dtype FCK_ORC_FP8: the caches hold one e4m3 byte per element: cache = fp8(value a 16-bit cache would hold / descale) */

/* fp32 -> e4m3 byte: round to nearest even, finite overflow saturates to +-448, NaN / inf give NaN */
uint8_t fck_orc_f32_to_fp8(float f);

/* Gather one sequence's first n rows of a paged cache into dst [n, Hk, D]. */
int fck_orc_gather_paged(const void* cache, const int32_t* pages, int page_size, int n, int hk, int d,
                         int elem_bytes, void* dst);

/* value of one e4m3 byte (NaN for 0x7f / 0xff) */
float fck_orc_fp8_to_f32(uint8_t x);

int fck_orc_num_threads(void);

#ifdef __cplusplus
}
#endif
#endif
