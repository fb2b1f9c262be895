/*
 * TEST INFRASTRUCTURE - NOT PART OF THE PRODUCT.  See fmha_oracle.h.
 *
 * The attention pipeline restated here is the ck_tile host reference that FlashCK's generated
 * harness includes (core/module/kernels/attention_kernels/fmha_common_jinja.h:80):
 *   S = Q.K^T, fp32 accumulate, sequential in k     ck_tile/host/reference/reference_batched_gemm.hpp:19-49
 *   S *= scale (accumulator element op)             same file, acc_element_op
 *   S = -inf where masked                           ck_tile/host/reference/reference_batched_masking.hpp:13-31
 *   P = softmax(S) in fp32, LSE = max + ln(sum)     ck_tile/host/reference/reference_batched_softmax.hpp:16-70
 *   P is stored in the data type                    fmha_common_jinja.h:120-189 (PDataType = data type)
 *   O = P.V, fp32 accumulate, stored in data type   reference_batched_gemm.hpp:19-49
 *
 * Pinned by tests/test_oracle_*.py against torch's scaled_dot_product_attention, brute-force numpy,
 * closed forms and the golden vectors under tests/golden/.
 */
#include "fmha_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------------------------------ */
/* element conversion                                                                           */
/* ------------------------------------------------------------------------------------------ */

static inline float bits_to_f32(uint32_t u)
{
    float f;
    memcpy(&f, &u, 4);
    return f;
}
static inline uint32_t f32_to_bits(float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}

static inline float bf16_to_f32(uint16_t x) { return bits_to_f32((uint32_t)x << 16); }

/* Round to nearest even: what static_cast<__bf16>(float) does, which is ck_tile's float_to_bf16 when it is
   built with the LLVM bf16 type (ck_tile/core/numeric/bfloat16.hpp:283-291, config.hpp:195-203: HIP >= 7). */
static inline uint16_t f32_to_bf16(float f)
{
    uint32_t u = f32_to_bits(f);
    if ((u & 0x7f800000u) == 0x7f800000u) { /* inf / nan */
        if (u & 0x007fffffu) return (uint16_t)((u >> 16) | 0x0040u);
        return (uint16_t)(u >> 16);
    }
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

static inline float fp16_to_f32(uint16_t h)
{
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    if (exp == 0) {
        if (man == 0) return bits_to_f32(sign);
        /* subnormal: value = man * 2^-24 */
        float v = (float)man * (1.0f / 16777216.0f);
        return sign ? -v : v;
    }
    if (exp == 31) return bits_to_f32(sign | 0x7f800000u | (man << 13));
    return bits_to_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

static inline uint16_t f32_to_fp16(float f)
{
    uint32_t u = f32_to_bits(f);
    uint32_t sign = (u >> 16) & 0x8000u;
    uint32_t au = u & 0x7fffffffu;
    if (au >= 0x7f800000u) { /* inf / nan */
        if (au > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((au >> 13) & 0x3ffu));
        return (uint16_t)(sign | 0x7c00u);
    }
    if (au >= 0x477ff000u) { /* >= 65520 rounds to inf */
        return (uint16_t)(sign | 0x7c00u);
    }
    if (au < 0x38800000u) { /* subnormal half or zero: |f| < 2^-14 */
        if (au < 0x33000000u) return (uint16_t)sign; /* < 2^-25 -> 0 */
        /* exact: scale to integer units of 2^-24 with round-to-nearest-even */
        float af = bits_to_f32(au);
        float scaled = af * 16777216.0f; /* exact power-of-two scaling */
        float r = nearbyintf(scaled);    /* default rounding mode: nearest even */
        return (uint16_t)(sign | (uint32_t)r);
    }
    uint32_t e = (au >> 23) - 112u;
    uint32_t m = au & 0x7fffffu;
    uint32_t h = (e << 10) | (m >> 13);
    uint32_t rem = m & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h += 1u;
    return (uint16_t)(sign | h);
}

/* OCP e4m3 ("e4m3fn"): 1 sign, 4 exponent (bias 7), 3 mantissa bits; no infinities, S.1111.111 is NaN, exponent 0 is
   subnormal (mantissa / 8 * 2^-6). */
float fck_orc_fp8_to_f32(uint8_t x)
{
    const int e = (x >> 3) & 15, m = x & 7;
    float v;
    if (e == 15 && m == 7)
        v = NAN;
    else if (e == 0)
        v = ldexpf((float)m, -9);
    else
        v = ldexpf(1.f + (float)m / 8.f, e - 7);
    return (x & 0x80) ? -v : v;
}

/* fp32 -> OCP e4m3, round to nearest even, saturating: finite values beyond +-448 give +-448 (0x7e), NaN and infinities
   give NaN (0x7f).  The software conversion of ck_tile (ck_tile/core/numeric/float8.hpp:249-470, run_cast_to_f8 with
   clip = true, no stochastic rounding) and, on the device, fmed3(x, 448, -448) on finite values followed by the RNE
   conversion instruction (same file :600-662). */
uint8_t fck_orc_f32_to_fp8(float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    const uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
    if ((u & 0x7f800000u) == 0x7f800000u) return (uint8_t)(sign | 0x7fu);
    float a = fabsf(f);
    if (a >= 448.f) return (uint8_t)(sign | 0x7eu);
    if (a == 0.f) return sign;
    /* the grid of representable values around a: spacing 2^(e-3) for a in [2^e, 2^(e+1)), e >= -6; 2^-9 below 2^-6 */
    int e;
    (void)frexpf(a, &e); /* a = m * 2^e, m in [0.5, 1) -> a in [2^(e-1), 2^e) */
    int ex = e - 1;
    if (ex < -6) ex = -6;
    const float q = ldexpf(a, 3 - ex);       /* a in units of the spacing: exact (a power-of-two scaling) */
    float r = rintf(q);                      /* round to nearest even (default rounding mode) */
    /* r in [0, 16]; r == 16 means the value rounded up into the next binade */
    int mant = (int)r, be = ex + 7;          /* biased exponent for normal numbers */
    if (ex == -6 && mant < 8) return (uint8_t)(sign | (uint8_t)mant); /* subnormal (or zero) */
    if (mant == 16) {
        mant = 8;
        be += 1;
    }
    if (be > 15 || (be == 15 && mant - 8 > 6)) return (uint8_t)(sign | 0x7eu); /* cannot happen below 448; kept for safety */
    return (uint8_t)(sign | (uint8_t)(be << 3) | (uint8_t)(mant - 8));
}

static inline float ld(const void* base, int64_t idx, int dtype)
{
    if (dtype == FCK_ORC_FP8) return fck_orc_fp8_to_f32(((const uint8_t*)base)[idx]);
    uint16_t x = ((const uint16_t*)base)[idx];
    return dtype == FCK_ORC_BF16 ? bf16_to_f32(x) : fp16_to_f32(x);
}
static inline uint16_t cvt(float f, int dtype) { return dtype == FCK_ORC_BF16 ? f32_to_bf16(f) : f32_to_fp16(f); }
static inline float rnd(float f, int dtype)
{
    if (dtype == FCK_ORC_FP8) return fck_orc_fp8_to_f32(fck_orc_f32_to_fp8(f));
    return dtype == FCK_ORC_BF16 ? bf16_to_f32(f32_to_bf16(f)) : fp16_to_f32(f32_to_fp16(f));
}
/* element idx of an output tensor.  fp8 outputs: o_acc_element_func = saturates<fp8_t> after scales{scale_o}
   (ck_tile/ops/fmha/kernel/fmha_fwd_kernel.hpp:1530-1538); the reference passes scale_o = 1
   (core/module/kernels/attention_kernels/fmha_fwd/fmha_fwd_jinja.h:327-328). */
static inline void st(void* base, int64_t idx, float f, int dtype, float o_scale)
{
    if (dtype == FCK_ORC_FP8)
        ((uint8_t*)base)[idx] = fck_orc_f32_to_fp8(f * (o_scale != 0.f ? o_scale : 1.f));
    else
        ((uint16_t*)base)[idx] = cvt(f, dtype);
}

int fck_orc_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ------------------------------------------------------------------------------------------ */
/* mask                                                                                         */
/* ------------------------------------------------------------------------------------------ */

/* make_generic_attention_mask_coordinates_from_lr_window + GenericAttentionMask::IsOutOfBound,
   ck_tile/ops/fmha/block/block_masking.hpp:608-628 and :359-373.  MASK_GENERIC uses the bottom-right
   anchoring, as every caller passes is_top_left = (mask_type == top_left). */
static void mask_coords(int mask_type, int64_t wl, int64_t wr, int sq, int sk, int64_t* y, int64_t* x)
{
    int top_left = (mask_type == FCK_ORC_MASK_TOP_LEFT);
    int64_t left_tmp = top_left ? sq - 1 : sk - 1;
    int64_t right_tmp = top_left ? sk - 1 : sq - 1;
    int64_t l = wl < 0 ? left_tmp : wl;
    int64_t r = wr < 0 ? right_tmp : wr;
    int64_t x_tmp = top_left ? 0 : sk - sq;
    int64_t y_tmp = top_left ? 0 : sq - sk;
    *x = 1 + r + x_tmp;
    *y = 1 + l + y_tmp;
}

static inline int visible_yx(int mask_type, int64_t y, int64_t x, int sk, int i, int j)
{
    if (mask_type == FCK_ORC_NO_MASK) return j < sk;
    int64_t x_start = -y + i + 1;
    int64_t x_end = i + x < sk ? i + x : sk;
    return !(j < x_start || j >= x_end);
}

int fck_orc_visible(int mask_type, int64_t wl, int64_t wr, int sq, int sk, int i, int j)
{
    int64_t y, x;
    mask_coords(mask_type, wl, wr, sq, sk, &y, &x);
    return visible_yx(mask_type, y, x, sk, i, j);
}

/* ------------------------------------------------------------------------------------------ */
/* K/V row lookup                                                                               */
/* ------------------------------------------------------------------------------------------ */

static int seq_q_len(const fck_orc_problem* p, int b)
{
    return p->seqstart_q ? p->seqstart_q[b + 1] - p->seqstart_q[b] : p->sq;
}
static int64_t seq_q_row0(const fck_orc_problem* p, int b)
{
    return p->seqstart_q ? p->seqstart_q[b] : (int64_t)b * p->sq;
}
static int seq_k_len(const fck_orc_problem* p, int b)
{
    switch (p->kv_mode) {
    case FCK_ORC_KV_BATCH: return p->seqlen_k ? p->seqlen_k[b] : p->sk;
    /* ck_tile/ops/fmha/kernel/fmha_fwd_splitkv_kernel.hpp:648-650: seqlen_k_ptr, when given, is the logical length of
       a packed sequence whose slot [seqstart_k[b], seqstart_k[b+1]) may hold padding behind it */
    case FCK_ORC_KV_GROUP: return p->seqlen_k ? p->seqlen_k[b] : p->seqstart_k[b + 1] - p->seqstart_k[b];
    case FCK_ORC_KV_BLOCK_TABLE: return p->seqlen_k[b];
    case FCK_ORC_KV_PAGE_LIST: {
        int np = p->kv_indptr[b + 1] - p->kv_indptr[b];
        if (np <= 0) return 0;
        int last = p->kv_last_page_lens ? p->kv_last_page_lens[b] : p->page_size;
        return (np - 1) * p->page_size + last;
    }
    }
    return 0;
}
/* physical row (in units of [Hk, D] rows) of logical key j of sequence b */
static int64_t kv_row(const fck_orc_problem* p, int b, int j)
{
    switch (p->kv_mode) {
    case FCK_ORC_KV_BATCH: {
        int64_t cb = p->cache_batch_idx ? p->cache_batch_idx[b] : b;
        return cb * p->sk + j;
    }
    case FCK_ORC_KV_GROUP: return (int64_t)p->seqstart_k[b] + j;
    case FCK_ORC_KV_BLOCK_TABLE: {
        /* fmha_fwd_split_kv_jinja.h:318,395-398: row b of the table, entry j / P */
        int64_t page = p->block_table[(int64_t)b * p->block_table_stride + j / p->page_size];
        return page * p->page_size + j % p->page_size;
    }
    case FCK_ORC_KV_PAGE_LIST: {
        int64_t page = p->kv_page_indices[p->kv_indptr[b] + j / p->page_size];
        return page * p->page_size + j % p->page_size;
    }
    }
    return 0;
}

/* ------------------------------------------------------------------------------------------ */
/* attention core: one query row over keys [k0, k1)                                             */
/* ------------------------------------------------------------------------------------------ */

typedef struct {
    float* s;      /* [cap] scores / probabilities */
    int64_t* rows; /* [cap] physical rows */
    float* qf;     /* [d] */
    float* of;     /* [dv] */
} scratch_t;

/* Returns lse through *lse_out; writes normalised fp32 output (P rounded to the data type first) into of[]. */
static void attend_row(const fck_orc_problem* p, const void* q, const void* k, const void* v, int b, int64_t qrow, int h,
                       const int64_t* rows, int k0, int k1, int i, int sq_b, int sk_b, scratch_t* sc, float* lse_out)
{
    const int d = p->d, dv = p->dv, hk = p->hk, dt = p->dtype;
    const int hkv = h / (p->hq / p->hk);
    int64_t y, x;
    mask_coords(p->mask_type, p->window_left, p->window_right, sq_b, sk_b, &y, &x);
    for (int t = 0; t < d; ++t) sc->qf[t] = ld(q, (qrow * p->hq + h) * d + t, dt);

    const int kv8 = p->kv_dtype == FCK_ORC_FP8 || dt == FCK_ORC_FP8; /* all-fp8 roles: Q, K, V, P and O are e4m3 */
    const float kd = (kv8 && p->k_descale != 0.f) ? p->k_descale : 1.f, vd = (kv8 && p->v_descale != 0.f) ? p->v_descale : 1.f;
    /* bias row of (b, h, i) / ALiBi slope of (b, h) */
    int64_t bias_row = 0;
    float slope = 0.f;
    int alibi_mode = 2;
    if (p->bias_type == 1) {
        bias_row = (int64_t)h * p->bias_head_stride +
                   (p->seqstart_q ? qrow * p->bias_row_stride : (int64_t)b * p->bias_batch_stride + (int64_t)i * p->bias_row_stride);
    } else if (p->bias_type == 2) {
        slope = ((const float*)p->bias)[(int64_t)b * p->bias_batch_stride + h];
        /* make_alibi_from_lr_mask: a causal window is VERTICAL, else the mask enum names the diagonal; no mask:
           FROM_BOTTOM_RIGHT */
        if (p->mask_type == 0)
            alibi_mode = 2;
        else if (p->window_left < 0 && p->window_right == 0)
            alibi_mode = 0;
        else
            alibi_mode = p->mask_type == 1 ? 1 : 2;
    }

    float vmax = -INFINITY;
    for (int j = k0; j < k1; ++j) {
        float acc = 0.f;
        const int64_t base = (rows[j] * hk + hkv) * d;
        if (kv8)
            for (int t = 0; t < d; ++t) acc += sc->qf[t] * fck_orc_fp8_to_f32(((const uint8_t*)k)[base + t]);
        else
            for (int t = 0; t < d; ++t) acc += sc->qf[t] * ld(k, base + t, dt);
        float sv = acc * (p->scale * kd);
        if (p->logits_soft_cap > 0.f) sv = p->logits_soft_cap * tanhf(sv / p->logits_soft_cap);
        if (p->bias_type == 1) {
            sv += dt == FCK_ORC_FP8 ? ((const float*)p->bias)[bias_row + j] : ld(p->bias, bias_row + j, dt); /* BiasDataType = float for fp8 */
        } else if (p->bias_type == 2) {
            /* Alibi::update (row major): VERTICAL adds slope * col; the two diagonal modes add -slope * |zero - col| with
               zero = row (top left) or row + sk - sq (bottom right: shift_right_down - shift_left_up = sk - sq) */
            if (alibi_mode == 0)
                sv += slope * (float)j;
            else
                sv += -slope * (float)labs((long)(alibi_mode == 1 ? i : i + sk_b - sq_b) - (long)j);
        }
        if (!visible_yx(p->mask_type, y, x, sk_b, i, j)) sv = -INFINITY;
        sc->s[j - k0] = sv;
        vmax = vmax < sv ? sv : vmax;
    }
    if (isinf(vmax) && vmax < 0) vmax = 0.f;
    float sum = 0.f;
    for (int j = k0; j < k1; ++j) sum += expf(sc->s[j - k0] - vmax);
    float inv = (sum == 0.f) ? 1.f : 1.f / sum;
    for (int t = 0; t < dv; ++t) sc->of[t] = 0.f;
    for (int j = k0; j < k1; ++j) {
        float pj = rnd(expf(sc->s[j - k0] - vmax) * inv, dt);
        if (pj == 0.f) continue; /* masked keys may sit in pages holding non-finite fill */
        const int64_t base = (rows[j] * hk + hkv) * dv;
        if (kv8)
            for (int t = 0; t < dv; ++t) sc->of[t] += pj * fck_orc_fp8_to_f32(((const uint8_t*)v)[base + t]);
        else
            for (int t = 0; t < dv; ++t) sc->of[t] += pj * ld(v, base + t, dt);
    }
    for (int t = 0; t < dv; ++t) sc->of[t] *= vd;
    /* softmax reference: lse = max + ln(sum); a row with no visible key gives ln(0) = -inf */
    *lse_out = (sum == 0.f) ? -INFINITY : vmax + logf(sum);
}

static int max_sk(const fck_orc_problem* p)
{
    int m = 1;
    for (int b = 0; b < p->batch; ++b) {
        int s = seq_k_len(p, b);
        if (s > m) m = s;
    }
    return m;
}

static int check(const fck_orc_problem* p)
{
    if (p->dtype != FCK_ORC_BF16 && p->dtype != FCK_ORC_FP16 && p->dtype != FCK_ORC_FP8) return -1;
    if (p->hk <= 0 || p->hq % p->hk) return -2;
    return 0;
}

static int64_t total_q_rows(const fck_orc_problem* p)
{
    return p->seqstart_q ? p->seqstart_q[p->batch] : (int64_t)p->batch * p->sq;
}

int fck_orc_fmha_fwd(const fck_orc_problem* p, const void* q, const void* k, const void* v, void* o, float* lse)
{
    int rc = check(p);
    if (rc) return rc;
    const int cap = max_sk(p);
    const int64_t tq = total_q_rows(p);
    for (int b = 0; b < p->batch; ++b) {
        const int sq_b = seq_q_len(p, b), sk_b = seq_k_len(p, b);
        const int64_t row0 = seq_q_row0(p, b);
        int64_t* rows = (int64_t*)malloc(sizeof(int64_t) * (size_t)(sk_b > 0 ? sk_b : 1));
        for (int j = 0; j < sk_b; ++j) rows[j] = kv_row(p, b, j);
        const int64_t ntask = (int64_t)p->hq * sq_b;
#pragma omp parallel
        {
            scratch_t sc;
            sc.s = (float*)malloc(sizeof(float) * (size_t)cap);
            sc.qf = (float*)malloc(sizeof(float) * (size_t)p->d);
            sc.of = (float*)malloc(sizeof(float) * (size_t)p->dv);
            sc.rows = 0;
#pragma omp for schedule(dynamic, 4)
            for (int64_t t = 0; t < ntask; ++t) {
                const int h = (int)(t / sq_b), i = (int)(t % sq_b);
                float l;
                attend_row(p, q, k, v, b, row0 + i, h, rows, 0, sk_b, i, sq_b, sk_b, &sc, &l);
                const int64_t orow = ((row0 + i) * p->hq + h) * p->dv;
                for (int c = 0; c < p->dv; ++c) st(o, orow + c, sc.of[c], p->dtype, p->o_scale);
                if (lse) {
                    if (p->seqstart_q)
                        lse[(int64_t)h * tq + row0 + i] = l;
                    else
                        lse[((int64_t)b * p->hq + h) * p->sq + i] = l;
                }
            }
            free(sc.s);
            free(sc.qf);
            free(sc.of);
        }
        free(rows);
    }
    return 0;
}

/* Split s of ns covers keys [s*ceil(sk/ns), min(sk, (s+1)*ceil(sk/ns))):
   GenericAttentionMask::GetTileRangeAlongX(..., num_splits, i_split), block_masking.hpp:312-326.
   Per split: O_acc normalised by that split's own sum, LSE_acc = max + ln(sum), -inf for a split without a
   visible key: ck_tile/ops/fmha/pipeline/block_fmha_fwd_splitkv_pipeline_qr_ks_vs.hpp:237-256,663-711.
   Workspace shapes: fmha_fwd_split_kv_jinja.h:543-547 and fmha_fwd_split_kv_combine_jinja.h:129-139. */
int fck_orc_fmha_splitkv(const fck_orc_problem* p, const void* q, const void* k, const void* v, int num_splits,
                         float* o_acc, float* lse_acc)
{
    int rc = check(p);
    if (rc) return rc;
    if (num_splits < 1) return -3;
    const int cap = max_sk(p);
    const int group = p->seqstart_q != 0;
    const int64_t Sq = group ? total_q_rows(p) : p->sq;
    for (int b = 0; b < p->batch; ++b) {
        const int sq_b = seq_q_len(p, b), sk_b = seq_k_len(p, b);
        const int64_t row0 = seq_q_row0(p, b);
        const int64_t wrow0 = group ? row0 : 0;
        const int64_t wb = group ? 0 : b;
        int64_t* rows = (int64_t*)malloc(sizeof(int64_t) * (size_t)(sk_b > 0 ? sk_b : 1));
        for (int j = 0; j < sk_b; ++j) rows[j] = kv_row(p, b, j);
        int per = (sk_b + num_splits - 1) / num_splits;
        if (per < 1) per = 1;
        const int64_t ntask = (int64_t)p->hq * sq_b * num_splits;
#pragma omp parallel
        {
            scratch_t sc;
            sc.s = (float*)malloc(sizeof(float) * (size_t)cap);
            sc.qf = (float*)malloc(sizeof(float) * (size_t)p->d);
            sc.of = (float*)malloc(sizeof(float) * (size_t)p->dv);
            sc.rows = 0;
#pragma omp for schedule(dynamic, 1)
            for (int64_t t = 0; t < ntask; ++t) {
                const int s = (int)(t % num_splits);
                const int i = (int)((t / num_splits) % sq_b);
                const int h = (int)(t / num_splits / sq_b);
                int k0 = per * s, k1 = k0 + per;
                if (k1 > sk_b) k1 = sk_b;
                if (k0 > k1) k0 = k1;
                float l;
                attend_row(p, q, k, v, b, row0 + i, h, rows, k0, k1, i, sq_b, sk_b, &sc, &l);
                const int64_t w = ((wb * p->hq + h) * num_splits + s) * Sq + wrow0 + i;
                lse_acc[w] = l;
                for (int c = 0; c < p->dv; ++c) o_acc[w * p->dv + c] = isinf(l) ? 0.f : sc.of[c];
            }
            free(sc.s);
            free(sc.qf);
            free(sc.of);
        }
        free(rows);
    }
    return 0;
}

/* ck_tile/ops/fmha/pipeline/block_fmha_fwd_splitkv_combine_pipeline.hpp:150-316:
   m = max_s lse_s; sum = sum_s exp(lse_s - m) (0 when m = -inf); LSE = ln(sum) + m (-inf when sum = 0);
   w_s = exp(lse_s - LSE) (0 when LSE = -inf); O = sum_s w_s * O_s, stored in the data type. */
int fck_orc_splitkv_combine(const float* lse_acc, const float* o_acc, void* o, float* lse, const int32_t* seqstart_q,
                            int batch, int sq, int hq, int dv, int num_splits, int dtype, float o_scale)
{
    if (dtype != FCK_ORC_BF16 && dtype != FCK_ORC_FP16 && dtype != FCK_ORC_FP8) return -1;
    const int group = seqstart_q != 0;
    const int64_t Sq = group ? seqstart_q[batch] : sq;
    const int Bs = group ? 1 : batch;
#pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < Bs; ++b)
        for (int h = 0; h < hq; ++h) {
            for (int64_t i = 0; i < Sq; ++i) {
                const int64_t w0 = (((int64_t)b * hq + h) * num_splits) * Sq + i;
                float m = -INFINITY;
                for (int s = 0; s < num_splits; ++s) {
                    float l = lse_acc[w0 + s * Sq];
                    m = m < l ? l : m;
                }
                float sum = 0.f;
                if (!(isinf(m) && m < 0))
                    for (int s = 0; s < num_splits; ++s) sum += expf(lse_acc[w0 + s * Sq] - m);
                float L = (sum == 0.f) ? -INFINITY : logf(sum) + m;
                const int64_t orow = (((int64_t)b * Sq + i) * hq + h) * dv;
                for (int c = 0; c < dv; ++c) {
                    float acc = 0.f;
                    for (int s = 0; s < num_splits; ++s) {
                        float w = (isinf(L) && L < 0) ? 0.f : expf(lse_acc[w0 + s * Sq] - L);
                        acc += w * o_acc[(w0 + s * Sq) * dv + c];
                    }
                    st(o, orow + c, acc, dtype, o_scale);
                }
                if (lse) lse[((int64_t)b * hq + h) * Sq + i] = L;
            }
        }
    return 0;
}

/* ------------------------------------------------------------------------------------------ */
/* rotary embedding, appendKV, gather                                                           */
/* ------------------------------------------------------------------------------------------ */

/* ck_tile/host/reference/reference_batched_rotary_position_embedding.hpp:29-70.  The three fp32 operations are
   rounded one by one (x*cos, other*sin, their sum): volatile keeps the compiler from contracting them. */
static void rope_row(const uint16_t* in, uint16_t* out, int d, const void* cos_tab, const void* sin_tab, int64_t pos,
                     int rotary_dim, int rope_mode, int dtype)
{
    const int half = rotary_dim / 2;
    for (int t = 0; t < d; ++t) {
        if (t >= rotary_dim || rope_mode == FCK_ORC_ROPE_NONE) {
            out[t] = in[t];
            continue;
        }
        int ci, other;
        float sign;
        if (rope_mode == FCK_ORC_ROPE_INTERLEAVED) {
            ci = t / 2;
            other = (t % 2 == 0) ? t + 1 : t - 1;
            sign = (t % 2 == 0) ? -1.f : 1.f;
        } else {
            ci = t % half;
            other = (t + half) % rotary_dim;
            sign = (other < half) ? 1.f : -1.f;
        }
        const float c = ld(cos_tab, pos * half + ci, dtype);
        const float s = ld(sin_tab, pos * half + ci, dtype);
        const float xin = dtype == FCK_ORC_BF16 ? bf16_to_f32(in[t]) : fp16_to_f32(in[t]);
        const float xo = sign * (dtype == FCK_ORC_BF16 ? bf16_to_f32(in[other]) : fp16_to_f32(in[other]));
        volatile float a = xin * c;
        volatile float bb = xo * s;
        volatile float r = a + bb;
        out[t] = cvt(r, dtype);
    }
}

int fck_orc_rope(void* x, int rows, int heads, int d, const int32_t* pos, const void* cos_tab, const void* sin_tab,
                 int rotary_dim, int rope_mode, int dtype)
{
    if (rotary_dim > d || rotary_dim % 2) return -1;
    uint16_t* tmp = (uint16_t*)malloc(sizeof(uint16_t) * (size_t)d);
    for (int r = 0; r < rows; ++r)
        for (int h = 0; h < heads; ++h) {
            uint16_t* row = (uint16_t*)x + ((int64_t)r * heads + h) * d;
            rope_row(row, tmp, d, cos_tab, sin_tab, pos[r], rotary_dim, rope_mode, dtype);
            memcpy(row, tmp, sizeof(uint16_t) * (size_t)d);
        }
    free(tmp);
    return 0;
}

/* ck_tile/ops/fmha/kernel/fmha_fwd_appendkv_kernel.hpp:455-466 (q rows use table row seqlen_k + has_mask * i),
   :510-521 (knew rows use seqlen_k + i) and pipeline/block_fmha_fwd_appendkv_pipeline.hpp:151-184 (new rows land
   at logical positions seqlen_k + i through the block table).  ck_tile takes one seqlen_knew for the whole
   batch; cu_seqlens_knew generalises it to a ragged batch. */
int fck_orc_appendkv(void* q, void* k_cache, void* v_cache, const void* knew, const void* vnew, const int32_t* seqlen_k,
                     const int32_t* cu_seqlens_knew, const void* cos_tab, const void* sin_tab, int rotary_dim,
                     int rope_mode, int has_mask, const int32_t* block_table, int block_table_stride, int page_size,
                     const int32_t* cache_batch_idx, int64_t cache_batch_stride_rows, int batch, int hq, int hk, int d,
                     int dv, int dtype, int kv_dtype, float k_descale, float v_descale)
{
    if (dtype != FCK_ORC_BF16 && dtype != FCK_ORC_FP16) return -1;
    if (kv_dtype != 0 && kv_dtype != FCK_ORC_FP8) return -1;
    const int kv8 = kv_dtype == FCK_ORC_FP8;
    uint16_t* tmp = (uint16_t*)malloc(sizeof(uint16_t) * (size_t)d);
    for (int b = 0; b < batch; ++b) {
        const int n0 = cu_seqlens_knew[b], n = cu_seqlens_knew[b + 1] - n0;
        const int L = seqlen_k[b];
        for (int i = 0; i < n; ++i) {
            const int t = L + i;
            int64_t prow;
            if (block_table) {
                int64_t page = block_table[(int64_t)b * block_table_stride + t / page_size];
                prow = page * page_size + t % page_size;
            } else {
                int64_t cb = cache_batch_idx ? cache_batch_idx[b] : b;
                prow = cb * cache_batch_stride_rows + t;
            }
            for (int h = 0; h < hk; ++h) {
                const uint16_t* src = (const uint16_t*)knew + ((int64_t)(n0 + i) * hk + h) * d;
                if (kv8) {
                    /* quantised cache: the row a 16-bit cache would hold (rotated, rounded to T), divided by the static
                       scale and converted to e4m3; V likewise without the rotation */
                    if (rope_mode != FCK_ORC_ROPE_NONE)
                        rope_row(src, tmp, d, cos_tab, sin_tab, t, rotary_dim, rope_mode, dtype);
                    else
                        memcpy(tmp, src, sizeof(uint16_t) * (size_t)d);
                    uint8_t* kd = (uint8_t*)k_cache + (prow * hk + h) * d;
                    for (int c = 0; c < d; ++c) kd[c] = fck_orc_f32_to_fp8(ld(tmp, c, dtype) / k_descale);
                    uint8_t* vd = (uint8_t*)v_cache + (prow * hk + h) * dv;
                    for (int c = 0; c < dv; ++c) vd[c] = fck_orc_f32_to_fp8(ld(vnew, ((int64_t)(n0 + i) * hk + h) * dv + c, dtype) / v_descale);
                    continue;
                }
                uint16_t* dst = (uint16_t*)k_cache + (prow * hk + h) * d;
                if (rope_mode != FCK_ORC_ROPE_NONE) {
                    rope_row(src, tmp, d, cos_tab, sin_tab, t, rotary_dim, rope_mode, dtype);
                    memcpy(dst, tmp, sizeof(uint16_t) * (size_t)d);
                } else {
                    memcpy(dst, src, sizeof(uint16_t) * (size_t)d);
                }
                memcpy((uint16_t*)v_cache + (prow * hk + h) * dv, (const uint16_t*)vnew + ((int64_t)(n0 + i) * hk + h) * dv,
                       sizeof(uint16_t) * (size_t)dv);
            }
            if (q && rope_mode != FCK_ORC_ROPE_NONE) {
                const int64_t qpos = L + (has_mask ? i : 0);
                for (int h = 0; h < hq; ++h) {
                    uint16_t* row = (uint16_t*)q + ((int64_t)(n0 + i) * hq + h) * d;
                    rope_row(row, tmp, d, cos_tab, sin_tab, qpos, rotary_dim, rope_mode, dtype);
                    memcpy(row, tmp, sizeof(uint16_t) * (size_t)d);
                }
            }
        }
    }
    free(tmp);
    return 0;
}

/* Logical token t of a sequence lives at (pages[t / P], t % P): fmha_fwd_split_kv_jinja.h:295-306,549-552. */
int fck_orc_gather_paged(const void* cache, const int32_t* pages, int page_size, int n, int hk, int d, int elem_bytes,
                         void* dst)
{
    const size_t rowb = (size_t)hk * d * elem_bytes;
    for (int t = 0; t < n; ++t) {
        int64_t prow = (int64_t)pages[t / page_size] * page_size + t % page_size;
        memcpy((char*)dst + (size_t)t * rowb, (const char*)cache + (size_t)prow * rowb, rowb);
    }
    return 0;
}
