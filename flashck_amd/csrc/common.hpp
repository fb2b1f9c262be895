// Shared device/host helpers for the gfx950 FMHA kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "gfx950_ops.hpp"

namespace fck {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4_t __attribute__((ext_vector_type(4)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef short s16x8_t __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// Element traits: storage is 16 bit; MFMA operands are 8 packed elements.
struct BF16 {
    typedef bf16x8_t vec8;
    typedef __bf16 elem;
    // round to nearest even (v_cvt_pk_bf16_f32 on gfx950)
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi)
    {
        typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
        bf2 v;
        v[0] = (__bf16)lo;
        v[1] = (__bf16)hi;
        return __builtin_bit_cast(uint32_t, v);
    }
    static __device__ __forceinline__ float to_f32(uint16_t x) { return __builtin_bit_cast(float, (uint32_t)x << 16); }
    static __device__ __forceinline__ uint16_t from_f32(float f) { return __builtin_bit_cast(uint16_t, (__bf16)f); }
    static __device__ __forceinline__ f32x4_t mfma16(vec8 a, vec8 b, f32x4_t c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ f32x16_t mfma32(vec8 a, vec8 b, f32x16_t c)
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    // 16x16x16: 4 packed elements per operand (for 16-key tiles)
    static __device__ __forceinline__ f32x4_t mfma16k16(u32x2_t a, u32x2_t b, f32x4_t c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4_t, a), __builtin_bit_cast(s16x4_t, b), c, 0, 0, 0);
    }
};

struct FP16 {
    typedef f16x8_t vec8;
    typedef _Float16 elem;
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi)
    {
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        h2 v;
        v[0] = (_Float16)lo;
        v[1] = (_Float16)hi;
        return __builtin_bit_cast(uint32_t, v);
    }
    static __device__ __forceinline__ float to_f32(uint16_t x) { return (float)__builtin_bit_cast(_Float16, x); }
    static __device__ __forceinline__ uint16_t from_f32(float f) { return __builtin_bit_cast(uint16_t, (_Float16)f); }
    static __device__ __forceinline__ f32x4_t mfma16(vec8 a, vec8 b, f32x4_t c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ f32x16_t mfma32(vec8 a, vec8 b, f32x16_t c)
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ f32x4_t mfma16k16(u32x2_t a, u32x2_t b, f32x4_t c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(f16x4_t, a), __builtin_bit_cast(f16x4_t, b), c, 0, 0, 0);
    }
};

template <typename V>
__device__ __forceinline__ V as_vec8(u32x4_t x)
{
    return __builtin_bit_cast(V, x);
}

// 16-byte global load through the vector memory path.
__device__ __forceinline__ u32x4_t ldg16(const void* p) { return *reinterpret_cast<const u32x4_t*>(p); }
// Loads of data that is read once (a K/V cache streamed by a decode step): the non-temporal hint keeps the lines from
// displacing what the L2 holds, and on this chip a chip-wide stream of such loads runs about 10 % faster than one of
// plain loads (6.4 against 5.8 TB/s for 256-byte pieces at a 2 KiB stride).
__device__ __forceinline__ u32x4_t ldg16_stream(const void* p) { return __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p)); }
__device__ __forceinline__ u32x2_t ldg8_stream(const void* p) { return __builtin_nontemporal_load(reinterpret_cast<const u32x2_t*>(p)); }

// Transposing LDS read: within each group of 16 lanes, lane i receives element (i % 4) of the 8 bytes that lane
// 4k + i/4 addressed, for k = 0..3.  When lanes 4k..4k+3 address 16 consecutive 16-bit columns of row k, lane i ends up
// with column i of rows 0..3.
__device__ __forceinline__ u32x2_t lds_read_tr16(const void FCK_LDS* p)
{
    s16x4_t v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4_t FCK_LDS*)p);
    return __builtin_bit_cast(u32x2_t, v);
}

// Cross-lane reductions on the VALU (swap32 / swap16 of gfx950_ops.hpp).
// over the lane pair (l, l ^ 32)
__device__ __forceinline__ float pair32_max(float x)
{
    float a, b;
    swap32(x, a, b);
    return fmaxf(a, b);
}
__device__ __forceinline__ float pair32_sum(float x)
{
    float a, b;
    swap32(x, a, b);
    return a + b;
}
// over the four lanes that share l % 16
__device__ __forceinline__ float quad16_max(float x)
{
    float a, b;
    swap16(x, a, b);
    return pair32_max(fmaxf(a, b));
}
__device__ __forceinline__ float quad16_sum(float x)
{
    float a, b;
    swap16(x, a, b);
    return pair32_sum(a + b);
}

// 8 e4m3 bytes (the two low dwords of v) widened to 8 elements of T; exact, every e4m3 value is a T value
template <typename T>
__device__ __forceinline__ u32x4_t fp8x8_to_t(u32x4_t v)
{
    const f32x2_t a0 = __builtin_amdgcn_cvt_pk_f32_fp8((int)v[0], false), a1 = __builtin_amdgcn_cvt_pk_f32_fp8((int)v[0], true);
    const f32x2_t a2 = __builtin_amdgcn_cvt_pk_f32_fp8((int)v[1], false), a3 = __builtin_amdgcn_cvt_pk_f32_fp8((int)v[1], true);
    return u32x4_t{T::pack2(a0[0], a0[1]), T::pack2(a1[0], a1[1]), T::pack2(a2[0], a2[1]), T::pack2(a3[0], a3[1])};
}

// fp32 -> e4m3 byte (OCP encoding): round to nearest even; finite values saturate at +-448, NaN and infinities are left
// to the conversion instruction (as ck_tile converts: ck_tile/core/numeric/float8.hpp:600-662)
__device__ __forceinline__ uint32_t f32_to_fp8_sat(float x)
{
    const bool finite = (__builtin_bit_cast(uint32_t, x) & 0x7f800000u) != 0x7f800000u;
    const float c = finite ? fminf(fmaxf(x, -448.f), 448.f) : x;
    return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(c, c, 0, false) & 0xffu;
}

// two fp32 values in [0, 448] rounded to the nearest e4m3 value (ties to even), as fp32 again
__device__ __forceinline__ f32x2_t round_to_fp8(float a, float b)
{
    return __builtin_amdgcn_cvt_pk_f32_fp8(__builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false), false);
}

// four fp32 values -> four e4m3 bytes (a in the lowest), each converted as f32_to_fp8_sat does
__device__ __forceinline__ uint32_t pack_fp8x4_sat(float a, float b, float c, float d)
{
    auto clamp = [](float x) {
        const bool finite = (__builtin_bit_cast(uint32_t, x) & 0x7f800000u) != 0x7f800000u;
        return finite ? fminf(fmaxf(x, -448.f), 448.f) : x;
    };
    const int lo = __builtin_amdgcn_cvt_pk_fp8_f32(clamp(a), clamp(b), 0, false);
    return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(clamp(c), clamp(d), lo, true);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

// LSE combine of the split-KV partials of one output row, 4 columns from column c on:
//   LSE = logsumexp_s lse_acc[s];  O = sum_s exp(lse_acc[s] - LSE) * o_acc[s]
// (ck_tile/ops/fmha/pipeline/block_fmha_fwd_splitkv_combine_pipeline.hpp:150-316), evaluated as
// O = (sum_s e^(lse_s - m) o_s) / (sum_s e^(lse_s - m)) with a running maximum m over batches of kCombineBatch splits, so
// that all loads of a batch are in flight together: the work is a chain of memory round trips, not arithmetic.
// w0 is the workspace row of split 0 and `step` the distance to the next split's row; rows whose splits are all empty
// (-inf) give zeros; a single split is passed through unchanged.  Shared by the combine kernel and by the fused tail of
// the split-KV kernel, so both produce the same bits.
constexpr int kCombineBatch = 16;

template <int DV>
__device__ __forceinline__ f32x4_t combine_splits(const float* lse_acc, const float* o_acc, int64_t w0, int64_t step, int ns, int c,
                                                  int dv = DV)  // dv: floats per partial row as stored (<= DV)
{
    float m_run = -INFINITY, sum = 0.f;
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
    for (int s0 = 0; s0 < ns; s0 += kCombineBatch) {
        float l[kCombineBatch];
        f32x4_t v[kCombineBatch];
#pragma unroll
        for (int j = 0; j < kCombineBatch; ++j) {
            const bool ok = s0 + j < ns;
            const int64_t w = w0 + (ok ? s0 + j : s0) * step;  // out-of-range slots re-read a valid one and are dropped
            const float lj = lse_acc[w];
            l[j] = ok ? lj : -INFINITY;
            v[j] = *reinterpret_cast<const f32x4_t*>(o_acc + w * dv + c);
        }
        float mb = l[0];
#pragma unroll
        for (int j = 1; j < kCombineBatch; ++j) mb = fmaxf(mb, l[j]);
        const float m_new = fmaxf(m_run, mb);
        if (m_new == -INFINITY) continue;
        const float keep = __expf(m_run - m_new);  // 0 for the first non-empty batch
        sum *= keep;
#pragma unroll
        for (int k = 0; k < 4; ++k) acc[k] *= keep;
#pragma unroll
        for (int j = 0; j < kCombineBatch; ++j) {
            const float wgt = __expf(l[j] - m_new);
            sum += wgt;
            if (wgt != 0.f) {  // an empty split's partial row may hold anything
#pragma unroll
                for (int k = 0; k < 4; ++k) acc[k] = __builtin_fmaf(wgt, v[j][k], acc[k]);
            }
        }
        m_run = m_new;
    }
    if (sum == 0.f) return f32x4_t{0.f, 0.f, 0.f, 0.f};
    if (ns == 1) return acc;  // weight exactly 1
    const float inv = 1.f / sum;
    return f32x4_t{acc[0] * inv, acc[1] * inv, acc[2] * inv, acc[3] * inv};
}

// Visible key range [lo, hi) of query row i: GenericAttentionMask::IsOutOfBound,
// ck_tile/ops/fmha/block/block_masking.hpp:359-373 with (y, x) from
// make_generic_attention_mask_coordinates_from_lr_window, same file :608-628.
struct MaskYX {
    int32_t y, x;  // only read when masking != 0
    int32_t masking;
};

__host__ __device__ inline MaskYX make_mask(uint32_t mask_type, int64_t wl, int64_t wr, int32_t sq, int32_t sk)
{
    MaskYX m;
    m.masking = mask_type != 0;
    const bool tl = mask_type == 1;
    const int64_t left_tmp = tl ? sq - 1 : sk - 1;
    const int64_t right_tmp = tl ? sk - 1 : sq - 1;
    const int64_t l = wl < 0 ? left_tmp : wl;
    const int64_t r = wr < 0 ? right_tmp : wr;
    int64_t x = 1 + r + (tl ? 0 : sk - sq);
    int64_t y = 1 + l + (tl ? 0 : sq - sk);
    // clamp: only comparisons against [0, sk] matter
    const int64_t big = (int64_t)1 << 30;
    x = x > big ? big : (x < -big ? -big : x);
    y = y > big ? big : (y < -big ? -big : y);
    m.x = (int32_t)x;
    m.y = (int32_t)y;
    return m;
}

__host__ __device__ inline int32_t mask_lo(const MaskYX& m, int32_t i)
{
    if (!m.masking) return 0;
    const int32_t v = i + 1 - m.y;
    return v > 0 ? v : 0;
}
__host__ __device__ inline int32_t mask_hi(const MaskYX& m, int32_t i, int32_t sk)
{
    if (!m.masking) return sk;
    const int64_t v = (int64_t)i + m.x;
    return v < sk ? (v > 0 ? (int32_t)v : 0) : sk;
}

// Optional score modifiers; an all-zero struct means none.  Order (ck_tile/ops/fmha/pipeline/
// block_fmha_pipeline_qr_ks_vs.hpp:391-449): x = scale * q.k; soft cap x = cap * tanh(x / cap)
// (ck_tile/ops/fmha/block/variants.hpp:208-209); bias added; then the mask.
//   elementwise bias: data dtype, element (b, h, i, j) at bias[b * batch_stride + h * head_stride + i * row_stride + j]
//                     (group mode: i counts from the first packed query row of the sequence, batch_stride unused):
//                     ck_tile/ops/fmha/kernel/fmha_fwd_splitkv_kernel.hpp:608-688,925-932
//   ALiBi:            fp32 slope of (b, h) at bias[b * batch_stride + h]; added term and mode as in
//                     ck_tile/ops/fmha/block/block_position_encoding.hpp:19-121,138-152 and
//                     ck_tile/ops/fmha/kernel/fmha_fwd_kernel.hpp:1482-1507
struct ScoreMod {
    const void* bias;
    int64_t batch_stride, head_stride, row_stride;
    int64_t cols;       // elementwise: columns of a bias row (0: not stated)
    int32_t bias_type;  // 0 none, 1 elementwise, 2 ALiBi
    float soft_cap;     // > 0: on
    float scale;        // the softmax scale in natural units (the soft cap is not linear, so it cannot be folded)
    int32_t bias_f32;   // elementwise: the bias holds fp32 (the e4m3 type roles), strides in floats; 0: the data type T
    __host__ __device__ bool active() const { return bias_type != 0 || soft_cap > 0.f; }
};

// ALiBi position modes (AlibiMode, block_position_encoding.hpp:38-43)
enum : int32_t { kAlibiVertical = 0, kAlibiTopLeft = 1, kAlibiBottomRight = 2 };

// mode of a problem: a causal window (left < 0, right == 0) under any mask type gives VERTICAL, otherwise the mask type
// names the diagonal; without a mask the diagonal ends at the bottom right corner
__host__ __device__ inline int32_t alibi_mode(uint32_t mask_type, int64_t wl, int64_t wr)
{
    if (mask_type == 0) return kAlibiBottomRight;
    if (wl < 0 && wr == 0) return kAlibiVertical;
    return mask_type == 1 ? kAlibiTopLeft : kAlibiBottomRight;
}

__device__ __forceinline__ float fast_tanh(float x)
{
    // 1 - 2 / (e^(2x) + 1): exact limits at +-inf, relative error of a few ulp elsewhere
    const float e = __builtin_amdgcn_exp2f(x * (2.f * kLog2e));
    return 1.f - 2.f * __builtin_amdgcn_rcpf(e + 1.f);
}

// The modifiers of one query row, set up once per row; score() maps a raw dot product to the log2-domain score
// (already multiplied by log2 e, so the caller's scale factor is 1).
template <typename T>
struct RowMod {
    const uint16_t* bias_row;  // elementwise: row (b, h, i) of the bias
    const float* bias_row32;   // the same when the bias holds fp32 (then bias_row is null)
    float slope;               // ALiBi: signed slope (positive for VERTICAL, negative otherwise)
    int32_t zero;              // ALiBi: column of distance 0 (unused for VERTICAL)
    int32_t mode;
    int32_t last_key;          // bias reads are clamped to the row's last key and to the last column of the bias
    float scale, cap, cap_rcp;
    int32_t bias_type;

    __device__ __forceinline__ void init(const ScoreMod& m, int b, int64_t first_row, int h, int i, int sq, int sk, uint32_t mask_type,
                                         int64_t wl, int64_t wr, bool group)
    {
        bias_type = m.bias_type;
        scale = m.scale;
        cap = m.soft_cap;
        cap_rcp = m.soft_cap > 0.f ? 1.f / m.soft_cap : 0.f;
        last_key = sk - 1;
        if (m.cols > 0 && m.cols - 1 < last_key) last_key = (int32_t)(m.cols - 1);
        bias_row = nullptr;
        bias_row32 = nullptr;
        slope = 0.f;
        zero = 0;
        mode = alibi_mode(mask_type, wl, wr);
        if (m.bias_type == 1) {
            const int64_t brow = (group ? first_row : 0) + i;
            const int64_t off = (group ? 0 : (int64_t)b * m.batch_stride) + (int64_t)h * m.head_stride + brow * m.row_stride;
            if (m.bias_f32)
                bias_row32 = reinterpret_cast<const float*>(m.bias) + off;
            else
                bias_row = reinterpret_cast<const uint16_t*>(m.bias) + off;
        } else if (m.bias_type == 2) {
            const float sl = reinterpret_cast<const float*>(m.bias)[(int64_t)b * m.batch_stride + h];
            slope = mode == kAlibiVertical ? sl : -sl;
            zero = mode == kAlibiBottomRight ? i + sk - sq : i;
        }
    }
    __device__ __forceinline__ float score(float qk, int key) const
    {
        float x = qk * scale;
        if (cap > 0.f) x = cap * fast_tanh(x * cap_rcp);
        if (bias_type == 1) {
            const int col = min(max(key, 0), last_key);
            x += bias_row32 ? bias_row32[col] : T::to_f32(bias_row[col]);
        } else if (bias_type == 2) {
            const int dist = mode == kAlibiVertical ? key : abs(zero - key);
            x = __builtin_fmaf(slope, (float)dist, x);
        }
        return x * kLog2e;
    }
};

// The modifiers that are pure arithmetic on a score (ALiBi, soft cap): RowMod without the elementwise bias, for the
// kernels whose vector phase has no room for a load per score.  Same formulas, same results.
struct ArithMod {
    float slope;
    int32_t zero, mode;
    float scale, cap, cap_rcp;
    bool alibi;

    __device__ __forceinline__ void init(const ScoreMod& m, int b, int h, int i, int sq, int sk, uint32_t mask_type, int64_t wl, int64_t wr)
    {
        scale = m.scale;
        cap = m.soft_cap;
        cap_rcp = m.soft_cap > 0.f ? 1.f / m.soft_cap : 0.f;
        alibi = m.bias_type == 2;
        slope = 0.f;
        zero = 0;
        mode = alibi_mode(mask_type, wl, wr);
        if (alibi) {
            const float sl = reinterpret_cast<const float*>(m.bias)[(int64_t)b * m.batch_stride + h];
            slope = mode == kAlibiVertical ? sl : -sl;
            zero = mode == kAlibiBottomRight ? i + sk - sq : i;
        }
    }
    __device__ __forceinline__ float score(float qk, int key) const
    {
        float x = qk * scale;
        if (cap > 0.f) x = cap * fast_tanh(x * cap_rcp);
        if (alibi) {
            const int dist = mode == kAlibiVertical ? key : abs(zero - key);
            x = __builtin_fmaf(slope, (float)dist, x);
        }
        return x * kLog2e;
    }
};

// Where the K/V rows of one sequence live.  `table` == nullptr: rows are contiguous from base_row.
// Otherwise logical key j sits at row table[j / page] * page + j % page.
struct KvSeq {
    const int32_t* table;
    int64_t base_row;
    int32_t len;  // number of keys
};

struct KvAddr {
    // mode 0: batch cache (+ cache_batch_idx); 1: group; 2: block table; 3: page list
    int32_t mode;
    int32_t page_size;
    int32_t page_shift;  // log2(page_size) when it is a power of two, else -1
    int32_t seqlen_k;    // batch mode: rows per cache sequence / default key count
    const int32_t* seqstart_k;
    const int32_t* seqlen_k_ptr;
    const int32_t* block_table;
    int32_t block_table_stride;
    const int32_t* cache_batch_idx;
    const int32_t* kv_indptr;
    const int32_t* kv_page_indices;
    const int32_t* kv_last_page_lens;
};

__device__ __forceinline__ KvSeq kv_seq(const KvAddr& a, int b)
{
    KvSeq s;
    if (a.mode == 0) {
        const int cb = a.cache_batch_idx ? a.cache_batch_idx[b] : b;
        s.table = nullptr;
        s.base_row = (int64_t)cb * a.seqlen_k;
        s.len = a.seqlen_k_ptr ? a.seqlen_k_ptr[b] : a.seqlen_k;
    } else if (a.mode == 1) {
        const int s0 = a.seqstart_k[b];
        s.table = nullptr;
        s.base_row = s0;
        // packed K/V with padding: the logical length comes from seqlen_k_ptr when it is given
        // (ck_tile/ops/fmha/kernel/fmha_fwd_splitkv_kernel.hpp:648-650)
        s.len = a.seqlen_k_ptr ? a.seqlen_k_ptr[b] : a.seqstart_k[b + 1] - s0;
    } else if (a.mode == 2) {
        s.table = a.block_table + (int64_t)b * a.block_table_stride;
        s.base_row = 0;
        s.len = a.seqlen_k_ptr[b];
    } else {
        const int p0 = a.kv_indptr[b], p1 = a.kv_indptr[b + 1];
        s.table = a.kv_page_indices + p0;
        s.base_row = 0;
        const int np = p1 - p0;
        const int last = a.kv_last_page_lens ? a.kv_last_page_lens[b] : a.page_size;
        s.len = np > 0 ? (np - 1) * a.page_size + last : 0;
    }
    return s;
}

__device__ __forceinline__ int64_t kv_row(const KvAddr& a, const KvSeq& s, int j)
{
    if (!s.table) return s.base_row + j;
    int pi, off;
    if (a.page_shift >= 0) {
        pi = j >> a.page_shift;
        off = j & (a.page_size - 1);
    } else {
        pi = j / a.page_size;
        off = j - pi * a.page_size;
    }
    return (int64_t)s.table[pi] * a.page_size + off;
}

}  // namespace fck
