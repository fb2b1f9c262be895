// Host side of the C ABI declared in include/flashck/fmha/fmha_c_api.h: argument validation, stride / workspace
// conventions of FlashCK's generated wrappers, kernel selection and launch.  No allocation, no synchronisation.
#include "flashck/fmha/fmha_c_api.h"

#include <hip/hip_runtime.h>

#include <climits>
#include <cmath>
#include <cstdlib>
#include <cstdarg>
#include <cstdio>
#include <mutex>

#include "kernels.hpp"

namespace {

thread_local char g_err[512] = "";
thread_local const char* g_kernel = "";  // kernel family of the calling thread's last launch

// "splitkv_decode_kernel<uniform_page|row_lookup[,head_pairs][,kv_fp8|,all_fp8][,score_mod][,padded_head_dim][,fused][,equal_chunks]>": the
// variant the calling thread's last split-KV launch took
void name_decode_kernel(bool uniform, int heads_per_workgroup, bool kv8, bool mod, bool padded, bool fused, bool chunks, bool q8 = false)
{
    thread_local char name[128];
    snprintf(name, sizeof(name), "splitkv_decode_kernel<%s%s%s%s%s%s%s>", uniform ? "uniform_page" : "row_lookup",
             heads_per_workgroup == 2 ? ",head_pairs" : "", q8 ? ",all_fp8" : kv8 ? ",kv_fp8" : "", mod && !padded ? ",score_mod" : "",
             padded ? ",padded_head_dim" : "", fused ? ",fused" : "", chunks ? ",equal_chunks" : "");
    g_kernel = name;
}

int fail(int code, const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

// The kernels keep counts and lengths in 32 bits: a larger argument would be cut down to some other, valid-looking
// problem, so it is refused instead.
template <typename... T>
int check_fit32(T... v)
{
    if (((v > (int64_t)INT32_MAX || v < (int64_t)INT32_MIN) || ...))
        return fail(FCK_ERR_INVALID_ARGUMENT, "a count, length or stride argument is beyond 32 bits");
    return FCK_OK;
}

int check_common(int64_t batch, int64_t hq, int64_t hk, int64_t d, int64_t dv, int32_t dtype)
{
    if (int rc = check_fit32(batch, hq, hk, d, dv)) return rc;
    if (dtype != FCK_DTYPE_FP16 && dtype != FCK_DTYPE_BF16 && dtype != FCK_DTYPE_FP8)
        return fail(FCK_ERR_UNSUPPORTED, "dtype %d: only FLOAT8 (1, e4m3), FLOAT16 (3) and BFLOAT16 (4) have kernels", dtype);
    if (dtype == FCK_DTYPE_FP8 && (d != dv || (d != 64 && d != 128 && d != 256)))
        return fail(FCK_ERR_UNSUPPORTED, "e4m3 queries need qk_head_dim = v_head_dim in {64, 128, 256}");
    if (batch <= 0 || hq <= 0 || hk <= 0) return fail(FCK_ERR_INVALID_ARGUMENT, "batch and head counts must be positive");
    if (hq % hk != 0) return fail(FCK_ERR_INVALID_ARGUMENT, "q_num_heads %ld is not a multiple of kv_num_heads %ld", (long)hq, (long)hk);
    // Kernels are built for head dims 64, 128 and 256; any other qk_head_dim / v_head_dim (the two may differ) that is a
    // multiple of 8 runs on the next larger one with the missing columns read as zeros (the reference's
    // is_pad_qk_head_dim / is_pad_v_head_dim traits, fmha_fwd_split_kv_codegen.h:106-107).
    if (d < 8 || dv < 8 || d > 256 || dv > 256 || d % 8 || dv % 8)
        return fail(FCK_ERR_UNSUPPORTED, "qk_head_dim %ld / v_head_dim %ld: head dims are multiples of 8 in [8, 256]", (long)d, (long)dv);
    return FCK_OK;
}

// Type the kernels compute a call in.  The all-fp8 roles (Q, K, V, P and O in e4m3) run on the bf16 instantiations: every
// e4m3 value is a bf16 value, so widening the operands is exact, and P is rounded to e4m3 before it is widened.
int compute_dtype(int32_t dtype) { return dtype == FCK_DTYPE_FP8 ? FCK_DTYPE_BF16 : dtype; }

// The all-fp8 roles of a call (dtype FLOAT8): what the K/V descales do not cover.  `at` may be null.
int fill_q8(int32_t& q8, float* o_scale, fck::ScoreMod& mod, const fck_fmha_attrs* at, int32_t dtype)
{
    q8 = 0;
    if (o_scale) *o_scale = 1.f;
    mod.bias_f32 = 0;
    if (dtype != FCK_DTYPE_FP8) return FCK_OK;
    // BiasDataType of the fp8 roles is float (fmha_common_jinja.h:157-171): an elementwise bias holds fp32, strides in floats
    if (mod.bias_type == FCK_BIAS_ELEMENTWISE) mod.bias_f32 = 1;
    const float os = at && at->o_scale != 0.f ? at->o_scale : 1.f;
    if (!(os > 0.f) || !std::isfinite(os)) return fail(FCK_ERR_INVALID_ARGUMENT, "o_scale must be positive and finite (0: 1)");
    if (!o_scale && os != 1.f)
        return fail(FCK_ERR_UNSUPPORTED, "o_scale applies where the output is written: the split-KV partial results are fp32 and "
                                         "fck_fmha_fwd_splitkv_combine writes e4m3 with scale 1, as the reference's wrapper does");
    q8 = 1;
    if (o_scale) *o_scale = os;
    return FCK_OK;
}

// head dim the kernels are instantiated for
int kernel_dim(int64_t d, int64_t dv)
{
    const int64_t m = d > dv ? d : dv;
    return m <= 64 ? 64 : m <= 128 ? 128 : 256;
}

// fp8 K/V with static per-tensor scales for the prefill entry points (after fill_mod): the K scale multiplies every
// score, the V scale the output
int fill_kv8(fck::PrefillArgs& a, const fck_fmha_attrs* at, int64_t d, int64_t dv, int32_t dtype)
{
    a.kv8 = 0;
    a.v_descale = 1.f;
    if (int rc = fill_q8(a.q8, &a.o_scale, a.mod, at, dtype)) return rc;
    const int32_t kvt = at ? at->kv_dtype : 0;
    if (!a.q8 && kvt == 0) return FCK_OK;  // e4m3 queries: "same as q" is e4m3 too
    if (kvt != 0 && kvt != FCK_DTYPE_FP8) return fail(FCK_ERR_UNSUPPORTED, "kv_dtype %d: only 0 (same as q) and FLOAT8 (1)", kvt);
    const float kd = !at || at->k_descale == 0.f ? 1.f : at->k_descale, vd = !at || at->v_descale == 0.f ? 1.f : at->v_descale;
    if (!(kd > 0.f) || !std::isfinite(kd) || !(vd > 0.f) || !std::isfinite(vd))
        return fail(FCK_ERR_INVALID_ARGUMENT, "k_descale and v_descale must be positive and finite (0: 1)");
    if (d != dv || d != kernel_dim(d, dv)) return fail(FCK_ERR_UNSUPPORTED, "an fp8 K/V cache needs qk_head_dim = v_head_dim in {64, 128, 256}");
    a.kv8 = 1;
    a.scale_log2 *= kd;
    a.mod.scale *= kd;
    a.v_descale = vd;
    return FCK_OK;
}

// tile variant of a prefill call (range only; whether the problem can take it is decided where the kernel is chosen)
int fill_variant(fck::PrefillArgs& a, const fck_fmha_attrs* at)
{
    a.variant = 0;
    if (!at || at->prefill_variant == 0) return FCK_OK;
    if (at->prefill_variant < 1 || at->prefill_variant > 4)
        return fail(FCK_ERR_INVALID_ARGUMENT, "prefill_variant %d out of range [0,4]", at->prefill_variant);
    a.variant = at->prefill_variant;
    return FCK_OK;
}

// Bias / ALiBi / soft cap of a call: `bias` is the positional pointer of the entry points that have one (else null).

int fill_mod(fck::ScoreMod& m, const void* bias, const fck_fmha_attrs* at, float scale, uint32_t mask_type, int64_t hq)
{
    m = fck::ScoreMod{};
    m.scale = scale;
    if (!at) {
        if (bias) return fail(FCK_ERR_UNSUPPORTED, "a bias pointer needs the _attrs entry point: fck_fmha_attrs says what it holds");
        return FCK_OK;
    }
    if (at->size != sizeof(fck_fmha_attrs))
        return fail(FCK_ERR_INVALID_ARGUMENT, "fck_fmha_attrs.size is %u, this library's struct has %zu bytes", at->size, sizeof(fck_fmha_attrs));
    if (!bias) bias = at->bias;
    if (at->bias && bias != at->bias) return fail(FCK_ERR_INVALID_ARGUMENT, "two different bias pointers (argument and fck_fmha_attrs.bias)");
    if (!(at->logits_soft_cap >= 0.f) || !std::isfinite(at->logits_soft_cap))
        return fail(FCK_ERR_INVALID_ARGUMENT, "logits_soft_cap must be finite and >= 0 (0: off)");
    switch (at->bias_type) {
    case FCK_BIAS_NONE:
        if (bias) return fail(FCK_ERR_INVALID_ARGUMENT, "a bias pointer with bias_type NO_BIAS");
        break;
    case FCK_BIAS_ELEMENTWISE:
        if (!bias) return fail(FCK_ERR_INVALID_ARGUMENT, "bias_type ELEMENTWISE_BIAS needs a bias pointer");
        if (reinterpret_cast<uintptr_t>(bias) & 1u) return fail(FCK_ERR_INVALID_ARGUMENT, "the bias must be 2-byte aligned");
        if (at->bias_row_stride <= 0 || at->bias_head_stride < 0 || at->bias_batch_stride < 0)
            return fail(FCK_ERR_INVALID_ARGUMENT, "elementwise bias: row stride must be positive, head and batch strides >= 0");
        if (at->bias_cols < 0 || at->bias_cols > at->bias_row_stride)
            return fail(FCK_ERR_INVALID_ARGUMENT, "elementwise bias: bias_cols %ld must be in [0, bias_row_stride %ld]", (long)at->bias_cols, (long)at->bias_row_stride);
        break;
    case FCK_BIAS_ALIBI:
        if (!bias) return fail(FCK_ERR_INVALID_ARGUMENT, "bias_type ALIBI needs the slopes pointer");
        if (reinterpret_cast<uintptr_t>(bias) & 3u) return fail(FCK_ERR_INVALID_ARGUMENT, "ALiBi slopes are fp32: the pointer must be 4-byte aligned");
        if (at->bias_batch_stride != 0 && at->bias_batch_stride < hq)
            return fail(FCK_ERR_INVALID_ARGUMENT, "ALiBi: bias_batch_stride is 0 (slopes shared by all batches) or >= q_num_heads");
        if (mask_type == FCK_MASK_GENERIC)
            return fail(FCK_ERR_UNSUPPORTED, "ALiBi with mask_type GENERIC: the reference defines the diagonal for top-left and bottom-right only");
        break;
    default: return fail(FCK_ERR_INVALID_ARGUMENT, "bias_type %d out of range [0,2]", at->bias_type);
    }
    m.bias = bias;
    m.bias_type = at->bias_type;
    m.batch_stride = at->bias_batch_stride;
    m.head_stride = at->bias_type == FCK_BIAS_ELEMENTWISE ? at->bias_head_stride : 0;
    m.row_stride = at->bias_type == FCK_BIAS_ELEMENTWISE ? at->bias_row_stride : 0;
    m.cols = at->bias_type == FCK_BIAS_ELEMENTWISE && at->bias_cols > 0 ? at->bias_cols : 0;
    m.soft_cap = at->logits_soft_cap;
    m.scale = scale;
    return FCK_OK;
}

int check_mask(uint32_t mask_type)
{
    if (mask_type > 3) return fail(FCK_ERR_INVALID_ARGUMENT, "mask_type %u out of range [0,3]", mask_type);
    return FCK_OK;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

int log2_exact(int64_t v)
{
    if (v <= 0 || (v & (v - 1))) return -1;
    int s = 0;
    while ((int64_t(1) << s) < v) ++s;
    return s;
}

int launch_status(hipError_t e, const char* what)
{
    if (e != hipSuccess) return fail(FCK_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
    return FCK_OK;
}

// compute units of the current device (looked up once per device)
int cu_count()
{
    constexpr int kMaxDev = 64;
    static int cus[kMaxDev];
    static std::once_flag once[kMaxDev];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDev) return 256;
    std::call_once(once[dev], [dev] {
        hipDeviceProp_t p;
        cus[dev] = hipGetDeviceProperties(&p, dev) == hipSuccess && p.multiProcessorCount > 0 ? p.multiProcessorCount : 256;
    });
    return cus[dev];
}

// The slice of the fused entry point's device array that `stream` uses on the current device: the one it was given on
// its first call, else the first free one; -1 when kDecodeScratchSlices other streams hold them all.  forget: empty the
// current device's table instead (returns 0).  Host memory only; a stream handle is just a key here, never dereferenced.
int fused_slice(hipStream_t stream, bool forget)
{
    constexpr int kMaxDev = 64;
    static std::mutex mu;
    static hipStream_t owner[kMaxDev][fck::kDecodeScratchSlices];
    static int used[kMaxDev];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDev) return -1;
    std::lock_guard<std::mutex> lock(mu);
    if (forget) {
        used[dev] = 0;
        return 0;
    }
    for (int i = 0; i < used[dev]; ++i)
        if (owner[dev][i] == stream) return i;
    if (used[dev] == fck::kDecodeScratchSlices) return -1;
    owner[dev][used[dev]] = stream;
    return used[dev]++;
}

}  // namespace

extern "C" {

const char* fck_last_error(void) { return g_err; }

const char* fck_fmha_version(void) { return "flashck-fmha-gfx950 0.2"; }

const char* fck_fmha_last_kernel(void) { return g_kernel; }

size_t fck_fmha_splitkv_workspace_bytes(int64_t shape_batch, int64_t hq, int64_t shape_sq, int64_t dv, int64_t num_splits)
{
    if (shape_batch <= 0 || hq <= 0 || shape_sq <= 0 || dv <= 0 || num_splits <= 0) return 0;
    const size_t rows = (size_t)shape_batch * hq * num_splits * shape_sq;
    return rows * dv * sizeof(float) + rows * sizeof(float);
}

int fck_fmha_num_splits_heuristic(int64_t batch, int64_t hq, int64_t hk, int64_t sq, int64_t max_sk, int64_t head_dim,
                                  int64_t num_cu)
{
    (void)head_dim;
    if (batch <= 0 || hq <= 0 || hk <= 0 || sq <= 0 || max_sk <= 0) return 1;
    // sizes no launch could have (the products below must stay inside 64 bits and away from zero)
    constexpr int64_t kMax = (int64_t)1 << 24;
    if (batch > kMax || hq > kMax || hk > hq || sq > kMax || num_cu > kMax) return 1;
    if (num_cu <= 0) num_cu = cu_count();
    // One workgroup streams one split of one KV head for 16..64 packed rows (query index x head-in-group).
    const int64_t g = hq / hk;
    const int64_t rows = sq * g;
    const int64_t m_tiles = rows <= 32 ? 1 : (rows + 63) / 64;
    const int64_t base = batch * hk * m_tiles;  // workgroups without splitting
    // Aim at >= 2 workgroups per CU so uneven sequence lengths even out, but keep at least 256 keys per split:
    // below that the merge and the workspace round trip outweigh the streaming.
    const int64_t want = (2 * num_cu + base - 1) / base;
    const int64_t cap = max_sk / 256 > 0 ? max_sk / 256 : 1;
    int64_t ns = want < cap ? want : cap;
    if (ns < 1) ns = 1;
    if (ns > 128) ns = 128;
    return (int)ns;
}

// Validation and argument block shared by the split-KV entry points (everything but the workspace / output pointers).
static int splitkv_setup(fck::SplitKvArgs& a, bool& uniform, int& rows_max, const void* q, const void* k, const void* v,
                         const void* bias, const int32_t* seqstart_q, const int32_t* seqstart_k, const int32_t* seqlen_k_ptr,
                         const int32_t* block_table, const int32_t* cache_batch_idx, int64_t batch, int64_t seqlen_q,
                         int64_t seqlen_k, int64_t hq, int64_t hk, int64_t d, int64_t dv, int64_t q_max_seq_len,
                         int64_t num_splits, int64_t max_num_page_blocks, int64_t page_block_size, float scale,
                         int64_t window_left, int64_t window_right, uint32_t mask_type, int32_t dtype, const fck_fmha_attrs* attrs)
{
    if (int rc = check_common(batch, hq, hk, d, dv, dtype)) return rc;
    if (int rc = check_mask(mask_type)) return rc;
    if (!q || !k || !v) return fail(FCK_ERR_INVALID_ARGUMENT, "q, k and v must not be null");
    if (!aligned16(q) || !aligned16(k) || !aligned16(v)) return fail(FCK_ERR_INVALID_ARGUMENT, "q, k and v must be 16-byte aligned");
    if (num_splits < 1 || num_splits > 128) return fail(FCK_ERR_INVALID_ARGUMENT, "num_splits %ld out of range [1,128]", (long)num_splits);
    if (!(scale > 0.f) || !std::isfinite(scale)) return fail(FCK_ERR_INVALID_ARGUMENT, "scale must be positive and finite");
    const bool group = seqstart_q != nullptr;
    if (!group && seqlen_q <= 0) return fail(FCK_ERR_INVALID_ARGUMENT, "seqlen_q must be positive in batch mode");
    if (group && seqlen_q <= 0) return fail(FCK_ERR_INVALID_ARGUMENT, "group mode: seqlen_q must carry total_q (workspace row count)");
    if (q_max_seq_len <= 0) q_max_seq_len = seqlen_q;
    if (q_max_seq_len <= 0) return fail(FCK_ERR_INVALID_ARGUMENT, "q_max_seq_len must be positive");
    if (int rc = check_fit32(seqlen_q, seqlen_k, q_max_seq_len, max_num_page_blocks, page_block_size, q_max_seq_len * (hq / hk))) return rc;

    a = fck::SplitKvArgs{};
    a.q = q;
    a.k = k;
    a.v = v;
    a.seqstart_q = seqstart_q;
    a.batch = (int32_t)batch;
    a.sq = (int32_t)seqlen_q;
    a.hq = (int32_t)hq;
    a.hk = (int32_t)hk;
    a.num_splits = (int32_t)num_splits;
    a.shape_sq = seqlen_q;  // group mode: seqlen_q carries total_q (the "shape" length of the FlashCK wrapper)
    a.d = (int32_t)d;
    a.dv = (int32_t)dv;
    const bool padded = d != dv || d != kernel_dim(d, dv);
    a.scale_log2 = scale * fck::kLog2e;
    a.mask_type = mask_type;
    a.window_left = window_left;
    a.window_right = window_right;
    if (int rc = fill_mod(a.mod, bias, attrs, scale, mask_type, hq)) return rc;
    a.v_descale = 1.f;
    if (attrs && attrs->decode_variant != 0) {
        const int32_t dvar = attrs->decode_variant;
        if (dvar < 1 || dvar > 4) return fail(FCK_ERR_INVALID_ARGUMENT, "decode_variant %d out of range [0,4]", dvar);
        if ((dvar == 2 || dvar == 4) && (hk % 2 || d > 128 || padded || q_max_seq_len * (hq / hk) > 16))
            return fail(FCK_ERR_INVALID_ARGUMENT, "decode_variant %d (head pairs) needs an even kv_num_heads, head dim 64 or 128 and at most 16 "
                                                  "packed query rows", dvar);
        if (dvar >= 3) {
            // splits of equal size in keys: a plain call over a block table with tile-aligned pages, one 16-row block
            if (!block_table || page_block_size % 32 || d > 128 || padded || q_max_seq_len * (hq / hk) > 16 || a.mod.active() || attrs->kv_dtype != 0)
                return fail(FCK_ERR_INVALID_ARGUMENT, "decode_variant %d (splits of equal size) needs a block table with pages a multiple of 32 keys, head "
                                                      "dim 64 or 128, at most 16 packed query rows and no bias / soft cap / fp8 cache", dvar);
            if (attrs->max_seqlen_k < 0) return fail(FCK_ERR_INVALID_ARGUMENT, "max_seqlen_k must be >= 0 (0: the block table's capacity)");
            const int64_t capacity = (batch > 0 ? max_num_page_blocks / batch : 0) * page_block_size;
            const int64_t bound = attrs->max_seqlen_k > 0 && attrs->max_seqlen_k < capacity ? attrs->max_seqlen_k : capacity;
            int64_t chunk = (bound + num_splits - 1) / num_splits;
            chunk = (chunk + 31) / 32 * 32;
            if (chunk <= 0 || chunk > INT32_MAX) return fail(FCK_ERR_INVALID_ARGUMENT, "decode_variant %d: no positive key-count bound", dvar);
            a.split_chunk = (int32_t)chunk;
        }
        a.variant = dvar;
    }
    if (int rc = fill_q8(a.q8, nullptr, a.mod, attrs, dtype)) return rc;
    if (a.q8 || (attrs && attrs->kv_dtype != 0)) {  // e4m3 queries: "same as q" is e4m3 too
        // fp8 K/V with static per-tensor scales: the K scale multiplies every score, the V scale the output
        const int32_t kvt = attrs ? attrs->kv_dtype : 0;
        if (kvt != 0 && kvt != FCK_DTYPE_FP8) return fail(FCK_ERR_UNSUPPORTED, "kv_dtype %d: only 0 (same as q) and FLOAT8 (1)", kvt);
        const float kd = !attrs || attrs->k_descale == 0.f ? 1.f : attrs->k_descale, vd = !attrs || attrs->v_descale == 0.f ? 1.f : attrs->v_descale;
        if (!(kd > 0.f) || !std::isfinite(kd) || !(vd > 0.f) || !std::isfinite(vd))
            return fail(FCK_ERR_INVALID_ARGUMENT, "k_descale and v_descale must be positive and finite (0: 1)");
        if (!aligned16(k) || !aligned16(v)) return fail(FCK_ERR_INVALID_ARGUMENT, "k and v must be 16-byte aligned");
        if (padded) return fail(FCK_ERR_UNSUPPORTED, "an fp8 K/V cache needs qk_head_dim = v_head_dim in {64, 128, 256}");
        a.kv8 = 1;
        a.scale_log2 *= kd;
        a.mod.scale *= kd;
        a.v_descale = vd;
    }

    uniform = true;
    fck::KvAddr& kv = a.kv;
    kv.seqlen_k_ptr = seqlen_k_ptr;
    kv.cache_batch_idx = cache_batch_idx;
    kv.page_shift = -1;
    if (block_table) {
        if (page_block_size <= 0) return fail(FCK_ERR_INVALID_ARGUMENT, "paged cache needs page_block_size > 0");
        if (!seqlen_k_ptr) return fail(FCK_ERR_INVALID_ARGUMENT, "paged cache needs per-sequence key counts (k_seq_len_ptr)");
        if (max_num_page_blocks < batch || max_num_page_blocks % batch)
            return fail(FCK_ERR_INVALID_ARGUMENT, "max_num_page_blocks %ld must be a positive multiple of batch %ld", (long)max_num_page_blocks, (long)batch);
        kv.mode = 2;
        kv.block_table = block_table;
        kv.block_table_stride = (int32_t)(max_num_page_blocks / batch);  // fmha_fwd_split_kv_jinja.h:318
        kv.page_size = (int32_t)page_block_size;
        kv.page_shift = log2_exact(page_block_size);
        uniform = page_block_size % 32 == 0;
    } else if (seqstart_k) {
        kv.mode = 1;
        kv.seqstart_k = seqstart_k;
    } else {
        if (seqlen_k <= 0) return fail(FCK_ERR_INVALID_ARGUMENT, "batch cache needs seqlen_k > 0");
        kv.mode = 0;
        kv.seqlen_k = (int32_t)seqlen_k;
    }
    rows_max = (int)(q_max_seq_len * (hq / hk));
    return FCK_OK;
}

int fck_fmha_fwd_splitkv(const void* q, const void* k, const void* v, const void* bias, void* lse_acc, void* o_acc,
                         const int32_t* seqstart_q, const int32_t* seqstart_k, const int32_t* seqlen_k_ptr,
                         const int32_t* block_table, const int32_t* cache_batch_idx, int64_t batch, int64_t seqlen_q,
                         int64_t seqlen_k, int64_t hq, int64_t hk, int64_t d, int64_t dv, int64_t q_max_seq_len,
                         int64_t num_splits, int64_t max_num_page_blocks, int64_t page_block_size, float scale,
                         int64_t window_left, int64_t window_right, uint32_t mask_type, int32_t dtype, void* stream)
{
    return fck_fmha_fwd_splitkv_attrs(q, k, v, bias, lse_acc, o_acc, seqstart_q, seqstart_k, seqlen_k_ptr, block_table, cache_batch_idx,
                                      batch, seqlen_q, seqlen_k, hq, hk, d, dv, q_max_seq_len, num_splits, max_num_page_blocks,
                                      page_block_size, scale, window_left, window_right, mask_type, dtype, nullptr, stream);
}

int fck_fmha_fwd_splitkv_attrs(const void* q, const void* k, const void* v, const void* bias, void* lse_acc, void* o_acc,
                               const int32_t* seqstart_q, const int32_t* seqstart_k, const int32_t* seqlen_k_ptr,
                               const int32_t* block_table, const int32_t* cache_batch_idx, int64_t batch, int64_t seqlen_q,
                               int64_t seqlen_k, int64_t hq, int64_t hk, int64_t d, int64_t dv, int64_t q_max_seq_len,
                               int64_t num_splits, int64_t max_num_page_blocks, int64_t page_block_size, float scale,
                               int64_t window_left, int64_t window_right, uint32_t mask_type, int32_t dtype,
                               const fck_fmha_attrs* attrs, void* stream)
{
    g_err[0] = 0;
    fck::SplitKvArgs a;
    bool uniform;
    int rows_max;
    if (int rc = splitkv_setup(a, uniform, rows_max, q, k, v, bias, seqstart_q, seqstart_k, seqlen_k_ptr, block_table,
                               cache_batch_idx, batch, seqlen_q, seqlen_k, hq, hk, d, dv, q_max_seq_len, num_splits,
                               max_num_page_blocks, page_block_size, scale, window_left, window_right, mask_type, dtype, attrs))
        return rc;
    if (!lse_acc || !o_acc) return fail(FCK_ERR_INVALID_ARGUMENT, "lse_acc and o_acc must not be null");
    if (!aligned16(o_acc)) return fail(FCK_ERR_INVALID_ARGUMENT, "o_acc must be 16-byte aligned");
    a.o_acc = static_cast<float*>(o_acc);
    a.lse_acc = static_cast<float*>(lse_acc);
    int hpw = 1;
    const hipError_t e = fck::launch_splitkv_decode(a, kernel_dim(d, dv), compute_dtype(dtype), rows_max, uniform, cu_count(), static_cast<hipStream_t>(stream), &hpw);
    name_decode_kernel(uniform, hpw, a.kv8 != 0, a.mod.active(), d != dv || d != kernel_dim(d, dv), false, a.split_chunk > 0, a.q8 != 0);
    return launch_status(e, "FmhaFwdSplitKV launch");
}

int fck_fmha_fwd_splitkv_fused(const void* q, const void* k, const void* v, const void* bias, void* o,
                               const int32_t* seqstart_q, const int32_t* seqstart_k, const int32_t* seqlen_k_ptr,
                               const int32_t* block_table, const int32_t* cache_batch_idx, int64_t batch, int64_t seqlen_q,
                               int64_t seqlen_k, int64_t hq, int64_t hk, int64_t d, int64_t dv, int64_t q_max_seq_len,
                               int64_t num_splits, int64_t max_num_page_blocks, int64_t page_block_size, float scale,
                               int64_t window_left, int64_t window_right, uint32_t mask_type, int32_t dtype, void* stream)
{
    g_err[0] = 0;
    if (dtype == FCK_DTYPE_FP8) return fail(FCK_ERR_UNSUPPORTED, "the fused split-KV entry point has no e4m3 kernels");
    // num_splits == 0: the split count comes from the CU count and the longest possible KV length (the capacity of
    // the block table, or seqlen_k), as fck_fmha_num_splits_heuristic gives it
    if (num_splits == 0) {
        const int64_t max_sk = block_table ? (batch > 0 ? max_num_page_blocks / batch : 0) * page_block_size : seqlen_k;
        if (max_sk <= 0) return fail(FCK_ERR_INVALID_ARGUMENT, "num_splits = 0 needs a positive key-count bound (seqlen_k or the block table's capacity)");
        num_splits = fck_fmha_num_splits_heuristic(batch, hq, hk, q_max_seq_len > 0 ? q_max_seq_len : seqlen_q, max_sk, d, 0);
    }
    fck::SplitKvArgs a;
    bool uniform;
    int rows_max;
    if (int rc = splitkv_setup(a, uniform, rows_max, q, k, v, bias, seqstart_q, seqstart_k, seqlen_k_ptr, block_table,
                               cache_batch_idx, batch, seqlen_q, seqlen_k, hq, hk, d, dv, q_max_seq_len, num_splits,
                               max_num_page_blocks, page_block_size, scale, window_left, window_right, mask_type, dtype, nullptr))
        return rc;
    if (!o) return fail(FCK_ERR_INVALID_ARGUMENT, "o must not be null");
    if (!aligned16(o)) return fail(FCK_ERR_INVALID_ARGUMENT, "o must be 16-byte aligned");
    if (d != dv || d != kernel_dim(d, dv))
        return fail(FCK_ERR_UNSUPPORTED, "the fused split-KV entry point needs qk_head_dim = v_head_dim in {64, 128, 256}");
    // The partial results and the arrival tickets live in a fixed device array of the library: nothing is allocated.
    const int64_t shape_batch = seqstart_q ? 1 : batch;
    const int64_t part_rows = shape_batch * hq * num_splits * seqlen_q;
    const int64_t m_tiles = fck::splitkv_decode_m_tiles(kernel_dim(d, dv), rows_max);
    const int64_t tickets = batch * hk * m_tiles;
    if (part_rows * (dv + 1) > fck::kDecodeScratchPartialFloats || tickets > fck::kDecodeScratchTickets)
        return fail(FCK_ERR_UNSUPPORTED,
                    "the fused split-KV entry point holds at most %ld partial floats (asked: %ld = rows %ld x (Dv + 1)) and %ld "
                    "tickets (asked: %ld); use fck_fmha_fwd_splitkv + fck_fmha_fwd_splitkv_combine with a caller-owned workspace",
                    (long)fck::kDecodeScratchPartialFloats, (long)(part_rows * (dv + 1)), (long)part_rows,
                    (long)fck::kDecodeScratchTickets, (long)tickets);
    float* scratch = nullptr;
    if (hipError_t e = fck::decode_scratch(&scratch); e != hipSuccess) return launch_status(e, "scratch symbol lookup");
    const int slice = fused_slice(static_cast<hipStream_t>(stream), false);
    if (slice < 0)
        return fail(FCK_ERR_UNSUPPORTED,
                    "the fused split-KV entry point serves at most %d streams per GPU (each owns a slice of the library's device "
                    "array); use one of them, or fck_fmha_fused_reset once no fused call is in flight, or fck_fmha_fwd_splitkv + "
                    "fck_fmha_fwd_splitkv_combine with a caller-owned workspace",
                    fck::kDecodeScratchSlices);
    a.tickets = reinterpret_cast<uint32_t*>(scratch) + slice * fck::kDecodeScratchTickets;
    a.o_acc = scratch + fck::kDecodeScratchSlices * fck::kDecodeScratchTickets + slice * fck::kDecodeScratchPartialFloats;
    a.lse_acc = a.o_acc + part_rows * dv;
    a.o = o;
    int hpw = 1;
    const hipError_t e = fck::launch_splitkv_decode(a, kernel_dim(d, dv), compute_dtype(dtype), rows_max, uniform, cu_count(), static_cast<hipStream_t>(stream), &hpw);
    name_decode_kernel(uniform, hpw, false, false, false, true, false);
    return launch_status(e, "FmhaFwdSplitKV (fused) launch");
}

int fck_fmha_fused_reset(void* stream)
{
    g_err[0] = 0;
    float* scratch = nullptr;
    if (hipError_t e = fck::decode_scratch(&scratch); e != hipSuccess) return launch_status(e, "scratch symbol lookup");
    fused_slice(nullptr, true);
    return launch_status(fck::launch_clear_tickets(reinterpret_cast<uint32_t*>(scratch),
                                                   (int)(fck::kDecodeScratchSlices * fck::kDecodeScratchTickets), static_cast<hipStream_t>(stream)),
                         "ticket reset launch");
}

int fck_fmha_validate_paged(const int32_t* seqlen_k, const int32_t* block_table, int64_t batch_stride_block_table,
                            const int32_t* kv_indptr, const int32_t* kv_page_indices, const int32_t* kv_last_page_lens,
                            int64_t batch, int64_t num_total_pages, int64_t page_block_size, int32_t* error_counts, void* stream)
{
    g_err[0] = 0;
    if (batch <= 0 || num_total_pages <= 0 || page_block_size <= 0 || batch > INT32_MAX || page_block_size > INT32_MAX)
        return fail(FCK_ERR_INVALID_ARGUMENT, "batch, num_total_pages and page_block_size must be positive");
    if (!error_counts) return fail(FCK_ERR_INVALID_ARGUMENT, "error_counts (int32[4], device memory) must not be null");
    if ((block_table != nullptr) == (kv_indptr != nullptr))
        return fail(FCK_ERR_INVALID_ARGUMENT, "give either a block table (with seqlen_k) or a page list (kv_indptr, kv_page_indices)");
    if (block_table && (!seqlen_k || batch_stride_block_table <= 0))
        return fail(FCK_ERR_INVALID_ARGUMENT, "a block table needs seqlen_k and batch_stride_block_table > 0");
    if (kv_indptr && !kv_page_indices) return fail(FCK_ERR_INVALID_ARGUMENT, "a page list needs kv_page_indices");
    fck::ValidateArgs a{};
    a.seqlen_k = seqlen_k;
    a.block_table = block_table;
    a.block_table_stride = batch_stride_block_table;
    a.kv_indptr = kv_indptr;
    a.kv_page_indices = kv_page_indices;
    a.kv_last_page_lens = kv_last_page_lens;
    a.num_total_pages = num_total_pages;
    a.page_size = (int32_t)page_block_size;
    a.batch = (int32_t)batch;
    a.counts = error_counts;
    return launch_status(fck::launch_validate_paged(a, static_cast<hipStream_t>(stream)), "paged-cache validation launch");
}

int fck_fmha_fwd_splitkv_combine(const void* lse_acc, const void* o_acc, void* o, const int32_t* seqstart_q, int64_t batch,
                                 int64_t seqlen_q, int64_t hq, int64_t dv, int64_t q_max_seq_len, int64_t num_splits,
                                 int32_t dtype, void* stream)
{
    g_err[0] = 0;
    (void)q_max_seq_len;
    if (dtype != FCK_DTYPE_FP16 && dtype != FCK_DTYPE_BF16 && dtype != FCK_DTYPE_FP8)
        return fail(FCK_ERR_UNSUPPORTED, "dtype %d: only FLOAT8 (1, e4m3), FLOAT16 (3) and BFLOAT16 (4) have kernels", dtype);
    if (!lse_acc || !o_acc || !o) return fail(FCK_ERR_INVALID_ARGUMENT, "lse_acc, o_acc and o must not be null");
    if (batch <= 0 || hq <= 0 || seqlen_q <= 0) return fail(FCK_ERR_INVALID_ARGUMENT, "batch, q_num_heads and seqlen_q must be positive");
    if (int rc = check_fit32(batch, seqlen_q, hq, dv, num_splits)) return rc;
    if (dv < 8 || dv > 256 || dv % 8) return fail(FCK_ERR_UNSUPPORTED, "v_head_dim %ld: a multiple of 8 in [8, 256]", (long)dv);
    if (num_splits < 1 || num_splits > 128) return fail(FCK_ERR_INVALID_ARGUMENT, "num_splits %ld out of range [1,128]", (long)num_splits);
    if (!aligned16(o_acc) || !aligned16(o)) return fail(FCK_ERR_INVALID_ARGUMENT, "o_acc and o must be 16-byte aligned");
    fck::CombineArgs a{};
    a.lse_acc = static_cast<const float*>(lse_acc);
    a.o_acc = static_cast<const float*>(o_acc);
    a.o = o;
    // group mode: one "batch" of total_q rows (seqlen_q carries total_q), fmha_fwd_split_kv_combine_jinja.h:118-119
    a.Sq = seqlen_q;
    a.rows = (seqstart_q ? 1 : batch) * seqlen_q;
    a.hq = (int32_t)hq;
    a.dv = (int32_t)dv;
    a.num_splits = (int32_t)num_splits;
    a.num_cu = cu_count();
    a.o_scale = 1.f;  // e4m3 output: the reference's wrapper has no scale argument either (fmha_fwd_split_kv_combine_jinja.h:78-92)
    return launch_status(fck::launch_splitkv_combine(a, dtype, static_cast<hipStream_t>(stream)), "FmhaFwdSplitKVCombine launch");
}

int fck_fmha_fwd_appendkv(void* q, void* k_cache, void* v_cache, const void* knew, const void* vnew, const int32_t* seqlen_k,
                          const int32_t* cu_seqlens_knew, int64_t seqlen_knew, const void* rotary_cos, const void* rotary_sin,
                          int64_t rotary_dim, int32_t rope_mode, int32_t has_mask, const int32_t* block_table,
                          int64_t batch_stride_block_table, int64_t page_block_size, const int32_t* cache_batch_idx,
                          int64_t seqlen_k_cache, int64_t batch, int64_t hq, int64_t hk, int64_t d, int64_t dv, int32_t dtype,
                          void* stream)
{
    return fck_fmha_fwd_appendkv_attrs(q, k_cache, v_cache, knew, vnew, seqlen_k, cu_seqlens_knew, seqlen_knew, rotary_cos, rotary_sin,
                                       rotary_dim, rope_mode, has_mask, block_table, batch_stride_block_table, page_block_size,
                                       cache_batch_idx, seqlen_k_cache, batch, hq, hk, d, dv, dtype, nullptr, stream);
}

int fck_fmha_fwd_appendkv_attrs(void* q, void* k_cache, void* v_cache, const void* knew, const void* vnew, const int32_t* seqlen_k,
                                const int32_t* cu_seqlens_knew, int64_t seqlen_knew, const void* rotary_cos, const void* rotary_sin,
                                int64_t rotary_dim, int32_t rope_mode, int32_t has_mask, const int32_t* block_table,
                                int64_t batch_stride_block_table, int64_t page_block_size, const int32_t* cache_batch_idx,
                                int64_t seqlen_k_cache, int64_t batch, int64_t hq, int64_t hk, int64_t d, int64_t dv, int32_t dtype,
                                const fck_fmha_attrs* attrs, void* stream)
{
    g_err[0] = 0;
    float k_descale = 1.f, v_descale = 1.f;
    int32_t kv8 = 0;
    if (attrs) {
        if (attrs->size != sizeof(fck_fmha_attrs))
            return fail(FCK_ERR_INVALID_ARGUMENT, "fck_fmha_attrs.size is %u, this library's struct has %zu bytes", attrs->size, sizeof(fck_fmha_attrs));
        if (attrs->bias_type != 0 || attrs->bias || attrs->logits_soft_cap != 0.f)
            return fail(FCK_ERR_INVALID_ARGUMENT, "appendKV takes no bias / soft cap: only kv_dtype, k_descale and v_descale of fck_fmha_attrs apply");
        if (attrs->kv_dtype != 0) {
            if (attrs->kv_dtype != FCK_DTYPE_FP8) return fail(FCK_ERR_UNSUPPORTED, "kv_dtype %d: only 0 (same as knew) and FLOAT8 (1)", attrs->kv_dtype);
            k_descale = attrs->k_descale == 0.f ? 1.f : attrs->k_descale;
            v_descale = attrs->v_descale == 0.f ? 1.f : attrs->v_descale;
            if (!(k_descale > 0.f) || !std::isfinite(k_descale) || !(v_descale > 0.f) || !std::isfinite(v_descale))
                return fail(FCK_ERR_INVALID_ARGUMENT, "k_descale and v_descale must be positive and finite (0: 1)");
            kv8 = 1;
        }
    }
    if (dtype != FCK_DTYPE_FP16 && dtype != FCK_DTYPE_BF16)
        return fail(FCK_ERR_UNSUPPORTED, "dtype %d: only FLOAT16 (3) and BFLOAT16 (4) have kernels", dtype);
    if (!k_cache || !v_cache || !knew || !vnew || !seqlen_k) return fail(FCK_ERR_INVALID_ARGUMENT, "k_cache, v_cache, knew, vnew and seqlen_k must not be null");
    if (batch <= 0 || hk <= 0 || d <= 0 || dv <= 0 || (q && hq <= 0)) return fail(FCK_ERR_INVALID_ARGUMENT, "sizes must be positive");
    if (d % 2 || dv % 2) return fail(FCK_ERR_INVALID_ARGUMENT, "head dims must be even");
    if (seqlen_knew <= 0) return fail(FCK_ERR_INVALID_ARGUMENT, "seqlen_knew (largest number of new tokens of a sequence) must be positive");
    if (int rc = check_fit32(batch, hq, hk, d, dv, seqlen_knew, rotary_dim, batch_stride_block_table, page_block_size, seqlen_k_cache)) return rc;
    if (rope_mode < 0 || rope_mode > 2) return fail(FCK_ERR_INVALID_ARGUMENT, "rope_mode %d out of range [0,2]", rope_mode);
    if (rope_mode != FCK_ROPE_NONE) {
        if (!rotary_cos || !rotary_sin) return fail(FCK_ERR_INVALID_ARGUMENT, "rotary tables must not be null when rope_mode != NONE");
        if (rotary_dim <= 0 || rotary_dim > d || rotary_dim % 2) return fail(FCK_ERR_INVALID_ARGUMENT, "rotary_dim %ld must be even and in (0, %ld]", (long)rotary_dim, (long)d);
    } else {
        rotary_dim = 0;
    }
    if (block_table) {
        if (page_block_size <= 0 || batch_stride_block_table <= 0) return fail(FCK_ERR_INVALID_ARGUMENT, "paged cache needs page_block_size and batch_stride_block_table > 0");
    } else if (seqlen_k_cache <= 0) {
        return fail(FCK_ERR_INVALID_ARGUMENT, "batch cache needs seqlen_k_cache > 0");
    }
    fck::AppendKvArgs a{};
    a.q = q;
    a.k_cache = k_cache;
    a.v_cache = v_cache;
    a.knew = knew;
    a.vnew = vnew;
    a.seqlen_k = seqlen_k;
    a.cu_seqlens_knew = cu_seqlens_knew;
    a.seqlen_knew = (int32_t)seqlen_knew;
    a.cos = rotary_cos;
    a.sin = rotary_sin;
    a.rotary_dim = (int32_t)rotary_dim;
    a.rope_mode = rope_mode;
    a.has_mask = has_mask;
    a.block_table = block_table;
    a.block_table_stride = (int32_t)batch_stride_block_table;
    a.page_size = (int32_t)page_block_size;
    a.cache_batch_idx = cache_batch_idx;
    a.seqlen_k_cache = seqlen_k_cache;
    a.batch = (int32_t)batch;
    a.hq = (int32_t)hq;
    a.hk = (int32_t)hk;
    a.d = (int32_t)d;
    a.dv = (int32_t)dv;
    a.kv8 = kv8;
    a.k_descale = k_descale;
    a.v_descale = v_descale;
    if (kv8) return launch_status(fck::launch_appendkv_fp8(a, dtype, (int)seqlen_knew, static_cast<hipStream_t>(stream)), "FmhaFwdAppendKV (fp8 cache) launch");
    return launch_status(fck::launch_appendkv(a, dtype, (int)seqlen_knew, static_cast<hipStream_t>(stream)), "FmhaFwdAppendKV launch");
}

static int prefill_common(fck::PrefillArgs& a, int64_t d_qk, int64_t dv, int32_t dtype, int64_t q_max_seq_len, bool uniform, void* stream,
                          const char* what)
{
    if (q_max_seq_len <= 0) return fail(FCK_ERR_INVALID_ARGUMENT, "q_max_seq_len must be positive");
    a.d = (int32_t)d_qk;
    a.dv = (int32_t)dv;
    const int64_t d = kernel_dim(d_qk, dv);
    // The direct-to-LDS kernels address a tile's rows with 32-bit byte offsets from the tile's first row.
    if ((int64_t)a.hk * d * 2 * 64 >= ((int64_t)1 << 31))
        return fail(FCK_ERR_INVALID_ARGUMENT, "kv_num_heads * head_dim = %ld is too large (64 cache rows must span < 2 GiB)", (long)(a.hk * d));
    // Long query runs at head dim <= 128 take the 8-wave ping-pong kernel (256 rows per workgroup).  Head dim 256
    // takes the 4-wave kernel that sends K/V tiles straight to LDS (128 rows per workgroup) when a 64-key tile never
    // straddles a page; short runs at head dim <= 128 and page sizes that are not a multiple of 64 take the 4-wave
    // kernel that stages K/V through registers.
    // Tile variants (2..4) exist for the plain ping-pong kernel on uniform pages; variant 1 names the default schedule of
    // whatever kernel the call takes.
    if (a.variant > 1 && !(d_qk == d && dv == d && d <= 128 && q_max_seq_len > 128 && uniform && !a.mod.active() && !a.kv8))
        return fail(FCK_ERR_INVALID_ARGUMENT, "prefill_variant %d needs the ping-pong kernel: head dim 64 or 128, query runs longer than 128, "
                                              "pages a multiple of 64 (or no pages), no bias / ALiBi / soft cap / fp8 cache", a.variant);
    if (d_qk != d || dv != d) {
        // Head dims other than 64 / 128 / 256, or qk_head_dim != v_head_dim: every kernel pads them (rows keep their stored
        // length in memory, the missing columns are zeros in LDS); which kernel follows the rules below, except that an
        // elementwise bias or a short query run takes the register-staged one.
        const bool fast = !(a.mod.active() && a.mod.bias_type == FCK_BIAS_ELEMENTWISE);
        if (fast && d <= 128 && q_max_seq_len > 128) {
            a.m_tiles = (int32_t)((q_max_seq_len + 255) / 256);
            g_kernel = uniform ? "prefill_pp_kernel<uniform_page,padded_head_dim>" : "prefill_pp_kernel<row_lookup,padded_head_dim>";
            return launch_status(fck::launch_prefill_pingpong(a, (int)d, compute_dtype(dtype), uniform, static_cast<hipStream_t>(stream)), what);
        }
        a.m_tiles = (int32_t)((q_max_seq_len + 127) / 128);
        if (fast && d == 256 && uniform) {
            g_kernel = "prefill_dma_kernel<uniform_page,padded_head_dim>";
            return launch_status(fck::launch_prefill_dma(a, (int)d, compute_dtype(dtype), static_cast<hipStream_t>(stream)), what);
        }
        g_kernel = uniform ? "prefill_kernel<uniform_page,padded_head_dim>" : "prefill_kernel<row_lookup,padded_head_dim>";
        return launch_status(fck::launch_prefill(a, (int)d, compute_dtype(dtype), uniform, static_cast<hipStream_t>(stream)), what);
    }
    if (a.kv8) {
        // an fp8 cache is widened on its way into LDS, which only the register-staged kernel can do
        a.m_tiles = (int32_t)((q_max_seq_len + 127) / 128);
        g_kernel = a.q8 ? (uniform ? "prefill_kernel<uniform_page,all_fp8>" : "prefill_kernel<row_lookup,all_fp8>")
                        : (uniform ? "prefill_kernel<uniform_page,kv_fp8>" : "prefill_kernel<row_lookup,kv_fp8>");
        return launch_status(fck::launch_prefill(a, (int)d, compute_dtype(dtype), uniform, static_cast<hipStream_t>(stream)), what);
    }
    const bool mod = a.mod.active();
    if (mod && a.mod.bias_type == FCK_BIAS_ELEMENTWISE) {
        // an elementwise bias costs a load per score: only the register-staged kernel reads it; ALiBi and the soft cap
        // are arithmetic on the score and every kernel applies them
        a.m_tiles = (int32_t)((q_max_seq_len + 127) / 128);
        g_kernel = uniform ? "prefill_kernel<uniform_page,score_mod>" : "prefill_kernel<row_lookup,score_mod>";
        return launch_status(fck::launch_prefill(a, (int)d, compute_dtype(dtype), uniform, static_cast<hipStream_t>(stream)), what);
    }
    if (d <= 128 && q_max_seq_len > 128) {
        a.m_tiles = (int32_t)((q_max_seq_len + 255) / 256);
        static const char* const variants[5] = {"prefill_pp_kernel<uniform_page>", "prefill_pp_kernel<uniform_page>",
                                                "prefill_pp_kernel<uniform_page,fast_requests>", "prefill_pp_kernel<uniform_page,max_in_matrix_phase>",
                                                "prefill_pp_kernel<uniform_page,fast_requests,max_in_matrix_phase>"};
        g_kernel = uniform ? (mod ? "prefill_pp_kernel<uniform_page,score_mod>" : variants[a.variant])
                           : (mod ? "prefill_pp_kernel<row_lookup,score_mod>" : "prefill_pp_kernel<row_lookup>");
        return launch_status(fck::launch_prefill_pingpong(a, (int)d, compute_dtype(dtype), uniform, static_cast<hipStream_t>(stream)), what);
    }
    a.m_tiles = (int32_t)((q_max_seq_len + 127) / 128);
    if (d == 256 && uniform) {
        g_kernel = mod ? "prefill_dma_kernel<uniform_page,score_mod>" : "prefill_dma_kernel<uniform_page>";
        return launch_status(fck::launch_prefill_dma(a, (int)d, compute_dtype(dtype), static_cast<hipStream_t>(stream)), what);
    }
    if (mod) {
        g_kernel = uniform ? "prefill_kernel<uniform_page,score_mod>" : "prefill_kernel<row_lookup,score_mod>";
        return launch_status(fck::launch_prefill(a, (int)d, compute_dtype(dtype), uniform, static_cast<hipStream_t>(stream)), what);
    }
    g_kernel = uniform ? "prefill_kernel<uniform_page>" : "prefill_kernel<row_lookup>";
    return launch_status(fck::launch_prefill(a, (int)d, compute_dtype(dtype), uniform, static_cast<hipStream_t>(stream)), what);
}

int fck_fmha_fwd(const void* q, const void* k, const void* v, const void* bias, void* o, const int32_t* seqstart_q,
                 const int32_t* seqstart_k, const int32_t* seqlen_k_ptr, int64_t batch, int64_t seqlen_q, int64_t seqlen_k,
                 int64_t hq, int64_t hk, int64_t d, int64_t dv, int64_t q_max_seq_len, float scale, int64_t window_left,
                 int64_t window_right, uint32_t mask_type, int32_t dtype, void* stream)
{
    return fck_fmha_fwd_attrs(q, k, v, bias, o, seqstart_q, seqstart_k, seqlen_k_ptr, batch, seqlen_q, seqlen_k, hq, hk, d, dv,
                              q_max_seq_len, scale, window_left, window_right, mask_type, dtype, nullptr, stream);
}

int fck_fmha_fwd_attrs(const void* q, const void* k, const void* v, const void* bias, void* o, const int32_t* seqstart_q,
                       const int32_t* seqstart_k, const int32_t* seqlen_k_ptr, int64_t batch, int64_t seqlen_q, int64_t seqlen_k,
                       int64_t hq, int64_t hk, int64_t d, int64_t dv, int64_t q_max_seq_len, float scale, int64_t window_left,
                       int64_t window_right, uint32_t mask_type, int32_t dtype, const fck_fmha_attrs* attrs, void* stream)
{
    g_err[0] = 0;
    if (int rc = check_common(batch, hq, hk, d, dv, dtype)) return rc;
    if (int rc = check_mask(mask_type)) return rc;
    if (!q || !k || !v || !o) return fail(FCK_ERR_INVALID_ARGUMENT, "q, k, v and o must not be null");
    if (int rc = check_fit32(seqlen_q, seqlen_k, q_max_seq_len)) return rc;
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(o)) return fail(FCK_ERR_INVALID_ARGUMENT, "q, k, v and o must be 16-byte aligned");
    if (!(scale > 0.f) || !std::isfinite(scale)) return fail(FCK_ERR_INVALID_ARGUMENT, "scale must be positive and finite");
    if ((seqstart_q == nullptr) != (seqstart_k == nullptr)) return fail(FCK_ERR_INVALID_ARGUMENT, "group mode needs both seqstart_q and seqstart_k");
    fck::PrefillArgs a{};
    a.q = q;
    a.k = k;
    a.v = v;
    a.o = o;
    a.seqstart_q = seqstart_q;
    a.batch = (int32_t)batch;
    a.sq = (int32_t)seqlen_q;
    a.hq = (int32_t)hq;
    a.hk = (int32_t)hk;
    a.scale_log2 = scale * fck::kLog2e;
    a.mask_type = mask_type;
    a.window_left = window_left;
    a.window_right = window_right;
    if (int rc = fill_mod(a.mod, bias, attrs, scale, mask_type, hq)) return rc;
    if (int rc = fill_kv8(a, attrs, d, dv, dtype)) return rc;
    if (int rc = fill_variant(a, attrs)) return rc;
    a.kv.page_shift = -1;
    a.kv.seqlen_k_ptr = seqlen_k_ptr;  // group mode: logical key counts of padded packed sequences
    if (seqstart_q) {
        a.kv.mode = 1;
        a.kv.seqstart_k = seqstart_k;
    } else {
        if (seqlen_q <= 0 || seqlen_k <= 0) return fail(FCK_ERR_INVALID_ARGUMENT, "batch mode needs seqlen_q, seqlen_k > 0");
        a.kv.mode = 0;
        a.kv.seqlen_k = (int32_t)seqlen_k;
        if (q_max_seq_len <= 0) q_max_seq_len = seqlen_q;
    }
    return prefill_common(a, d, dv, dtype, q_max_seq_len, true, stream, "FmhaFwd launch");
}

int fck_fmha_batch_prefill(const void* q, const void* k_cache, const void* v_cache, void* o, const int32_t* seqstart_q,
                           const int32_t* kv_indptr, const int32_t* kv_page_indices, const int32_t* kv_last_page_lens,
                           int64_t num_total_pages, int64_t page_block_size, int64_t batch, int64_t hq, int64_t hk, int64_t d,
                           int64_t dv, int64_t q_max_seq_len, float scale, int64_t window_left, int64_t window_right,
                           uint32_t mask_type, int32_t dtype, void* stream)
{
    return fck_fmha_batch_prefill_attrs(q, k_cache, v_cache, o, seqstart_q, kv_indptr, kv_page_indices, kv_last_page_lens,
                                        num_total_pages, page_block_size, batch, hq, hk, d, dv, q_max_seq_len, scale, window_left,
                                        window_right, mask_type, dtype, nullptr, stream);
}

int fck_fmha_batch_prefill_attrs(const void* q, const void* k_cache, const void* v_cache, void* o, const int32_t* seqstart_q,
                                 const int32_t* kv_indptr, const int32_t* kv_page_indices, const int32_t* kv_last_page_lens,
                                 int64_t num_total_pages, int64_t page_block_size, int64_t batch, int64_t hq, int64_t hk,
                                 int64_t d, int64_t dv, int64_t q_max_seq_len, float scale, int64_t window_left,
                                 int64_t window_right, uint32_t mask_type, int32_t dtype, const fck_fmha_attrs* attrs, void* stream)
{
    g_err[0] = 0;
    if (int rc = check_common(batch, hq, hk, d, dv, dtype)) return rc;
    if (int rc = check_mask(mask_type)) return rc;
    if (!q || !k_cache || !v_cache || !o || !seqstart_q || !kv_indptr || !kv_page_indices)
        return fail(FCK_ERR_INVALID_ARGUMENT, "q, k_cache, v_cache, o, seqstart_q, kv_indptr and kv_page_indices must not be null");
    if (!aligned16(q) || !aligned16(k_cache) || !aligned16(v_cache) || !aligned16(o)) return fail(FCK_ERR_INVALID_ARGUMENT, "q, k_cache, v_cache and o must be 16-byte aligned");
    if (page_block_size <= 0 || num_total_pages <= 0) return fail(FCK_ERR_INVALID_ARGUMENT, "page_block_size and num_total_pages must be positive");
    if (int rc = check_fit32(page_block_size, num_total_pages, q_max_seq_len)) return rc;
    if (!(scale > 0.f) || !std::isfinite(scale)) return fail(FCK_ERR_INVALID_ARGUMENT, "scale must be positive and finite");
    fck::PrefillArgs a{};
    a.q = q;
    a.k = k_cache;
    a.v = v_cache;
    a.o = o;
    a.seqstart_q = seqstart_q;
    a.batch = (int32_t)batch;
    a.hq = (int32_t)hq;
    a.hk = (int32_t)hk;
    a.scale_log2 = scale * fck::kLog2e;
    a.mask_type = mask_type;
    a.window_left = window_left;
    a.window_right = window_right;
    if (int rc = fill_mod(a.mod, nullptr, attrs, scale, mask_type, hq)) return rc;
    if (int rc = fill_kv8(a, attrs, d, dv, dtype)) return rc;
    if (int rc = fill_variant(a, attrs)) return rc;
    a.kv.mode = 3;
    a.kv.kv_indptr = kv_indptr;
    a.kv.kv_page_indices = kv_page_indices;
    a.kv.kv_last_page_lens = kv_last_page_lens;
    a.kv.page_size = (int32_t)page_block_size;
    a.kv.page_shift = log2_exact(page_block_size);
    if (num_total_pages * page_block_size > INT32_MAX)
        return fail(FCK_ERR_INVALID_ARGUMENT, "a pool of %ld x %ld cache rows exceeds the 2^31 - 1 rows the kernels index", (long)num_total_pages, (long)page_block_size);
    return prefill_common(a, d, dv, dtype, q_max_seq_len, page_block_size % 64 == 0, stream, "FmhaFwdBatchPrefill launch");
}

int fck_fmha_fwd_pagedkv(const void* q, const void* k_cache, const void* v_cache, void* o, const int32_t* seqstart_q,
                         const int32_t* seqlen_k_ptr, const int32_t* block_table, int64_t batch_stride_block_table,
                         int64_t page_block_size, int64_t batch, int64_t seqlen_q, int64_t hq, int64_t hk, int64_t d,
                         int64_t dv, int64_t q_max_seq_len, float scale, int64_t window_left, int64_t window_right,
                         uint32_t mask_type, int32_t dtype, void* stream)
{
    return fck_fmha_fwd_pagedkv_attrs(q, k_cache, v_cache, o, seqstart_q, seqlen_k_ptr, block_table, batch_stride_block_table,
                                      page_block_size, batch, seqlen_q, hq, hk, d, dv, q_max_seq_len, scale, window_left, window_right,
                                      mask_type, dtype, nullptr, stream);
}

int fck_fmha_fwd_pagedkv_attrs(const void* q, const void* k_cache, const void* v_cache, void* o, const int32_t* seqstart_q,
                               const int32_t* seqlen_k_ptr, const int32_t* block_table, int64_t batch_stride_block_table,
                               int64_t page_block_size, int64_t batch, int64_t seqlen_q, int64_t hq, int64_t hk, int64_t d,
                               int64_t dv, int64_t q_max_seq_len, float scale, int64_t window_left, int64_t window_right,
                               uint32_t mask_type, int32_t dtype, const fck_fmha_attrs* attrs, void* stream)
{
    g_err[0] = 0;
    if (int rc = check_common(batch, hq, hk, d, dv, dtype)) return rc;
    if (int rc = check_mask(mask_type)) return rc;
    if (!q || !k_cache || !v_cache || !o || !seqlen_k_ptr || !block_table)
        return fail(FCK_ERR_INVALID_ARGUMENT, "q, k_cache, v_cache, o, seqlen_k and block_table must not be null");
    if (!aligned16(q) || !aligned16(k_cache) || !aligned16(v_cache) || !aligned16(o)) return fail(FCK_ERR_INVALID_ARGUMENT, "q, k_cache, v_cache and o must be 16-byte aligned");
    if (page_block_size <= 0 || batch_stride_block_table <= 0) return fail(FCK_ERR_INVALID_ARGUMENT, "page_block_size and batch_stride_block_table must be positive");
    if (int rc = check_fit32(page_block_size, batch_stride_block_table, seqlen_q, q_max_seq_len)) return rc;
    if (!(scale > 0.f) || !std::isfinite(scale)) return fail(FCK_ERR_INVALID_ARGUMENT, "scale must be positive and finite");
    if (!seqstart_q && seqlen_q <= 0) return fail(FCK_ERR_INVALID_ARGUMENT, "batch mode needs seqlen_q > 0");
    fck::PrefillArgs a{};
    a.q = q;
    a.k = k_cache;
    a.v = v_cache;
    a.o = o;
    a.seqstart_q = seqstart_q;
    a.batch = (int32_t)batch;
    a.sq = (int32_t)seqlen_q;
    a.hq = (int32_t)hq;
    a.hk = (int32_t)hk;
    a.scale_log2 = scale * fck::kLog2e;
    a.mask_type = mask_type;
    a.window_left = window_left;
    a.window_right = window_right;
    if (int rc = fill_mod(a.mod, nullptr, attrs, scale, mask_type, hq)) return rc;
    if (int rc = fill_kv8(a, attrs, d, dv, dtype)) return rc;
    if (int rc = fill_variant(a, attrs)) return rc;
    a.kv.mode = 2;
    a.kv.block_table = block_table;
    a.kv.block_table_stride = (int32_t)batch_stride_block_table;
    a.kv.seqlen_k_ptr = seqlen_k_ptr;
    a.kv.page_size = (int32_t)page_block_size;
    a.kv.page_shift = log2_exact(page_block_size);
    if (q_max_seq_len <= 0) q_max_seq_len = seqlen_q;
    return prefill_common(a, d, dv, dtype, q_max_seq_len, page_block_size % 64 == 0, stream, "FmhaFwdPagedKV launch");
}

}  // extern "C"
