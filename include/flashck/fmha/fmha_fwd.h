/*
 * C++ header API of the FMHA forward family, in the style of FlashCK's `flashck::naive::<op>_fwd<T>` functions
 * (include/flashck/norm/layer_norm.h:29-76: typed raw device pointers in, validation of null / non-GPU pointers and
 * sizes, failures as std::runtime_error).  The reference keeps an empty file at this path
 * (include/flashck/fmha/fmha_fwd.h); these templates are a thin layer over the C ABI of fmha_c_api.h.
 *
 * Differences from the LayerNorm template, which returns a buffer owned by FlashCK's graph runtime: outputs and
 * workspaces are caller-owned device memory passed in (the boundary of this library allocates nothing), and every call
 * takes the stream to launch on.  The output pointer is returned for chaining.
 *
 * Element types: _Float16 (fp16) and unsigned short / __bf16 (bf16 storage) - the reference instantiates its operators
 * for `_Float16` and `ushort` (layer_norm.h:19).
 */
#pragma once

#include <hip/hip_runtime_api.h>

#include <array>
#include <cstdint>
#include <stdexcept>
#include <string>
#include <type_traits>

#include "flashck/fmha/fmha_c_api.h"

namespace flashck {

namespace naive {

/* One e4m3 byte (OCP encoding): the element type that selects the all-fp8 roles (Q, K, V, P and O in e4m3,
 * FCK_DTYPE_FP8) in the functions below, where the C ABI has kernels for them. */
struct fp8_e4m3 {
    unsigned char bits;
};

namespace fmha_detail {

template <typename T>
struct DTypeOf;
template <>
struct DTypeOf<_Float16> {
    static constexpr int32_t value = FCK_DTYPE_FP16;
};
template <>
struct DTypeOf<unsigned short> {
    static constexpr int32_t value = FCK_DTYPE_BF16;
};
template <>
struct DTypeOf<fp8_e4m3> {
    static constexpr int32_t value = FCK_DTYPE_FP8;
};
#if defined(__clang__)
template <>
struct DTypeOf<__bf16> {
    static constexpr int32_t value = FCK_DTYPE_BF16;
};
#endif

/* true when the pointer is device (or managed) memory of some GPU; false for host memory and when no GPU is present */
inline bool IsGpuPointer(const void* p)
{
    hipPointerAttribute_t attr;
    if (hipPointerGetAttributes(&attr, p) != hipSuccess) {
        (void)hipGetLastError();  // the failed query must not be reported by the next HIP call
        return false;
    }
    return attr.type == hipMemoryTypeDevice || attr.type == hipMemoryTypeManaged;
}

struct Ptr {
    const void* p;
    const char* name;
    bool optional;
};

/* null checks for every pointer first, then the GPU-pointer checks, as the reference's header functions order them
 * (layer_norm.h:31-41) */
template <size_t N>
inline void Require(const char* op, const Ptr (&ptrs)[N])
{
    for (const Ptr& x : ptrs)
        if (x.p == nullptr && !x.optional) throw std::runtime_error(std::string(op) + ": null " + x.name);
    for (const Ptr& x : ptrs)
        if (x.p != nullptr && !IsGpuPointer(x.p))
            throw std::runtime_error(std::string(op) + ": " + x.name + " must be a GPU pointer");
}

inline void Check(int rc, const char* op)
{
    if (rc != FCK_OK) throw std::runtime_error(std::string(op) + " execution failed: " + fck_last_error());
}

}  // namespace fmha_detail

/**
 * @brief Dense attention forward, batch mode
 * @tparam T Data type (_Float16, unsigned short as bf16 storage)
 * @param q Query [batch, q_seq_len, q_num_heads, qk_head_dim]
 * @param k Key [batch, kv_seq_len, kv_num_heads, qk_head_dim]
 * @param v Value [batch, kv_seq_len, kv_num_heads, v_head_dim]
 * @param o Output [batch, q_seq_len, q_num_heads, v_head_dim]
 * @param scale Softmax scale; 0 selects 1/sqrt(qk_head_dim)
 * @param window_size {left, right}, -1 = unbounded (with a mask type: {-1, 0} is causal)
 * @param mask_type FCK_MASK_*
 * @return o
 */
template <typename T>
T* fmha_fwd(const T* q, const T* k, const T* v, T* o, int64_t batch, int64_t q_seq_len, int64_t kv_seq_len,
            int64_t q_num_heads, int64_t kv_num_heads, int64_t qk_head_dim, int64_t v_head_dim, float scale = 0.f,
            std::array<int64_t, 2> window_size = {-1, -1}, uint32_t mask_type = FCK_MASK_NONE,
            const int32_t* k_seq_len = nullptr, hipStream_t stream = nullptr)
{
    using namespace fmha_detail;
    Require("FmhaFwd", {
        {q, "query tensor q", false},
        {k, "key tensor k", false},
        {v, "value tensor v", false},
        {o, "output tensor o", false},
        {k_seq_len, "k_seq_len", true}});
    if (scale == 0.f && qk_head_dim > 0) scale = 1.f / __builtin_sqrtf((float)qk_head_dim);
    Check(fck_fmha_fwd(q, k, v, nullptr, o, nullptr, nullptr, k_seq_len, batch, q_seq_len, kv_seq_len, q_num_heads,
                       kv_num_heads, qk_head_dim, v_head_dim, q_seq_len, scale, window_size[0], window_size[1], mask_type,
                       DTypeOf<T>::value, stream),
          "FmhaFwd");
    return o;
}

/**
 * @brief Dense attention forward, group mode: q [total_q, Hq, D], k/v [total_k, Hk, D] packed by the prefix sums
 * q_seq_start / k_seq_start (int32 [batch + 1], device memory)
 */
template <typename T>
T* fmha_fwd_varlen(const T* q, const T* k, const T* v, T* o, const int32_t* q_seq_start, const int32_t* k_seq_start,
                   int64_t batch, int64_t total_q, int64_t total_k, int64_t q_max_seq_len, int64_t q_num_heads,
                   int64_t kv_num_heads, int64_t qk_head_dim, int64_t v_head_dim, float scale = 0.f,
                   std::array<int64_t, 2> window_size = {-1, -1}, uint32_t mask_type = FCK_MASK_NONE,
                   hipStream_t stream = nullptr)
{
    using namespace fmha_detail;
    Require("FmhaFwd", {
        {q, "query tensor q", false},
        {k, "key tensor k", false},
        {v, "value tensor v", false},
        {o, "output tensor o", false},
        {q_seq_start, "q_seq_start", false},
        {k_seq_start, "k_seq_start", false}});
    if (scale == 0.f && qk_head_dim > 0) scale = 1.f / __builtin_sqrtf((float)qk_head_dim);
    Check(fck_fmha_fwd(q, k, v, nullptr, o, q_seq_start, k_seq_start, nullptr, batch, total_q, total_k, q_num_heads,
                       kv_num_heads, qk_head_dim, v_head_dim, q_max_seq_len, scale, window_size[0], window_size[1],
                       mask_type, DTypeOf<T>::value, stream),
          "FmhaFwd");
    return o;
}

/**
 * @brief Split-KV forward over a paged cache: per-split partials into the caller's fp32 workspaces
 * @param k_cache, v_cache [num_pages, page_block_size, kv_num_heads, head_dim]
 * @param k_seq_len int32 [batch] keys per sequence; block_table int32 [batch, max_num_page_blocks / batch]
 * @param o_acc fp32 [batch, Hq, num_splits, q_seq_len, Dv]; lse_acc fp32 [batch, Hq, num_splits, q_seq_len]
 *        (fck_fmha_splitkv_workspace_bytes gives their combined size)
 * @param num_splits 0 asks the heuristic (needs max_kv_seq_len); the count used is returned
 */
template <typename T>
int fmha_fwd_splitkv(const T* q, const T* k_cache, const T* v_cache, float* o_acc, float* lse_acc, const int32_t* k_seq_len,
                     const int32_t* block_table, int64_t batch, int64_t q_seq_len, int64_t q_num_heads,
                     int64_t kv_num_heads, int64_t qk_head_dim, int64_t v_head_dim, int64_t num_splits,
                     int64_t max_num_page_blocks, int64_t page_block_size, int64_t max_kv_seq_len = 0, float scale = 0.f,
                     std::array<int64_t, 2> window_size = {-1, -1}, uint32_t mask_type = FCK_MASK_NONE,
                     hipStream_t stream = nullptr)
{
    using namespace fmha_detail;
    Require("FmhaFwdSplitKV", {
        {q, "query tensor q", false},
        {k_cache, "k_cache", false},
        {v_cache, "v_cache", false},
        {o_acc, "workspace o_acc", false},
        {lse_acc, "workspace lse_acc", false},
        {k_seq_len, "k_seq_len", false},
        {block_table, "block_table", false}});
    if (num_splits <= 0) {
        if (max_kv_seq_len <= 0 && batch > 0) max_kv_seq_len = max_num_page_blocks / batch * page_block_size;
        num_splits = fck_fmha_num_splits_heuristic(batch, q_num_heads, kv_num_heads, q_seq_len, max_kv_seq_len, qk_head_dim, 0);
    }
    if (scale == 0.f && qk_head_dim > 0) scale = 1.f / __builtin_sqrtf((float)qk_head_dim);
    Check(fck_fmha_fwd_splitkv(q, k_cache, v_cache, nullptr, lse_acc, o_acc, nullptr, nullptr, k_seq_len, block_table, nullptr,
                               batch, q_seq_len, 0, q_num_heads, kv_num_heads, qk_head_dim, v_head_dim, q_seq_len,
                               num_splits, max_num_page_blocks, page_block_size, scale, window_size[0], window_size[1],
                               mask_type, DTypeOf<T>::value, stream),
          "FmhaFwdSplitKV");
    return (int)num_splits;
}

/** @brief LSE combine of split-KV partials -> o [batch, q_seq_len, q_num_heads, v_head_dim]; returns o */
template <typename T>
T* fmha_fwd_splitkv_combine(const float* lse_acc, const float* o_acc, T* o, int64_t batch, int64_t q_seq_len,
                            int64_t q_num_heads, int64_t v_head_dim, int64_t num_splits, hipStream_t stream = nullptr)
{
    using namespace fmha_detail;
    Require("FmhaFwdSplitKVCombine", {
        {lse_acc, "lse_acc", false},
        {o_acc, "o_acc", false},
        {o, "output tensor o", false}});
    Check(fck_fmha_fwd_splitkv_combine(lse_acc, o_acc, o, nullptr, batch, q_seq_len, q_num_heads, v_head_dim, q_seq_len,
                                       num_splits, DTypeOf<T>::value, stream),
          "FmhaFwdSplitKVCombine");
    return o;
}

/**
 * @brief Rotate knew (and q, in place) and append knew / vnew to a paged cache behind k_seq_len[b] tokens
 * @param q, knew, vnew packed [total_new, H, D] with cu_seqlens_knew (int32 [batch + 1]); q may be null
 * @param rotary_cos, rotary_sin T [max position + 1, rotary_dim / 2]; ignored when rope_mode == FCK_ROPE_NONE
 */
template <typename T>
void fmha_fwd_appendkv(T* q, T* k_cache, T* v_cache, const T* knew, const T* vnew, const int32_t* k_seq_len,
                       const int32_t* cu_seqlens_knew, int64_t max_seqlen_knew, const T* rotary_cos, const T* rotary_sin,
                       int64_t rotary_dim, int32_t rope_mode, const int32_t* block_table, int64_t batch_stride_block_table,
                       int64_t page_block_size, int64_t batch, int64_t q_num_heads, int64_t kv_num_heads,
                       int64_t qk_head_dim, int64_t v_head_dim, bool has_mask = true, hipStream_t stream = nullptr)
{
    using namespace fmha_detail;
    Require("FmhaFwdAppendKV", {
        {q, "query tensor q", true},
        {k_cache, "k_cache", false},
        {v_cache, "v_cache", false},
        {knew, "knew", false},
        {vnew, "vnew", false},
        {k_seq_len, "k_seq_len", false},
        {cu_seqlens_knew, "cu_seqlens_knew", true},
        {block_table, "block_table", false},
        {rotary_cos, "rotary_cos", rope_mode == FCK_ROPE_NONE},
        {rotary_sin, "rotary_sin", rope_mode == FCK_ROPE_NONE}});
    Check(fck_fmha_fwd_appendkv(q, k_cache, v_cache, knew, vnew, k_seq_len, cu_seqlens_knew, max_seqlen_knew, rotary_cos,
                                rotary_sin, rotary_dim, rope_mode, has_mask ? 1 : 0, block_table, batch_stride_block_table,
                                page_block_size, nullptr, 0, batch, q_num_heads, kv_num_heads, qk_head_dim, v_head_dim,
                                DTypeOf<T>::value, stream),
          "FmhaFwdAppendKV");
}

/**
 * @brief Varlen causal prefill over a page list: q/o [total_q, Hq, D] packed by q_seq_start; sequence b owns pages
 * kv_page_indices[kv_indptr[b] .. kv_indptr[b+1]) of the cache [num_total_pages, page_block_size, Hk, D]; returns o
 */
template <typename T>
T* fmha_batch_prefill(const T* q, const T* k_cache, const T* v_cache, T* o, const int32_t* q_seq_start,
                      const int32_t* kv_indptr, const int32_t* kv_page_indices, const int32_t* kv_last_page_lens,
                      int64_t num_total_pages, int64_t page_block_size, int64_t batch, int64_t q_num_heads,
                      int64_t kv_num_heads, int64_t qk_head_dim, int64_t v_head_dim, int64_t q_max_seq_len, float scale = 0.f,
                      std::array<int64_t, 2> window_size = {-1, 0}, uint32_t mask_type = FCK_MASK_BOTTOM_RIGHT,
                      hipStream_t stream = nullptr)
{
    using namespace fmha_detail;
    Require("FmhaFwdBatchPrefill", {
        {q, "query tensor q", false},
        {k_cache, "k_cache", false},
        {v_cache, "v_cache", false},
        {o, "output tensor o", false},
        {q_seq_start, "q_seq_start", false},
        {kv_indptr, "kv_indptr", false},
        {kv_page_indices, "kv_page_indices", false},
        {kv_last_page_lens, "kv_last_page_lens", true}});
    if (scale == 0.f && qk_head_dim > 0) scale = 1.f / __builtin_sqrtf((float)qk_head_dim);
    Check(fck_fmha_batch_prefill(q, k_cache, v_cache, o, q_seq_start, kv_indptr, kv_page_indices, kv_last_page_lens,
                                 num_total_pages, page_block_size, batch, q_num_heads, kv_num_heads, qk_head_dim, v_head_dim,
                                 q_max_seq_len, scale, window_size[0], window_size[1], mask_type, DTypeOf<T>::value, stream),
          "FmhaFwdBatchPrefill");
    return o;
}

/**
 * @brief Causal prefill over a block table (chunked prefill: the q_seq_len new queries of a sequence attend to its
 * k_seq_len[b] cached keys); q_seq_start null = batch mode q [batch, q_seq_len, Hq, D]; returns o
 */
template <typename T>
T* fmha_fwd_pagedkv(const T* q, const T* k_cache, const T* v_cache, T* o, const int32_t* q_seq_start, const int32_t* k_seq_len,
                    const int32_t* block_table, int64_t batch_stride_block_table, int64_t page_block_size, int64_t batch,
                    int64_t q_seq_len, int64_t q_num_heads, int64_t kv_num_heads, int64_t qk_head_dim, int64_t v_head_dim,
                    int64_t q_max_seq_len, float scale = 0.f, std::array<int64_t, 2> window_size = {-1, 0},
                    uint32_t mask_type = FCK_MASK_BOTTOM_RIGHT, hipStream_t stream = nullptr)
{
    using namespace fmha_detail;
    Require("FmhaFwdPagedKV", {
        {q, "query tensor q", false},
        {k_cache, "k_cache", false},
        {v_cache, "v_cache", false},
        {o, "output tensor o", false},
        {q_seq_start, "q_seq_start", true},
        {k_seq_len, "k_seq_len", false},
        {block_table, "block_table", false}});
    if (scale == 0.f && qk_head_dim > 0) scale = 1.f / __builtin_sqrtf((float)qk_head_dim);
    Check(fck_fmha_fwd_pagedkv(q, k_cache, v_cache, o, q_seq_start, k_seq_len, block_table, batch_stride_block_table,
                               page_block_size, batch, q_seq_len, q_num_heads, kv_num_heads, qk_head_dim, v_head_dim,
                               q_max_seq_len, scale, window_size[0], window_size[1], mask_type, DTypeOf<T>::value, stream),
          "FmhaFwdPagedKV");
    return o;
}

}  // namespace naive

}  // namespace flashck
