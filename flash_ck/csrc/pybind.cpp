// Compiled Python module `flash_ck.flash_ck`: the FMHA operators as functions of torch tensors, in the way the
// reference's module exposes layer_norm_fwd (core/pybind/pybind.cc:13-58, core/pybind/norm/layer_norm.h:13-31):
// TORCH_CHECK validation, outputs allocated with torch, work enqueued on torch's current stream.  Everything below the
// tensors is the C ABI of include/flashck/fmha/fmha_c_api.h; there is no other implementation behind these names.
#include <torch/extension.h>

#include <c10/hip/HIPStream.h>

#include <cmath>
#include <optional>
#include <tuple>

#include "flashck/fmha/fmha_c_api.h"

namespace flashck {
namespace pytorch {

using at::Tensor;
typedef std::optional<Tensor> OptTensor;

namespace {

// FLASH_CK_HOST_TENSORS: test build that binds the same glue to the CPU emulator build of the kernels (tests/emu), where
// tensors live in host memory and there is no stream; the shipped module is built without it.
#ifdef FLASH_CK_HOST_TENSORS
void* current_stream() { return nullptr; }
constexpr bool kHostTensors = true;
#else
void* current_stream() { return static_cast<void*>(c10::hip::getCurrentHIPStream().stream()); }
constexpr bool kHostTensors = false;
#endif

// float8_e4m3fn: the all-fp8 roles (Q, K, V, P and O in e4m3), where the library has kernels for them
int32_t dtype_id(at::ScalarType t)
{
    TORCH_CHECK(t == at::kHalf || t == at::kBFloat16 || t == at::kFloat8_e4m3fn, "FMHA supports float16, bfloat16 and float8_e4m3fn, got ", t);
    return t == at::kHalf ? FCK_DTYPE_FP16 : t == at::kBFloat16 ? FCK_DTYPE_BF16 : FCK_DTYPE_FP8;
}

int32_t dtype_id(const Tensor& t)
{
    return dtype_id(t.scalar_type());
}

void check_gpu(const Tensor& t, const char* name, int64_t ndim = -1)
{
    TORCH_CHECK(t.is_cuda() != kHostTensors, name, " must be a GPU tensor");
    TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
    TORCH_CHECK(ndim < 0 || t.dim() == ndim, name, " must have ", ndim, " dimensions, got ", t.dim());
}

const int32_t* index_ptr(const OptTensor& t, const char* name)
{
    if (!t.has_value()) return nullptr;
    check_gpu(*t, name);
    TORCH_CHECK(t->scalar_type() == at::kInt, name, " must be int32");
    return t->data_ptr<int32_t>();
}

void check(int rc, const char* what)
{
    TORCH_CHECK(rc == FCK_OK, what, ": ", fck_last_error());
}

float default_scale(double scale, int64_t d) { return scale > 0 ? (float)scale : 1.f / std::sqrt((float)d); }

void check_kv(const Tensor& q, const Tensor& k, const Tensor& v)
{
    TORCH_CHECK(k.scalar_type() == q.scalar_type() && v.scalar_type() == q.scalar_type(), "q, k and v must have one dtype");
    TORCH_CHECK(k.size(-1) == q.size(-1), "k head dim ", k.size(-1), " != q head dim ", q.size(-1));
    TORCH_CHECK(k.size(-2) == v.size(-2) && k.size(-2) > 0 && q.size(-2) % k.size(-2) == 0, "q heads must be a multiple of kv heads");
}

}  // namespace

// q [B, sq, Hq, D], k / v [B, sk, Hk, D / Dv] -> o [B, sq, Hq, Dv]
Tensor fmha_fwd(const Tensor& q, const Tensor& k, const Tensor& v, double scale, int64_t mask_type, int64_t window_left, int64_t window_right)
{
    check_gpu(q, "q", 4);
    check_gpu(k, "k", 4);
    check_gpu(v, "v", 4);
    check_kv(q, k, v);
    TORCH_CHECK(k.size(0) == q.size(0) && v.size(0) == q.size(0) && v.size(1) == k.size(1), "k / v do not match q's batch or each other's length");
    Tensor o = at::empty({q.size(0), q.size(1), q.size(2), v.size(3)}, q.options());
    check(fck_fmha_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), nullptr, o.data_ptr(), nullptr, nullptr, nullptr, q.size(0), q.size(1), k.size(1),
                       q.size(2), k.size(2), q.size(3), v.size(3), q.size(1), default_scale(scale, q.size(3)), window_left, window_right,
                       (uint32_t)mask_type, dtype_id(q), current_stream()),
          "fmha_fwd");
    return o;
}

// packed q [total_q, Hq, D], k / v [total_k, Hk, D / Dv] with cu_seqlens (int32 [B + 1])
Tensor fmha_fwd_varlen(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor& cu_seqlens_q, const Tensor& cu_seqlens_k,
                       int64_t max_seqlen_q, double scale, int64_t mask_type, int64_t window_left, int64_t window_right)
{
    check_gpu(q, "q", 3);
    check_gpu(k, "k", 3);
    check_gpu(v, "v", 3);
    check_kv(q, k, v);
    TORCH_CHECK(max_seqlen_q > 0, "max_seqlen_q must be positive");
    TORCH_CHECK(cu_seqlens_q.numel() >= 2 && cu_seqlens_k.numel() == cu_seqlens_q.numel(), "cu_seqlens_q and cu_seqlens_k must have batch + 1 entries");
    Tensor o = at::empty({q.size(0), q.size(1), v.size(2)}, q.options());
    check(fck_fmha_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), nullptr, o.data_ptr(), index_ptr(cu_seqlens_q, "cu_seqlens_q"),
                       index_ptr(cu_seqlens_k, "cu_seqlens_k"), nullptr, cu_seqlens_q.numel() - 1, q.size(0), k.size(0), q.size(1), k.size(1),
                       q.size(2), v.size(2), max_seqlen_q, default_scale(scale, q.size(2)), window_left, window_right, (uint32_t)mask_type,
                       dtype_id(q), current_stream()),
          "fmha_fwd_varlen");
    return o;
}

// paged split-KV forward: q [B, sq, Hq, D] or packed [total_q, Hq, D] (cu_seqlens_q), caches [pages, P, Hk, D / Dv]
// -> (o_acc fp32 [Bs, Hq, ns, Sq, Dv], lse_acc fp32 [Bs, Hq, ns, Sq])
std::tuple<Tensor, Tensor> fmha_fwd_splitkv(const Tensor& q, const Tensor& k_cache, const Tensor& v_cache, int64_t num_splits, const Tensor& seqlen_k,
                                            const Tensor& block_table, const OptTensor& cu_seqlens_q, int64_t max_seqlen_q, double scale,
                                            int64_t mask_type, int64_t window_left, int64_t window_right)
{
    const bool group = cu_seqlens_q.has_value();
    check_gpu(q, "q", group ? 3 : 4);
    check_gpu(k_cache, "k_cache", 4);
    check_gpu(v_cache, "v_cache", 4);
    check_gpu(block_table, "block_table", 2);
    check_kv(q, k_cache, v_cache);
    TORCH_CHECK(num_splits >= 1, "num_splits must be >= 1 (fmha_num_splits_heuristic proposes one)");
    const int64_t B = seqlen_k.numel(), Hq = q.size(-2), D = q.size(-1), Hk = k_cache.size(2), Dv = v_cache.size(3);
    TORCH_CHECK(block_table.size(0) == B, "block_table must have one row per sequence");
    TORCH_CHECK(!group || max_seqlen_q > 0, "group mode needs max_seqlen_q");
    const int64_t sq = group ? q.size(0) : q.size(1), bs = group ? 1 : q.size(0);
    TORCH_CHECK(group ? cu_seqlens_q->numel() == B + 1 : q.size(0) == B, "seqlen_k must have one entry per sequence of q");
    auto f32 = q.options().dtype(at::kFloat);
    Tensor o_acc = at::empty({bs, Hq, num_splits, sq, Dv}, f32), lse_acc = at::empty({bs, Hq, num_splits, sq}, f32);
    check(fck_fmha_fwd_splitkv(q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), nullptr, lse_acc.data_ptr(), o_acc.data_ptr(),
                               index_ptr(cu_seqlens_q, "cu_seqlens_q"), nullptr, index_ptr(seqlen_k, "seqlen_k"), index_ptr(block_table, "block_table"),
                               nullptr, B, sq, 0, Hq, Hk, D, Dv, group ? max_seqlen_q : sq, num_splits, block_table.numel(), k_cache.size(1),
                               default_scale(scale, D), window_left, window_right, (uint32_t)mask_type, dtype_id(q), current_stream()),
          "fmha_fwd_splitkv");
    return {o_acc, lse_acc};
}

Tensor fmha_fwd_splitkv_combine(const Tensor& lse_acc, const Tensor& o_acc, at::ScalarType dtype, const OptTensor& cu_seqlens_q, int64_t max_seqlen_q)
{
    check_gpu(lse_acc, "lse_acc", 4);
    check_gpu(o_acc, "o_acc", 5);
    TORCH_CHECK(lse_acc.scalar_type() == at::kFloat && o_acc.scalar_type() == at::kFloat, "the partials are float32");
    const int32_t out_dtype = dtype_id(dtype);
    const int64_t bs = o_acc.size(0), Hq = o_acc.size(1), ns = o_acc.size(2), sq = o_acc.size(3), Dv = o_acc.size(4);
    TORCH_CHECK(lse_acc.sizes() == at::IntArrayRef({bs, Hq, ns, sq}), "lse_acc does not match o_acc");
    const bool group = cu_seqlens_q.has_value();
    TORCH_CHECK(!group || bs == 1, "group mode partials have shape batch 1");
    Tensor o = group ? at::empty({sq, Hq, Dv}, o_acc.options().dtype(dtype)) : at::empty({bs, sq, Hq, Dv}, o_acc.options().dtype(dtype));
    check(fck_fmha_fwd_splitkv_combine(lse_acc.data_ptr(), o_acc.data_ptr(), o.data_ptr(), index_ptr(cu_seqlens_q, "cu_seqlens_q"),
                                       group ? cu_seqlens_q->numel() - 1 : bs, sq, Hq, Dv, max_seqlen_q > 0 ? max_seqlen_q : sq, ns,
                                       out_dtype, current_stream()),
          "fmha_fwd_splitkv_combine");
    return o;
}

// in place: rotates q and knew, writes knew / vnew behind seqlen_k[b] tokens of the paged cache
void fmha_fwd_appendkv(const OptTensor& q, Tensor& k_cache, Tensor& v_cache, const Tensor& knew, const Tensor& vnew, const Tensor& seqlen_k,
                       const Tensor& block_table, const OptTensor& cu_seqlens_knew, int64_t max_seqlen_knew, const OptTensor& rotary_cos,
                       const OptTensor& rotary_sin, int64_t rope_mode, bool has_mask)
{
    const bool packed = cu_seqlens_knew.has_value();
    check_gpu(knew, "knew", packed ? 3 : 4);
    check_gpu(vnew, "vnew", packed ? 3 : 4);
    check_gpu(k_cache, "k_cache", 4);
    check_gpu(v_cache, "v_cache", 4);
    check_gpu(block_table, "block_table", 2);
    if (q.has_value()) check_gpu(*q, "q", packed ? 3 : 4);
    TORCH_CHECK(k_cache.scalar_type() == knew.scalar_type() && v_cache.scalar_type() == knew.scalar_type() && vnew.scalar_type() == knew.scalar_type(),
                "caches and new tokens must have one dtype");
    const int64_t B = seqlen_k.numel(), Hk = knew.size(-2), D = knew.size(-1), Dv = vnew.size(-1);
    TORCH_CHECK(k_cache.size(2) == Hk && k_cache.size(3) == D && v_cache.size(2) == Hk && v_cache.size(3) == Dv, "caches do not match the new tokens");
    TORCH_CHECK(block_table.size(0) == B, "block_table must have one row per sequence");
    const int64_t n = packed ? max_seqlen_knew : knew.size(1);
    TORCH_CHECK(n > 0, "packed new tokens need max_seqlen_knew");
    int64_t rotary_dim = 0;
    if (rope_mode != FCK_ROPE_NONE) {
        TORCH_CHECK(rotary_cos.has_value() && rotary_sin.has_value(), "rope_mode != 0 needs rotary_cos and rotary_sin");
        check_gpu(*rotary_cos, "rotary_cos", 2);
        check_gpu(*rotary_sin, "rotary_sin", 2);
        TORCH_CHECK(rotary_cos->scalar_type() == knew.scalar_type() && rotary_sin->sizes() == rotary_cos->sizes(), "rotary tables: knew's dtype, equal shapes");
        rotary_dim = rotary_cos->size(1) * 2;
    }
    check(fck_fmha_fwd_appendkv(q.has_value() ? q->data_ptr() : nullptr, k_cache.data_ptr(), v_cache.data_ptr(), knew.data_ptr(), vnew.data_ptr(),
                                index_ptr(seqlen_k, "seqlen_k"), index_ptr(cu_seqlens_knew, "cu_seqlens_knew"), n,
                                rotary_cos.has_value() ? rotary_cos->data_ptr() : nullptr, rotary_sin.has_value() ? rotary_sin->data_ptr() : nullptr,
                                rotary_dim, (int32_t)rope_mode, has_mask ? 1 : 0, index_ptr(block_table, "block_table"), block_table.size(1),
                                k_cache.size(1), nullptr, 0, B, q.has_value() ? q->size(-2) : 0, Hk, D, Dv, dtype_id(knew), current_stream()),
          "fmha_fwd_appendkv");
}

// varlen prefill over a page list: q [total_q, Hq, D]
Tensor fmha_batch_prefill(const Tensor& q, const Tensor& k_cache, const Tensor& v_cache, const Tensor& cu_seqlens_q, const Tensor& kv_indptr,
                          const Tensor& kv_page_indices, const OptTensor& kv_last_page_lens, int64_t max_seqlen_q, double scale, int64_t mask_type,
                          int64_t window_left, int64_t window_right)
{
    check_gpu(q, "q", 3);
    check_gpu(k_cache, "k_cache", 4);
    check_gpu(v_cache, "v_cache", 4);
    check_kv(q, k_cache, v_cache);
    const int64_t B = cu_seqlens_q.numel() - 1;
    TORCH_CHECK(B >= 1 && kv_indptr.numel() == B + 1, "cu_seqlens_q and kv_indptr must have batch + 1 entries");
    TORCH_CHECK(max_seqlen_q > 0, "max_seqlen_q must be positive");
    Tensor o = at::empty({q.size(0), q.size(1), v_cache.size(3)}, q.options());
    check(fck_fmha_batch_prefill(q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), o.data_ptr(), index_ptr(cu_seqlens_q, "cu_seqlens_q"),
                                 index_ptr(kv_indptr, "kv_indptr"), index_ptr(kv_page_indices, "kv_page_indices"),
                                 index_ptr(kv_last_page_lens, "kv_last_page_lens"), k_cache.size(0), k_cache.size(1), B, q.size(1), k_cache.size(2),
                                 q.size(2), v_cache.size(3), max_seqlen_q, default_scale(scale, q.size(2)), window_left, window_right,
                                 (uint32_t)mask_type, dtype_id(q), current_stream()),
          "fmha_batch_prefill");
    return o;
}

// prefill over a block table: q [B, sq, Hq, D] or packed with cu_seqlens_q
Tensor fmha_fwd_pagedkv(const Tensor& q, const Tensor& k_cache, const Tensor& v_cache, const Tensor& seqlen_k, const Tensor& block_table,
                        const OptTensor& cu_seqlens_q, int64_t max_seqlen_q, double scale, int64_t mask_type, int64_t window_left, int64_t window_right)
{
    const bool group = cu_seqlens_q.has_value();
    check_gpu(q, "q", group ? 3 : 4);
    check_gpu(k_cache, "k_cache", 4);
    check_gpu(v_cache, "v_cache", 4);
    check_gpu(block_table, "block_table", 2);
    check_kv(q, k_cache, v_cache);
    const int64_t B = seqlen_k.numel();
    TORCH_CHECK(block_table.size(0) == B, "block_table must have one row per sequence");
    TORCH_CHECK(group ? (cu_seqlens_q->numel() == B + 1 && max_seqlen_q > 0) : q.size(0) == B, "q does not match seqlen_k (group mode needs max_seqlen_q)");
    const int64_t sq = group ? 0 : q.size(1);
    std::vector<int64_t> shape(q.sizes().begin(), q.sizes().end());
    shape.back() = v_cache.size(3);
    Tensor o = at::empty(shape, q.options());
    check(fck_fmha_fwd_pagedkv(q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), o.data_ptr(), index_ptr(cu_seqlens_q, "cu_seqlens_q"),
                               index_ptr(seqlen_k, "seqlen_k"), index_ptr(block_table, "block_table"), block_table.size(1), k_cache.size(1), B, sq,
                               q.size(-2), k_cache.size(2), q.size(-1), v_cache.size(3), group ? max_seqlen_q : sq, default_scale(scale, q.size(-1)),
                               window_left, window_right, (uint32_t)mask_type, dtype_id(q), current_stream()),
          "fmha_fwd_pagedkv");
    return o;
}

}  // namespace pytorch

namespace py = pybind11;

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m)
{
    m.doc() = "FlashCK PyTorch Extension: FMHA forward family on gfx950";
    m.def("fmha_version", [] { return std::string(fck_fmha_version()); });
    m.def("fmha_last_kernel", [] { return std::string(fck_fmha_last_kernel()); });
    m.def("fmha_num_splits_heuristic", &fck_fmha_num_splits_heuristic, py::arg("batch"), py::arg("q_num_heads"), py::arg("kv_num_heads"),
          py::arg("seqlen_q"), py::arg("max_seqlen_k"), py::arg("head_dim"), py::arg("num_cu") = 0,
          "Split count from the CU count and the KV length");
    m.def("fmha_fwd", &pytorch::fmha_fwd, "Dense attention forward", py::arg("q"), py::arg("k"), py::arg("v"), py::arg("scale") = 0.0,
          py::arg("mask_type") = 0, py::arg("window_left") = -1, py::arg("window_right") = -1);
    m.def("fmha_fwd_varlen", &pytorch::fmha_fwd_varlen, "Packed (group mode) attention forward", py::arg("q"), py::arg("k"), py::arg("v"),
          py::arg("cu_seqlens_q"), py::arg("cu_seqlens_k"), py::arg("max_seqlen_q"), py::arg("scale") = 0.0, py::arg("mask_type") = 0,
          py::arg("window_left") = -1, py::arg("window_right") = -1);
    m.def("fmha_fwd_splitkv", &pytorch::fmha_fwd_splitkv, "Split-KV forward over a paged cache -> (o_acc, lse_acc)", py::arg("q"),
          py::arg("k_cache"), py::arg("v_cache"), py::arg("num_splits"), py::arg("seqlen_k"), py::arg("block_table"),
          py::arg("cu_seqlens_q") = py::none(), py::arg("max_seqlen_q") = 0, py::arg("scale") = 0.0, py::arg("mask_type") = 0,
          py::arg("window_left") = -1, py::arg("window_right") = -1);
    m.def("fmha_fwd_splitkv_combine", &pytorch::fmha_fwd_splitkv_combine, "LSE combine of split-KV partials", py::arg("lse_acc"), py::arg("o_acc"),
          py::arg("dtype"), py::arg("cu_seqlens_q") = py::none(), py::arg("max_seqlen_q") = 0);
    m.def("fmha_fwd_appendkv", &pytorch::fmha_fwd_appendkv, "Rotary embedding + paged-cache append, in place", py::arg("q"), py::arg("k_cache"),
          py::arg("v_cache"), py::arg("knew"), py::arg("vnew"), py::arg("seqlen_k"), py::arg("block_table"),
          py::arg("cu_seqlens_knew") = py::none(), py::arg("max_seqlen_knew") = 0, py::arg("rotary_cos") = py::none(),
          py::arg("rotary_sin") = py::none(), py::arg("rope_mode") = 0, py::arg("has_mask") = true);
    m.def("fmha_batch_prefill", &pytorch::fmha_batch_prefill, "Varlen prefill over a page list", py::arg("q"), py::arg("k_cache"), py::arg("v_cache"),
          py::arg("cu_seqlens_q"), py::arg("kv_indptr"), py::arg("kv_page_indices"), py::arg("kv_last_page_lens") = py::none(),
          py::arg("max_seqlen_q") = 0, py::arg("scale") = 0.0, py::arg("mask_type") = 2, py::arg("window_left") = -1, py::arg("window_right") = 0);
    m.def("fmha_fwd_pagedkv", &pytorch::fmha_fwd_pagedkv, "Prefill over a block table", py::arg("q"), py::arg("k_cache"), py::arg("v_cache"),
          py::arg("seqlen_k"), py::arg("block_table"), py::arg("cu_seqlens_q") = py::none(), py::arg("max_seqlen_q") = 0, py::arg("scale") = 0.0,
          py::arg("mask_type") = 2, py::arg("window_left") = -1, py::arg("window_right") = 0);
}

}  // namespace flashck
