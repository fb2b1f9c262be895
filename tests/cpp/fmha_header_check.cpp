// Host-only check of include/flashck/fmha/fmha_fwd.h: every template instantiates for both element types, and the
// validation that precedes a launch reports null and non-GPU pointers the way the reference's header API does
// (std::runtime_error with the operation name).  Needs no GPU: every call here must fail before anything is launched.
#include "flashck/fmha/fmha_fwd.h"

#include <cstdio>
#include <cstring>

template <typename F>
static int expect_throw(F f, const char* needle)
{
    try {
        f();
    } catch (const std::runtime_error& e) {
        if (std::strstr(e.what(), needle)) return 0;
        std::printf("wrong message: '%s' (wanted '%s')\n", e.what(), needle);
        return 1;
    }
    std::printf("no exception (wanted '%s')\n", needle);
    return 1;
}

template <typename T>
static int run()
{
    namespace n = flashck::naive;
    int bad = 0;
    T host[64] = {};
    float hostf[64] = {};
    int32_t hosti[8] = {};
    bad += expect_throw([&] { n::fmha_fwd<T>(nullptr, host, host, host, 1, 1, 1, 1, 1, 64, 64); }, "FmhaFwd: null query tensor q");
    bad += expect_throw([&] { n::fmha_fwd<T>(host, host, host, nullptr, 1, 1, 1, 1, 1, 64, 64); }, "FmhaFwd: null output tensor o");
    bad += expect_throw([&] { n::fmha_fwd<T>(host, host, host, host, 1, 1, 1, 1, 1, 64, 64); }, "query tensor q must be a GPU pointer");
    bad += expect_throw([&] { n::fmha_fwd_varlen<T>(host, host, host, host, nullptr, hosti, 1, 1, 1, 1, 1, 1, 64, 64); }, "FmhaFwd: null q_seq_start");
    bad += expect_throw([&] { n::fmha_fwd_varlen<T>(host, host, host, host, hosti, hosti, 1, 1, 1, 1, 1, 1, 64, 64); }, "must be a GPU pointer");
    bad += expect_throw([&] { n::fmha_fwd_splitkv<T>(host, host, host, nullptr, hostf, hosti, hosti, 1, 1, 8, 2, 128, 128, 0, 4, 128); }, "FmhaFwdSplitKV: null workspace o_acc");
    bad += expect_throw([&] { n::fmha_fwd_splitkv<T>(host, host, host, hostf, hostf, hosti, hosti, 1, 1, 8, 2, 128, 128, 0, 4, 128); }, "FmhaFwdSplitKV: query tensor q must be a GPU pointer");
    bad += expect_throw([&] { n::fmha_fwd_splitkv<T>(nullptr, host, host, hostf, hostf, hosti, hosti, 1, 1, 8, 2, 128, 128, 2, 4, 128); }, "FmhaFwdSplitKV: null query tensor q");
    bad += expect_throw([&] { n::fmha_fwd_splitkv_combine<T>(nullptr, hostf, host, 1, 1, 8, 128, 2); }, "FmhaFwdSplitKVCombine: null lse_acc");
    bad += expect_throw([&] { n::fmha_fwd_appendkv<T>(nullptr, nullptr, host, host, host, hosti, hosti, 1, host, host, 64, FCK_ROPE_HALF_ROTATED, hosti, 4, 16, 1, 8, 2, 64, 64); }, "FmhaFwdAppendKV: null k_cache");
    bad += expect_throw([&] { n::fmha_batch_prefill<T>(host, host, host, host, hosti, nullptr, hosti, nullptr, 4, 16, 1, 8, 2, 64, 64, 1); }, "FmhaFwdBatchPrefill: null kv_indptr");
    bad += expect_throw([&] { n::fmha_batch_prefill<T>(host, host, host, host, hosti, hosti, hosti, nullptr, 4, 16, 1, 8, 2, 64, 64, 1); }, "must be a GPU pointer");
    bad += expect_throw([&] { n::fmha_fwd_pagedkv<T>(host, host, host, host, nullptr, nullptr, hosti, 4, 16, 1, 1, 8, 2, 64, 64, 1); }, "FmhaFwdPagedKV: null k_seq_len");
    bad += expect_throw([&] { n::fmha_fwd_pagedkv<T>(host, host, host, host, nullptr, hosti, hosti, 4, 16, 1, 1, 8, 2, 64, 64, 1); }, "must be a GPU pointer");
    return bad;
}

int main()
{
    const int bad = run<_Float16>() + run<unsigned short>();
    static_assert(flashck::naive::fmha_detail::DTypeOf<_Float16>::value == FCK_DTYPE_FP16, "fp16 id");
    static_assert(flashck::naive::fmha_detail::DTypeOf<unsigned short>::value == FCK_DTYPE_BF16, "bf16 id");
    static_assert(flashck::naive::fmha_detail::DTypeOf<flashck::naive::fp8_e4m3>::value == FCK_DTYPE_FP8 && sizeof(flashck::naive::fp8_e4m3) == 1,
                  "e4m3 id, one byte per element");
    std::printf(bad ? "FAILED: %d checks\n" : "OK\n", bad);
    return bad != 0;
}
