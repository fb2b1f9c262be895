// Generator of the golden vectors under tests/golden/: runs ck_tile's own HOST reference functions (the
// "CPU host reference attention" FlashCK's generated harness includes through ck_tile/host.hpp,
// core/module/kernels/attention_kernels/fmha_common_jinja.h:80) on small seeded inputs and stores inputs and
// outputs.  ck_tile is the third-party dependency that holds the arithmetic of FlashCK's FMHA path; the copy used
// here is the header-only one this image ships under /opt/rocm/include (ROCm 7.2.0).  Nothing from it is copied
// into the repository: the headers are only included at build time by make_golden.sh.
//
// File format (little endian): repeated records  [u32 name_len][name][u32 dtype: 0=f32 3=fp16 4=bf16 6=i32]
// [u32 ndim][u32 dims...][raw data].
#include <functional>
#include <optional>

#include "ck_tile/core.hpp"
#include "ck_tile/host/host_tensor.hpp"
#include "ck_tile/host/reference/reference_batched_gemm.hpp"
#include "ck_tile/host/reference/reference_batched_masking.hpp"
#include "ck_tile/host/reference/reference_batched_rotary_position_embedding.hpp"
#include "ck_tile/host/reference/reference_batched_softmax.hpp"
#include "ck_tile/ops/fmha/block/block_masking.hpp"

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <random>
#include <string>
#include <vector>

static FILE* g_out;

template <typename T> struct dtype_code;
template <> struct dtype_code<float> { static constexpr uint32_t v = 0; };
template <> struct dtype_code<ck_tile::fp16_t> { static constexpr uint32_t v = 3; };
template <> struct dtype_code<ck_tile::bf16_t> { static constexpr uint32_t v = 4; };
template <> struct dtype_code<int32_t> { static constexpr uint32_t v = 6; };

template <typename T>
static void put(const std::string& name, const ck_tile::HostTensor<T>& t)
{
    const uint32_t nl = name.size(), code = dtype_code<T>::v, nd = t.get_num_of_dimension();
    fwrite(&nl, 4, 1, g_out);
    fwrite(name.data(), 1, nl, g_out);
    fwrite(&code, 4, 1, g_out);
    fwrite(&nd, 4, 1, g_out);
    for (uint32_t i = 0; i < nd; ++i) {
        const uint32_t d = t.get_length(i);
        fwrite(&d, 4, 1, g_out);
    }
    fwrite(t.mData.data(), sizeof(T), t.mData.size(), g_out);
}

template <typename T>
static void fill_normal(ck_tile::HostTensor<T>& t, std::mt19937& g, float sd = 1.f)
{
    std::normal_distribution<float> d(0.f, sd);
    for (auto& v : t.mData) v = ck_tile::type_convert<T>(d(g));
}

// rotary tables with random angles, as FlashCK's harness builds them (fmha_common_jinja.h:191-229)
template <typename T>
static void rope_case(const std::string& tag, int seq, int heads, int d, int rotary_dim, bool interleaved, std::mt19937& g)
{
    ck_tile::HostTensor<T> x({heads, seq, d}), y({heads, seq, d}), c({seq, rotary_dim / 2}), s({seq, rotary_dim / 2});
    fill_normal(x, g);
    std::uniform_real_distribution<float> ang(0.f, 6.2831853f);
    for (size_t i = 0; i < c.mData.size(); ++i) {
        const float a = ang(g);
        c.mData[i] = ck_tile::type_convert<T>(std::cos(a));
        s.mData[i] = ck_tile::type_convert<T>(std::sin(a));
    }
    ck_tile::reference_batched_rotary_position_embedding(x, c, s, interleaved, y);
    put(tag + ".x", x);
    put(tag + ".cos", c);
    put(tag + ".sin", s);
    put(tag + ".y", y);
}

// The attention chain of the ck_tile FMHA harness: S = Q.K^T (fp32 acc, scaled) -> mask -> softmax (fp32, LSE) with P
// stored in the data type -> O = P.V (fp32 acc) stored in the data type.
template <typename T>
static void attn_case(const std::string& tag, int bh, int sq, int sk, int d, int dv, float scale, int mask_type,
                      int wl, int wr, std::mt19937& g)
{
    ck_tile::HostTensor<T> q({bh, sq, d}), k({bh, sk, d}), vt({bh, dv, sk}), p({bh, sq, sk}), o({bh, sq, dv});
    ck_tile::HostTensor<float> s({bh, sq, sk}), lse({bh, sq});
    fill_normal(q, g);
    fill_normal(k, g);
    fill_normal(vt, g);
    ck_tile::reference_batched_gemm<T, T, float, float>(q, k, s, ck_tile::identity{}, ck_tile::identity{},
                                                        ck_tile::scales(scale));
    if (mask_type != 0) {
        using Mask = ck_tile::GenericAttentionMask<true, true>;
        const auto m = ck_tile::make_generic_attention_mask_from_lr_window<Mask>(wl, wr, sq, sk, mask_type == 1);
        ck_tile::reference_batched_masking(s, m);
    }
    ck_tile::reference_batched_softmax<float, float, T>(s, p, ck_tile::identity{}, std::ref(lse));
    ck_tile::reference_batched_gemm<T, T, float, T>(p, vt, o);
    ck_tile::HostTensor<int32_t> meta({4});
    meta.mData = {mask_type, wl, wr, 0};
    ck_tile::HostTensor<float> sc({1});
    sc.mData = {scale};
    put(tag + ".q", q);
    put(tag + ".k", k);
    put(tag + ".vt", vt);
    put(tag + ".mask", meta);
    put(tag + ".scale", sc);
    put(tag + ".p", p);
    put(tag + ".lse", lse);
    put(tag + ".o", o);
}

int main(int argc, char** argv)
{
    if (argc < 2) return 2;
    g_out = fopen(argv[1], "wb");
    if (!g_out) return 3;
    std::mt19937 g(42);  // FC_TUNING_SEED, core/utils/flags.cc:225
    using bf16 = ck_tile::bf16_t;
    using fp16 = ck_tile::fp16_t;
    rope_case<bf16>("rope_half_bf16", 4, 2, 128, 128, false, g);
    rope_case<bf16>("rope_inter_bf16", 4, 2, 128, 128, true, g);
    rope_case<fp16>("rope_half_fp16_partial", 5, 3, 128, 64, false, g);
    rope_case<fp16>("rope_inter_fp16_partial", 5, 3, 64, 32, true, g);
    attn_case<bf16>("attn_bf16_nomask", 3, 9, 13, 32, 32, 1.f / std::sqrt(32.f), 0, -1, -1, g);
    attn_case<bf16>("attn_bf16_causal_br", 3, 9, 13, 32, 32, 1.f / std::sqrt(32.f), 2, -1, 0, g);
    attn_case<bf16>("attn_bf16_causal_tl", 3, 9, 13, 32, 32, 1.f / std::sqrt(32.f), 1, -1, 0, g);
    attn_case<bf16>("attn_bf16_window_br", 2, 12, 20, 64, 64, 0.125f, 2, 3, 1, g);
    attn_case<bf16>("attn_bf16_causal_sq_gt_sk", 2, 11, 6, 32, 32, 1.f / std::sqrt(32.f), 2, -1, 0, g);
    attn_case<fp16>("attn_fp16_nomask", 4, 16, 16, 64, 64, 0.125f, 0, -1, -1, g);
    attn_case<fp16>("attn_fp16_window_tl", 2, 10, 17, 32, 32, 1.f / std::sqrt(32.f), 1, 4, 2, g);
    // qk_head_dim != v_head_dim, head dims off the 64 / 128 / 256 grid (appended last: the records above keep their bytes)
    attn_case<bf16>("attn_bf16_d40_dv72_causal_br", 2, 9, 14, 40, 72, 1.f / std::sqrt(40.f), 2, -1, 0, g);
    attn_case<fp16>("attn_fp16_d192_dv128_nomask", 2, 5, 11, 192, 128, 1.f / std::sqrt(192.f), 0, -1, -1, g);
    fclose(g_out);
    return 0;
}
