// AppendKV into a quantised cache (gfx950): rotary embedding of the new K rows and of Q as in appendkv_rope.hip, with the
// new K/V rows written as one e4m3 byte per element: cache = fp8(x / descale), x being the element a 16-bit cache would
// receive (the rotated K row rounded to T, the V row as given), round to nearest even, saturating at +-448.  Static
// per-tensor scales, as the reference's fp8 type configuration uses them
// (core/module/kernels/attention_kernels/fmha_common_jinja.h:157-171, is_static_quant).
//
// A kernel of its own next to the 16-bit one, which stays exactly the arithmetic that is bit-identical to ck_tile's
// host rotary reference; this one adds a division and a conversion per element behind it.  Launch-latency bound like
// the 16-bit kernel: one workgroup per (new token, sequence), one wave per row, a thread owns a rotation pair.
#include "common.hpp"
#include "kernels.hpp"

namespace fck {

// Rotates one row (rope_mode 0: copies it) and hands every element, rounded to T, to `put(index, bits)`.
template <typename T, typename Put>
__device__ __forceinline__ void rotated_elements(const uint16_t* in, int d, const uint16_t* cos_row, const uint16_t* sin_row,
                                                 int rotary_dim, int rope_mode, int lane, Put put)
{
#pragma clang fp contract(off)
    const int half = rotary_dim >> 1;
    for (int p = lane; p < (d >> 1); p += 64) {
        if (p < half && rope_mode != 0) {
            const int t1 = rope_mode == 1 ? 2 * p : p;            // interleaved: (2p, 2p+1); half rotated: (p, p + rotary_dim/2)
            const int t2 = rope_mode == 1 ? 2 * p + 1 : p + half;
            const float x1 = T::to_f32(in[t1]), x2 = T::to_f32(in[t2]);
            const float c = T::to_f32(cos_row[p]), s = T::to_f32(sin_row[p]);
            const float a1 = x1 * c, b1 = -x2 * s;
            const float a2 = x2 * c, b2 = x1 * s;
            const float o1 = a1 + b1;
            const float o2 = a2 + b2;
            put(t1, T::from_f32(o1));
            put(t2, T::from_f32(o2));
        } else {
            const int base = (rope_mode != 0) ? rotary_dim + 2 * (p - half) : 2 * p;
            put(base, in[base]);
            put(base + 1, in[base + 1]);
        }
    }
}

template <typename T>
__global__ __launch_bounds__(256) void appendkv_fp8_kernel(const AppendKvArgs a)
{
    const int i = blockIdx.x;  // index of the new token inside its sequence
    const int b = blockIdx.y;
    int n0, n;
    if (a.cu_seqlens_knew) {
        n0 = a.cu_seqlens_knew[b];
        n = a.cu_seqlens_knew[b + 1] - n0;
    } else {
        n0 = b * a.seqlen_knew;
        n = a.seqlen_knew;
    }
    if (i >= n) return;
    const int L = a.seqlen_k[b];
    const int t = L + i;
    int64_t prow;
    if (a.block_table) {
        const int pi = t / a.page_size;
        prow = (int64_t)a.block_table[(int64_t)b * a.block_table_stride + pi] * a.page_size + (t - pi * a.page_size);
    } else {
        const int64_t cb = a.cache_batch_idx ? a.cache_batch_idx[b] : b;
        prow = cb * a.seqlen_k_cache + t;
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint16_t* cosb = reinterpret_cast<const uint16_t*>(a.cos);
    const uint16_t* sinb = reinterpret_cast<const uint16_t*>(a.sin);
    const int half = a.rotary_dim >> 1;
    const int64_t src_row = n0 + i;
    const int items = a.hk * 2 + (a.q ? a.hq : 0);
    for (int it = wave; it < items; it += 4) {
        if (it < a.hk) {
            const uint16_t* src = reinterpret_cast<const uint16_t*>(a.knew) + (src_row * a.hk + it) * a.d;
            uint8_t* dst = reinterpret_cast<uint8_t*>(a.k_cache) + (prow * a.hk + it) * a.d;
            const float ds = a.k_descale;
            rotated_elements<T>(src, a.d, cosb + (int64_t)t * half, sinb + (int64_t)t * half, a.rotary_dim, a.rope_mode, lane,
                                [&](int e, uint16_t bits) { dst[e] = (uint8_t)f32_to_fp8_sat(T::to_f32(bits) / ds); });
        } else if (it < 2 * a.hk) {
            const int h = it - a.hk;
            const uint16_t* src = reinterpret_cast<const uint16_t*>(a.vnew) + (src_row * a.hk + h) * a.dv;
            uint8_t* dst = reinterpret_cast<uint8_t*>(a.v_cache) + (prow * a.hk + h) * a.dv;
            for (int e = lane; e < a.dv; e += 64) dst[e] = (uint8_t)f32_to_fp8_sat(T::to_f32(src[e]) / a.v_descale);
        } else if (a.rope_mode != 0) {
            const int h = it - 2 * a.hk;
            uint16_t* row = reinterpret_cast<uint16_t*>(a.q) + (src_row * a.hq + h) * a.d;
            const int64_t qpos = L + (a.has_mask ? i : 0);
            // in place: a thread reads both elements of its pair before it writes them
            rotated_elements<T>(row, a.d, cosb + qpos * half, sinb + qpos * half, a.rotary_dim, a.rope_mode, lane,
                                [&](int e, uint16_t bits) { row[e] = bits; });
        }
    }
}

hipError_t launch_appendkv_fp8(const AppendKvArgs& a, int dtype, int max_new, hipStream_t st)
{
    const dim3 grid(max_new, a.batch);
    if (dtype == 4)
        hipLaunchKernelGGL((appendkv_fp8_kernel<BF16>), grid, dim3(256), 0, st, a);
    else
        hipLaunchKernelGGL((appendkv_fp8_kernel<FP16>), grid, dim3(256), 0, st, a);
    return hipGetLastError();
}

}  // namespace fck
