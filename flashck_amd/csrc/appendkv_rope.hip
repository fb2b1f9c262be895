// AppendKV: rotary embedding of the new K rows (and of Q, in place) plus the write of the new K/V rows into the
// (paged) cache behind the tokens each sequence already holds (gfx950).
//
// The operation is launch-latency bound (a few MB), so the kernel favours exactness over width: one workgroup per
// (new token, sequence); a thread owns one rotation pair, reads both inputs, and writes both outputs, which makes
// the in-place Q rotation race free.  Arithmetic is fp32 with each product and the sum rounded on its own
// (floating-point contraction is switched off for the rotation, so no FMA is formed), then rounded to nearest
// even into T: the result is bit-identical to ck_tile's host rotary reference
// (ck_tile/host/reference/reference_batched_rotary_position_embedding.hpp:29-70).
#include "common.hpp"
#include "kernels.hpp"

namespace fck {

template <typename T>
__device__ __forceinline__ void rotate_row(const uint16_t* in, uint16_t* out, int d, const uint16_t* cos_row,
                                           const uint16_t* sin_row, int rotary_dim, int rope_mode, int tid, int nthreads)
{
#pragma clang fp contract(off)
    const int half = rotary_dim >> 1;
    for (int p = tid; p < (d >> 1); p += nthreads) {
        int t1, t2;
        if (p < half && rope_mode != 0) {
            if (rope_mode == 1) {  // interleaved: (2p, 2p+1)
                t1 = 2 * p;
                t2 = t1 + 1;
            } else {  // half rotated: (p, p + rotary_dim/2)
                t1 = p;
                t2 = p + half;
            }
            const float x1 = T::to_f32(in[t1]), x2 = T::to_f32(in[t2]);
            const float c = T::to_f32(cos_row[p]), s = T::to_f32(sin_row[p]);
            const float a1 = x1 * c, b1 = -x2 * s;
            const float a2 = x2 * c, b2 = x1 * s;
            const float o1 = a1 + b1;
            const float o2 = a2 + b2;
            out[t1] = T::from_f32(o1);
            out[t2] = T::from_f32(o2);
        } else {
            // not rotated: with rope on these are the tail elements rotary_dim .. d-1, else the whole row
            const int base = (rope_mode != 0) ? rotary_dim + 2 * (p - half) : 2 * p;
            const uint16_t a0 = in[base], a1 = in[base + 1];
            out[base] = a0;
            out[base + 1] = a1;
        }
    }
}

template <typename T>
__global__ __launch_bounds__(256) void appendkv_rope_kernel(const AppendKvArgs a)
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
    const int t = L + i;  // logical position of the new token
    int64_t prow;
    if (a.block_table) {
        const int pi = t / a.page_size;
        const int64_t page = a.block_table[(int64_t)b * a.block_table_stride + pi];
        prow = page * a.page_size + (t - pi * a.page_size);
    } else {
        const int64_t cb = a.cache_batch_idx ? a.cache_batch_idx[b] : b;
        prow = cb * a.seqlen_k_cache + t;
    }
    const int tid = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint16_t* cosb = reinterpret_cast<const uint16_t*>(a.cos);
    const uint16_t* sinb = reinterpret_cast<const uint16_t*>(a.sin);
    const int half = a.rotary_dim >> 1;
    const int64_t src_row = n0 + i;

    // work items of this token: Hk key rows, Hk value rows, Hq query rows; one wave per row at a time
    const int items = a.hk * 2 + (a.q ? a.hq : 0);
    for (int it = wave; it < items; it += 4) {
        if (it < a.hk) {
            const int h = it;
            const uint16_t* src = reinterpret_cast<const uint16_t*>(a.knew) + (src_row * a.hk + h) * a.d;
            uint16_t* dst = reinterpret_cast<uint16_t*>(a.k_cache) + (prow * a.hk + h) * a.d;
            rotate_row<T>(src, dst, a.d, cosb + (int64_t)t * half, sinb + (int64_t)t * half, a.rotary_dim, a.rope_mode,
                          tid, 64);
        } else if (it < 2 * a.hk) {
            const int h = it - a.hk;
            const uint16_t* src = reinterpret_cast<const uint16_t*>(a.vnew) + (src_row * a.hk + h) * a.dv;
            uint16_t* dst = reinterpret_cast<uint16_t*>(a.v_cache) + (prow * a.hk + h) * a.dv;
            for (int e = tid; e < a.dv; e += 64) dst[e] = src[e];
        } else if (a.rope_mode != 0) {
            const int h = it - 2 * a.hk;
            uint16_t* row = reinterpret_cast<uint16_t*>(a.q) + (src_row * a.hq + h) * a.d;
            const int64_t qpos = L + (a.has_mask ? i : 0);
            rotate_row<T>(row, row, a.d, cosb + qpos * half, sinb + qpos * half, a.rotary_dim, a.rope_mode, tid, 64);
        }
    }
}

hipError_t launch_appendkv(const AppendKvArgs& a, int dtype, int max_new, hipStream_t st)
{
    const dim3 grid(max_new, a.batch);
    if (dtype == 4)
        hipLaunchKernelGGL((appendkv_rope_kernel<BF16>), grid, dim3(256), 0, st, a);
    else
        hipLaunchKernelGGL((appendkv_rope_kernel<FP16>), grid, dim3(256), 0, st, a);
    return hipGetLastError();
}

}  // namespace fck
