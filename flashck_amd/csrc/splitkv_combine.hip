// LSE combine of split-KV partial results (gfx950).
//   LSE = logsumexp_s lse_acc[s];  O = sum_s exp(lse_acc[s] - LSE) * o_acc[s]  -> T
// A pure streaming reduce: DV/4 lanes own one output row with float4 loads of each split's partial row.
// Layouts: o_acc [Bs, Hq, ns, Sq, Dv], lse_acc [Bs, Hq, ns, Sq], o [Bs*Sq, Hq, Dv].  Dv is any multiple of 8 up to 256: the
// kernel is instantiated for DV = 64 / 128 / 256 and the lanes past Dv of a row's group idle.
// The work is a short chain of dependent loads per row, so what matters is how many CUs share it: workgroups are
// 256 threads when that still gives every CU a few of them, one wave (64 threads) otherwise - a decode step of 256
// output rows then runs on 128 workgroups instead of 32.
#include "common.hpp"
#include "kernels.hpp"

#include <type_traits>

namespace fck {

// output type tag: one e4m3 byte per element, O = saturate(a.o_scale * o) (the all-fp8 roles)
struct FP8Out {};

template <typename T, int DV, int NT = 256>
__global__ __launch_bounds__(NT) void splitkv_combine_kernel(const CombineArgs a)
{
    constexpr int TPR = DV / 4;     // threads per output row
    constexpr int RPB = NT / TPR;   // rows per block
    const int64_t item = (int64_t)blockIdx.x * RPB + threadIdx.x / TPR;  // (row, head) pair
    const int c = (threadIdx.x % TPR) * 4;
    if (item >= a.rows * a.hq || c >= a.dv) return;
    const int64_t row = item / a.hq;  // b * Sq + i
    const int h = (int)(item % a.hq);
    const int64_t b = row / a.Sq, i = row % a.Sq;
    const int ns = a.num_splits;
    const int64_t w0 = ((b * a.hq + h) * ns) * a.Sq + i;  // split 0; next split is Sq further

    const f32x4_t acc = combine_splits<DV>(a.lse_acc, a.o_acc, w0, a.Sq, ns, c, a.dv);
    if constexpr (std::is_same<T, FP8Out>::value) {
        *reinterpret_cast<uint32_t*>(reinterpret_cast<uint8_t*>(a.o) + (row * a.hq + h) * a.dv + c) =
            pack_fp8x4_sat(acc[0] * a.o_scale, acc[1] * a.o_scale, acc[2] * a.o_scale, acc[3] * a.o_scale);
    } else {
        u32x2_t out;
        out[0] = T::pack2(acc[0], acc[1]);
        out[1] = T::pack2(acc[2], acc[3]);
        *reinterpret_cast<u32x2_t*>(reinterpret_cast<uint16_t*>(a.o) + (row * a.hq + h) * a.dv + c) = out;
    }
}

template <typename T, int DV>
static hipError_t launch_dv(const CombineArgs& a, hipStream_t st)
{
    constexpr int RPB = 256 / (DV / 4), RPW = 64 / (DV / 4);  // rows per 256-thread / per 64-thread workgroup
    const int64_t items = a.rows * a.hq;
    const int64_t wide = (items + RPB - 1) / RPB;
    if (wide < 4 * (int64_t)a.num_cu) {
        hipLaunchKernelGGL((splitkv_combine_kernel<T, DV, 64>), dim3((unsigned)((items + RPW - 1) / RPW)), dim3(64), 0, st, a);
    } else {
        hipLaunchKernelGGL((splitkv_combine_kernel<T, DV, 256>), dim3((unsigned)wide), dim3(256), 0, st, a);
    }
    return hipGetLastError();
}

template <typename T>
static hipError_t launch_t(const CombineArgs& a, hipStream_t st)
{
    if (a.dv <= 0 || a.dv > 256 || a.dv % 8) return hipErrorInvalidValue;
    if (a.dv <= 64) return launch_dv<T, 64>(a, st);
    if (a.dv <= 128) return launch_dv<T, 128>(a, st);
    return launch_dv<T, 256>(a, st);
}

hipError_t launch_splitkv_combine(const CombineArgs& a, int dtype, hipStream_t st)
{
    if (dtype == 1) return launch_t<FP8Out>(a, st);
    return dtype == 4 ? launch_t<BF16>(a, st) : launch_t<FP16>(a, st);
}

}  // namespace fck
