// Self-test kernels of the wave64 emulator (test infrastructure): small kernels written against the documented
// semantics of the instructions the emulator models, with results that tests/test_emu_selftest.py checks on the host.
#include <hip/hip_runtime.h>

#include "common.hpp"

using namespace fck;

// D = A . B + C with the operand layouts of v_mfma_f32_32x32x16_bf16 / 16x16x32 / 16x16x16: A [M][K], B [K][M] row major in memory
template <int M, int K>
__global__ void mfma_kernel(const uint16_t* a, const uint16_t* b, float* d)
{
    const int l = threadIdx.x;
    constexpr int E = K / (64 / M);  // elements per lane
    uint16_t av[8] = {}, bv[8] = {};
    for (int j = 0; j < E; ++j) {
        const int k = (l / M) * E + j;
        av[j] = a[(l % M) * K + k];
        bv[j] = b[k * M + (l % M)];
    }
    if constexpr (M == 32) {
        f32x16_t acc;
        for (int v = 0; v < 16; ++v) acc[v] = 1.f;
        u32x4_t ax, bx;
        memcpy(&ax, av, 16);
        memcpy(&bx, bv, 16);
        acc = BF16::mfma32(as_vec8<bf16x8_t>(ax), as_vec8<bf16x8_t>(bx), acc);
        for (int v = 0; v < 16; ++v) d[((v / 4) * 8 + (l / 32) * 4 + v % 4) * 32 + l % 32] = acc[v];
    } else if constexpr (K == 32) {
        f32x4_t acc = {1.f, 1.f, 1.f, 1.f};
        u32x4_t ax, bx;
        memcpy(&ax, av, 16);
        memcpy(&bx, bv, 16);
        acc = BF16::mfma16(as_vec8<bf16x8_t>(ax), as_vec8<bf16x8_t>(bx), acc);
        for (int v = 0; v < 4; ++v) d[((l / 16) * 4 + v) * 16 + l % 16] = acc[v];
    } else {
        f32x4_t acc = {1.f, 1.f, 1.f, 1.f};
        u32x2_t ax, bx;
        memcpy(&ax, av, 8);
        memcpy(&bx, bv, 8);
        acc = BF16::mfma16k16(ax, bx, acc);
        for (int v = 0; v < 4; ++v) d[((l / 16) * 4 + v) * 16 + l % 16] = acc[v];
    }
}

// out[0..63] = pair32_sum(lane), out[64..127] = quad16_max(lane * 7 % 64), out[128..191] = readlane(lane * 3, 63 - lane % 4),
// out[192] = ballot(lane % 3 == 0) low word, out[193] = high word
__global__ void lanes_kernel(float* out)
{
    const int l = threadIdx.x;
    out[l] = pair32_sum((float)l);
    out[64 + l] = quad16_max((float)(l * 7 % 64));
    out[128 + l] = (float)__builtin_amdgcn_readlane(l * 3, 63 - l % 4);
    const uint64_t m = __builtin_amdgcn_ballot_w64(l % 3 == 0);
    if (l == 0) {
        out[192] = (float)(uint32_t)(m & 0xffffu);
        out[193] = (float)(uint32_t)(m >> 48);
    }
}

// Transposing LDS read: a 16 x 16 tile of 16-bit values (row r, column c) = r * 16 + c; every 16-lane group reads rows
// 4g..4g+3: lane i addresses row 4g + i / 4, columns (i % 4) * 4 .. + 3 and must receive column i of rows 4g .. 4g + 3.
__global__ void transpose_kernel(uint16_t* out)
{
    FCK_DYNAMIC_LDS(smem);
    uint16_t* tile = reinterpret_cast<uint16_t*>(smem);
    const int l = threadIdx.x;
    for (int e = l; e < 256; e += 64) tile[e] = (uint16_t)e;
    __syncthreads();
    const int g = l / 16, i = l % 16;
    const u32x2_t v = lds_read_tr16((char FCK_LDS*)smem + ((4 * g + i / 4) * 16 + (i % 4) * 4) * 2);
    uint16_t r[4];
    memcpy(r, &v, 8);
    for (int k = 0; k < 4; ++k) out[l * 4 + k] = r[k];
}

// Asynchronous global -> LDS copies: wave 0 requests two 1 KiB blocks, waits as told, barrier, wave 1 reads both.
// wait_keep = 0: both blocks must have landed; 1: only the first is guaranteed; 2: none.
template <int KEEP>
__global__ void async_kernel(const uint32_t* src, uint32_t* out)
{
    FCK_DYNAMIC_LDS(smem);
    const int l = threadIdx.x & 63, w = threadIdx.x >> 6;
    if (w == 0) {
        load_to_lds(lds_address((char FCK_LDS*)smem), src, (uint32_t)l * 16u);
        load_to_lds(lds_address((char FCK_LDS*)smem + 1024), src + 256, (uint32_t)l * 16u);
        wait_vm<KEEP>();
    }
    __syncthreads();
    if (w == 1) {
        const uint32_t* lds = reinterpret_cast<const uint32_t*>(smem);
        for (int e = l; e < 512; e += 64) out[e] = lds[e];
    }
    __syncthreads();
    if (w == 0) wait_vm<0>();
}

// A missing barrier: each of two waves writes its number + 1 into its own LDS word and reads the other wave's word with
// no barrier in between.  Whichever wave runs first sees the poison the emulator fills LDS with; the other one gets away
// with the race.  out[w] = what wave w read.
__global__ void race_kernel(uint32_t* out)
{
    FCK_DYNAMIC_LDS(smem);
    uint32_t* lds = reinterpret_cast<uint32_t*>(smem);
    const int l = threadIdx.x & 63, w = threadIdx.x >> 6;
    if (l == 0) {
        lds[w] = (uint32_t)w + 1u;
        out[w] = lds[w ^ 1];
    }
}

// A global -> LDS instruction that `real` lanes of the wave take part in and the others are masked off for.
__global__ void masked_kernel(const uint32_t* src, int real)
{
    FCK_DYNAMIC_LDS(smem);
    const int l = threadIdx.x & 63;
    if (l < real)
        load_to_lds(lds_address((char FCK_LDS*)smem), src, (uint32_t)l * 16u);
    else
        FCK_LOAD_TO_LDS_MASKED();
    wait_vm<0>();
}

extern "C" {
__attribute__((visibility("default"))) int emu_selftest_masked(const uint32_t* src, int real)
{
    hipLaunchKernelGGL(masked_kernel, dim3(1), dim3(64), 1024, nullptr, src, real);
    return (int)hipGetLastError();
}
__attribute__((visibility("default"))) int emu_selftest_race(uint32_t* out)
{
    hipLaunchKernelGGL(race_kernel, dim3(1), dim3(128), 8, nullptr, out);
    return (int)hipGetLastError();
}
__attribute__((visibility("default"))) int emu_selftest_mfma(int shape, const uint16_t* a, const uint16_t* b, float* d)
{
    if (shape == 0) hipLaunchKernelGGL((mfma_kernel<32, 16>), dim3(1), dim3(64), 0, nullptr, a, b, d);
    if (shape == 1) hipLaunchKernelGGL((mfma_kernel<16, 32>), dim3(1), dim3(64), 0, nullptr, a, b, d);
    if (shape == 2) hipLaunchKernelGGL((mfma_kernel<16, 16>), dim3(1), dim3(64), 0, nullptr, a, b, d);
    return (int)hipGetLastError();
}
__attribute__((visibility("default"))) int emu_selftest_lanes(float* out)
{
    hipLaunchKernelGGL(lanes_kernel, dim3(1), dim3(64), 0, nullptr, out);
    return (int)hipGetLastError();
}
__attribute__((visibility("default"))) int emu_selftest_transpose(uint16_t* out)
{
    hipLaunchKernelGGL(transpose_kernel, dim3(1), dim3(64), 512, nullptr, out);
    return (int)hipGetLastError();
}
__attribute__((visibility("default"))) int emu_selftest_async(int keep, const uint32_t* src, uint32_t* out)
{
    if (keep == 0) hipLaunchKernelGGL((async_kernel<0>), dim3(1), dim3(128), 2048, nullptr, src, out);
    if (keep == 1) hipLaunchKernelGGL((async_kernel<1>), dim3(1), dim3(128), 2048, nullptr, src, out);
    if (keep == 2) hipLaunchKernelGGL((async_kernel<2>), dim3(1), dim3(128), 2048, nullptr, src, out);
    return (int)hipGetLastError();
}
__attribute__((visibility("default"))) int emu_selftest_late_loads(void) { return emu::late_loads() ? 1 : 0; }
}
