// Argument blocks and launchers shared between the C ABI (fmha_api.cpp) and the kernel translation units.
#pragma once

#include "common.hpp"

#include <mutex>

namespace fck {

// Launch `Kern` with `lds` bytes of dynamic LDS.  More than 64 KiB needs an opt-in per kernel and device; it is made
// once per device under std::call_once, so concurrent first calls from several host threads are safe, and every later
// call is a plain launch (nothing but the launch itself reaches the stream, so a warmed-up call can be captured).
template <auto Kern, typename Args>
inline hipError_t launch_with_lds(dim3 grid, dim3 block, size_t lds, hipStream_t st, const Args& a)
{
    constexpr int kMaxDev = 64;
    static std::once_flag once[kMaxDev];
    static hipError_t status[kMaxDev];
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= kMaxDev) return hipErrorInvalidDevice;
    std::call_once(once[dev], [&] {
        status[dev] = hipFuncSetAttribute((const void*)Kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    });
    if (status[dev] != hipSuccess) return status[dev];
    hipLaunchKernelGGL(Kern, grid, block, lds, st, a);
    return hipGetLastError();
}

struct SplitKvArgs {
    const void* q;
    const void* k;
    const void* v;
    float* o_acc;
    float* lse_acc;
    const int32_t* seqstart_q;
    KvAddr kv;
    int32_t batch, sq, hq, hk, num_splits;
    int32_t m_tiles;     // row tiles per (sequence, KV head); set by the launcher
    uint32_t* tickets;   // non-null: the last workgroup of a (sequence, head group, row tile) merges the splits into `o`
    void* o;
    int64_t shape_sq;  // Sq of the workspace: sq (batch mode) or total_q (group mode)
    float scale_log2;  // scale * log2(e)
    uint32_t mask_type;
    int64_t window_left, window_right;
    ScoreMod mod;      // bias / ALiBi / soft cap; all zero: none
    int32_t variant;   // 0: chosen by the launcher; 1 / 3: one KV head per workgroup; 2 / 4: head pairs (3, 4: with split_chunk)
    int32_t split_chunk;  // > 0: keys per split, the same for every sequence (variants 3 and 4); 0: num_splits equal parts per sequence
    int32_t kv8;       // K and V are fp8 (e4m3); the K scale is folded into scale_log2 / mod.scale by the caller
    float v_descale;   // factor on the output (1 unless V is quantised)
    int32_t longest_first;  // set by the launcher: workgroups take the sequences in order of decreasing key count
    int32_t d, dv;     // head dims of Q/K and of V/O as stored (multiples of 8); the kernel's D is the next of 64 / 128 / 256
    int32_t q8;        // with kv8: Q is e4m3 too and P is rounded to e4m3 before the second product (all-fp8 roles)
};

struct CombineArgs {
    const float* lse_acc;
    const float* o_acc;
    void* o;
    int64_t rows;  // Bs * Sq
    int64_t Sq;
    int32_t hq, dv, num_splits;
    int32_t num_cu;  // compute units of the device (decides the workgroup size)
    float o_scale;   // e4m3 output: O = saturate(o_scale * o)
};

struct AppendKvArgs {
    void* q;
    void* k_cache;
    void* v_cache;
    const void* knew;
    const void* vnew;
    const int32_t* seqlen_k;
    const int32_t* cu_seqlens_knew;
    int32_t seqlen_knew;
    const void* cos;
    const void* sin;
    int32_t rotary_dim, rope_mode, has_mask;
    const int32_t* block_table;
    int32_t block_table_stride, page_size;
    const int32_t* cache_batch_idx;
    int64_t seqlen_k_cache;
    int32_t batch, hq, hk, d, dv;
    int32_t kv8;                 // the caches hold e4m3 bytes: cache = fp8(value / descale)
    float k_descale, v_descale;
};

struct PrefillArgs {
    const void* q;
    const void* k;
    const void* v;
    void* o;
    const int32_t* seqstart_q;
    KvAddr kv;
    int32_t batch, sq, hq, hk;
    int32_t m_tiles;
    float scale_log2;
    uint32_t mask_type;
    int64_t window_left, window_right;
    ScoreMod mod;  // bias / ALiBi / soft cap; all zero: none (an elementwise bias only in the 4-wave kernel of prefill.hip)
    int32_t d, dv;  // head dims of Q/K and of V/O as stored; other than the kernel's D only in the 4-wave kernel of prefill.hip
    int32_t variant;  // tile variant of the ping-pong kernel: 0 / 1 the default schedule, 2..4 see prefill_pingpong.hip
    int32_t kv8;      // K and V are fp8 (e4m3); the K scale is folded into scale_log2 / mod.scale by the caller (4-wave kernel only)
    float v_descale;  // factor on the output (1 unless V is quantised)
    int32_t q8;       // with kv8: Q and O are e4m3 too, P is rounded to e4m3 before the second product (all-fp8 roles)
    float o_scale;    // q8: O = saturate(o_scale * o)
};

// arguments of the paged-cache checker: a block table (block_table != nullptr: seqlen_k, block_table_stride) or a page
// list (kv_indptr, kv_page_indices, optional kv_last_page_lens)
struct ValidateArgs {
    const int32_t* seqlen_k;
    const int32_t* block_table;
    int64_t block_table_stride;
    const int32_t* kv_indptr;
    const int32_t* kv_page_indices;
    const int32_t* kv_last_page_lens;
    int64_t num_total_pages;
    int32_t page_size, batch;
    int32_t* counts;  // int32[4], device memory of the caller
};
hipError_t launch_validate_paged(const ValidateArgs& a, hipStream_t st);
hipError_t launch_clear_tickets(uint32_t* tickets, int n, hipStream_t st);

// heads_per_workgroup (may be null): receives the kernel variant the launcher took, 1 or 2 KV heads per workgroup
hipError_t launch_splitkv_decode(const SplitKvArgs& a, int d, int dtype, int rows_max, bool uniform_page, int num_cu,
                                 hipStream_t st, int* heads_per_workgroup = nullptr);
// Device memory the fused split-KV entry point uses instead of a caller-owned workspace: a fixed array in the library
// (one copy per GPU), cut into kDecodeScratchSlices equal slices so that calls on different streams of a GPU never share
// one (a stream keeps the slice it got on its first call).  Layout: the arrival counters of all slices
// (kDecodeScratchTickets each, self-resetting), then the partial results of all slices (kDecodeScratchPartialFloats each).
constexpr int64_t kDecodeScratchTickets = 16384;
constexpr int64_t kDecodeScratchPartialFloats = (int64_t)4 << 20;  // 16 MiB
constexpr int kDecodeScratchSlices = 4;
constexpr int64_t kDecodeScratchFloats = kDecodeScratchSlices * (kDecodeScratchTickets + kDecodeScratchPartialFloats);
// address of the array on the current device (looked up once per device)
hipError_t decode_scratch(float** ptr);
// row tiles per (sequence, KV head) the split-KV launcher uses for `rows_max` packed query rows
int splitkv_decode_m_tiles(int d, int rows_max);
hipError_t launch_splitkv_combine(const CombineArgs& a, int dtype, hipStream_t st);
hipError_t launch_appendkv(const AppendKvArgs& a, int dtype, int max_new, hipStream_t st);
// a.kv8: the caches hold e4m3 bytes
hipError_t launch_appendkv_fp8(const AppendKvArgs& a, int dtype, int max_new, hipStream_t st);
hipError_t launch_prefill(const PrefillArgs& a, int d, int dtype, bool uniform_page, hipStream_t st);
// Tiles of a sequence whose first rows the direct-to-LDS prefill kernels cache in LDS; tiles past them are looked up one
// by one.
constexpr int kPrefillPageCache = 4096;
constexpr int kPrefillKeyTile = 64;
// 256-row workgroups (a.m_tiles counts 256-row tiles); head dims 64 and 128
hipError_t launch_prefill_pingpong(const PrefillArgs& a, int d, int dtype, bool uniform_page, hipStream_t st);

// Head dim 256 with the K/V tiles sent global -> LDS directly (128-row workgroups; a.m_tiles counts 128-row tiles);
// uniform pages only.
hipError_t launch_prefill_dma(const PrefillArgs& a, int d, int dtype, hipStream_t st);

}  // namespace fck
