// Tile machinery shared by the prefill kernels that send K/V tiles global -> LDS directly (prefill_pingpong.hip,
// prefill_dma.hip): the XOR swizzles of a staged tile and the per-workgroup cache of every key tile's first cache
// row (the global -> LDS instruction itself and the wait on a wave's own loads are in gfx950_ops.hpp).
#pragma once
#include "common.hpp"
#include "kernels.hpp"

namespace fck {
namespace tiles {

// XOR swizzles of the 16-byte chunk index of a staged row of D elements.  They keep both LDS read patterns free of
// bank conflicts whether the LDS serves 128 or 256 bytes per clock: K is read by 8/16 consecutive lanes = consecutive
// rows at one logical chunk; V (transposing read) by 16/32 lanes = 4 rows x (2 or 4) adjacent chunks.
template <int D>
__device__ __forceinline__ int k_swz(int row)
{
    if constexpr (D >= 128)
        return row & 15;
    else
        return ((row & 7) + ((row >> 3) & 1)) & 7;
}
template <int D>
__device__ __forceinline__ int v_swz(int row, int lc)
{
    if constexpr (D >= 128)
        return ((row & 3) << 1) ^ (((lc >> 1) & 1) << 3);
    else
        return (row & 3) << 1;
}
// Logical V chunk that lands at physical chunk pc of `row`: the inverse of lc -> lc ^ v_swz(row, lc).  The swizzle is
// applied on the global side: lane l of a global -> LDS instruction always lands at byte l*16 of its 1 KiB block, so it
// fetches the chunk that belongs there.
template <int D>
__device__ __forceinline__ int v_chunk_at(int row, int pc)
{
    const int t = pc ^ ((row & 3) << 1);
    return D >= 128 ? (t ^ (((t >> 1) & 1) << 3)) : t;
}

using fck::load_to_lds;
using fck::wait_vm;

// First cache row of key tile i (BN keys, local index from t_begin) of a paged sequence whose tiles never straddle a
// page.  fill() computes the first CACHE of them once per workgroup into LDS (a barrier must follow); row0()
// then costs a v_readlane: lane l keeps the entry of tile chunk * 64 + l in a register and LDS is read once per 64
// tiles (an LDS read per tile would queue behind the operand reads of the matrix work).  Tiles past the cached ones of
// a very long sequence are looked up one by one, with a scalar load through the constant address space (the table is
// an input, never written here) that is consumed on the spot, so that the wait it needs stays there.
template <int BN, int CACHE = kPrefillPageCache>
struct FirstRows {
    int FCK_LDS* rows;
    int vec = 0, chunk = -1;

    __device__ __forceinline__ static int table_row(const KvAddr& kv, const int32_t* table, int kb)
    {
        const int pi = kv.page_shift >= 0 ? kb >> kv.page_shift : kb / kv.page_size;
        return table[pi] * kv.page_size + (kb - pi * kv.page_size);
    }
    __device__ __forceinline__ void fill(const KvAddr& kv, const KvSeq& ks, int t_begin, int n, int tid, int nthreads)
    {
        if (ks.table != nullptr)
            for (int i = tid; i < min(n, CACHE); i += nthreads) rows[i] = table_row(kv, ks.table, (t_begin + i) * BN);
    }
    __device__ __forceinline__ int64_t row0(const KvAddr& kv, const KvSeq& ks, int t_begin, int i, int lane)
    {
        if (ks.table != nullptr) {
            if (i >= CACHE) {
                const int kb = (t_begin + i) * BN;
                const int pi = kv.page_shift >= 0 ? kb >> kv.page_shift : kb / kv.page_size;
                int page = const_load(ks.table, pi);
                FCK_PIN_SGPR(page);
                return (int64_t)page * kv.page_size + (kb - pi * kv.page_size);
            }
            if ((i >> 6) != chunk) {
                chunk = i >> 6;
                vec = rows[min(chunk * 64 + lane, CACHE - 1)];
            }
            return __builtin_amdgcn_readlane(vec, i & 63);
        }
        return ks.base_row + (t_begin + i) * BN;
    }
};

}  // namespace tiles
}  // namespace fck
