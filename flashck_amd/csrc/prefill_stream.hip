// Forward attention for long query runs, streaming variant of the ping-pong kernel (gfx950).
//
// Same tile machinery as prefill_pingpong.hip - 8 waves = two groups that alternate matrix and vector phases, 64-key K/V
// tiles sent global -> LDS into rings of four buffers, operands fetched two MFMA pairs ahead - but the grid is
// persistent: one workgroup per CU walks a list of work items (256 query rows of one head each), and the K/V tile
// stream does not stop at an item boundary: the last requests of an item fetch the first tiles of the next one, and the
// phase that finishes an item (O^T += V^T.P^T of its last tile, normalise, store) also starts the next (S^T = K.Q^T of
// its first tile).  What a one-item-per-workgroup grid pays per item - dispatch, the chain of dependent metadata loads,
// the cold first tiles, an idle half pipeline at both ends - is paid once per workgroup.
//
// Work list.  Slots (row tile, sequence x KV head, query head in group) are ordered heaviest row tile first, as in the
// ping-pong kernel, and dealt to the XCDs the same way (all workgroups that stream one (sequence, KV head) sit on one
// XCD).  Every workgroup scans the slots of its XCD, keeps the valid ones in that order (ordered compaction) and takes
// those whose rank falls to it when the ranks are dealt to the XCD's workgroups back and forth (0..W-1, W-1..0, ...):
// with costs sorted in descending order this keeps the per-workgroup totals within a few percent of each other without
// any atomic counter.
//
// Phases of one item with n tiles at stream position pos (tile t lives in ring buffer (pos + t) % 4), per wave:
//   [cold start only: request K0 V0 K1 K2 V1; wait; barrier; barrier; M(-1) = {S = K0.Q}; barrier]
//   for i in 0 .. n-2:  V(i) = {request K_{i+3}, V_{i+2}; softmax(i)}; barrier; M(i) = {PV(i); S = K_{i+1}.Q}; wait; barrier
//   V(n-1) = {request K_{n+2}, V_{n+1}; softmax(n-1)}; barrier
//   M(n-1) = {PV(n-1); normalise and store O; [hand-off: next item's Q; S = K_n.Q]}; wait; barrier
//   (an item with no visible tile: store zeros; barrier; barrier)
// A tile index >= n addresses the next item (hand-off) when this item has at least 4 tiles and the next at least 3;
// otherwise such requests are left out, the wait that follows drains the queue, and the next item starts cold.  Group 1
// runs one barrier behind group 0 throughout (one extra barrier at kernel start, group 0 one at the end); a cold start
// therefore passes two barriers after its wait, which is what it takes for each group to see the other's share.
#include "common.hpp"
#include "kernels.hpp"

#include <type_traits>

namespace fck {
namespace stream {

template <int D>
struct Shape {
    static constexpr int BM = 256;
    static constexpr int BN = 64;
    static constexpr int NB = BN / 32;   // 32-key blocks per tile
    static constexpr int KT = D / 16;    // k-steps of the QK product
    static constexpr int DVB = D / 32;   // 32-column blocks of the output
    static constexpr int ROWB = D * 2;   // bytes per staged row
    static constexpr int TILEB = BN * ROWB;
    static constexpr int LD = TILEB / 1024 / 8;  // 1 KiB global->LDS instructions per wave and tile
    static constexpr int RING = 4;               // LDS buffers per operand (a power of two)
    static_assert(TILEB % 8192 == 0, "a tile is split evenly over the 8 waves");
};

// XOR swizzles of the 16-byte chunk index (conflict-free for the K read by rows and the transposing V read).
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

// wave-uniform description of one work item
struct Item {
    int b, h, hkv, q_row0, sq_b, m0, sk_b, t_begin, n;
    const int32_t* table;
    int64_t base_row;
    MaskYX mk;
};

// Uniform metadata reads (sequence starts, page-list bounds, lengths) go through the constant address space, so that
// they become scalar loads: they wait on their own counter and issue together, instead of one vector load and one
// full drain of the vector-memory queue per value.  The arrays are inputs of the launch and never written by it.
__device__ __forceinline__ int32_t ldc(const int32_t* p, int64_t i)
{
    return ((const __attribute__((address_space(4))) int32_t*)p)[i];
}
// kv_seq() of common.hpp with constant-space reads
__device__ __forceinline__ KvSeq kv_seq_c(const KvAddr& a, int b)
{
    KvSeq s;
    if (a.mode == 0) {
        const int cb = a.cache_batch_idx ? ldc(a.cache_batch_idx, b) : b;
        s.table = nullptr;
        s.base_row = (int64_t)cb * a.seqlen_k;
        s.len = a.seqlen_k_ptr ? ldc(a.seqlen_k_ptr, b) : a.seqlen_k;
    } else if (a.mode == 1) {
        const int s0 = ldc(a.seqstart_k, b);
        s.table = nullptr;
        s.base_row = s0;
        s.len = a.seqlen_k_ptr ? ldc(a.seqlen_k_ptr, b) : ldc(a.seqstart_k, b + 1) - s0;
    } else if (a.mode == 2) {
        s.table = a.block_table + (int64_t)b * a.block_table_stride;
        s.base_row = 0;
        s.len = ldc(a.seqlen_k_ptr, b);
    } else {
        const int p0 = ldc(a.kv_indptr, b), p1 = ldc(a.kv_indptr, b + 1);
        s.table = a.kv_page_indices + p0;
        s.base_row = 0;
        const int np = p1 - p0;
        const int last = a.kv_last_page_lens ? ldc(a.kv_last_page_lens, b) : a.page_size;
        s.len = np > 0 ? (np - 1) * a.page_size + last : 0;
    }
    return s;
}

// first-row cache of a tile stream: lane l holds the first cache row of tile chunk * 64 + l of the item in buffer buf
struct RowCache {
    int vec, chunk, buf;
};

template <typename T, int D>
__global__ __launch_bounds__(512) void prefill_stream_kernel(const PrefillArgs a)
{
    typedef Shape<D> S;
    typedef typename T::vec8 vec8;
    constexpr int BN = S::BN;
    constexpr int kRing = S::RING;
    constexpr int kRows = kPrefillStreamRowCache;
    constexpr int kItems = kPrefillStreamMaxItems;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    char FCK_LDS* lds = (char FCK_LDS*)smem;  // K ring | V ring | first rows (2 items) | item list | scan scratch
    char FCK_LDS* const k_ring = lds;
    char FCK_LDS* const v_ring = lds + kRing * S::TILEB;
    int FCK_LDS* const row_lds = (int FCK_LDS*)(lds + 2 * kRing * S::TILEB);
    int FCK_LDS* const my_items = row_lds + 2 * kRows;
    int FCK_LDS* const scan = my_items + kItems;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int group = wave >> 2;
    const int wg = wave & 3;
    const int l32 = lane & 31;
    const int half = lane >> 5;

    // ---- work list of this workgroup ----------------------------------------------------------------------------
    constexpr int kXcd = 8;
    const int g = a.hq / a.hk;
    const int xcd = blockIdx.x % kXcd;
    const int wgx = blockIdx.x / kXcd;      // this workgroup among those of its XCD
    const int nwx = gridDim.x / kXcd;       // workgroups per XCD
    const int groups = a.batch * a.hk;
    const int gx = (groups + kXcd - 1) / kXcd;  // (sequence, KV head) pairs per XCD
    const int slots = g * gx * a.m_tiles;
    int total = 0;  // valid slots of this XCD
    for (int c0 = 0; c0 < slots; c0 += 512) {
        const int s = c0 + tid;
        bool valid = false;
        if (s < slots) {
            const int gk = (s / g) % gx;
            const int mt = a.m_tiles - 1 - s / (g * gx);
            const int gid = gk * kXcd + xcd;
            if (gid < groups) {
                const int b = gid / a.hk;
                const int rows = a.seqstart_q ? a.seqstart_q[b + 1] - a.seqstart_q[b] : a.sq;
                valid = mt * S::BM < rows;
            }
        }
        const uint64_t vote = __builtin_amdgcn_ballot_w64(valid);
        if (lane == 0) scan[wave] = __builtin_popcountll(vote);
        __syncthreads();
        int before = 0, chunk_total = 0;
#pragma unroll
        for (int w = 0; w < 8; ++w) {
            const int c = scan[w];
            before += (w < wave) ? c : 0;
            chunk_total += c;
        }
        if (valid) {
            const int k = total + before + __builtin_popcountll(vote & ((1ull << lane) - 1));  // rank among the valid slots
            const int m = k % (2 * nwx);
            const int which = (m == wgx) ? 0 : ((m == 2 * nwx - 1 - wgx) ? 1 : -1);
            const int pos = 2 * (k / (2 * nwx)) + which;
            if (which >= 0 && pos < kItems) my_items[pos] = s;
        }
        total += chunk_total;
        __syncthreads();  // scan[] is rewritten by the next chunk
    }
    const int rem = total % (2 * nwx);
    int my_count = 2 * (total / (2 * nwx)) + (rem > wgx ? 1 : 0) + (rem > 2 * nwx - 1 - wgx ? 1 : 0);
    my_count = min(my_count, kItems);  // the launcher only starts this kernel when the list cannot overflow
    if (my_count == 0) return;

    auto load_item = [&](int pos) __attribute__((always_inline)) {
        Item it;
        const int s = __builtin_amdgcn_readfirstlane(my_items[pos]);
        const int hh = s % g;
        const int gk = (s / g) % gx;
        const int mt = a.m_tiles - 1 - s / (g * gx);
        const int gid = gk * kXcd + xcd;
        it.b = gid / a.hk;
        it.hkv = gid % a.hk;
        it.h = it.hkv * g + hh;
        if (a.seqstart_q) {
            it.q_row0 = ldc(a.seqstart_q, it.b);
            it.sq_b = ldc(a.seqstart_q, it.b + 1) - it.q_row0;
        } else {
            it.q_row0 = it.b * a.sq;
            it.sq_b = a.sq;
        }
        it.m0 = mt * S::BM;
        const KvSeq ks = kv_seq_c(a.kv, it.b);
        it.table = ks.table;
        it.base_row = ks.base_row;
        it.sk_b = ks.len;
        it.mk = make_mask(a.mask_type, a.window_left, a.window_right, it.sq_b, it.sk_b);
        // tiles the workgroup walks (a group also walks the few tiles only the other group can see: they mask to zero)
        it.t_begin = mask_lo(it.mk, it.m0) / BN;
        const int t_end = (mask_hi(it.mk, min(it.m0 + S::BM, it.sq_b) - 1, it.sk_b) + BN - 1) / BN;
        it.n = max(t_end - it.t_begin, 0);
        return it;
    };
    // first cache row of every tile of an item, into half `buf` of the row cache (every thread writes its entries)
    auto fill_rows = [&](const Item& it, int buf) __attribute__((always_inline)) {
        if (it.table != nullptr)
            for (int i = tid; i < min(it.n, kRows); i += 512) {
                const int kb = (it.t_begin + i) * BN;
                const int pi = a.kv.page_shift >= 0 ? kb >> a.kv.page_shift : kb / a.kv.page_size;
                row_lds[buf * kRows + i] = it.table[pi] * a.kv.page_size + (kb - pi * a.kv.page_size);
            }
    };
    auto tile_row0 = [&](const Item& it, int buf, int i, RowCache& c) __attribute__((always_inline)) -> int64_t {
        if (it.table != nullptr) {
            if (buf != c.buf || (i >> 6) != c.chunk) {
                c.buf = buf;
                c.chunk = i >> 6;
                c.vec = row_lds[buf * kRows + min(c.chunk * 64 + lane, kRows - 1)];
            }
            return __builtin_amdgcn_readlane(c.vec, i & 63);
        }
        return it.base_row + (it.t_begin + i) * BN;
    };

    // ---- per-lane state of the current item ----------------------------------------------------------------------
    int t_begin = 0, lo_r = 0, hi_r = 0, w_lo_max = 0, w_hi_min = 0, r = 0;
    bool row_ok = false;
    auto enter = [&](const Item& it) __attribute__((always_inline)) {
        t_begin = it.t_begin;
        r = it.m0 + group * 128 + wg * 32 + l32;  // this lane's query row
        row_ok = r < it.sq_b;
        lo_r = row_ok ? mask_lo(it.mk, r) : 0;
        hi_r = row_ok ? mask_hi(it.mk, r, it.sk_b) : it.sk_b;
        // wave-uniform: keys in [w_lo_max, w_hi_min) are visible to every valid row of the wave
        const int wr0 = it.m0 + group * 128 + wg * 32;
        const bool wave_ok = wr0 < it.sq_b;
        const int wr1 = min(wr0 + 32, it.sq_b) - 1;
        w_lo_max = wave_ok ? mask_lo(it.mk, wr1) : 0;
        w_hi_min = wave_ok ? mask_hi(it.mk, wr0, it.sk_b) : it.sk_b;
    };
    // Q fragments (B operand of S^T = K . Q^T): lane (row = l32, k-group = half)
    auto load_q = [&](const Item& it, u32x4_t (&dst)[S::KT]) __attribute__((always_inline)) {
        const int row = it.m0 + group * 128 + wg * 32 + l32;
        const bool ok = row < it.sq_b;
        const uint16_t* qp =
            reinterpret_cast<const uint16_t*>(a.q) + ((int64_t)(it.q_row0 + (ok ? row : 0)) * a.hq + it.h) * D + half * 8;
#pragma unroll
        for (int t = 0; t < S::KT; ++t) {
            dst[t] = u32x4_t{0u, 0u, 0u, 0u};
            if (ok) dst[t] = ldg16(qp + t * 16);
        }
    };

    u32x4_t qf[S::KT], qnext[S::KT];
    f32x16_t oacc[S::DVB];
    float m_run = -INFINITY, l_run = 0.f;
    auto reset_acc = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < S::DVB; ++i)
#pragma unroll
            for (int j = 0; j < 16; ++j) oacc[i][j] = 0.f;
        m_run = -INFINITY;
        l_run = 0.f;
    };
    reset_acc();
    f32x16_t s[S::NB];          // scores of the tile between its M and V phase
    u32x4_t pfrag[2 * S::NB];   // probabilities of the tile between its V phase and the next M phase

    const uint16_t* kp = reinterpret_cast<const uint16_t*>(a.k);
    const uint16_t* vp = reinterpret_cast<const uint16_t*>(a.v);
    const int64_t row_stride = (int64_t)a.hk * D;

    // global -> LDS assignment: wave w fills the 1 KiB blocks w, w+8, ... of a tile; lane l of an instruction lands at
    // byte l*16 of its block, i.e. at (row, physical chunk) below, and fetches the logical chunk that the swizzle maps
    // there.
    int cp_row[S::LD], cp_k[S::LD], cp_v[S::LD];  // tile row, element offsets (row-relative) of the K and V chunk
#pragma unroll
    for (int u = 0; u < S::LD; ++u) {
        const int off = (wave + 8 * u) * 1024 + lane * 16;
        const int row = off / S::ROWB;
        const int pc = (off % S::ROWB) >> 4;
        cp_row[u] = row;
        cp_k[u] = (pc ^ k_swz<D>(row)) * 8;
        const int t = pc ^ ((row & 3) << 1);
        cp_v[u] = (D >= 128 ? (t ^ (((t >> 1) & 1) << 3)) : t) * 8;  // inverse of lc -> lc ^ v_swz(row, lc)
    }
    // byte offsets of this lane's chunks from the first row of a tile whose 64 rows all exist
    uint32_t cp_koff[S::LD], cp_voff[S::LD];
#pragma unroll
    for (int u = 0; u < S::LD; ++u) {
        cp_koff[u] = (uint32_t)(cp_row[u] * (int)row_stride + cp_k[u]) * 2u;
        cp_voff[u] = (uint32_t)(cp_row[u] * (int)row_stride + cp_v[u]) * 2u;
    }
    // request this wave's share of tile `tile` of item `it` (first cache row row0) into ring buffer `slot`
    auto request = [&](const uint16_t* base, char FCK_LDS* ring, int slot, const Item& it, int tile, int64_t row0,
                       const int (&cp_c)[S::LD], const uint32_t (&cp_off)[S::LD]) __attribute__((always_inline)) {
        const int room = it.sk_b - 1 - (it.t_begin + tile) * BN;
        const bool whole = room >= BN - 1;  // every row of the tile exists (all tiles but the last of a sequence)
#pragma unroll
        for (int u = 0; u < S::LD; ++u) {
            // Written as assembly on purpose: a load the compiler knows about makes it drain the whole load queue
            // before the next LDS read it cannot prove disjoint.  m0 carries the LDS address of the block and is
            // put back afterwards, since the compiler does not expect it to change.
            uint32_t m0_saved;
            const uint32_t dst = (uint32_t)(uintptr_t)(ring + slot * S::TILEB + (wave + 8 * u) * 1024);
            const uint16_t* tb = base + (row0 * row_stride + it.hkv * D);
            uint32_t off = cp_off[u];
            if (!whole)  // rows past the last key repeat it (their scores are masked)
                off = (uint32_t)(min(cp_row[u], room) * (int)row_stride + cp_c[u]) * 2u;
            asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %3\n\ts_mov_b32 m0, %0"
                         : "=&s"(m0_saved)
                         : "s"(dst), "v"(off), "s"(tb)
                         : "memory");
        }
    };
    // wait until at most `keep` of this wave's vector-memory operations are outstanding (they complete in order)
    auto wait_vm = [&](auto keep) __attribute__((always_inline)) {
        constexpr int N = decltype(keep)::value;
        __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
    };

    // per-lane LDS read offsets
    // K (A operand): row = key (mbk * 32 + l32), chunk = t * 2 + half
    const int k_rd = l32 * S::ROWB;
    const int k_sw = k_swz<D>(l32);  // rows mbk*32 + l32 share the swizzle of l32 (32 is a multiple of 16)
    // V^T (A operand, transposing read): 16-lane group q4 = lane / 16 covers columns (q4 & 1) * 16 .. +15 of a
    // 32-column block; lane i of the group addresses row half * 4 + i / 4, columns (i % 4) * 4 .. +3
    const int i16 = lane & 15;
    const int q4 = lane >> 4;
    const int v_row = half * 4 + (i16 >> 2);
    const int v_rd = v_row * S::ROWB + ((i16 & 1) << 3);
    const int v_c0 = (q4 & 1) * 2 + ((i16 & 3) >> 1);  // chunk inside the 32-column block (4 chunks)

    // Matrix phase: O^T += V^T . P^T from the V tile in `vt` (when PV), then S^T = K . Q^T from the K tile in `kt`
    // (when QK), as one sequence of steps of two MFMAs; the LDS operands of a step are requested two steps ahead.
    constexpr int kPvSteps = 2 * S::NB * (S::DVB / 2);
    auto matrix = [&](auto PV, auto QK, const char FCK_LDS* vt, const char FCK_LDS* kt) __attribute__((always_inline)) {
        constexpr bool kPv = decltype(PV)::value, kQk = decltype(QK)::value;
        constexpr int kP = kPv ? kPvSteps : 0;
        constexpr int kSteps = kP + (kQk ? S::KT : 0);
        u32x4_t bf[3][2];
        auto fetch = [&](int m, u32x4_t (&d)[2]) __attribute__((always_inline)) {
            if (m < kP) {
                const int ks4 = m / (S::DVB / 2), pr = m % (S::DVB / 2);  // 16 keys ks4*16..+15; rows +{0,8}+v_row share v_row's swizzle
                const char FCK_LDS* vb = vt + ks4 * 16 * S::ROWB + v_rd;
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    const int lc = (pr * 2 + e) * 4 + v_c0;
                    const int coff = ((lc ^ v_swz<D>(v_row, lc)) << 4);
                    const u32x2_t lo4 = lds_read_tr16(vb + coff);
                    const u32x2_t hi4 = lds_read_tr16(vb + 8 * S::ROWB + coff);
                    d[e] = u32x4_t{lo4[0], lo4[1], hi4[0], hi4[1]};
                }
            } else {
                const int t = m - kP;
#pragma unroll
                for (int mbk = 0; mbk < 2; ++mbk)
                    d[mbk] = *(const u32x4_t FCK_LDS*)(kt + mbk * 32 * S::ROWB + k_rd + (((t * 2 + half) ^ k_sw) << 4));
            }
        };
        auto mma = [&](int m, const u32x4_t (&d)[2]) __attribute__((always_inline)) {
            if (m < kP) {
                const int ks4 = m / (S::DVB / 2), pr = m % (S::DVB / 2);
                const vec8 pf = as_vec8<vec8>(pfrag[ks4]);
#pragma unroll
                for (int e = 0; e < 2; ++e) oacc[pr * 2 + e] = T::mfma32(as_vec8<vec8>(d[e]), pf, oacc[pr * 2 + e]);
            } else {
                const int t = m - kP;
                const vec8 qv = as_vec8<vec8>(qf[t]);
#pragma unroll
                for (int mbk = 0; mbk < 2; ++mbk) {
                    if (t == 0) {
                        f32x16_t z;
#pragma unroll
                        for (int j = 0; j < 16; ++j) z[j] = 0.f;
                        s[mbk] = T::mfma32(as_vec8<vec8>(d[mbk]), qv, z);
                    } else {
                        s[mbk] = T::mfma32(as_vec8<vec8>(d[mbk]), qv, s[mbk]);
                    }
                }
            }
        };
        fetch(0, bf[0]);
        if (kSteps > 1) fetch(1, bf[1]);
        // The wave in its matrix phase outranks the wave it shares the SIMD with (in its vector phase): at equal
        // priority the vector-phase wave always has an instruction ready and wins the issue slot, the matrix pipe
        // starves and the two phases run one after the other instead of side by side.
        __builtin_amdgcn_s_setprio(3);
#pragma unroll
        for (int m = 0; m < kSteps; ++m) {
            if (m + 2 < kSteps) fetch(m + 2, bf[(m + 2) % 3]);
            mma(m, bf[m % 3]);
            __builtin_amdgcn_sched_barrier(0);
        }
        __builtin_amdgcn_s_setprio(0);
    };

    // online softmax of local tile i: s -> pfrag
    auto softmax = [&](int i) __attribute__((always_inline)) {
        const int kb = (t_begin + i) * S::BN;
        const bool need_mask = (kb < w_lo_max) || (kb + S::BN > w_hi_min);
        if (need_mask) {
#pragma unroll
            for (int mbk = 0; mbk < S::NB; ++mbk)
#pragma unroll
                for (int j = 0; j < 16; ++j) {
                    const int key = kb + mbk * 32 + (j >> 2) * 8 + half * 4 + (j & 3);
                    const bool vis = key >= lo_r && key < hi_r;
                    s[mbk][j] = vis ? s[mbk][j] : -INFINITY;
                }
        }
        float tmax = -INFINITY;
#pragma unroll
        for (int mbk = 0; mbk < S::NB; ++mbk)
#pragma unroll
            for (int j = 0; j < 16; ++j) tmax = fmaxf(tmax, s[mbk][j]);
        tmax = pair32_max(tmax);
        tmax *= a.scale_log2;  // scale > 0: max commutes with the scaling
        // Lazy rescale: the reference m_run only moves when some row's maximum outgrows it by more than kLazy (log2
        // units).  Softmax is shift invariant, so a stale reference is exact; it bounds the exponentials by 2^kLazy.
        constexpr float kLazy = 8.f;
        if (__builtin_amdgcn_ballot_w64(tmax > m_run + kLazy) != 0) {
            const float m_new = fmaxf(m_run, tmax);
            const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
            const float alpha = fast_exp2(m_run - m_use);
            m_run = m_new;
            l_run *= alpha;
#pragma unroll
            for (int q = 0; q < S::DVB; ++q) oacc[q] *= alpha;
        }
        const float m_ref = (m_run == -INFINITY) ? 0.f : m_run;
        float psum = 0.f;
        // 8 scores at a time: exponentiate, add up, pack - the fp32 scores die as soon as their packed pair exists
#pragma unroll
        for (int ks4 = 0; ks4 < 2 * S::NB; ++ks4) {
            const int mbk = ks4 >> 1, j0 = (ks4 & 1) * 8;
            float p[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                p[e] = fast_exp2(__builtin_fmaf(s[mbk][j0 + e], a.scale_log2, -m_ref));
                psum += p[e];
            }
            pfrag[ks4][0] = T::pack2(p[0], p[1]);
            pfrag[ks4][1] = T::pack2(p[2], p[3]);
            pfrag[ks4][2] = T::pack2(p[4], p[5]);
            pfrag[ks4][3] = T::pack2(p[6], p[7]);
            __builtin_amdgcn_sched_barrier(0);
        }
        l_run += psum;
        // Pin the packed probabilities here: without a use before the barrier that ends this phase, the exponentials
        // are sunk past it into the matrix phase and the two wave groups stop overlapping.
#pragma unroll
        for (int ks4 = 0; ks4 < 2 * S::NB; ++ks4)
            asm volatile("" : "+v"(pfrag[ks4][0]), "+v"(pfrag[ks4][1]), "+v"(pfrag[ks4][2]), "+v"(pfrag[ks4][3]));
        asm volatile("" : "+v"(l_run));
    };


    // ---- epilogue of an item: normalise and store its rows -------------------------------------------------------
    auto finish = [&](const Item& it) __attribute__((always_inline)) {
        const float l_all = pair32_sum(l_run);
        if (row_ok) {
            const float inv = (l_all == 0.f) ? 0.f : 1.f / l_all;
            uint16_t* op = reinterpret_cast<uint16_t*>(a.o) + ((int64_t)(it.q_row0 + r) * a.hq + it.h) * D;
#pragma unroll
            for (int dvb = 0; dvb < S::DVB; ++dvb)
#pragma unroll
                for (int j4 = 0; j4 < 4; ++j4) {
                    u32x2_t out;
                    out[0] = T::pack2(oacc[dvb][j4 * 4 + 0] * inv, oacc[dvb][j4 * 4 + 1] * inv);
                    out[1] = T::pack2(oacc[dvb][j4 * 4 + 2] * inv, oacc[dvb][j4 * 4 + 3] * inv);
                    *reinterpret_cast<u32x2_t*>(op + dvb * 32 + j4 * 8 + half * 4) = out;
                }
        }
    };

    typedef std::integral_constant<int, 0> Keep0;
    typedef std::integral_constant<int, 2 * S::LD> KeepBatch;  // one batch = this wave's share of one K and one V tile

    // ---- the stream ----------------------------------------------------------------------------------------------
    Item A = load_item(0);
    fill_rows(A, 0);
    load_q(A, qf);
#pragma unroll
    for (int t = 0; t < S::KT; ++t) asm volatile("" : "+v"(qf[t]));  // landed before the loop: no wait for them inside it
    enter(A);
    __syncthreads();                  // item 0's first rows are in LDS
    if (group == 1) __syncthreads();  // skew: group 1 runs one barrier behind from here on
    RowCache kc = {0, -1, -1}, vc = {0, -1, -1};  // first-row caches of the K and the V request streams
    int pos = 0;                      // stream position of A's tile 0
    bool warm = false;                // A's first three K tiles and first two V tiles were requested by its predecessor
    for (int ii = 0; ii < my_count; ++ii) {
        const int cur = ii & 1, nxt = cur ^ 1;
        const bool has_next = ii + 1 < my_count;
        Item B = A;
        if (has_next) {
            // next item: description, first rows (read again no earlier than two barriers from here) and Q fragments
            B = load_item(ii + 1);
            if (kc.buf == nxt) kc.chunk = -1;  // that half of the row cache changes hands
            if (vc.buf == nxt) vc.chunk = -1;
            load_q(B, qnext);  // requested before the page-table reads below, so one wait covers both
            fill_rows(B, nxt);
#pragma unroll
            for (int t = 0; t < S::KT; ++t) asm volatile("" : "+v"(qnext[t]));  // have them landed here, not at the hand-off
        }
        const int n = A.n;
        const bool handoff = has_next && n >= 4 && B.n >= 3;
        // (item, tile, buffer of its first rows) a request for tile index `want` of the stream refers to
        auto issue = [&](const uint16_t* base, char FCK_LDS* ring, int want, RowCache& c, const int (&cp_c)[S::LD],
                         const uint32_t (&cp_off)[S::LD]) __attribute__((always_inline)) {
            if (want < n) {
                const int64_t row0 = tile_row0(A, cur, want, c);
                request(base, ring, (pos + want) & (kRing - 1), A, want, row0, cp_c, cp_off);
            } else if (handoff) {
                const int64_t row0 = tile_row0(B, nxt, want - n, c);
                request(base, ring, (pos + want) & (kRing - 1), B, want - n, row0, cp_c, cp_off);
            }
        };
        if (n > 0) {
            if (!warm) {
                issue(kp, k_ring, 0, kc, cp_k, cp_koff);
                issue(vp, v_ring, 0, vc, cp_v, cp_voff);
                issue(kp, k_ring, 1, kc, cp_k, cp_koff);
                issue(kp, k_ring, 2, kc, cp_k, cp_koff);
                issue(vp, v_ring, 1, vc, cp_v, cp_voff);
                if (n >= 3 || handoff)
                    wait_vm(KeepBatch{});
                else
                    wait_vm(Keep0{});
                __syncthreads();
                __syncthreads();  // second barrier: the other group, one barrier behind, has passed its wait too
                matrix(std::false_type{}, std::true_type{}, v_ring, k_ring + (pos & (kRing - 1)) * S::TILEB);
                __syncthreads();
            }
            for (int i = 0; i + 1 < n; ++i) {
                issue(kp, k_ring, i + 3, kc, cp_k, cp_koff);
                issue(vp, v_ring, i + 2, vc, cp_v, cp_voff);
                softmax(i);
                __syncthreads();
                matrix(std::true_type{}, std::true_type{}, v_ring + ((pos + i) & (kRing - 1)) * S::TILEB,
                       k_ring + ((pos + i + 1) & (kRing - 1)) * S::TILEB);
                if (handoff || i + 3 < n)
                    wait_vm(KeepBatch{});  // a full batch was requested in this iteration: it may stay in flight
                else
                    wait_vm(Keep0{});
                __syncthreads();
            }
            if (handoff) {
                issue(kp, k_ring, n + 2, kc, cp_k, cp_koff);
                issue(vp, v_ring, n + 1, vc, cp_v, cp_voff);
            }
            softmax(n - 1);
            __syncthreads();
            matrix(std::true_type{}, std::false_type{}, v_ring + ((pos + n - 1) & (kRing - 1)) * S::TILEB, k_ring);
        }
        finish(A);
        reset_acc();
        if (has_next) {
#pragma unroll
            for (int t = 0; t < S::KT; ++t) qf[t] = qnext[t];
            enter(B);
        }
        if (n > 0) {
            if (handoff) {
                matrix(std::false_type{}, std::true_type{}, v_ring, k_ring + ((pos + n) & (kRing - 1)) * S::TILEB);
                wait_vm(KeepBatch{});
            } else {
                wait_vm(Keep0{});
            }
            __syncthreads();
        } else {
            // an item without visible tiles: keep two barriers between writing the next item's first rows (above) and
            // reading them (its cold start), one for each group's share
            __syncthreads();
            __syncthreads();
        }
        pos += n;
        warm = handoff;
        A = B;
    }
    if (group == 0) __syncthreads();  // both groups pass the same number of barriers
}

template <typename T, int D>
static hipError_t launch_d(const PrefillArgs& a, int num_cu, hipStream_t st)
{
    const int nwx = num_cu / 8 > 0 ? num_cu / 8 : 1;
    const dim3 grid(8 * nwx);
    constexpr size_t lds = (size_t)2 * Shape<D>::RING * Shape<D>::TILEB + 2 * kPrefillStreamRowCache * 4 +
                           kPrefillStreamMaxItems * 4 + 64;
    return launch_with_lds<prefill_stream_kernel<T, D>>(grid, dim3(512), lds, st, a);
}

}  // namespace stream

bool prefill_stream_fits(const PrefillArgs& a, int num_cu)
{
    const int nwx = num_cu / 8 > 0 ? num_cu / 8 : 1;
    const int64_t g = a.hq / a.hk, gx = ((int64_t)a.batch * a.hk + 7) / 8;
    // a workgroup takes at most two of every 2 * nwx valid slots, plus two from the last partial round
    return g * gx * a.m_tiles / nwx + 2 <= kPrefillStreamMaxItems;
}

// `a.m_tiles` must count 256-row tiles; head dims 64 and 128; uniform pages (page size a multiple of the key tile).
hipError_t launch_prefill_stream(const PrefillArgs& a, int d, int dtype, int num_cu, hipStream_t st)
{
    if (!prefill_stream_fits(a, num_cu)) return hipErrorInvalidValue;
    if (d == 64) return dtype == 4 ? stream::launch_d<BF16, 64>(a, num_cu, st) : stream::launch_d<FP16, 64>(a, num_cu, st);
    if (d == 128) return dtype == 4 ? stream::launch_d<BF16, 128>(a, num_cu, st) : stream::launch_d<FP16, 128>(a, num_cu, st);
    return hipErrorInvalidValue;
}

}  // namespace fck
