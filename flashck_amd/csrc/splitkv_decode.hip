// Split-KV forward for short query lengths (decode): hand-written gfx950 kernel.
//
// Work decomposition
//   grid  = 1-D; workgroup id = head group + NG * (split + num_splits * (row tile + m_tiles * sequence)), so the head
//           groups that stream the same token rows are dispatched side by side.  A workgroup owns one split of HG
//           adjacent KV heads of one sequence and the 16*MB packed query rows (query index, head-in-group) of each.
//   waves = NW per workgroup, all independent: wave w walks the TK-key tiles w, w+NW, ... of the split for all HG heads
//           with its own online-softmax states; the NW partial states are merged through LDS at the end.
// Data path per tile (TK = 32 / HG keys), no workgroup barrier anywhere in the loop
//   K, V  global -> VGPR in whole HG*2*D-byte pieces of a token row (HG = 2 at head dim <= 128 reads 512 contiguous
//       bytes per token: HBM serves that access shape ~8 % faster than 256-byte pieces at a 2 KiB stride), then into
//       the wave's own XOR-swizzled LDS tile.  The registers form a rolling window: as soon as a register of tile i+1
//       has been written to LDS it becomes the destination of the matching load of tile i+2, so a wave always has a
//       full burst of loads outstanding and the memory queue never runs dry between tiles.  K is read back with
//       ds_read_b128 as the A operand of S^T = K . Q^T, V is read back transposed (ds_read_b64_tr_b16) as the A operand
//       of O^T += V^T . P^T;
//   S^T = K . Q^T with v_mfma_f32_16x16x32, so that each lane keeps the scores of one query row and the
//       probabilities it produces are already laid out as the B operand of the second product (v_mfma_f32_16x16x32
//       for 32-key tiles, v_mfma_f32_16x16x16 for 16-key tiles).
// Optional tail (fused entry point): the workgroup that is last to deliver its partial result for a (sequence, head
// group, row tile) - found with a device-scope ticket - merges the splits of those rows and writes the final output, so
// no second launch is needed.
#include "common.hpp"
#include "kernels.hpp"

#include <type_traits>

namespace fck {

template <int D, int HG>
struct DecodeShape {
    static constexpr int TK = 32 / HG;        // keys per wave tile
    static constexpr int NBK = TK / 16;       // 16-key blocks per tile
    static constexpr int LPR = D / 8;         // lanes that cover one head row with 16-byte pieces
    static constexpr int LPT = LPR * HG;      // lanes that cover the head group's piece of one token row
    static constexpr int KPI = 64 / LPT;      // token rows per load instruction
    static constexpr int VN = TK / KPI;       // load instructions per operand and tile
    static constexpr int KT = D / 32;         // MFMA k-steps of the QK product
    static constexpr int DB = D / 16;         // 16-column blocks of the output
    static constexpr int VROW = D * 2;        // bytes per staged head row
    static constexpr int HTILE = TK * VROW;   // staged bytes of one head's share of a tile
    static constexpr int TILE = HG * HTILE;   // staged bytes of one operand of a tile (32 * D * 2 for every HG)
    static constexpr int OSTRIDE = D + 4;     // floats per row of the merge buffer (bank spread)
    static_assert(LPT <= 64 && TK % KPI == 0, "a load instruction covers whole token-row pieces");
};

template <int D, int NW, int HG>
constexpr size_t decode_lds_bytes()
{
    typedef DecodeShape<D, HG> S;
    const size_t stage = (size_t)NW * 2 * S::TILE;
    const size_t merge = (size_t)NW * 16 * S::OSTRIDE * 4 + (size_t)NW * 2 * 16 * 4 + 16;
    return stage > merge ? stage : merge;
}

template <int LPR>
__device__ __forceinline__ int v_swizzle(int key)
{
    return ((key & 7) << 1) & (LPR - 1);
}

// kKv8: K and V are stored as fp8 (e4m3, one byte per element) and widened to T on their way into LDS; everything after
// the staging tile is the 16-bit path.  A lane then loads 8 bytes where the 16-bit path loads 16.
// a.q8 (instantiations with kMod and kKv8 only): the all-fp8 roles.  Q is e4m3 as well (widened to T like K and V: exact)
// and every probability is rounded to e4m3 before the second product (the row sum keeps the unrounded values).  The
// partial results stay fp32; the e4m3 output is written by the combine kernel.
// kPad: the stored head dims (a.d for Q/K, a.dv for V and the output; multiples of 8) are smaller than D: rows are
// a.d / a.dv elements apart, and the 16-byte pieces past a row's end are zeros instead of loads (a zero column of Q and K
// adds nothing to a score, a zero column of V gives an output column that is not stored).
// kChunk: the key ranges of the splits are chunks of a.split_chunk keys, the same for every sequence (split s of a
// sequence covers [s * chunk, (s + 1) * chunk), the last split also whatever lies beyond), instead of num_splits equal
// parts of each sequence: work items of equal size for a ragged batch; the splits a short sequence does not reach are
// empty.
template <typename T, int D, int NW, int MB, int HG, bool kUniformPage, bool kMod = false, bool kKv8 = false, bool kPad = false,
          bool kChunk = false>
__global__ __launch_bounds__(NW * 64) void splitkv_decode_kernel(const SplitKvArgs a)
{
    static_assert(!kPad || (HG == 1 && !kKv8), "padded head dims: one KV head per workgroup, 16-bit cache");
    const int dq = kPad ? a.d : D;   // elements per stored Q / K row
    const int dvs = kPad ? a.dv : D;  // elements per stored V / partial-output row
    typedef DecodeShape<D, HG> S;
    typedef typename T::vec8 vec8;
    FCK_DYNAMIC_LDS(smem);

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int l16 = lane & 15;
    const int kg = lane >> 4;

    const int ng = a.hk / HG;  // head groups
    int wg = blockIdx.x;
    const int hgrp = wg % ng;
    wg /= ng;
    const int split = wg % a.num_splits;
    wg /= a.num_splits;
    const int mtile = wg % a.m_tiles;
    int b = wg / a.m_tiles;
    if (a.longest_first) {
        // The grid holds more workgroups than the chip runs at once, and the hardware starts them in id order: the
        // ids are therefore dealt to the sequences longest first, so that the workgroups that start last are the short
        // ones (a ragged batch in its given order ends with whatever length comes last, on a chip that is half idle).
        // Lane j holds the key count of sequence j; a sequence's place is the number of sequences ahead of it.
        const int len_j = lane < a.batch ? kv_seq(a.kv, lane).len : -1;
        int place = 0;
        for (int i = 0; i < a.batch; ++i) {
            const int len_i = __builtin_amdgcn_readlane(len_j, i);
            place += (len_i > len_j || (len_i == len_j && i < lane)) ? 1 : 0;
        }
        const uint64_t hit = __ballot(lane < a.batch && place == b);  // exactly one lane
        b = __builtin_amdgcn_readfirstlane((int)__builtin_ctzll(hit));
    }
    const int hkv0 = hgrp * HG;
    const int g = a.hq / a.hk;

    // The first 256 entries of this sequence's block-table row, requested before anything else: lane l holds entries
    // 4l .. 4l+3.  The request does not depend on the key count, so it is in flight while that count is read, and a
    // tile's page id is then a register read instead of a load in the chain that leads to the first K/V request.
    u32x4_t tbl_vec = {0u, 0u, 0u, 0u};
    int tbl_cached = 0;  // entries held in tbl_vec
    if constexpr (kUniformPage) {
        if (a.kv.mode == 2 && (a.kv.block_table_stride & 3) == 0) {
            tbl_cached = min(a.kv.block_table_stride, 256);
            if (lane * 4 < tbl_cached) tbl_vec = ldg16(a.kv.block_table + (int64_t)b * a.kv.block_table_stride + lane * 4);
        }
    }

    // ---- per-sequence geometry (uniform) -------------------------------------------------------------
    int q_row0, sq_b;
    if (a.seqstart_q) {
        q_row0 = a.seqstart_q[b];
        sq_b = a.seqstart_q[b + 1] - q_row0;
    } else {
        q_row0 = b * a.sq;
        sq_b = a.sq;
    }
    const KvSeq ks = kv_seq(a.kv, b);
    const int sk_b = ks.len;
    const int R = sq_b * g;  // packed rows of one (sequence, kv head)
    const int r_tile0 = mtile * 16 * MB;
    if (r_tile0 >= R) return;

    // Split geometry: num_splits equal ranges of ceil(sk / num_splits) keys (the last ones may be empty)
    const int per = kChunk ? a.split_chunk : max(1, (sk_b + a.num_splits - 1) / a.num_splits);
    const int n_active = a.num_splits;
    const int k0 = (int)min((int64_t)per * split, (int64_t)sk_b);
    const int k1 = (kChunk && split == a.num_splits - 1) ? sk_b : min(k0 + per, sk_b);

    const MaskYX mk = make_mask(a.mask_type, a.window_left, a.window_right, sq_b, sk_b);

    // rows of this lane (one per 16-row block); the HG heads of the group share them
    int row_i[MB], row_hl[MB], lo[MB], hi[MB];
    bool row_ok[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        const int r = r_tile0 + mb * 16 + l16;
        row_ok[mb] = r < R;
        const int rc = row_ok[mb] ? r : 0;
        row_i[mb] = rc / g;
        row_hl[mb] = rc % g;
        lo[mb] = max(mask_lo(mk, row_i[mb]), k0);
        hi[mb] = min(mask_hi(mk, row_i[mb], sk_b), k1);
        if (!row_ok[mb]) {
            lo[mb] = 0;
            hi[mb] = 0;
        }
    }
    // bias / ALiBi / soft cap of this lane's rows
    RowMod<T> rmod[HG][MB];  // per head of the group: slopes and bias rows differ between heads
    if constexpr (kMod) {
#pragma unroll
        for (int hl = 0; hl < HG; ++hl)
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
                rmod[hl][mb].init(a.mod, b, q_row0, (hkv0 + hl) * g + row_hl[mb], row_i[mb], sq_b, sk_b, a.mask_type, a.window_left,
                                  a.window_right, a.seqstart_q != nullptr);
    }
    // key range any row of the tile can see (uniform)
    const int i_first = r_tile0 / g;
    const int i_last = (min(r_tile0 + 16 * MB, R) - 1) / g;
    const int vis_lo = max(mask_lo(mk, i_first), k0);
    const int vis_hi = min(mask_hi(mk, i_last, sk_b), k1);

    const int Sq = (int)a.shape_sq;
    const int wb = a.seqstart_q ? 0 : b;
    const int wrow0 = a.seqstart_q ? q_row0 : 0;

    const int t_begin = vis_lo / S::TK;
    const int t_end = (vis_hi + S::TK - 1) / S::TK;

    // ---- Q as the B operand: lane (row = l16, k-group = kg) holds 8 consecutive head-dim elements per k-step -----
    vec8 qf[HG][MB][S::KT];
    {
        const uint16_t* qp = reinterpret_cast<const uint16_t*>(a.q);
#pragma unroll
        for (int hl = 0; hl < HG; ++hl)
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) {
                const int64_t off = ((int64_t)(q_row0 + row_i[mb]) * a.hq + (hkv0 + hl) * g + row_hl[mb]) * dq + kg * 8;
                if constexpr (kMod && kKv8) {
                    if (a.q8) {  // one byte per element
                        const uint8_t* qp8 = reinterpret_cast<const uint8_t*>(a.q) + off;
#pragma unroll
                        for (int t = 0; t < S::KT; ++t) {
                            u32x2_t v = {0u, 0u};
                            if (row_ok[mb]) v = *reinterpret_cast<const u32x2_t*>(qp8 + t * 32);
                            qf[hl][mb][t] = as_vec8<vec8>(fp8x8_to_t<T>(u32x4_t{v[0], v[1], 0u, 0u}));
                        }
                        continue;
                    }
                }
#pragma unroll
                for (int t = 0; t < S::KT; ++t) {
                    u32x4_t v = {0u, 0u, 0u, 0u};
                    if (row_ok[mb] && (!kPad || t * 32 + kg * 8 < dq)) v = ldg16(qp + off + t * 32);
                    qf[hl][mb][t] = as_vec8<vec8>(v);
                }
            }
    }

    // ---- online softmax state ------------------------------------------------------------------------------
    float m_run[HG][MB], l_run[HG][MB];
    f32x4_t oacc[HG][MB][S::DB];
#pragma unroll
    for (int hl = 0; hl < HG; ++hl)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            m_run[hl][mb] = -INFINITY;
            l_run[hl][mb] = 0.f;
#pragma unroll
            for (int db = 0; db < S::DB; ++db) oacc[hl][mb][db] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
        }

    typedef typename std::conditional<kKv8, uint8_t, uint16_t>::type kv_elem;
    const kv_elem* kp = reinterpret_cast<const kv_elem*>(a.k);
    const kv_elem* vp = reinterpret_cast<const kv_elem*>(a.v);
    // one lane's piece of a K/V row: 8 elements, as they come from memory and as they go to LDS
    auto fetch = [](const kv_elem* p) -> u32x4_t {
        if constexpr (kKv8) {
            const u32x2_t v = ldg8_stream(p);
            return u32x4_t{v[0], v[1], 0u, 0u};
        } else {
            return ldg16_stream(p);
        }
    };
    auto staged = [](u32x4_t v) -> u32x4_t {
        if constexpr (kKv8) {
            const f32x2_t a0 = __builtin_amdgcn_cvt_pk_f32_fp8((int)v[0], false), a1 = __builtin_amdgcn_cvt_pk_f32_fp8((int)v[0], true);
            const f32x2_t a2 = __builtin_amdgcn_cvt_pk_f32_fp8((int)v[1], false), a3 = __builtin_amdgcn_cvt_pk_f32_fp8((int)v[1], true);
            return u32x4_t{T::pack2(a0[0], a0[1]), T::pack2(a1[0], a1[1]), T::pack2(a2[0], a2[1]), T::pack2(a3[0], a3[1])};
        } else {
            return v;
        }
    };
    const int last_key = sk_b - 1;

    // ---- this wave's staging tiles and its lanes' places in them -----------------------------------------------------
    char FCK_LDS* kstage = (char FCK_LDS*)(smem) + wave * 2 * S::TILE;
    char FCK_LDS* vstage = kstage + S::TILE;
    // load instruction u of an operand: token row u * KPI + lane / LPT of the tile, piece lane % LPT of the group's
    // HG * 2 * D bytes = (head lane % LPT / LPR, 16-byte chunk lane % LPR)
    const int ld_key = lane / S::LPT;
    const int ld_piece = lane % S::LPT;
    int vw_off[S::VN], kw_off[S::VN];
#pragma unroll
    for (int u = 0; u < S::VN; ++u) {
        const int key = u * S::KPI + ld_key;
        const int hl = ld_piece / S::LPR;
        const int chunk = ld_piece % S::LPR;
        vw_off[u] = (hl * S::TK + key) * S::VROW + ((chunk ^ v_swizzle<S::LPR>(key)) << 4);
        kw_off[u] = (hl * S::TK + key) * S::VROW + ((chunk ^ (key & 7)) << 4);
    }
    // K as the A operand: lane (key = nb * 16 + l16, k-group kg) reads chunk t * 4 + kg of its key row
    const int kr_off = l16 * S::VROW;
    const int kr_sw = l16 & 7;
    const int tr_key = kg * 4 + (l16 >> 2);
    const int tr_sw = v_swizzle<S::LPR>(tr_key);
    const int tr_base = tr_key * S::VROW + ((l16 & 2) << 3) + ((l16 & 1) << 3);

    const int n_tiles = t_end - t_begin;  // tiles of the workgroup (may be <= 0)

    // registers of the rolling window: VN loads of K, then VN loads of V
    struct Frag {
        u32x4_t a[2 * S::VN];
    };

    // Tile order: wave w takes tiles w, w + NW, ...
    int next_tile = wave;
    auto claim = [&]() -> int {
        const int c = next_tile;
        next_tile += NW;
        return c;
    };
    auto page_index = [&](int key) { return a.kv.page_shift >= 0 ? key >> a.kv.page_shift : key / a.kv.page_size; };
    // First cache row of tile c on the uniform-page path.  The page id is a scalar load through the constant address
    // space (the table is an input, never written here): it waits on its own counter, so asking for it one tile ahead
    // does not disturb the window of vector loads.
    auto tile_row0 = [&](int c) -> int64_t {
        const int kb = (t_begin + min(c, max(n_tiles - 1, 0))) * S::TK;
        if (ks.table != nullptr) {
            const int pi = page_index(kb);
            int page;
            if (pi < tbl_cached) {
                const uint32_t e0 = __builtin_amdgcn_readlane(tbl_vec[0], pi >> 2), e1 = __builtin_amdgcn_readlane(tbl_vec[1], pi >> 2);
                const uint32_t e2 = __builtin_amdgcn_readlane(tbl_vec[2], pi >> 2), e3 = __builtin_amdgcn_readlane(tbl_vec[3], pi >> 2);
                page = (int)((pi & 2) ? ((pi & 1) ? e3 : e2) : ((pi & 1) ? e1 : e0));
            } else {
                page = const_load(ks.table, pi);
            }
            return (int64_t)page * a.kv.page_size + (kb - pi * a.kv.page_size);
        }
        return ks.base_row + kb;
    };
    // global offset (in elements) of this lane's piece for load instruction u of tile c (first cache row row0)
    // (dim: elements per stored row of the operand, dq for K and dvs for V)
    auto src_off = [&](int c, int u, int64_t row0, int dim) -> int64_t {
        const int kb = (t_begin + c) * S::TK;
        if constexpr (kUniformPage) {
            // the whole tile lies in one page (or the cache is contiguous): one row base per tile;
            // rows past the last key repeat it (their scores are masked)
            const int kl = min(u * S::KPI + ld_key, last_key - kb);
            return ((row0 + kl) * a.hk + hkv0) * dim + ld_piece * 8;
        } else {
            const int key = min(kb + u * S::KPI + ld_key, last_key);
            return (kv_row(a.kv, ks, key) * a.hk + hkv0) * dim + ld_piece * 8;
        }
    };
    const bool k_piece = !kPad || ld_piece * 8 < dq, v_piece = !kPad || ld_piece * 8 < dvs;  // this lane's piece exists
    auto fetch_k = [&](int c, int u, int64_t row0) -> u32x4_t {
        if constexpr (kPad) {
            if (!k_piece) return u32x4_t{0u, 0u, 0u, 0u};
        }
        return fetch(kp + src_off(c, u, row0, dq));
    };
    auto fetch_v = [&](int c, int u, int64_t row0) -> u32x4_t {
        if constexpr (kPad) {
            if (!v_piece) return u32x4_t{0u, 0u, 0u, 0u};
        }
        return fetch(vp + src_off(c, u, row0, dvs));
    };
    auto load_tile = [&](int c, int64_t row0, Frag& f) {
#pragma unroll
        for (int u = 0; u < S::VN; ++u) f.a[u] = fetch_k(c, u, row0);
#pragma unroll
        for (int u = 0; u < S::VN; ++u) f.a[S::VN + u] = fetch_v(c, u, row0);
    };
    auto store_tile = [&](const Frag& f) {
#pragma unroll
        for (int u = 0; u < S::VN; ++u) *(u32x4_t FCK_LDS*)(kstage + kw_off[u]) = staged(f.a[u]);
#pragma unroll
        for (int u = 0; u < S::VN; ++u) *(u32x4_t FCK_LDS*)(vstage + vw_off[u]) = staged(f.a[S::VN + u]);
    };
    // write the tile held in f to LDS and request tile c_next into the same registers, one register at a time
    auto refill_tile = [&](int c_next, int64_t row0, Frag& f) {
#pragma unroll
        for (int u = 0; u < S::VN; ++u) {
            *(u32x4_t FCK_LDS*)(kstage + kw_off[u]) = staged(f.a[u]);
            f.a[u] = fetch_k(c_next, u, row0);
            __builtin_amdgcn_sched_barrier(0);  // keep the store / load pairs interleaved in this order
        }
#pragma unroll
        for (int u = 0; u < S::VN; ++u) {
            *(u32x4_t FCK_LDS*)(vstage + vw_off[u]) = staged(f.a[S::VN + u]);
            f.a[S::VN + u] = fetch_v(c_next, u, row0);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    auto compute_tile = [&](int c) {
        const int kb = (t_begin + c) * S::TK;
        FCK_WAVE_LDS_ORDER();  // the staging tile was written by all lanes of this wave; the reads below come after
#pragma unroll
        for (int hl = 0; hl < HG; ++hl) {
            const char FCK_LDS* kh = kstage + hl * S::HTILE;
            const char FCK_LDS* vh = vstage + hl * S::HTILE;
            // S^T[key][row] = K . Q^T
            u32x4_t kfrag[S::NBK][S::KT];
#pragma unroll
            for (int nb = 0; nb < S::NBK; ++nb)
#pragma unroll
                for (int t = 0; t < S::KT; ++t)
                    kfrag[nb][t] = *(const u32x4_t FCK_LDS*)(kh + nb * 16 * S::VROW + kr_off + (((t * 4 + kg) ^ kr_sw) << 4));
            f32x4_t s[MB][S::NBK];
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int nb = 0; nb < S::NBK; ++nb) {
                    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int t = 0; t < S::KT; ++t) acc = T::mfma16(as_vec8<vec8>(kfrag[nb][t]), qf[hl][mb][t], acc);
                    s[mb][nb] = acc;
                }

            uint32_t pk[MB][2 * S::NBK];  // probabilities, two per register: keys nb * 16 + kg * 4 + (0..3)
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) {
                float x[4 * S::NBK];
                float tmax = -INFINITY;
#pragma unroll
                for (int nb = 0; nb < S::NBK; ++nb)
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const int key = kb + nb * 16 + kg * 4 + j;
                        const bool vis = key >= lo[mb] && key < hi[mb];
                        float v;
                        if constexpr (kMod)
                            v = vis ? rmod[hl][mb].score(s[mb][nb][j], key) : -INFINITY;
                        else
                            v = vis ? s[mb][nb][j] * a.scale_log2 : -INFINITY;
                        x[nb * 4 + j] = v;
                        tmax = fmaxf(tmax, v);
                    }
                tmax = quad16_max(tmax);
                const float m_new = fmaxf(m_run[hl][mb], tmax);
                const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
                const float alpha = fast_exp2(m_run[hl][mb] - m_use);
                m_run[hl][mb] = m_new;
                float psum = 0.f;
                float p[4 * S::NBK];
#pragma unroll
                for (int e = 0; e < 4 * S::NBK; ++e) {
                    p[e] = fast_exp2(x[e] - m_use);
                    psum += p[e];
                }
                l_run[hl][mb] = l_run[hl][mb] * alpha + psum;
                if constexpr (kMod && kKv8) {
                    if (a.q8) {  // 0 <= p <= 1: the conversion never saturates
#pragma unroll
                        for (int e = 0; e < 4 * S::NBK; e += 2) {
                            const f32x2_t p8 = round_to_fp8(p[e], p[e + 1]);
                            p[e] = p8[0];
                            p[e + 1] = p8[1];
                        }
                    }
                }
#pragma unroll
                for (int db = 0; db < S::DB; ++db) oacc[hl][mb][db] *= alpha;
#pragma unroll
                for (int e = 0; e < 2 * S::NBK; ++e) pk[mb][e] = T::pack2(p[2 * e], p[2 * e + 1]);
            }

            // O^T[dv][row] += V^T . P^T
#pragma unroll
            for (int db = 0; db < S::DB; ++db) {
                const int coff = tr_base + ((((db * 2) ^ tr_sw)) << 4);
                const u32x2_t lo4 = lds_read_tr16(vh + coff);
                if constexpr (S::NBK == 2) {
                    const u32x2_t hi4 = lds_read_tr16(vh + coff + 16 * S::VROW);
                    const u32x4_t av = {lo4[0], lo4[1], hi4[0], hi4[1]};
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb) {
                        const u32x4_t pv = {pk[mb][0], pk[mb][1], pk[mb][2], pk[mb][3]};
                        oacc[hl][mb][db] = T::mfma16(as_vec8<vec8>(av), as_vec8<vec8>(pv), oacc[hl][mb][db]);
                    }
                } else {
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb) {
                        const u32x2_t pv = {pk[mb][0], pk[mb][1]};
                        oacc[hl][mb][db] = T::mfma16k16(lo4, pv, oacc[hl][mb][db]);
                    }
                }
            }
        }
    };

    // Software pipeline over the tiles this wave claims.  Tile c0 sits in the wave's LDS tiles while tile c1 is in flight
    // in the rolling window; c2 is claimed and its first row looked up one iteration before it is requested.  LDS
    // operations of one wave execute in order, so the wave's own reads of a tile are done before its writes of the
    // next one land and no barrier is needed.
    {
        int c0 = claim();
        int c1 = claim();
        if (c0 < n_tiles) {
            Frag f;
            int64_t r1 = 0;
            if constexpr (kUniformPage) {
                const int64_t r0 = tile_row0(c0);
                r1 = tile_row0(c1);
                load_tile(c0, r0, f);
            } else {
                load_tile(c0, 0, f);
            }
            int c2 = claim();
            while (c1 < n_tiles) {
                int64_t r2 = 0;
                if constexpr (kUniformPage) r2 = tile_row0(c2);
                const int c3 = claim();
                refill_tile(c1, r1, f);  // c0 -> LDS, c1 -> window
                compute_tile(c0);
                c0 = c1;
                c1 = c2;
                c2 = c3;
                r1 = r2;
            }
            store_tile(f);
            compute_tile(c0);
        }
    }

    // ---- merge the NW partial states --------------------------------------------------------------------------
    // each lane owns a partial row sum over its key slots per tile: fold the 4 lanes of a row
#pragma unroll
    for (int hl = 0; hl < HG; ++hl)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) l_run[hl][mb] = quad16_sum(l_run[hl][mb]);

    float* obuf = reinterpret_cast<float*>(smem);                       // [NW][16][OSTRIDE]
    float* mlbuf = obuf + NW * 16 * S::OSTRIDE;                         // [NW][2][16]
    constexpr int NT = NW * 64;
    float* o_acc = a.o_acc;
    float* lse_acc = a.lse_acc;

#pragma unroll
    for (int hl = 0; hl < HG; ++hl)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            __syncthreads();  // staging tiles (or the previous block's merge data) are no longer read
            float* ow = obuf + (wave * 16 + l16) * S::OSTRIDE + kg * 4;
#pragma unroll
            for (int db = 0; db < S::DB; ++db) *reinterpret_cast<f32x4_t*>(ow + db * 16) = oacc[hl][mb][db];
            if (kg == 0) {
                mlbuf[(wave * 2 + 0) * 16 + l16] = m_run[hl][mb];
                mlbuf[(wave * 2 + 1) * 16 + l16] = l_run[hl][mb];
            }
            __syncthreads();
            for (int e = threadIdx.x; e < 16 * D; e += NT) {
                const int rr = e / D, c = e % D;
                const int r = r_tile0 + mb * 16 + rr;
                if (r >= R) continue;
                if constexpr (kPad) {
                    if (c >= dvs) continue;
                }
                float mmax = -INFINITY;
#pragma unroll
                for (int w = 0; w < NW; ++w) mmax = fmaxf(mmax, mlbuf[(w * 2 + 0) * 16 + rr]);
                const float muse = (mmax == -INFINITY) ? 0.f : mmax;
                float L = 0.f, acc = 0.f;
#pragma unroll
                for (int w = 0; w < NW; ++w) {
                    const float sc = fast_exp2(mlbuf[(w * 2 + 0) * 16 + rr] - muse);
                    L += mlbuf[(w * 2 + 1) * 16 + rr] * sc;
                    acc += obuf[(w * 16 + rr) * S::OSTRIDE + c] * sc;
                }
                const int i = r / g, h = (hkv0 + hl) * g + r % g;
                const int64_t wofs = ((int64_t)(wb * a.hq + h) * a.num_splits + split) * Sq + wrow0 + i;
                o_acc[wofs * dvs + c] = (L == 0.f) ? 0.f : acc / L * a.v_descale;
                if (c == 0) lse_acc[wofs] = (L == 0.f) ? -INFINITY : (mmax + fast_log2(L)) * kLn2;
            }
        }

    // ---- optional tail: the last workgroup to arrive for these rows merges their splits ----------------------------
    if (a.tickets == nullptr) return;
    // Publishing protocol.  Device-scope cache maintenance is expensive on this chip (every XCD has its own L2), so it
    // is done by one thread per workgroup: the barrier orders every thread's partial results before thread 0, whose
    // release fence makes them visible device-wide before it takes the ticket; only the last workgroup to arrive runs
    // the matching acquire fence before the barrier behind which its threads read the other workgroups' results.
    __syncthreads();
    uint32_t* flag = reinterpret_cast<uint32_t*>(mlbuf + NW * 2 * 16);
    uint32_t* ticket = a.tickets + ((int64_t)b * ng + hgrp) * a.m_tiles + mtile;
    if (threadIdx.x == 0) {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
        const uint32_t arrived = __hip_atomic_fetch_add(ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (arrived == (uint32_t)(n_active - 1)) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
        *flag = arrived;
    }
    __syncthreads();
    if (*flag != (uint32_t)(n_active - 1)) return;
    {
        constexpr int TPR = D / 4;  // threads per output row
        const int rows_here = min(16 * MB, R - r_tile0);
        const int items = HG * rows_here * TPR;
        for (int e = threadIdx.x; e < items; e += NT) {
            const int c = (e % TPR) * 4;
            const int rr = (e / TPR) % rows_here;
            const int hl = e / (TPR * rows_here);
            const int r = r_tile0 + rr;
            const int i = r / g, h = (hkv0 + hl) * g + r % g;
            const int64_t w0 = ((int64_t)(wb * a.hq + h) * a.num_splits) * Sq + wrow0 + i;  // split 0; next split is Sq further
            const f32x4_t acc = combine_splits<D>(lse_acc, o_acc, w0, Sq, n_active, c);
            u32x2_t out;
            out[0] = T::pack2(acc[0], acc[1]);
            out[1] = T::pack2(acc[2], acc[3]);
            *reinterpret_cast<u32x2_t*>(reinterpret_cast<uint16_t*>(a.o) + ((int64_t)(q_row0 + i) * a.hq + h) * D + c) = out;
        }
    }
    if (threadIdx.x == 0) *ticket = 0u;  // left clean for the next launch
}

// ------------------------------------------------------------------------------------------------------
// Workspace of the fused entry point.  In host code the array's name is only a handle: its device address is looked up
// per device with hipGetSymbolAddress, and only that address is ever handed to a kernel.
static __device__ __align__(256) float g_decode_scratch[kDecodeScratchFloats];

hipError_t decode_scratch(float** ptr)
{
    constexpr int kMaxDev = 64;
    static std::once_flag once[kMaxDev];
    static hipError_t status[kMaxDev];
    static float* addr[kMaxDev];
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= kMaxDev) return hipErrorInvalidDevice;
    std::call_once(once[dev], [&] {
        void* p = nullptr;
        status[dev] = hipGetSymbolAddress(&p, HIP_SYMBOL(g_decode_scratch));
        addr[dev] = static_cast<float*>(p);
    });
    *ptr = addr[dev];
    return status[dev];
}

template <typename T, int D, int NW, int MB, int HG>
static hipError_t launch_cfg(const SplitKvArgs& a, bool uniform, hipStream_t st)
{
    const dim3 grid((unsigned)((int64_t)(a.hk / HG) * a.num_splits * a.m_tiles * a.batch));
    const dim3 block(NW * 64);
    constexpr size_t lds = decode_lds_bytes<D, NW, HG>();
    if (a.q8 && (!a.kv8 || a.tickets || a.d != D || a.dv != D)) return hipErrorInvalidValue;  // refused by the caller
    if constexpr (HG == 1) {
        if (a.d != D || a.dv != D) {  // padded head dims: the general kernel (modifiers on, identity when there are none)
            if (a.kv8 || a.tickets) return hipErrorInvalidValue;  // refused by the caller
            if (uniform) return launch_with_lds<splitkv_decode_kernel<T, D, NW, MB, HG, true, true, false, true>>(grid, block, lds, st, a);
            return launch_with_lds<splitkv_decode_kernel<T, D, NW, MB, HG, false, true, false, true>>(grid, block, lds, st, a);
        }
    }
    if (a.mod.active() || a.q8) {  // q8 (all-fp8 roles) lives in the general fp8 kernels only
        if (a.kv8) {
            if (uniform) return launch_with_lds<splitkv_decode_kernel<T, D, NW, MB, HG, true, true, true>>(grid, block, lds, st, a);
            return launch_with_lds<splitkv_decode_kernel<T, D, NW, MB, HG, false, true, true>>(grid, block, lds, st, a);
        }
        if (uniform) return launch_with_lds<splitkv_decode_kernel<T, D, NW, MB, HG, true, true>>(grid, block, lds, st, a);
        return launch_with_lds<splitkv_decode_kernel<T, D, NW, MB, HG, false, true>>(grid, block, lds, st, a);
    }
    if (a.kv8) {
        if (uniform) return launch_with_lds<splitkv_decode_kernel<T, D, NW, MB, HG, true, false, true>>(grid, block, lds, st, a);
        return launch_with_lds<splitkv_decode_kernel<T, D, NW, MB, HG, false, false, true>>(grid, block, lds, st, a);
    }
    if (a.split_chunk > 0) {  // validated by the caller: plain call, uniform pages, one 16-row block, head dim 64 or 128
        if constexpr (NW == 8 && MB == 1 && D <= 128) {
            if (!uniform || a.tickets) return hipErrorInvalidValue;
            return launch_with_lds<splitkv_decode_kernel<T, D, NW, MB, HG, true, false, false, false, true>>(grid, block, lds, st, a);
        } else {
            return hipErrorInvalidValue;
        }
    }
    if (uniform) return launch_with_lds<splitkv_decode_kernel<T, D, NW, MB, HG, true>>(grid, block, lds, st, a);
    return launch_with_lds<splitkv_decode_kernel<T, D, NW, MB, HG, false>>(grid, block, lds, st, a);
}

// Head pairs (HG = 2) stream HBM faster, but halve the number of workgroups: they are used when the grid still
// covers the CUs.
static bool use_head_pairs(const SplitKvArgs& a, int m_tiles, int num_cu)
{
    if (a.variant != 0) return a.variant == 2 || a.variant == 4;  // validated by the caller
    if (a.hk % 2 || a.d != a.dv || (a.d != 64 && a.d != 128)) return false;
    return (int64_t)(a.hk / 2) * a.num_splits * m_tiles * a.batch >= num_cu;
}

template <typename T, int D>
static hipError_t launch_mb(SplitKvArgs a, int rows_max, bool uniform, int num_cu, hipStream_t st, int* heads_per_workgroup)
{
    *heads_per_workgroup = 1;
    // 8 waves (2 per SIMD, 256 VGPRs each) when one 16-row block is enough; 4 waves (512 VGPRs) when a lane carries
    // the accumulators of several row blocks or of a 256-wide head.
    a.m_tiles = splitkv_decode_m_tiles(D, rows_max);
    // Between one and two workgroups per CU (one workgroup fills a CU's LDS) the start order matters, see the kernel:
    // the short sequences then fill in behind the first workgroups to finish (ragged batch of 32, 384 workgroups:
    // 63.8 us against 69.3 us in the given order).  With more rounds than two, longest first ends in a train of small
    // workgroups that are all start-up and merge, and the given order, which mixes them with long ones, is faster.
    auto set_order = [&](int hg) {
        const int64_t wgs = (int64_t)(a.hk / hg) * a.num_splits * a.m_tiles * a.batch;
        a.longest_first = a.batch > 1 && a.batch <= 64 && wgs > num_cu && wgs <= 2 * (int64_t)num_cu;
    };
    set_order(1);
    if constexpr (D == 256) {
        if (rows_max <= 16) return launch_cfg<T, D, 4, 1, 1>(a, uniform, st);
        return launch_cfg<T, D, 4, 2, 1>(a, uniform, st);
    } else {
        if (rows_max <= 16) {
            if (use_head_pairs(a, 1, num_cu)) {
                set_order(2);
                *heads_per_workgroup = 2;
                return launch_cfg<T, D, 8, 1, 2>(a, uniform, st);
            }
            return launch_cfg<T, D, 8, 1, 1>(a, uniform, st);
        }
        if (rows_max <= 32) return launch_cfg<T, D, 4, 2, 1>(a, uniform, st);
        return launch_cfg<T, D, 4, 4, 1>(a, uniform, st);
    }
}

template <typename T>
static hipError_t launch_d(const SplitKvArgs& a, int d, int rows_max, bool uniform, int num_cu, hipStream_t st, int* hpw)
{
    switch (d) {
    case 64: return launch_mb<T, 64>(a, rows_max, uniform, num_cu, st, hpw);
    case 128: return launch_mb<T, 128>(a, rows_max, uniform, num_cu, st, hpw);
    case 256: return launch_mb<T, 256>(a, rows_max, uniform, num_cu, st, hpw);
    }
    return hipErrorInvalidValue;
}

int splitkv_decode_m_tiles(int d, int rows_max)
{
    if (d == 256) return rows_max <= 16 ? 1 : (rows_max + 31) / 32;
    return rows_max <= 32 ? 1 : (rows_max + 63) / 64;
}

hipError_t launch_splitkv_decode(const SplitKvArgs& a, int d, int dtype, int rows_max, bool uniform_page, int num_cu,
                                 hipStream_t st, int* heads_per_workgroup)
{
    int hpw = 1;
    const hipError_t e = dtype == 4 ? launch_d<BF16>(a, d, rows_max, uniform_page, num_cu, st, &hpw)
                                    : launch_d<FP16>(a, d, rows_max, uniform_page, num_cu, st, &hpw);
    if (heads_per_workgroup) *heads_per_workgroup = hpw;
    return e;
}

}  // namespace fck
