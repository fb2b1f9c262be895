// Forward attention for long query runs, ping-pong variant (gfx950): two groups of four waves share the SIMDs of a CU
// and are kept half an iteration apart, so that while one group feeds the matrix cores the other runs its softmax on
// the vector ALUs.
//
// Work decomposition
//   grid  = 1-D, XCD-aware order; a workgroup of 8 waves owns 256 query rows of one head: group g = wave / 4 owns rows
//           [g*128, g*128+128), 32 rows per wave.  Waves w and w+4 sit on the same SIMD.
// Phases (one workgroup barrier after each); tile i = the i-th key tile of the visible range
//   matrix phase  M(i) = { O^T += V^T.P^T of tile i ; S^T = K.Q^T of tile i+1 }
//   vector phase  V(i) = { online softmax of tile i: S -> P }
//   group 0 runs M(i) in phase 2i+2 and V(i) in phase 2i+1; group 1 runs the same instruction stream one phase later
//   (it passes one extra barrier before its first matrix phase, group 0 one extra after its last), so every phase pairs
//   one M with one V on each SIMD and no branch inside the loop depends on the group.
// Data path
//   K, V tiles: global -> LDS directly (global_load_lds_dwordx4, 1 KiB per wave instruction), rings of kRing buffers
//   each; the XOR swizzle of the staged tile is applied on the global side (lane l of an instruction always lands at
//   LDS byte l*16 of its block, so it fetches the chunk that belongs there).  In M(i) every wave requests its share of
//   K_{i+3} and V_{i+2} into the buffers M(i-1) was the last to read, and before the barrier that ends M(i) it waits
//   until its share of K_{i+2} and V_{i+1} has landed.  No register is a load destination, so nothing the compiler
//   schedules can wait on these loads by accident.  K is read with ds_read_b128 as the A operand of
//   v_mfma_f32_32x32x16, V with the transposing ds_read_b64_tr_b16, both two MFMA pairs ahead of their use; Q stays in
//   registers; P never leaves registers because the accumulator layout of the first product is the B-operand layout of
//   the second.
#include "common.hpp"
#include "kernels.hpp"
#include "lds_tiles.hpp"

#include <type_traits>

namespace fck {

template <int D, int BN_>
struct PPShape {
    static constexpr int BM = 256;
    static constexpr int BN = BN_;
    static constexpr int NB = BN_ / 32;  // 32-key blocks per tile
    static constexpr int KT = D / 16;   // k-steps of the QK product
    static constexpr int DVB = D / 32;  // 32-column blocks of the output
    static constexpr int ROWB = D * 2;  // bytes per staged row
    static constexpr int CH = D / 8;    // 16-byte chunks per row
    static constexpr int TILEB = BN * ROWB;
    static constexpr int LD = TILEB / 1024 / 8;  // 1 KiB global->LDS instructions per wave and tile
    static constexpr int RING = 4;               // LDS buffers per operand (a power of two)
    static_assert(TILEB % 8192 == 0, "a tile is split evenly over the 8 waves");
};

using tiles::k_swz;
using tiles::v_swz;

// kMod: ALiBi and / or the logits soft cap are applied to every score in the vector phase (ArithMod; an elementwise
// bias needs a load per score and stays with the register-staged kernel).
// kVar: tile variants a tuner can choose between (fck_fmha_attrs.prefill_variant - 1; 0 is the default schedule):
//   bit 0  requests of a tile whose 64 rows all exist use byte offsets computed once per workgroup (no clamp and no
//          multiply per request; the scalar base carries the tile)
//   bit 1  the per-lane maximum of a tile's raw scores is taken at the end of the matrix phase that produced them,
//          which shortens the (longer) vector phase by that much; tiles that need masking take it again after the mask
// kPad: the stored head dims (a.d for Q / K, a.dv for V / O; multiples of 8) are smaller than D.  Rows are a.d / a.dv
//   elements apart in memory; a lane whose 16-byte piece lies past a row's end requests nothing, and the LDS bytes it
//   would have filled are zeroed once per workgroup (the swizzle maps them to the same places in every tile): zero
//   columns of Q and K add nothing to a score, zero columns of V give output columns that are not stored.  Always
//   together with kMod (the identity when no modifier is set).
template <typename T, int D, int BN, bool kUniformPage, bool kMod = false, int kVar = 0, bool kPad = false>
__global__ __launch_bounds__(512) void prefill_pp_kernel(const PrefillArgs a)
{
    constexpr bool kFastRequests = (kVar & 1) != 0, kMaxInMatrixPhase = (kVar & 2) != 0;
    static_assert(kVar == 0 || (kUniformPage && !kMod), "tile variants exist for the plain uniform-page kernel");
    static_assert(!kPad || kMod, "padded head dims: the general kernel");
    const int dq = kPad ? a.d : D;    // elements per stored Q / K row
    const int dvs = kPad ? a.dv : D;  // elements per stored V / O row
    typedef PPShape<D, BN> S;
    typedef typename T::vec8 vec8;
    static_assert(S::NB == 2, "the matrix phase is written for 64-key tiles");
    constexpr int kRing = S::RING;
    FCK_DYNAMIC_LDS(smem);
    char FCK_LDS* lds = (char FCK_LDS*)smem;  // K ring | V ring | page ids (kPrefillPageCache x int32)
    char FCK_LDS* const k_ring = lds;
    char FCK_LDS* const v_ring = lds + kRing * S::TILEB;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int group = wave >> 2;
    const int wg = wave & 3;
    const int l32 = lane & 31;
    const int half = lane >> 5;

    // XCD-aware work order.  Workgroups are handed to the 8 XCDs round-robin by linear id, and each XCD has its own L2.
    // All workgroups that stream the same K/V (the g query heads of one KV head, every row tile of the sequence) are
    // therefore given ids that are congruent modulo 8, so they run on one XCD and share its L2; (sequence, KV head)
    // pairs are dealt round-robin to the XCDs.  Inside an XCD the heaviest row tiles of all sequences come first.
    constexpr int kXcd = 8;
    const int g = a.hq / a.hk;
    const int xcd = blockIdx.x % kXcd;
    const int slot = blockIdx.x / kXcd;
    const int groups = a.batch * a.hk;
    const int gx = (groups + kXcd - 1) / kXcd;  // (sequence, KV head) pairs per XCD
    const int hh = slot % g;
    const int gk = (slot / g) % gx;
    const int mt = a.m_tiles - 1 - slot / (g * gx);
    const int gid = gk * kXcd + xcd;
    if (gid >= groups) return;
    const int b = gid / a.hk;
    const int hkv = gid % a.hk;
    const int h = hkv * g + hh;

    int q_row0, sq_b;
    if (a.seqstart_q) {
        q_row0 = a.seqstart_q[b];
        sq_b = a.seqstart_q[b + 1] - q_row0;
    } else {
        q_row0 = b * a.sq;
        sq_b = a.sq;
    }
    // Row tiles are aligned to the END of the sequence: tile mt covers rows [mt * BM - pad, (mt + 1) * BM - pad) with
    // pad = (-sq) mod BM, so the ragged tile is the first one.  Under a causal mask the first tile sees the fewest keys,
    // so the rows that do not exist cost little there, and the last, most expensive tile is always full.
    const int tiles_b = (sq_b + S::BM - 1) / S::BM;
    if (mt >= tiles_b) return;
    const int m0 = mt * S::BM - (tiles_b * S::BM - sq_b);  // negative for a ragged first tile
    const KvSeq ks = kv_seq(a.kv, b);
    const int sk_b = ks.len;
    const MaskYX mk = make_mask(a.mask_type, a.window_left, a.window_right, sq_b, sk_b);

    // this lane's query row
    const int r = m0 + group * 128 + wg * 32 + l32;
    const bool row_ok = r >= 0 && r < sq_b;
    const int lo_r = row_ok ? mask_lo(mk, r) : 0;
    const int hi_r = row_ok ? mask_hi(mk, r, sk_b) : sk_b;
    ArithMod amod;
    if constexpr (kMod) amod.init(a.mod, b, h, row_ok ? r : 0, sq_b, sk_b, a.mask_type, a.window_left, a.window_right);
    // wave-uniform: keys in [w_lo_max, w_hi_min) are visible to every valid row of the wave
    const int wr0 = max(m0 + group * 128 + wg * 32, 0);
    const int wr1 = min(m0 + group * 128 + wg * 32 + 32, sq_b) - 1;
    const bool wave_ok = wr1 >= wr0;
    const int w_lo_max = wave_ok ? mask_lo(mk, wr1) : 0;
    const int w_hi_min = wave_ok ? mask_hi(mk, wr0, sk_b) : sk_b;
    // tiles the workgroup walks (a group also walks the few tiles only the other group can see: they mask to zero)
    const int t_begin = mask_lo(mk, max(m0, 0)) / S::BN;
    const int t_end = (mask_hi(mk, min(m0 + S::BM, sq_b) - 1, sk_b) + S::BN - 1) / S::BN;
    const int n = t_end - t_begin;  // number of tiles (may be <= 0)

    // ---- Q fragments (B operand of S^T = K . Q^T): lane (row = l32, k-group = half) ------------------------------
    u32x4_t qf[S::KT];
    {
        const uint16_t* qp =
            reinterpret_cast<const uint16_t*>(a.q) + ((int64_t)(q_row0 + (row_ok ? r : 0)) * a.hq + h) * dq + half * 8;
#pragma unroll
        for (int t = 0; t < S::KT; ++t) {
            qf[t] = u32x4_t{0u, 0u, 0u, 0u};
            if (row_ok && (!kPad || t * 16 + half * 8 < dq)) qf[t] = ldg16(qp + t * 16);
        }
    }

    f32x16_t oacc[S::DVB];
#pragma unroll
    for (int i = 0; i < S::DVB; ++i)
#pragma unroll
        for (int j = 0; j < 16; ++j) oacc[i][j] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;
    f32x16_t s[S::NB];          // scores of the tile between its M and V phase
    u32x4_t pfrag[2 * S::NB];   // probabilities of the tile between its V phase and the next M phase
    float tmax_pre = -INFINITY;  // kMaxInMatrixPhase: per-lane maximum of s, from the matrix phase that produced it

    const uint16_t* kp = reinterpret_cast<const uint16_t*>(a.k);
    const uint16_t* vp = reinterpret_cast<const uint16_t*>(a.v);
    const int64_t row_stride = (int64_t)a.hk * D;
    const int64_t rs_k = kPad ? (int64_t)a.hk * dq : row_stride, rs_v = kPad ? (int64_t)a.hk * dvs : row_stride;
    const int last_key = sk_b - 1;

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
        cp_v[u] = tiles::v_chunk_at<D>(row, pc) * 8;
    }

    // kFastRequests: byte offsets of a whole tile's requests
    uint32_t cp_koff[S::LD], cp_voff[S::LD];
    if constexpr (kFastRequests) {
#pragma unroll
        for (int u = 0; u < S::LD; ++u) {
            cp_koff[u] = (uint32_t)(cp_row[u] * (int)row_stride + cp_k[u]) * 2u;
            cp_voff[u] = (uint32_t)(cp_row[u] * (int)row_stride + cp_v[u]) * 2u;
        }
    }

    // First cache row of every tile (uniform-page path), cached per workgroup (see tiles::FirstRows)
    tiles::FirstRows<S::BN> first_rows{(int FCK_LDS*)(lds + 2 * kRing * S::TILEB)};
    if constexpr (kUniformPage) first_rows.fill(a.kv, ks, t_begin, n, tid, 512);
    auto tile_row0 = [&](int i) __attribute__((always_inline)) -> int64_t { return first_rows.row0(a.kv, ks, t_begin, i, lane); };
    auto tile = [&](int i) __attribute__((always_inline)) { return min(i, n - 1); };  // requests past the end re-read the last tile
    // request this wave's share of local tile `want` into ring buffer want % kRing (past the last tile: that tile
    // again); row0 = tile_row0(tile(want)) on the uniform-page path
    auto request = [&](const uint16_t* base, char FCK_LDS* ring, int want, int64_t row0, const int (&cp_c)[S::LD],
                       const uint32_t (&cp_off)[S::LD]) __attribute__((always_inline)) {
        const int i = tile(want);
        const int kb = (t_begin + i) * S::BN;
        const int room = last_key - kb;
        const int slot_ = want & (kRing - 1);
#pragma unroll
        for (int u = 0; u < S::LD; ++u) {
            const int row = min(cp_row[u], room);  // rows past the last key repeat it (their scores are masked)
            const uint32_t dst = lds_address(ring + slot_ * S::TILEB + (wave + 8 * u) * 1024);
            if constexpr (kPad) {
                // rows are a.d / a.dv elements apart; a piece past the stored row's end is not requested (its place in the
                // tile was zeroed once).  The waits below count instructions per wave, so every one of the S::LD
                // instructions must still be issued by every wave: it is, because a 1 KiB block holds whole rows, the
                // swizzle only permutes the pieces of a row, and piece 0 of a row is always stored (dim >= 8), so no
                // instruction has all its lanes skipped.
                const int64_t rs = base == kp ? rs_k : rs_v;
                const int dim = base == kp ? dq : dvs;
                if (cp_c[u] >= dim) {
                    FCK_LOAD_TO_LDS_MASKED();
                    continue;
                }
                if constexpr (kUniformPage)
                    tiles::load_to_lds(dst, base + (row0 * rs + hkv * dim), (uint32_t)(row * (int)rs + cp_c[u]) * 2u);
                else
                    tiles::load_to_lds(dst, base + kv_row(a.kv, ks, kb + row) * rs + hkv * dim + cp_c[u]);
            } else if constexpr (kUniformPage) {
                const uint16_t* tb = base + (row0 * row_stride + hkv * D);
                if (kFastRequests && room >= S::BN - 1)
                    tiles::load_to_lds(dst, tb, cp_off[u]);
                else
                    tiles::load_to_lds(dst, tb, (uint32_t)(row * (int)row_stride + cp_c[u]) * 2u);
            } else {
                tiles::load_to_lds(dst, base + kv_row(a.kv, ks, kb + row) * row_stride + hkv * D + cp_c[u]);
            }
        }
    };
    // wait until at most `keep` of this wave's vector-memory operations are outstanding (they complete in order)
    auto wait_vm = [&](auto keep) __attribute__((always_inline)) { tiles::wait_vm<decltype(keep)::value>(); };

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
        if constexpr (kMaxInMatrixPhase && kQk) {
            float t = s[0][0];
#pragma unroll
            for (int mbk = 0; mbk < S::NB; ++mbk)
#pragma unroll
                for (int j = 0; j < 16; ++j) t = fmaxf(t, s[mbk][j]);
            FCK_PIN_VGPR(t);  // stays in this phase
            tmax_pre = t;
        }
    };

    // online softmax of local tile i: s -> pfrag
    auto softmax = [&](int i) __attribute__((always_inline)) {
        const int kb = (t_begin + i) * S::BN;
        if constexpr (kMod) {
#pragma unroll
            for (int mbk = 0; mbk < S::NB; ++mbk)
#pragma unroll
                for (int j = 0; j < 16; ++j) s[mbk][j] = amod.score(s[mbk][j], kb + mbk * 32 + (j >> 2) * 8 + half * 4 + (j & 3));
        }
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
        if (kMaxInMatrixPhase && !need_mask) {
            tmax = tmax_pre;
        } else {
#pragma unroll
            for (int mbk = 0; mbk < S::NB; ++mbk)
#pragma unroll
                for (int j = 0; j < 16; ++j) tmax = fmaxf(tmax, s[mbk][j]);
        }
        tmax = pair32_max(tmax);
        if constexpr (!kMod) tmax *= a.scale_log2;  // scale > 0: max commutes with the scaling (modified scores are in the log2 domain already)
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
                if constexpr (kMod)
                    p[e] = fast_exp2(s[mbk][j0 + e] - m_ref);
                else
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
            FCK_PIN_VGPR4(pfrag[ks4][0], pfrag[ks4][1], pfrag[ks4][2], pfrag[ks4][3]);
        FCK_PIN_VGPR(l_run);
    };

    if constexpr (kPad) {
        // the LDS bytes no request of this lane will ever fill, in every ring buffer (the same lane and instruction slot of
        // every tile): nobody else writes them, and the barriers ahead of the first matrix phase publish them
        const u32x4_t zero = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int slot_ = 0; slot_ < kRing; ++slot_)
#pragma unroll
            for (int u = 0; u < S::LD; ++u) {
                const int off = slot_ * S::TILEB + (wave + 8 * u) * 1024 + lane * 16;
                if (cp_k[u] >= dq) *(u32x4_t FCK_LDS*)(k_ring + off) = zero;
                if (cp_v[u] >= dvs) *(u32x4_t FCK_LDS*)(v_ring + off) = zero;
            }
    }
    if (n > 0) {
        typedef std::integral_constant<int, 0> Keep0;
        typedef std::integral_constant<int, 2 * S::LD> KeepBatch;  // one batch = this wave's share of one K and one V tile
        if constexpr (kUniformPage) __syncthreads();  // the row cache is in LDS
        // Batch j = (K_{j+3}, V_{j+2}) is requested in the vector phase V(j), where the wave has issue slots to spare,
        // and has landed when the wave leaves M(j+1); M(j+2) is the first phase that reads it.  Tile t lives in ring
        // buffer t % kRing: while batch j is requested the other group may still read K_j and V_{j-1}, and K_{j+1},
        // K_{j+2}, V_j, V_{j+1} are waiting or in flight, hence four buffers per operand.
        int64_t r0 = 0, r1 = 0, r2 = 0;
        if constexpr (kUniformPage) {
            r0 = tile_row0(0);
            r1 = tile_row0(tile(1));
            r2 = tile_row0(tile(2));
        }
        request(kp, k_ring, 0, r0, cp_k, cp_koff);
        request(vp, v_ring, 0, r0, cp_v, cp_voff);
        request(kp, k_ring, 1, r1, cp_k, cp_koff);
        request(kp, k_ring, 2, r2, cp_k, cp_koff);  // batch -1
        request(vp, v_ring, 1, r1, cp_v, cp_voff);
        wait_vm(KeepBatch{});
        __syncthreads();
        if (group == 1) __syncthreads();  // skew: group 1 idles through phase 0
        matrix(std::false_type{}, std::true_type{}, v_ring, k_ring);
        __syncthreads();
        int64_t row_v = r2;  // first row of tile(i + 2): the tile whose K went out with the previous batch
        for (int i = 0; i + 1 < n; ++i) {
            int64_t row_k = 0;
            if constexpr (kUniformPage) row_k = tile_row0(tile(i + 3));
            request(kp, k_ring, i + 3, row_k, cp_k, cp_koff);
            request(vp, v_ring, i + 2, row_v, cp_v, cp_voff);
            row_v = row_k;
            softmax(i);
            __syncthreads();
            matrix(std::true_type{}, std::true_type{}, v_ring + (i & (kRing - 1)) * S::TILEB,
                   k_ring + ((i + 1) & (kRing - 1)) * S::TILEB);
            wait_vm(KeepBatch{});
            __syncthreads();
        }
        softmax(n - 1);
        __syncthreads();
        matrix(std::true_type{}, std::false_type{}, v_ring + ((n - 1) & (kRing - 1)) * S::TILEB, k_ring);
        wait_vm(Keep0{});  // nothing may still be landing in LDS when the workgroup retires
        __syncthreads();
        if (group == 0) __syncthreads();  // both groups pass the same number of barriers
    }

    // ---- epilogue ----------------------------------------------------------------------------------------------------
    l_run = pair32_sum(l_run);
    if (row_ok) {
        const float inv = (l_run == 0.f) ? 0.f : 1.f / l_run;
        uint16_t* op = reinterpret_cast<uint16_t*>(a.o) + ((int64_t)(q_row0 + r) * a.hq + h) * dvs;
#pragma unroll
        for (int dvb = 0; dvb < S::DVB; ++dvb)
#pragma unroll
            for (int j4 = 0; j4 < 4; ++j4) {
                if constexpr (kPad) {
                    if (dvb * 32 + j4 * 8 + half * 4 >= dvs) continue;
                }
                u32x2_t out;
                out[0] = T::pack2(oacc[dvb][j4 * 4 + 0] * inv, oacc[dvb][j4 * 4 + 1] * inv);
                out[1] = T::pack2(oacc[dvb][j4 * 4 + 2] * inv, oacc[dvb][j4 * 4 + 3] * inv);
                *reinterpret_cast<u32x2_t*>(op + dvb * 32 + j4 * 8 + half * 4) = out;
            }
    }
}

template <typename T, int D, int BN>
static hipError_t launch_d(const PrefillArgs& a, bool uniform, hipStream_t st)
{
    const int g = a.hq / a.hk, gx = (a.batch * a.hk + 7) / 8;
    const dim3 grid(8 * a.m_tiles * gx * g);
    constexpr size_t lds = (size_t)2 * PPShape<D, BN>::RING * PPShape<D, BN>::TILEB + kPrefillPageCache * 4;
    if (a.mod.bias_type == 1) return hipErrorInvalidValue;  // elementwise bias: not in this kernel (the caller routes it away)
    if (a.d != D || a.dv != D) {  // padded head dims
        if (uniform) return launch_with_lds<prefill_pp_kernel<T, D, BN, true, true, 0, true>>(grid, dim3(512), lds, st, a);
        return launch_with_lds<prefill_pp_kernel<T, D, BN, false, true, 0, true>>(grid, dim3(512), lds, st, a);
    }
    if (a.mod.active()) {
        if (uniform) return launch_with_lds<prefill_pp_kernel<T, D, BN, true, true>>(grid, dim3(512), lds, st, a);
        return launch_with_lds<prefill_pp_kernel<T, D, BN, false, true>>(grid, dim3(512), lds, st, a);
    }
    if (a.variant > 0) {  // validated by the caller: plain call, uniform pages, variant in [1, 4]
        if (!uniform) return hipErrorInvalidValue;
        switch (a.variant) {
        case 1: break;  // the default schedule, by name
        case 2: return launch_with_lds<prefill_pp_kernel<T, D, BN, true, false, 1>>(grid, dim3(512), lds, st, a);
        case 3: return launch_with_lds<prefill_pp_kernel<T, D, BN, true, false, 2>>(grid, dim3(512), lds, st, a);
        case 4: return launch_with_lds<prefill_pp_kernel<T, D, BN, true, false, 3>>(grid, dim3(512), lds, st, a);
        default: return hipErrorInvalidValue;
        }
    }
    if (uniform) return launch_with_lds<prefill_pp_kernel<T, D, BN, true>>(grid, dim3(512), lds, st, a);
    return launch_with_lds<prefill_pp_kernel<T, D, BN, false>>(grid, dim3(512), lds, st, a);
}

// `a.m_tiles` must count 256-row tiles.  Key tile: 64 at head dim 64, 32 at head dim 128 (register budget of two
// waves per SIMD).
hipError_t launch_prefill_pingpong(const PrefillArgs& a, int d, int dtype, bool uniform_page, hipStream_t st)
{
    if (d == 64) return dtype == 4 ? launch_d<BF16, 64, 64>(a, uniform_page, st) : launch_d<FP16, 64, 64>(a, uniform_page, st);
    if (d == 128) return dtype == 4 ? launch_d<BF16, 128, 64>(a, uniform_page, st) : launch_d<FP16, 128, 64>(a, uniform_page, st);
    return hipErrorInvalidValue;
}

}  // namespace fck
