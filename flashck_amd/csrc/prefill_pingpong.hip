// Forward attention for long query runs, ping-pong variant (gfx950): two groups of four waves share the SIMDs of a CU
// and are kept half an iteration apart, so that while one group feeds the matrix cores the other runs its softmax on
// the vector ALUs.
//
// Work decomposition
//   grid  = 1-D, XCD-aware order; a workgroup of 8 waves owns 256 query rows of one head: group g = wave / 4 owns rows
//           [g*128, g*128+128), 32 rows per wave.  Waves w and w+4 sit on the same SIMD.
// Phases (one workgroup barrier after each); tile i = the i-th key tile of the visible range
//   group 0, phase 2i   : matrix phase  M(i) = { O^T += V^T.P^T of tile i-1 ; S^T = K.Q^T of tile i }
//   group 0, phase 2i+1 : vector phase  V(i) = { online softmax of tile i: S -> P }
//   group 1 runs the same instruction stream one phase later (it passes one extra barrier before its first matrix
//   phase, group 0 one extra after its last), so every phase pairs one M with one V on each SIMD and no branch inside
//   the loop depends on the group.
// Data path
//   K, V tiles: global -> VGPR (whole rows, 16 B per lane) -> swizzled LDS, two buffers each; the loads of a tile are
//   issued six phases (three tiles) before they are written to LDS.  K is read with ds_read_b128 as the A operand of
//   v_mfma_f32_32x32x16, V with the transposing ds_read_b64_tr_b16; Q is parked in LDS; P never leaves registers
//   because the accumulator layout of the first product is the B-operand layout of the second.
#include "common.hpp"
#include "kernels.hpp"

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
    static constexpr int NCH = BN * CH;                    // 16-byte chunks per tile
    static constexpr int LD = (NCH + 511) / 512;           // 16-byte loads per thread and tile (threads past NCH idle)
};

// XOR swizzles of the 16-byte chunk index.  They keep both LDS read patterns free of bank conflicts whether the LDS
// serves 128 or 256 bytes per clock: K is read by 8/16 consecutive lanes = consecutive rows at one logical chunk; V by
// 16/32 lanes = 4 rows x (2 or 4) adjacent chunks.
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

template <typename T, int D, int BN, bool kUniformPage>
__global__ __launch_bounds__(512) void prefill_pp_kernel(const PrefillArgs a)
{
    typedef PPShape<D, BN> S;
    typedef typename T::vec8 vec8;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    char FCK_LDS* lds = (char FCK_LDS*)smem;  // K0 | K1 | V0 | V1 | Q fragments (8 waves x KT x 1 KiB) | page ids (kPrefillPageCache x int32)

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
    const int m0 = mt * S::BM;
    if (m0 >= sq_b) return;
    const KvSeq ks = kv_seq(a.kv, b);
    const int sk_b = ks.len;
    const MaskYX mk = make_mask(a.mask_type, a.window_left, a.window_right, sq_b, sk_b);

    // this lane's query row
    const int r = m0 + group * 128 + wg * 32 + l32;
    const bool row_ok = r < sq_b;
    const int lo_r = row_ok ? mask_lo(mk, r) : 0;
    const int hi_r = row_ok ? mask_hi(mk, r, sk_b) : sk_b;
    // wave-uniform: keys in [w_lo_max, w_hi_min) are visible to every valid row of the wave
    const int wr0 = m0 + group * 128 + wg * 32;
    const bool wave_ok = wr0 < sq_b;
    const int wr1 = min(wr0 + 32, sq_b) - 1;
    const int w_lo_max = wave_ok ? mask_lo(mk, wr1) : 0;
    const int w_hi_min = wave_ok ? mask_hi(mk, wr0, sk_b) : sk_b;
    // tiles the workgroup walks (a group also walks the few tiles only the other group can see: they mask to zero)
    const int t_begin = mask_lo(mk, m0) / S::BN;
    const int t_end = (mask_hi(mk, min(m0 + S::BM, sq_b) - 1, sk_b) + S::BN - 1) / S::BN;
    const int n = t_end - t_begin;  // number of tiles (may be <= 0)

    // ---- Q fragments (B operand of S^T = K . Q^T): lane (row = l32, k-group = half) ------------------------------
    // They are parked in a wave-private LDS area, lane-linear, and re-read in every matrix phase: the 4*KT registers
    // they would occupy are what lets three K/V tiles be in flight from global memory.
    char FCK_LDS* qlds = lds + 4 * S::TILEB + wave * (S::KT * 1024) + lane * 16;
    {
        const uint16_t* qp =
            reinterpret_cast<const uint16_t*>(a.q) + ((int64_t)(q_row0 + (row_ok ? r : 0)) * a.hq + h) * D + half * 8;
#pragma unroll
        for (int t = 0; t < S::KT; ++t) {
            u32x4_t v = {0u, 0u, 0u, 0u};
            if (row_ok) v = ldg16(qp + t * 16);
            *(u32x4_t FCK_LDS*)(qlds + t * 1024) = v;
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

    const uint16_t* kp = reinterpret_cast<const uint16_t*>(a.k);
    const uint16_t* vp = reinterpret_cast<const uint16_t*>(a.v);
    const int64_t row_stride = (int64_t)a.hk * D;
    const int last_key = sk_b - 1;

    // global -> LDS copy assignment: 16-byte chunk (row, c) per thread and step
    int cp_row[S::LD], cp_c[S::LD], cp_koff[S::LD], cp_voff[S::LD];
#pragma unroll
    for (int u = 0; u < S::LD; ++u) {
        const int cid = min(tid + 512 * u, S::NCH - 1);  // threads past the tile repeat its last chunk (same bytes)
        cp_row[u] = cid / S::CH;
        cp_c[u] = cid % S::CH;
        cp_koff[u] = cp_row[u] * S::ROWB + ((cp_c[u] ^ k_swz<D>(cp_row[u])) << 4);
        cp_voff[u] = cp_row[u] * S::ROWB + ((cp_c[u] ^ v_swz<D>(cp_row[u], cp_c[u])) << 4);
    }

    struct Regs {
        u32x4_t k[S::LD], v[S::LD];
    };

    // Page ids (uniform-page path): the pages of this workgroup's tiles are copied into LDS once, so that the lookups
    // of the main loop are LDS reads (lgkmcnt) and never wait on the vector loads in flight (vmcnt is shared by all
    // global loads of a wave and counts in order).  The host only selects this path when a sequence cannot have more
    // than kPrefillPageCache tiles.
    constexpr int kPageCache = kPrefillPageCache;
    int FCK_LDS* page_lds = (int FCK_LDS*)(lds + 4 * S::TILEB + 8 * S::KT * 1024);
    auto page_index = [&](int key) __attribute__((always_inline)) {
        return a.kv.page_shift >= 0 ? key >> a.kv.page_shift : key / a.kv.page_size;
    };
    if constexpr (kUniformPage) {
        if (ks.table != nullptr)
            for (int i = tid; i < min(n, kPageCache); i += 512) page_lds[i] = ks.table[page_index((t_begin + i) * S::BN)];
    }
    auto tile_row0 = [&](int i) __attribute__((always_inline)) -> int64_t {
        const int kb = (t_begin + i) * S::BN;
        if (ks.table != nullptr) {
            const int page = __builtin_amdgcn_readfirstlane(page_lds[i]);
            return (int64_t)page * a.kv.page_size + (kb - page_index(kb) * a.kv.page_size);
        }
        return ks.base_row + kb;
    };
    // Every step of the main loop requests exactly one K tile and one V tile, unconditionally (tile indices past the
    // end are clamped and re-read the last tile): with a fixed number of loads per step the compiler can count how many
    // younger loads may stay outstanding when a tile is written to LDS, instead of draining the counter to zero.
    auto load_tile = [&](const uint16_t* base, int i, int64_t row0, u32x4_t (&dst)[S::LD]) __attribute__((always_inline)) {
        const int kb = (t_begin + i) * S::BN;
        if constexpr (kUniformPage) {
            const int room = last_key - kb;
#pragma unroll
            for (int u = 0; u < S::LD; ++u)
                dst[u] = ldg16(base + (row0 + min(cp_row[u], room)) * row_stride + hkv * D + cp_c[u] * 8);
        } else {
#pragma unroll
            for (int u = 0; u < S::LD; ++u)
                dst[u] = ldg16(base + kv_row(a.kv, ks, min(kb + cp_row[u], last_key)) * row_stride + hkv * D + cp_c[u] * 8);
        }
    };
    auto store_k = [&](int i, const Regs& R) __attribute__((always_inline)) {
        char FCK_LDS* kd = lds + (i & 1) * S::TILEB;
#pragma unroll
        for (int u = 0; u < S::LD; ++u) *(u32x4_t FCK_LDS*)(kd + cp_koff[u]) = R.k[u];
    };
    auto store_v = [&](int i, const Regs& R) __attribute__((always_inline)) {
        char FCK_LDS* vd = lds + (2 + (i & 1)) * S::TILEB;
#pragma unroll
        for (int u = 0; u < S::LD; ++u) *(u32x4_t FCK_LDS*)(vd + cp_voff[u]) = R.v[u];
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

    // S^T = K . Q^T of local tile i
    auto qk = [&](int i) __attribute__((always_inline)) {
        const char FCK_LDS* kt = lds + (i & 1) * S::TILEB;
#pragma unroll
        for (int mbk = 0; mbk < S::NB; ++mbk)
#pragma unroll
            for (int j = 0; j < 16; ++j) s[mbk][j] = 0.f;
#pragma unroll
        for (int t = 0; t < S::KT; ++t) {
            const vec8 qv = as_vec8<vec8>(*(const u32x4_t FCK_LDS*)(qlds + t * 1024));
#pragma unroll
            for (int mbk = 0; mbk < S::NB; ++mbk) {
                const u32x4_t kv = *(const u32x4_t FCK_LDS*)(kt + mbk * 32 * S::ROWB + k_rd + (((t * 2 + half) ^ k_sw) << 4));
                s[mbk] = T::mfma32(as_vec8<vec8>(kv), qv, s[mbk]);
            }
        }
    };
    // O^T += V^T . P^T of local tile i
    auto pv = [&](int i) __attribute__((always_inline)) {
        const char FCK_LDS* vt = lds + (2 + (i & 1)) * S::TILEB;
#pragma unroll
        for (int ks4 = 0; ks4 < 2 * S::NB; ++ks4) {  // 16 keys per step; rows ks4*16 + {0,8} + v_row share v_row's swizzle
            const vec8 pf = as_vec8<vec8>(pfrag[ks4]);
            const char FCK_LDS* vb = vt + ks4 * 16 * S::ROWB + v_rd;
#pragma unroll
            for (int dvb = 0; dvb < S::DVB; ++dvb) {
                const int lc = dvb * 4 + v_c0;
                const int coff = ((lc ^ v_swz<D>(v_row, lc)) << 4);
                const u32x2_t lo4 = lds_read_tr16(vb + coff);
                const u32x2_t hi4 = lds_read_tr16(vb + 8 * S::ROWB + coff);
                const u32x4_t av = {lo4[0], lo4[1], hi4[0], hi4[1]};
                oacc[dvb] = T::mfma32(as_vec8<vec8>(av), pf, oacc[dvb]);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
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

    if (n > 0) {
        // Three tiles are in flight from global memory: set (i % 3) holds (K_{i+1}, V_i) from step(i-3) until step(i).
        Regs R0, R1, R2;
        if constexpr (kUniformPage) __syncthreads();  // page ids are in LDS
        auto tile = [&](int i) __attribute__((always_inline)) { return min(i, n - 1); };  // clamp past-the-end requests
        {
            int64_t r[4] = {0, 0, 0, 0};
            if constexpr (kUniformPage) {
#pragma unroll
                for (int t = 0; t < 4; ++t) r[t] = tile_row0(tile(t));
            }
            load_tile(kp, 0, r[0], R0.k);
            store_k(0, R0);  // K_0 goes straight to LDS
            load_tile(kp, tile(1), r[1], R0.k);
            load_tile(vp, 0, r[0], R0.v);
            load_tile(kp, tile(2), r[2], R1.k);
            load_tile(vp, tile(1), r[1], R1.v);
            load_tile(kp, tile(3), r[3], R2.k);
            load_tile(vp, tile(2), r[2], R2.v);
        }
        __syncthreads();
        // step(i, R), right after the matrix phase of tile i: write this thread's chunks of (K_{i+1}, V_i) from R and
        // request (K_{i+4}, V_{i+3}) into the same registers.  Group 0 does this in phase 2i, group 1 in phase 2i+1;
        // both halves are in LDS before phase 2i+2, the first one that reads them.
        auto step = [&](int i, Regs& R, int64_t rk, int64_t rv) __attribute__((always_inline)) {
            if (i + 1 < n) store_k(i + 1, R);
            store_v(i, R);
            load_tile(kp, tile(i + 4), rk, R.k);
            load_tile(vp, tile(i + 3), rv, R.v);
        };
        // row bases of the tiles step(i) will request, looked up one matrix phase earlier
        auto rows_for = [&](int i, int64_t& rk, int64_t& rv) __attribute__((always_inline)) {
            rk = 0;
            rv = 0;
            if constexpr (kUniformPage) {
                rv = tile_row0(tile(i + 3));
                rk = tile_row0(tile(i + 4));
            }
        };
        if (group == 1) __syncthreads();  // skew: group 1 idles through phase 0
        int64_t rk, rv;
        rows_for(0, rk, rv);
        qk(0);
        step(0, R0, rk, rv);
        __syncthreads();
        int i = 0;
        while (true) {
            if (i + 1 >= n) break;
            softmax(i);
            __syncthreads();
            rows_for(i + 1, rk, rv);
            pv(i);
            qk(i + 1);
            step(i + 1, R1, rk, rv);
            __syncthreads();
            ++i;
            if (i + 1 >= n) break;
            softmax(i);
            __syncthreads();
            rows_for(i + 1, rk, rv);
            pv(i);
            qk(i + 1);
            step(i + 1, R2, rk, rv);
            __syncthreads();
            ++i;
            if (i + 1 >= n) break;
            softmax(i);
            __syncthreads();
            rows_for(i + 1, rk, rv);
            pv(i);
            qk(i + 1);
            step(i + 1, R0, rk, rv);
            __syncthreads();
            ++i;
        }
        softmax(n - 1);
        __syncthreads();
        pv(n - 1);
        __syncthreads();
        if (group == 0) __syncthreads();  // both groups pass the same number of barriers
    }

    // ---- epilogue ----------------------------------------------------------------------------------------------------
    l_run = pair32_sum(l_run);
    if (row_ok) {
        const float inv = (l_run == 0.f) ? 0.f : 1.f / l_run;
        uint16_t* op = reinterpret_cast<uint16_t*>(a.o) + ((int64_t)(q_row0 + r) * a.hq + h) * D;
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
}

template <typename T, int D, int BN>
static hipError_t launch_d(const PrefillArgs& a, bool uniform, hipStream_t st)
{
    const int g = a.hq / a.hk, gx = (a.batch * a.hk + 7) / 8;
    const dim3 grid(8 * a.m_tiles * gx * g);
    constexpr size_t lds = (size_t)4 * PPShape<D, BN>::TILEB + 8 * PPShape<D, BN>::KT * 1024 + kPrefillPageCache * 4;
    hipError_t e;
    if (uniform) {
        auto kern = prefill_pp_kernel<T, D, BN, true>;
        static bool once = false;
        if (!once) {
            e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return e;
            once = true;
        }
        hipLaunchKernelGGL(kern, grid, dim3(512), lds, st, a);
    } else {
        auto kern = prefill_pp_kernel<T, D, BN, false>;
        static bool once = false;
        if (!once) {
            e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return e;
            once = true;
        }
        hipLaunchKernelGGL(kern, grid, dim3(512), lds, st, a);
    }
    return hipGetLastError();
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
