// Forward attention for long query runs at head dim 256 (gfx950): the 4-wave, 128-row kernel of prefill.hip with the
// K/V tiles sent global -> LDS directly instead of through registers.
//
// At head dim 256 the register-staged kernel needs 64 VGPRs just to hold one K and one V tile in flight next to 128
// accumulator and 64 query registers, and the compiler spills into the accumulation registers' half of the file.  Here a
// tile never passes through a register: wave w requests the 1 KiB blocks w, w+4, ... of the next tile
// (global_load_lds_dwordx4, XOR swizzle applied on the global side, conflict-free read patterns as in
// prefill_pingpong.hip) into the buffer the previous iteration read, at the top of an iteration, and waits for them at
// its bottom, before the one barrier per tile.  The first cache row of every tile is computed once per workgroup into
// LDS (a per-tile page-table load would sit on the critical path and drain the load queue each time).  The grid is 1-D in
// XCD-aware order: all workgroups that stream one (sequence, KV head) run on one XCD, heaviest row tiles first.
//
// Limits: uniform pages only (page size a multiple of the 64-key tile, or no paging; the caller takes prefill.hip
// otherwise); the first rows of the first kPrefillPageCache key tiles are cached, later tiles are looked up one by one.
#include "common.hpp"
#include "kernels.hpp"
#include "lds_tiles.hpp"

#include <type_traits>

namespace fck {
namespace dma {

template <int D>
struct Shape {
    static constexpr int BM = 128;
    static constexpr int BN = 64;
    static constexpr int KT = D / 16;    // k-steps of the QK product
    static constexpr int DVB = D / 32;   // 32-column blocks of the output
    static constexpr int ROWB = D * 2;   // bytes per staged row
    static constexpr int TILEB = BN * ROWB;
    static constexpr int LD = TILEB / 1024 / 4;  // 1 KiB global->LDS instructions per wave and tile
    static_assert(D >= 128, "swizzles below are those of rows of at least 256 bytes");
};

// swizzles of rows of at least 256 bytes (see lds_tiles.hpp)
__device__ __forceinline__ int k_swz(int row) { return tiles::k_swz<256>(row); }
__device__ __forceinline__ int v_swz(int row, int lc) { return tiles::v_swz<256>(row, lc); }

// kMod: ALiBi and / or the logits soft cap applied to every score (ArithMod)
// kPad: the stored head dims (a.d for Q / K, a.dv for V / O; multiples of 8) are smaller than D: rows are a.d / a.dv
//   elements apart, a lane whose 16-byte piece lies past a row's end requests nothing and the LDS bytes it would have
//   filled are zeroed once per workgroup (zero columns of Q and K add nothing to a score, zero columns of V give output
//   columns that are not stored).  Always together with kMod (the identity when no modifier is set).
template <typename T, int D, bool kMod = false, bool kPad = false>
__global__ __launch_bounds__(256, 1) void prefill_dma_kernel(const PrefillArgs a)
{
    static_assert(!kPad || kMod, "padded head dims: the general kernel");
    const int dq = kPad ? a.d : D;    // elements per stored Q / K row
    const int dvs = kPad ? a.dv : D;  // elements per stored V / O row
    typedef Shape<D> S;
    typedef typename T::vec8 vec8;
    constexpr int BN = S::BN;
    FCK_DYNAMIC_LDS(smem);
    char FCK_LDS* lds = (char FCK_LDS*)smem;  // K0 | K1 | V0 | V1 | first rows (kPrefillPageCache x int32)
    int FCK_LDS* const row_lds = (int FCK_LDS*)(lds + 4 * S::TILEB);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31;
    const int half = lane >> 5;

    // XCD-aware work order (workgroups go to the 8 XCDs round-robin by linear id)
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
    // Row tiles are aligned to the END of the sequence (the ragged tile is the first one, where a causal mask leaves
    // the fewest keys): tile mt covers rows [mt * BM - pad, (mt + 1) * BM - pad), pad = (-sq) mod BM.
    const int tiles_b = (sq_b + S::BM - 1) / S::BM;
    if (mt >= tiles_b) return;
    const int m0 = mt * S::BM - (tiles_b * S::BM - sq_b);  // negative for a ragged first tile
    const KvSeq ks = kv_seq(a.kv, b);
    const int sk_b = ks.len;
    const MaskYX mk = make_mask(a.mask_type, a.window_left, a.window_right, sq_b, sk_b);

    // this lane's query row
    const int r = m0 + wave * 32 + l32;
    const bool row_ok = r >= 0 && r < sq_b;
    const int lo_r = row_ok ? mask_lo(mk, r) : 0;
    const int hi_r = row_ok ? mask_hi(mk, r, sk_b) : sk_b;
    ArithMod amod;
    if constexpr (kMod) amod.init(a.mod, b, h, row_ok ? r : 0, sq_b, sk_b, a.mask_type, a.window_left, a.window_right);
    // wave-uniform bounds: keys in [w_lo_max, w_hi_min) are visible to every valid row of the wave
    const int wr0 = max(m0 + wave * 32, 0);
    const int wr1 = min(m0 + wave * 32 + 32, sq_b) - 1;
    const bool wave_ok = wr1 >= wr0;
    const int w_lo_max = wave_ok ? mask_lo(mk, wr1) : 0;
    const int w_hi_min = wave_ok ? mask_hi(mk, wr0, sk_b) : sk_b;
    // workgroup-uniform visible range
    const int t_begin = mask_lo(mk, max(m0, 0)) / BN;
    const int t_end = (mask_hi(mk, min(m0 + S::BM, sq_b) - 1, sk_b) + BN - 1) / BN;
    const int n = t_end - t_begin;  // number of tiles (may be <= 0)

    // ---- Q fragments (B operand of S^T = K . Q^T): lane (row = l32, k-group = half) ------------------------------
    vec8 qf[S::KT];
    {
        const uint16_t* qp = reinterpret_cast<const uint16_t*>(a.q) + ((int64_t)(q_row0 + (row_ok ? r : 0)) * a.hq + h) * dq +
                             half * 8;
#pragma unroll
        for (int t = 0; t < S::KT; ++t) {
            u32x4_t v = {0u, 0u, 0u, 0u};
            if (row_ok && (!kPad || t * 16 + half * 8 < dq)) v = ldg16(qp + t * 16);
            qf[t] = as_vec8<vec8>(v);
        }
    }

    f32x16_t oacc[S::DVB];
#pragma unroll
    for (int i = 0; i < S::DVB; ++i)
#pragma unroll
        for (int j = 0; j < 16; ++j) oacc[i][j] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;

    const uint16_t* kp = reinterpret_cast<const uint16_t*>(a.k);
    const uint16_t* vp = reinterpret_cast<const uint16_t*>(a.v);
    const int64_t row_stride = (int64_t)a.hk * D;

    // global -> LDS assignment: wave w fills the 1 KiB blocks w, w+4, ... of a tile; lane l of an instruction lands at
    // byte l*16 of its block, i.e. at (row, physical chunk) below, and fetches the logical chunk the swizzle maps there.
    // A 1 KiB block is two rows here, so block w + 4u holds rows cp_row0 + 8u (+1): the physical chunk is the same for
    // every u, the K swizzle (row & 15) alternates with the parity of u and the V swizzle (row & 3) does not change.
    // Three offset registers therefore serve all 16 instructions of a tile; the 8u rows go into the scalar base.
    static_assert(S::ROWB == 512, "two rows per 1 KiB block");
    const int cp_row0 = wave * 2 + (lane >> 5);
    const int cp_pc = lane & 31;
    const int cp_kc0 = (cp_pc ^ k_swz(cp_row0)) * 8;      // K chunk (element offset in the row), even u
    const int cp_kc1 = (cp_pc ^ k_swz(cp_row0 + 8)) * 8;  // odd u
    const int cp_vc = tiles::v_chunk_at<256>(cp_row0, cp_pc) * 8;  // V chunk
    const uint32_t cp_koff0 = (uint32_t)(cp_row0 * (int)row_stride + cp_kc0) * 2u;  // bytes from row 8u of the tile
    const uint32_t cp_koff1 = (uint32_t)(cp_row0 * (int)row_stride + cp_kc1) * 2u;
    const uint32_t cp_voff = (uint32_t)(cp_row0 * (int)row_stride + cp_vc) * 2u;

    // first cache row of every tile of this workgroup (see tiles::FirstRows)
    tiles::FirstRows<BN> first_rows{row_lds};
    first_rows.fill(a.kv, ks, t_begin, n, tid, 256);
    auto tile_row0 = [&](int i) __attribute__((always_inline)) -> int64_t { return first_rows.row0(a.kv, ks, t_begin, i, lane); };
    if constexpr (kPad) {
        // the LDS bytes no request of this lane will ever fill, in both buffers of each operand
        const u32x4_t zero = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int buf = 0; buf < 2; ++buf)
#pragma unroll
            for (int u = 0; u < S::LD; ++u) {
                const int off = (wave + 4 * u) * 1024 + lane * 16;
                if (((u & 1) ? cp_kc1 : cp_kc0) >= dq) *(u32x4_t FCK_LDS*)(lds + buf * S::TILEB + off) = zero;
                if (cp_vc >= dvs) *(u32x4_t FCK_LDS*)(lds + (2 + buf) * S::TILEB + off) = zero;
            }
    }
    // request this wave's share of the K and V tile i (local index) into buffer buf
    auto request = [&](int i, int buf) __attribute__((always_inline)) {
        const int room = sk_b - 1 - (t_begin + i) * BN;
        const bool whole = room >= BN - 1;  // every row of the tile exists (all tiles but the last of a sequence)
        const int64_t row0 = tile_row0(i);
        if constexpr (kPad) {
            // rows are a.d / a.dv elements apart; a piece past the stored row's end is not requested
#pragma unroll
            for (int kv = 0; kv < 2; ++kv) {
                const int64_t rs = (int64_t)a.hk * (kv == 0 ? dq : dvs);
                const int dim = kv == 0 ? dq : dvs;
                const uint16_t* tb = (kv == 0 ? kp : vp) + (row0 * rs + hkv * dim);
                char FCK_LDS* dst0 = lds + ((kv == 0 ? 0 : 2) + buf) * S::TILEB;
#pragma unroll
                for (int u = 0; u < S::LD; ++u) {
                    const int c = kv == 0 ? ((u & 1) ? cp_kc1 : cp_kc0) : cp_vc;
                    if (c >= dim) {
                        FCK_LOAD_TO_LDS_MASKED();
                        continue;
                    }
                    const int row = min(cp_row0 + 8 * u, room);  // rows past the last key repeat it (their scores are masked)
                    tiles::load_to_lds(lds_address(dst0 + (wave + 4 * u) * 1024), tb, (uint32_t)(row * (int)rs + c) * 2u);
                }
            }
            return;
        }
        const int64_t tile_off = row0 * row_stride + hkv * D;
#pragma unroll
        for (int kv = 0; kv < 2; ++kv) {
            char FCK_LDS* dst0 = lds + ((kv == 0 ? 0 : 2) + buf) * S::TILEB;
#pragma unroll
            for (int u = 0; u < S::LD; ++u) {
                const uint16_t* tb = (kv == 0 ? kp : vp) + tile_off;
                uint32_t off;
                if (whole) {
                    tb += (int64_t)(8 * u) * row_stride;  // rows 8u .. of the tile, in the scalar base
                    off = kv == 0 ? ((u & 1) ? cp_koff1 : cp_koff0) : cp_voff;
                } else {  // rows past the last key repeat it (their scores are masked)
                    const int row = min(cp_row0 + 8 * u, room);
                    off = (uint32_t)(row * (int)row_stride + (kv == 0 ? ((u & 1) ? cp_kc1 : cp_kc0) : cp_vc)) * 2u;
                }
                tiles::load_to_lds(lds_address(dst0 + (wave + 4 * u) * 1024), tb, off);
            }
        }
    };
    // wait until none of this wave's vector-memory operations is outstanding
    auto wait_all = [&]() __attribute__((always_inline)) { tiles::wait_vm<0>(); };

    // per-lane LDS read offsets
    // K (A operand): row = key (mbk * 32 + l32), chunk = t * 2 + half
    const int k_rd = l32 * S::ROWB;
    const int k_sw = k_swz(l32);  // rows mbk*32 + l32 share the swizzle of l32 (32 is a multiple of 16)
    // V^T (A operand, transposing read): 16-lane group q4 = lane / 16 covers columns (q4 & 1) * 16 .. +15 of a
    // 32-column block; lane i of the group addresses row half * 4 + i / 4, columns (i % 4) * 4 .. +3
    const int i16 = lane & 15;
    const int q4 = lane >> 4;
    const int v_row = half * 4 + (i16 >> 2);
    const int v_rd = v_row * S::ROWB + ((i16 & 1) << 3);
    const int v_c0 = (q4 & 1) * 2 + ((i16 & 3) >> 1);  // chunk inside the 32-column block (4 chunks)

    if (n > 0) {
        __syncthreads();  // the first rows are in LDS
        request(0, 0);
        wait_all();
        __syncthreads();
    }
    for (int i = 0; i < n; ++i) {
        const int buf = i & 1;
        const int kb = (t_begin + i) * BN;
        if (i + 1 < n) request(i + 1, buf ^ 1);  // the other buffer was last read before the barrier that ended tile i-1

        const char FCK_LDS* kt = lds + buf * S::TILEB;
        const char FCK_LDS* vt = lds + (2 + buf) * S::TILEB;

        // ---- S^T = K . Q^T -------------------------------------------------------------------------------------
        f32x16_t s[2];
#pragma unroll
        for (int mbk = 0; mbk < 2; ++mbk) {
#pragma unroll
            for (int j = 0; j < 16; ++j) s[mbk][j] = 0.f;
#pragma unroll
            for (int t = 0; t < S::KT; ++t) {
                const u32x4_t kv = *(const u32x4_t FCK_LDS*)(kt + mbk * 32 * S::ROWB + k_rd + (((t * 2 + half) ^ k_sw) << 4));
                s[mbk] = T::mfma32(as_vec8<vec8>(kv), qf[t], s[mbk]);
            }
        }

        // ---- online softmax (exp2 domain) ---------------------------------------------------------------------
        if constexpr (kMod) {
#pragma unroll
            for (int mbk = 0; mbk < 2; ++mbk)
#pragma unroll
                for (int j = 0; j < 16; ++j) s[mbk][j] = amod.score(s[mbk][j], kb + mbk * 32 + (j >> 2) * 8 + half * 4 + (j & 3));
        }
        const bool need_mask = (kb < w_lo_max) || (kb + BN > w_hi_min);
        float tmax = -INFINITY;
        if (need_mask) {
#pragma unroll
            for (int mbk = 0; mbk < 2; ++mbk)
#pragma unroll
                for (int j = 0; j < 16; ++j) {
                    const int key = kb + mbk * 32 + (j >> 2) * 8 + half * 4 + (j & 3);
                    const bool vis = key >= lo_r && key < hi_r;
                    s[mbk][j] = vis ? s[mbk][j] : -INFINITY;
                }
        }
#pragma unroll
        for (int mbk = 0; mbk < 2; ++mbk)
#pragma unroll
            for (int j = 0; j < 16; ++j) tmax = fmaxf(tmax, s[mbk][j]);
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
            // The output accumulator lives in the accumulation half of the register file (the MFMAs update it there).
            // It is scaled through explicit accumulator reads and writes inside this branch: a plain `oacc[q] *= alpha`
            // makes the compiler copy all of it into vector registers at the top of every iteration.
#pragma unroll
            for (int q = 0; q < S::DVB; ++q)
#pragma unroll
                for (int j = 0; j < 16; ++j) FCK_ACC_SCALE(oacc[q][j], alpha);
        }
        const float m_ref = (m_run == -INFINITY) ? 0.f : m_run;
        float psum = 0.f;
#pragma unroll
        for (int mbk = 0; mbk < 2; ++mbk)
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                const float p = kMod ? fast_exp2(s[mbk][j] - m_ref) : fast_exp2(__builtin_fmaf(s[mbk][j], a.scale_log2, -m_ref));
                s[mbk][j] = p;
                psum += p;
            }
        l_run += psum;

        // ---- O^T += V^T . P^T ---------------------------------------------------------------------------------------
#pragma unroll
        for (int ks4 = 0; ks4 < 4; ++ks4) {  // 16 keys per step; rows ks4*16 + {0,8} + v_row share v_row's swizzle
            const int mbk = ks4 >> 1, j0 = (ks4 & 1) * 8;
            u32x4_t pk;
            pk[0] = T::pack2(s[mbk][j0 + 0], s[mbk][j0 + 1]);
            pk[1] = T::pack2(s[mbk][j0 + 2], s[mbk][j0 + 3]);
            pk[2] = T::pack2(s[mbk][j0 + 4], s[mbk][j0 + 5]);
            pk[3] = T::pack2(s[mbk][j0 + 6], s[mbk][j0 + 7]);
            const vec8 pf = as_vec8<vec8>(pk);
            const char FCK_LDS* vb = vt + ks4 * 16 * S::ROWB + v_rd;
#pragma unroll
            for (int dvb = 0; dvb < S::DVB; ++dvb) {
                const int lc = dvb * 4 + v_c0;
                const int coff = ((lc ^ v_swz(v_row, lc)) << 4);
                const u32x2_t lo4 = lds_read_tr16(vb + coff);
                const u32x2_t hi4 = lds_read_tr16(vb + 8 * S::ROWB + coff);
                const u32x4_t av = {lo4[0], lo4[1], hi4[0], hi4[1]};
                oacc[dvb] = T::mfma32(as_vec8<vec8>(av), pf, oacc[dvb]);
            }
        }

        wait_all();       // this wave's share of tile i+1 has landed
        __syncthreads();  // ... and so has everyone's; nobody reads tile i any more
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

template <typename T, int D>
static hipError_t launch_d(const PrefillArgs& a, hipStream_t st)
{
    const int g = a.hq / a.hk, gx = (a.batch * a.hk + 7) / 8;
    const dim3 grid(8 * a.m_tiles * gx * g);
    constexpr size_t lds = (size_t)4 * Shape<D>::TILEB + kPrefillPageCache * 4;
    if (a.mod.bias_type == 1) return hipErrorInvalidValue;  // elementwise bias: not in this kernel (the caller routes it away)
    if (a.d != D || a.dv != D) return launch_with_lds<prefill_dma_kernel<T, D, true, true>>(grid, dim3(256), lds, st, a);
    if (a.mod.active()) return launch_with_lds<prefill_dma_kernel<T, D, true>>(grid, dim3(256), lds, st, a);
    return launch_with_lds<prefill_dma_kernel<T, D>>(grid, dim3(256), lds, st, a);
}

}  // namespace dma

// `a.m_tiles` must count 128-row tiles; head dim 256; uniform pages, at most kPrefillPageCache key tiles per sequence.
hipError_t launch_prefill_dma(const PrefillArgs& a, int d, int dtype, hipStream_t st)
{
    if (d != 256) return hipErrorInvalidValue;
    return dtype == 4 ? dma::launch_d<BF16, 256>(a, st) : dma::launch_d<FP16, 256>(a, st);
}

}  // namespace fck
