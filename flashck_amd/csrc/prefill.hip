// Forward attention for long query runs (dense, varlen and paged prefill): hand-written gfx950 kernel.
//
// Work decomposition
//   grid  = (m_tiles, Hq, B); a workgroup of 4 waves owns 128 query rows of one head (32 rows per wave) and walks
//           the visible keys in tiles of 64; heavy (late) row tiles are scheduled first.
// Data path per 64-key tile
//   K, V  global -> VGPR (whole rows, 16 B per lane) -> XOR-swizzled LDS tiles, double buffered, shared by the
//         four waves; the loads of tile j+1 are in flight while tile j is consumed;
//   S^T = K . Q^T   v_mfma_f32_32x32x16, K read from LDS with ds_read_b128, Q resident in registers;
//   online softmax in the exp2 domain, one query row per lane pair (l, l^32);
//   O^T += V^T . P^T  V read from LDS transposed (ds_read_b64_tr_b16); P stays in registers because the
//         accumulator layout of the first product is the B-operand layout of the second.
#include "common.hpp"
#include "kernels.hpp"

#include <type_traits>

namespace fck {

template <int D>
struct PrefillShape {
    static constexpr int BM = 128;
    static constexpr int BN = 64;
    static constexpr int KT = D / 16;   // k-steps of the QK product
    static constexpr int DVB = D / 32;  // 32-column blocks of the output
    static constexpr int ROWB = D * 2;  // bytes per staged row
    static constexpr int CH = D / 8;    // 16-byte chunks per row
    static constexpr int TILEB = BN * ROWB;
    static constexpr int LD = BN * CH / 256;  // 16-byte loads per thread and tile
};

template <int D>
constexpr size_t prefill_lds_bytes()
{
    return (size_t)4 * PrefillShape<D>::TILEB;
}

// kPad: the stored head dims (a.d for Q/K, a.dv for V/O; multiples of 8) are smaller than D.  Rows are a.d / a.dv
// elements apart and the 16-byte pieces past a row's end are zeros instead of loads: zero columns of Q and K add
// nothing to a score, zero columns of V give output columns that are not stored.
// kKv8: K and V are stored as fp8 (e4m3, one byte per element, static per-tensor scales) and widened to T on their way
// into LDS; a lane then loads 8 bytes where the 16-bit path loads 16.  The K scale arrives folded into the softmax
// scale, the V scale multiplies the output.  Always together with kMod (the identity when no modifier is set).
// a.q8 (kKv8 instantiations only): the all-fp8 roles.  Q is e4m3 as well (widened to T like K and V: exact), every
// probability is rounded to e4m3 before the second product (the row sum keeps the unrounded values), and O is stored as
// e4m3, saturate(o_scale * o).  The matrix instructions are the 16-bit ones: what the roles save here is memory
// traffic, not matrix time.
template <typename T, int D, bool kUniformPage, bool kMod = false, bool kPad = false, bool kKv8 = false>
__global__ __launch_bounds__(256, (D == 256 ? 1 : 2)) void prefill_kernel(const PrefillArgs a)
{
    static_assert(!kKv8 || (kMod && !kPad), "fp8 cache: the general kernel, stored head dims equal to D");
    const int dq = kPad ? a.d : D;    // elements per stored Q / K row
    const int dvs = kPad ? a.dv : D;  // elements per stored V / O row
    typedef PrefillShape<D> S;
    typedef typename T::vec8 vec8;
    FCK_DYNAMIC_LDS(smem);
    char FCK_LDS* lds = (char FCK_LDS*)smem;  // K0 | K1 | V0 | V1

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31;
    const int half = lane >> 5;

    const int mt = a.m_tiles - 1 - blockIdx.x;  // heavy tiles first
    const int h = blockIdx.y;
    const int b = blockIdx.z;
    const int hkv = h / (a.hq / a.hk);

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
    const int r = m0 + wave * 32 + l32;
    const bool row_ok = r < sq_b;
    const int lo_r = row_ok ? mask_lo(mk, r) : 0;
    const int hi_r = row_ok ? mask_hi(mk, r, sk_b) : sk_b;
    // bias / ALiBi / soft cap of this lane's row; scores then come out in the log2 domain, so the scale becomes 1
    RowMod<T> rmod;
    if constexpr (kMod)
        rmod.init(a.mod, b, q_row0, h, row_ok ? r : 0, sq_b, sk_b, a.mask_type, a.window_left, a.window_right, a.seqstart_q != nullptr);
    const float scl = kMod ? 1.f : a.scale_log2;
    // wave-uniform bounds: keys in [w_lo_max, w_hi_min) are visible to every valid row of the wave
    const int wr0 = m0 + wave * 32;
    const int wr1 = min(wr0 + 32, sq_b) - 1;  // last valid row of the wave (may be < wr0 when the wave is empty)
    const bool wave_ok = wr0 < sq_b;
    const int w_lo_max = wave_ok ? mask_lo(mk, wr1) : 0;
    const int w_hi_min = wave_ok ? mask_hi(mk, wr0, sk_b) : sk_b;
    // workgroup-uniform visible range
    const int g_last = min(m0 + S::BM, sq_b) - 1;
    const int vis_lo = mask_lo(mk, m0);
    const int vis_hi = mask_hi(mk, g_last, sk_b);
    const int t_begin = vis_lo / S::BN;
    const int t_end = (vis_hi + S::BN - 1) / S::BN;

    // ---- Q fragments (B operand of S^T = K . Q^T): lane (row = l32, k-group = half) ------------------------------
    vec8 qf[S::KT];
    {
        const uint16_t* qp = reinterpret_cast<const uint16_t*>(a.q) + ((int64_t)(q_row0 + (row_ok ? r : 0)) * a.hq + h) * dq +
                             half * 8;
        bool q_done = false;
        if constexpr (kKv8) {
            if (a.q8) {  // one byte per element
                const uint8_t* qp8 = reinterpret_cast<const uint8_t*>(a.q) + ((int64_t)(q_row0 + (row_ok ? r : 0)) * a.hq + h) * D + half * 8;
#pragma unroll
                for (int t = 0; t < S::KT; ++t) {
                    u32x2_t v = {0u, 0u};
                    if (row_ok) v = *reinterpret_cast<const u32x2_t*>(qp8 + t * 16);
                    qf[t] = as_vec8<vec8>(fp8x8_to_t<T>(u32x4_t{v[0], v[1], 0u, 0u}));
                }
                q_done = true;
            }
        }
        if (!q_done) {
#pragma unroll
            for (int t = 0; t < S::KT; ++t) {
                u32x4_t v = {0u, 0u, 0u, 0u};
                if (row_ok && (!kPad || t * 16 + half * 8 < dq)) v = ldg16(qp + t * 16);
                qf[t] = as_vec8<vec8>(v);
            }
        }
    }

    f32x16_t oacc[S::DVB];
#pragma unroll
    for (int i = 0; i < S::DVB; ++i)
#pragma unroll
        for (int j = 0; j < 16; ++j) oacc[i][j] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;

    typedef typename std::conditional<kKv8, uint8_t, uint16_t>::type kv_elem;
    const kv_elem* kp = reinterpret_cast<const kv_elem*>(a.k);
    const kv_elem* vp = reinterpret_cast<const kv_elem*>(a.v);
    const int last_key = sk_b - 1;
    // this thread's piece u of a K / V row: offset inside the row's cache line-up, or zeros when the row ends before it
    auto load_piece = [&](const kv_elem* base, int64_t row, int c, int dim) -> u32x4_t {
        if constexpr (kPad) {
            if (c * 8 >= dim) return u32x4_t{0u, 0u, 0u, 0u};
        }
        if constexpr (kKv8) {
            const u32x2_t v = *reinterpret_cast<const u32x2_t*>(base + (row * a.hk + hkv) * dim + c * 8);
            return u32x4_t{v[0], v[1], 0u, 0u};
        } else {
            return ldg16(base + (row * a.hk + hkv) * dim + c * 8);
        }
    };
    auto staged = [](u32x4_t v) -> u32x4_t {
        if constexpr (kKv8)
            return fp8x8_to_t<T>(v);
        else
            return v;
    };

    // global -> LDS copy assignment: 16-byte chunk (row, c) per thread and step
    int cp_row[S::LD], cp_c[S::LD], cp_koff[S::LD], cp_voff[S::LD];
#pragma unroll
    for (int u = 0; u < S::LD; ++u) {
        const int cid = tid + 256 * u;
        cp_row[u] = cid / S::CH;
        cp_c[u] = cid % S::CH;
        cp_koff[u] = cp_row[u] * S::ROWB + ((cp_c[u] ^ (cp_row[u] & 7)) << 4);
        cp_voff[u] = cp_row[u] * S::ROWB + ((cp_c[u] ^ (((cp_row[u] & 7) << 1) & (S::CH - 1))) << 4);
    }

    u32x4_t kreg[S::LD], vreg[S::LD];
    auto load_tile = [&](int tile) {
        const int kb = tile * S::BN;
        if constexpr (kUniformPage) {
            const int kbc = min(kb, last_key);
            const int64_t row0 = kv_row(a.kv, ks, kbc) - (kbc - kb);
            const int room = last_key - kb;
#pragma unroll
            for (int u = 0; u < S::LD; ++u) {
                const int64_t row = row0 + min(cp_row[u], room);
                kreg[u] = load_piece(kp, row, cp_c[u], dq);
                vreg[u] = load_piece(vp, row, cp_c[u], dvs);
            }
        } else {
#pragma unroll
            for (int u = 0; u < S::LD; ++u) {
                const int key = min(kb + cp_row[u], last_key);
                const int64_t row = kv_row(a.kv, ks, key);
                kreg[u] = load_piece(kp, row, cp_c[u], dq);
                vreg[u] = load_piece(vp, row, cp_c[u], dvs);
            }
        }
    };
    auto store_tile = [&](int buf) {
        char FCK_LDS* kd = lds + buf * S::TILEB;
        char FCK_LDS* vd = lds + (2 + buf) * S::TILEB;
#pragma unroll
        for (int u = 0; u < S::LD; ++u) {
            *(u32x4_t FCK_LDS*)(kd + cp_koff[u]) = staged(kreg[u]);
            *(u32x4_t FCK_LDS*)(vd + cp_voff[u]) = staged(vreg[u]);
        }
    };

    // per-lane LDS read offsets
    // K (A operand): row = key (mbk * 32 + l32), chunk = t * 2 + half, swizzle key & 7
    const int k_sw = l32 & 7;
    const int k_rd = l32 * S::ROWB;
    // V^T (A operand, transposing read): 16-lane group q4 = lane / 16 covers columns (q4 & 1) * 16 .. +15 of a
    // 32-column block; lane i of the group addresses row half * 4 + i / 4, columns (i % 4) * 4 .. +3
    const int i16 = lane & 15;
    const int q4 = lane >> 4;
    const int v_row = half * 4 + (i16 >> 2);
    const int v_sw = ((v_row & 7) << 1) & (S::CH - 1);
    const int v_rd = v_row * S::ROWB + ((i16 & 1) << 3);
    const int v_c0 = (q4 & 1) * 2 + ((i16 & 3) >> 1);  // chunk inside the 32-column block (4 chunks)

    if (t_begin < t_end) {
        load_tile(t_begin);
        store_tile(0);
    }
    __syncthreads();

    for (int tile = t_begin; tile < t_end; ++tile) {
        const int buf = (tile - t_begin) & 1;
        const int kb = tile * S::BN;
        const bool more = tile + 1 < t_end;
        if (more) load_tile(tile + 1);

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
                for (int j = 0; j < 16; ++j)
                    s[mbk][j] = rmod.score(s[mbk][j], kb + mbk * 32 + (j >> 2) * 8 + half * 4 + (j & 3));
        }
        const bool need_mask = (kb < w_lo_max) || (kb + S::BN > w_hi_min);
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
        tmax *= scl;  // scale > 0: max commutes with the scaling
        // Lazy rescale: the running reference m_run only moves when some row's maximum outgrows it by more than
        // kLazy (in log2 units).  Softmax is shift invariant, so keeping a stale reference is exact; it bounds the
        // exponentials by 2^kLazy and saves the accumulator rescale on almost every tile.
        constexpr float kLazy = 8.f;
        if (__builtin_amdgcn_ballot_w64(tmax > m_run + kLazy) != 0) {
            const float m_new = fmaxf(m_run, tmax);
            const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
            const float alpha = fast_exp2(m_run - m_use);
            m_run = m_new;
            l_run *= alpha;
#pragma unroll
            for (int i = 0; i < S::DVB; ++i) oacc[i] *= alpha;
        }
        const float m_ref = (m_run == -INFINITY) ? 0.f : m_run;
        float psum = 0.f;
#pragma unroll
        for (int mbk = 0; mbk < 2; ++mbk)
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                const float p = fast_exp2(__builtin_fmaf(s[mbk][j], scl, -m_ref));
                s[mbk][j] = p;
                psum += p;
            }
        l_run += psum;
        if constexpr (kKv8) {
            if (a.q8) {  // 0 <= p <= 2^kLazy = 256 < 448: the conversion never saturates
#pragma unroll
                for (int mbk = 0; mbk < 2; ++mbk)
#pragma unroll
                    for (int j = 0; j < 16; j += 2) {
                        const f32x2_t p8 = round_to_fp8(s[mbk][j], s[mbk][j + 1]);
                        s[mbk][j] = p8[0];
                        s[mbk][j + 1] = p8[1];
                    }
            }
        }

        // ---- O^T += V^T . P^T ---------------------------------------------------------------------------------------
#pragma unroll
        for (int ks4 = 0; ks4 < 4; ++ks4) {  // 16 keys per step
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
                const int coff = (((dvb * 4 + v_c0) ^ v_sw) << 4);
                const u32x2_t lo4 = lds_read_tr16(vb + coff);
                const u32x2_t hi4 = lds_read_tr16(vb + 8 * S::ROWB + coff);
                const u32x4_t av = {lo4[0], lo4[1], hi4[0], hi4[1]};
                oacc[dvb] = T::mfma32(as_vec8<vec8>(av), pf, oacc[dvb]);
            }
        }

        if (more) store_tile(buf ^ 1);
        __syncthreads();
    }

    // ---- epilogue ----------------------------------------------------------------------------------------------------
    l_run = pair32_sum(l_run);
    if (row_ok) {
        float inv = (l_run == 0.f) ? 0.f : 1.f / l_run;
        if constexpr (kKv8) inv *= a.v_descale;
        if constexpr (kKv8) {
            if (a.q8) {  // four e4m3 bytes per store
                inv *= a.o_scale;
                uint8_t* op8 = reinterpret_cast<uint8_t*>(a.o) + ((int64_t)(q_row0 + r) * a.hq + h) * D;
#pragma unroll
                for (int dvb = 0; dvb < S::DVB; ++dvb)
#pragma unroll
                    for (int j4 = 0; j4 < 4; ++j4)
                        *reinterpret_cast<uint32_t*>(op8 + dvb * 32 + j4 * 8 + half * 4) =
                            pack_fp8x4_sat(oacc[dvb][j4 * 4 + 0] * inv, oacc[dvb][j4 * 4 + 1] * inv, oacc[dvb][j4 * 4 + 2] * inv,
                                           oacc[dvb][j4 * 4 + 3] * inv);
                return;
            }
        }
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
static hipError_t launch_d(const PrefillArgs& a, bool uniform, hipStream_t st)
{
    const dim3 grid(a.m_tiles, a.hq, a.batch);
    constexpr size_t lds = prefill_lds_bytes<D>();
    if (a.q8 && !a.kv8) return hipErrorInvalidValue;  // refused by the caller
    if (a.kv8) {  // fp8 cache: the general kernel with the widening load (the caller refuses padded head dims)
        if (a.d != D || a.dv != D) return hipErrorInvalidValue;
        if (uniform) return launch_with_lds<prefill_kernel<T, D, true, true, false, true>>(grid, dim3(256), lds, st, a);
        return launch_with_lds<prefill_kernel<T, D, false, true, false, true>>(grid, dim3(256), lds, st, a);
    }
    if (a.d != D || a.dv != D) {  // padded head dims: the general kernel (modifiers on, identity when there are none)
        if (uniform) return launch_with_lds<prefill_kernel<T, D, true, true, true>>(grid, dim3(256), lds, st, a);
        return launch_with_lds<prefill_kernel<T, D, false, true, true>>(grid, dim3(256), lds, st, a);
    }
    if (a.mod.active()) {
        if (uniform) return launch_with_lds<prefill_kernel<T, D, true, true>>(grid, dim3(256), lds, st, a);
        return launch_with_lds<prefill_kernel<T, D, false, true>>(grid, dim3(256), lds, st, a);
    }
    if (uniform) {
        // plain calls over tile-aligned pages at head dim 256 belong to the direct-to-LDS kernel: no instantiation here
        if constexpr (D == 256)
            return hipErrorInvalidValue;
        else
            return launch_with_lds<prefill_kernel<T, D, true>>(grid, dim3(256), lds, st, a);
    }
    return launch_with_lds<prefill_kernel<T, D, false>>(grid, dim3(256), lds, st, a);
}

template <typename T>
static hipError_t launch_t(const PrefillArgs& a, int d, bool uniform, hipStream_t st)
{
    switch (d) {
    case 64: return launch_d<T, 64>(a, uniform, st);
    case 128: return launch_d<T, 128>(a, uniform, st);
    case 256: return launch_d<T, 256>(a, uniform, st);
    }
    return hipErrorInvalidValue;
}

hipError_t launch_prefill(const PrefillArgs& a, int d, int dtype, bool uniform_page, hipStream_t st)
{
    return dtype == 4 ? launch_t<BF16>(a, d, uniform_page, st) : launch_t<FP16>(a, d, uniform_page, st);
}

}  // namespace fck
