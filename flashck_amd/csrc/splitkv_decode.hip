// Split-KV forward for short query lengths (decode): hand-written gfx950 kernel.
//
// Work decomposition
//   grid  = (m_tiles * num_splits, Hk, B); one workgroup owns one split of one KV head of one sequence and the
//           16*MB packed query rows (query index, head-in-group) that share that KV head.
//   waves = NW per workgroup; wave w walks the 32-key tiles w, w+NW, ... of the split with its own online-softmax
//           state; the NW partial states are merged through LDS at the end.
// Data path per step (one 32-key tile per wave)
//   K, V  global -> VGPR with whole 2*D-byte rows per D/8 lanes (every 128-byte line is touched by one instruction).
//       Waves work in pairs: the even wave fetches the K rows of both tiles of the pair (64 consecutive keys), the odd
//       wave fetches the V rows, so every wave streams from one array in bursts of 2*D/16 loads - measured to be the
//       access shape the HBM system sustains best, whereas one wave alternating between the K and the V pool is
//       15-20 % slower.  The rows are staged in per-wave, XOR-swizzled LDS tiles; K is read back with ds_read_b128
//       as the A operand of S^T = K . Q^T, V is read back transposed (ds_read_b64_tr_b16) as the A operand of
//       O^T += V^T . P^T;
//   S^T = K . Q^T with v_mfma_f32_16x16x32, so that each lane keeps the scores of one query row and the
//       probabilities it produces are already laid out as the B operand of the second product.
// The loads of step i+1 are in flight while step i is computed from LDS.
#include "common.hpp"
#include "kernels.hpp"

namespace fck {

template <int D>
struct DecodeShape {
    static constexpr int TK = 32;          // keys per tile
    static constexpr int LPR = D / 8;      // lanes that cover one V row with 16-byte pieces
    static constexpr int KPI = 64 / LPR;   // keys per V load instruction
    static constexpr int VN = TK / KPI;    // V load instructions per tile
    static constexpr int KT = D / 32;      // MFMA k-steps of the QK product
    static constexpr int DB = D / 16;      // 16-column blocks of the output
    static constexpr int VROW = D * 2;     // bytes per staged V row
    static constexpr int VTILE = TK * VROW;
    static constexpr int OSTRIDE = D + 4;  // floats per row of the merge buffer (bank spread)
};

template <int D, int NW>
constexpr size_t decode_lds_bytes()
{
    typedef DecodeShape<D> S;
    const size_t stage = (size_t)NW * 2 * S::VTILE;
    const size_t merge = (size_t)NW * 16 * S::OSTRIDE * 4 + (size_t)NW * 2 * 16 * 4;
    return stage > merge ? stage : merge;
}

template <int LPR>
__device__ __forceinline__ int v_swizzle(int key)
{
    return ((key & 7) << 1) & (LPR - 1);
}

template <typename T, int D, int NW, int MB, bool kUniformPage>
__global__ __launch_bounds__(NW * 64) void splitkv_decode_kernel(const SplitKvArgs a)
{
    typedef DecodeShape<D> S;
    typedef typename T::vec8 vec8;
    extern __shared__ __attribute__((aligned(16))) char smem[];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int l16 = lane & 15;
    const int kg = lane >> 4;

    const int split = blockIdx.x % a.num_splits;
    const int mtile = blockIdx.x / a.num_splits;
    const int hkv = blockIdx.y;
    const int b = blockIdx.z;
    const int g = a.hq / a.hk;

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
    const int R = sq_b * g;  // packed rows of this (sequence, kv head)
    const int r_tile0 = mtile * 16 * MB;
    if (r_tile0 >= R) return;

    const int per = max(1, (sk_b + a.num_splits - 1) / a.num_splits);
    const int k0 = min(per * split, sk_b);
    const int k1 = min(k0 + per, sk_b);

    const MaskYX mk = make_mask(a.mask_type, a.window_left, a.window_right, sq_b, sk_b);

    // rows of this lane (one per 16-row block)
    int row_i[MB], row_h[MB], lo[MB], hi[MB];
    bool row_ok[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        const int r = r_tile0 + mb * 16 + l16;
        row_ok[mb] = r < R;
        const int rc = row_ok[mb] ? r : 0;
        row_i[mb] = rc / g;
        row_h[mb] = hkv * g + rc % g;
        lo[mb] = max(mask_lo(mk, row_i[mb]), k0);
        hi[mb] = min(mask_hi(mk, row_i[mb], sk_b), k1);
        if (!row_ok[mb]) {
            lo[mb] = 0;
            hi[mb] = 0;
        }
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
    vec8 qf[MB][S::KT];
    {
        const uint16_t* qp = reinterpret_cast<const uint16_t*>(a.q);
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            const int64_t off = ((int64_t)(q_row0 + row_i[mb]) * a.hq + row_h[mb]) * D + kg * 8;
#pragma unroll
            for (int t = 0; t < S::KT; ++t) {
                u32x4_t v = {0u, 0u, 0u, 0u};
                if (row_ok[mb]) v = ldg16(qp + off + t * 32);
                qf[mb][t] = as_vec8<vec8>(v);
            }
        }
    }

    // ---- online softmax state ------------------------------------------------------------------------------
    float m_run[MB], l_run[MB];
    f32x4_t oacc[MB][S::DB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        m_run[mb] = -INFINITY;
        l_run[mb] = 0.f;
#pragma unroll
        for (int db = 0; db < S::DB; ++db) oacc[mb][db] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
    }

    const uint16_t* kp = reinterpret_cast<const uint16_t*>(a.k);
    const uint16_t* vp = reinterpret_cast<const uint16_t*>(a.v);
    const int64_t krow_stride = (int64_t)a.hk * D;
    const int last_key = sk_b - 1;

    // per-lane constants of the V staging tile
    char FCK_LDS* kstage = (char FCK_LDS*)(smem) + wave * 2 * S::VTILE;
    char FCK_LDS* vstage = kstage + S::VTILE;
    int vw_off[S::VN], kw_off[S::VN];
#pragma unroll
    for (int u = 0; u < S::VN; ++u) {
        const int key = u * S::KPI + lane / S::LPR;
        const int chunk = lane % S::LPR;
        vw_off[u] = key * S::VROW + ((chunk ^ v_swizzle<S::LPR>(key)) << 4);
        kw_off[u] = key * S::VROW + ((chunk ^ (key & 7)) << 4);
    }
    // K as the A operand: lane (key = nb * 16 + l16, k-group kg) reads chunk t * 4 + kg of its key row
    const int kr_off = l16 * S::VROW;
    const int kr_sw = l16 & 7;
    const int tr_key = kg * 4 + (l16 >> 2);
    const int tr_sw = v_swizzle<S::LPR>(tr_key);
    const int tr_base = tr_key * S::VROW + ((l16 & 2) << 3) + ((l16 & 1) << 3);

    // ---- loading roles -------------------------------------------------------------------------------------------
    // pair p = waves (2p, 2p+1); in step `it` they own tiles tA = t_begin + 2p + it * NW and tA + 1
    const int role = wave & 1;         // 0: fetches K for the pair, 1: fetches V
    const int pair0 = wave & ~1;       // even wave of the pair
    const int n_iter = (t_end - t_begin + NW - 1) / NW;  // steps of the workgroup (uniform)
    const uint16_t* src = role ? vp : kp;
    char FCK_LDS* stageA = (char FCK_LDS*)(smem) + pair0 * 2 * S::VTILE + role * S::VTILE;  // tile of wave 2p
    char FCK_LDS* stageB = stageA + 2 * S::VTILE;                                           // tile of wave 2p+1

    struct Frag {
        u32x4_t a[2 * S::VN];
    };

    // Page ids of the pair's tiles, 64 steps at a time: lane j holds the pages of step it0 + j, so the loop reads them
    // with v_readlane instead of a dependent scalar load per step.
    int page_regA = 0, page_regB = 0;
    auto page_index = [&](int key) { return a.kv.page_shift >= 0 ? key >> a.kv.page_shift : key / a.kv.page_size; };
    auto clamp_tile = [&](int t) { return min(t, t_end - 1); };
    auto fetch_pages = [&](int it0) {
        const int it = it0 + lane;
        if (ks.table != nullptr && it < n_iter) {
            const int tA = t_begin + pair0 + it * NW;
            page_regA = ks.table[page_index(clamp_tile(tA) * S::TK)];
            page_regB = ks.table[page_index(clamp_tile(tA + 1) * S::TK)];
        }
    };

    auto load_step = [&](int it, Frag& f) {
        if constexpr (kUniformPage) {
            if ((it & 63) == 0) fetch_pages(it);
        }
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            const int tile = clamp_tile(t_begin + pair0 + half + it * NW);
            const int kb = tile * S::TK;
            if constexpr (kUniformPage) {
                // the whole tile lies in one page (or the cache is contiguous): one row base per tile
                int64_t row0;
                if (ks.table != nullptr) {
                    const int page = __builtin_amdgcn_readlane(half ? page_regB : page_regA, it & 63);
                    row0 = (int64_t)page * a.kv.page_size + (kb - page_index(kb) * a.kv.page_size);
                } else {
                    row0 = ks.base_row + kb;
                }
                const int room = last_key - kb;  // largest valid local key
#pragma unroll
                for (int u = 0; u < S::VN; ++u) {
                    const int kl = min(u * S::KPI + lane / S::LPR, room);
                    f.a[half * S::VN + u] = ldg16(src + (row0 + kl) * krow_stride + hkv * D + (lane % S::LPR) * 8);
                }
            } else {
#pragma unroll
                for (int u = 0; u < S::VN; ++u) {
                    const int key = min(kb + u * S::KPI + lane / S::LPR, last_key);
                    f.a[half * S::VN + u] = ldg16(src + kv_row(a.kv, ks, key) * krow_stride + hkv * D + (lane % S::LPR) * 8);
                }
            }
        }
    };
    auto store_step = [&](const Frag& f) {
#pragma unroll
        for (int u = 0; u < S::VN; ++u) {
            const int off = role ? vw_off[u] : kw_off[u];
            *(u32x4_t FCK_LDS*)(stageA + off) = f.a[u];
            *(u32x4_t FCK_LDS*)(stageB + off) = f.a[S::VN + u];
        }
    };

    auto compute_tile = [&](int it) {
        const int kb = (t_begin + wave + it * NW) * S::TK;

        // S^T[key][row] = K . Q^T
        u32x4_t kfrag[2][S::KT];
#pragma unroll
        for (int nb = 0; nb < 2; ++nb)
#pragma unroll
            for (int t = 0; t < S::KT; ++t)
                kfrag[nb][t] = *(const u32x4_t FCK_LDS*)(kstage + nb * 16 * S::VROW + kr_off + (((t * 4 + kg) ^ kr_sw) << 4));
        f32x4_t s[MB][2];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) {
                f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int t = 0; t < S::KT; ++t) acc = T::mfma16(as_vec8<vec8>(kfrag[nb][t]), qf[mb][t], acc);
                s[mb][nb] = acc;
            }

        vec8 pf[MB];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            float x[8];
            float tmax = -INFINITY;
#pragma unroll
            for (int nb = 0; nb < 2; ++nb)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int key = kb + nb * 16 + kg * 4 + j;
                    const bool vis = key >= lo[mb] && key < hi[mb];
                    const float v = vis ? s[mb][nb][j] * a.scale_log2 : -INFINITY;
                    x[nb * 4 + j] = v;
                    tmax = fmaxf(tmax, v);
                }
            tmax = quad16_max(tmax);
            const float m_new = fmaxf(m_run[mb], tmax);
            const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
            const float alpha = fast_exp2(m_run[mb] - m_use);
            m_run[mb] = m_new;
            float psum = 0.f;
            float p[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                p[e] = fast_exp2(x[e] - m_use);
                psum += p[e];
            }
            l_run[mb] = l_run[mb] * alpha + psum;
#pragma unroll
            for (int db = 0; db < S::DB; ++db) oacc[mb][db] *= alpha;
            u32x4_t pk;
            pk[0] = T::pack2(p[0], p[1]);
            pk[1] = T::pack2(p[2], p[3]);
            pk[2] = T::pack2(p[4], p[5]);
            pk[3] = T::pack2(p[6], p[7]);
            pf[mb] = as_vec8<vec8>(pk);
        }

        // O^T[dv][row] += V^T . P^T
#pragma unroll
        for (int db = 0; db < S::DB; ++db) {
            const int coff = tr_base + ((((db * 2) ^ tr_sw)) << 4);
            const u32x2_t lo4 = lds_read_tr16(vstage + coff);
            const u32x2_t hi4 = lds_read_tr16(vstage + coff + 16 * S::VROW);
            u32x4_t av = {lo4[0], lo4[1], hi4[0], hi4[1]};
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) oacc[mb][db] = T::mfma16(as_vec8<vec8>(av), pf[mb], oacc[mb][db]);
        }
    };

    // Software pipeline over the steps of the workgroup.  The last step is peeled so that the prefetch is unconditional
    // inside the loop (a conditional prefetch makes the wait counters at the join cover both paths, which serialises
    // load and compute).  Two workgroup barriers per step: all tiles read / next tiles written.
    if (n_iter > 0) {
        {
            Frag f0;
            load_step(0, f0);
            store_step(f0);
        }
        __syncthreads();
        int it = 0;
        for (; it + 1 < n_iter; ++it) {
            Frag pre;
            load_step(it + 1, pre);
            if (t_begin + wave + it * NW < t_end) compute_tile(it);
            __syncthreads();
            store_step(pre);
            __syncthreads();
        }
        if (t_begin + wave + it * NW < t_end) compute_tile(it);
    }

    // ---- merge the NW partial states --------------------------------------------------------------------------
    // each lane owns a partial row sum over its 8 key slots per tile: fold the 4 lanes of a row
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        l_run[mb] = quad16_sum(l_run[mb]);
    }

    float* obuf = reinterpret_cast<float*>(smem);                       // [NW][16][OSTRIDE]
    float* mlbuf = obuf + NW * 16 * S::OSTRIDE;                         // [NW][2][16]
    constexpr int NT = NW * 64;
    float* o_acc = a.o_acc;
    float* lse_acc = a.lse_acc;

#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        __syncthreads();  // staging tiles (or the previous block's merge data) are no longer read
        float* ow = obuf + (wave * 16 + l16) * S::OSTRIDE + kg * 4;
#pragma unroll
        for (int db = 0; db < S::DB; ++db) *reinterpret_cast<f32x4_t*>(ow + db * 16) = oacc[mb][db];
        if (kg == 0) {
            mlbuf[(wave * 2 + 0) * 16 + l16] = m_run[mb];
            mlbuf[(wave * 2 + 1) * 16 + l16] = l_run[mb];
        }
        __syncthreads();
        for (int e = threadIdx.x; e < 16 * D; e += NT) {
            const int rr = e / D, c = e % D;
            const int r = r_tile0 + mb * 16 + rr;
            if (r >= R) continue;
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
            const int i = r / g, h = hkv * g + r % g;
            const int64_t wofs = ((int64_t)(wb * a.hq + h) * a.num_splits + split) * Sq + wrow0 + i;
            o_acc[wofs * D + c] = (L == 0.f) ? 0.f : acc / L;
            if (c == 0) lse_acc[wofs] = (L == 0.f) ? -INFINITY : (mmax + fast_log2(L)) * kLn2;
        }
    }
}

// ------------------------------------------------------------------------------------------------------
template <typename T, int D, int NW, int MB>
static hipError_t launch_cfg(const SplitKvArgs& a, int m_tiles, bool uniform, hipStream_t st)
{
    const dim3 grid(m_tiles * a.num_splits, a.hk, a.batch);
    const dim3 block(NW * 64);
    constexpr size_t lds = decode_lds_bytes<D, NW>();
    hipError_t e;
    if (uniform) {
        auto kern = splitkv_decode_kernel<T, D, NW, MB, true>;
        static bool once = false;
        if (!once) {
            e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return e;
            once = true;
        }
        hipLaunchKernelGGL(kern, grid, block, lds, st, a);
    } else {
        auto kern = splitkv_decode_kernel<T, D, NW, MB, false>;
        static bool once = false;
        if (!once) {
            e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return e;
            once = true;
        }
        hipLaunchKernelGGL(kern, grid, block, lds, st, a);
    }
    return hipGetLastError();
}

template <typename T, int D>
static hipError_t launch_mb(const SplitKvArgs& a, int rows_max, bool uniform, hipStream_t st)
{
    // 8 waves (2 per SIMD, 256 VGPRs each) when one 16-row block is enough; 4 waves (512 VGPRs) when a lane carries
    // the accumulators of several row blocks or of a 256-wide head.
    if constexpr (D == 256) {
        if (rows_max <= 16) return launch_cfg<T, D, 4, 1>(a, 1, uniform, st);
        return launch_cfg<T, D, 4, 2>(a, (rows_max + 31) / 32, uniform, st);
    } else {
        if (rows_max <= 16) return launch_cfg<T, D, 8, 1>(a, 1, uniform, st);
        if (rows_max <= 32) return launch_cfg<T, D, 4, 2>(a, 1, uniform, st);
        return launch_cfg<T, D, 4, 4>(a, (rows_max + 63) / 64, uniform, st);
    }
}

template <typename T>
static hipError_t launch_d(const SplitKvArgs& a, int d, int rows_max, bool uniform, hipStream_t st)
{
    switch (d) {
    case 64: return launch_mb<T, 64>(a, rows_max, uniform, st);
    case 128: return launch_mb<T, 128>(a, rows_max, uniform, st);
    case 256: return launch_mb<T, 256>(a, rows_max, uniform, st);
    }
    return hipErrorInvalidValue;
}

hipError_t launch_splitkv_decode(const SplitKvArgs& a, int d, int dtype, int rows_max, bool uniform_page,
                                 hipStream_t st)
{
    if (dtype == 4) return launch_d<BF16>(a, d, rows_max, uniform_page, st);
    return launch_d<FP16>(a, d, rows_max, uniform_page, st);
}

}  // namespace fck
