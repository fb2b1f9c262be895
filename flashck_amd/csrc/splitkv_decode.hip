// Split-KV forward for short query lengths (decode): hand-written gfx950 kernel.
//
// Work decomposition
//   grid  = (m_tiles * num_splits, Hk, B); one workgroup owns one split of one KV head of one sequence and the
//           16*MB packed query rows (query index, head-in-group) that share that KV head.
//   waves = NW per workgroup; wave w walks the 32-key tiles w, w+NW, ... of the split with its own online-softmax
//           state; the NW partial states are merged through LDS at the end.
// Data path per 32-key tile and wave
//   K   global -> VGPR directly in MFMA operand order (16 keys x 64 B per load instruction);
//   V   global -> VGPR with whole 2*D-byte rows per 16*D/128 lanes, staged in a wave-private, XOR-swizzled LDS tile
//       and read back transposed (ds_read_b64_tr_b16) as the A operand of O^T += V^T . P^T;
//   S^T = K . Q^T with v_mfma_f32_16x16x32, so that each lane keeps the scores of one query row and the
//       probabilities it produces are already laid out as the B operand of the second product.
// Loads of tile i+1 are issued before the arithmetic of tile i.
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
    const size_t stage = (size_t)NW * S::VTILE;
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
    char FCK_LDS* vstage = (char FCK_LDS*)(smem) + wave * S::VTILE;
    int vw_off[S::VN];
#pragma unroll
    for (int u = 0; u < S::VN; ++u) {
        const int key = u * S::KPI + lane / S::LPR;
        const int chunk = lane % S::LPR;
        vw_off[u] = key * S::VROW + ((chunk ^ v_swizzle<S::LPR>(key)) << 4);
    }
    const int tr_key = kg * 4 + (l16 >> 2);
    const int tr_sw = v_swizzle<S::LPR>(tr_key);
    const int tr_base = tr_key * S::VROW + ((l16 & 2) << 3) + ((l16 & 1) << 3);

    struct Frag {
        u32x4_t k[2][S::KT];
        u32x4_t v[S::VN];
    };

    auto load_tile = [&](int tile, Frag& f) {
        const int kb = tile * S::TK;
        if constexpr (kUniformPage) {
            // the whole tile lies in one page (or the cache is contiguous): one row base per tile
            const int kbc = min(kb, last_key);
            const int64_t row0 = kv_row(a.kv, ks, kbc) - (kbc - kb);
            const int room = last_key - kb;  // largest valid local key
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) {
                const int kl = min(nb * 16 + l16, room);
                const uint16_t* p = kp + (row0 + kl) * krow_stride + hkv * D + kg * 8;
#pragma unroll
                for (int t = 0; t < S::KT; ++t) f.k[nb][t] = ldg16(p + t * 32);
            }
#pragma unroll
            for (int u = 0; u < S::VN; ++u) {
                const int kl = min(u * S::KPI + lane / S::LPR, room);
                f.v[u] = ldg16(vp + (row0 + kl) * krow_stride + hkv * D + (lane % S::LPR) * 8);
            }
        } else {
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) {
                const int key = min(kb + nb * 16 + l16, last_key);
                const uint16_t* p = kp + kv_row(a.kv, ks, key) * krow_stride + hkv * D + kg * 8;
#pragma unroll
                for (int t = 0; t < S::KT; ++t) f.k[nb][t] = ldg16(p + t * 32);
            }
#pragma unroll
            for (int u = 0; u < S::VN; ++u) {
                const int key = min(kb + u * S::KPI + lane / S::LPR, last_key);
                f.v[u] = ldg16(vp + kv_row(a.kv, ks, key) * krow_stride + hkv * D + (lane % S::LPR) * 8);
            }
        }
    };

    auto compute_tile = [&](int tile, const Frag& f) {
        const int kb = tile * S::TK;
        // stage V (wave private): write rows, then read them back transposed
#pragma unroll
        for (int u = 0; u < S::VN; ++u) *(u32x4_t FCK_LDS*)(vstage + vw_off[u]) = f.v[u];

        // S^T[key][row] = K . Q^T
        f32x4_t s[MB][2];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) {
                f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int t = 0; t < S::KT; ++t) acc = T::mfma16(as_vec8<vec8>(f.k[nb][t]), qf[mb][t], acc);
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
            tmax = fmaxf(tmax, __shfl_xor(tmax, 16));
            tmax = fmaxf(tmax, __shfl_xor(tmax, 32));
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
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int db = 0; db < S::DB; ++db) {
            const int coff = tr_base + ((((db * 2) ^ tr_sw)) << 4);
            const u32x2_t lo4 = lds_read_tr16(vstage + coff);
            const u32x2_t hi4 = lds_read_tr16(vstage + coff + 16 * S::VROW);
            u32x4_t av = {lo4[0], lo4[1], hi4[0], hi4[1]};
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) oacc[mb][db] = T::mfma16(as_vec8<vec8>(av), pf[mb], oacc[mb][db]);
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    };

    {
        int tile = t_begin + wave;
        if (tile < t_end) {
            Frag cur;
            load_tile(tile, cur);
            while (true) {
                const int nxt = tile + NW;
                const bool more = nxt < t_end;
                Frag pre;
                if (more) load_tile(nxt, pre);
                compute_tile(tile, cur);
                if (!more) break;
                cur = pre;
                tile = nxt;
            }
        }
    }

    // ---- merge the NW partial states --------------------------------------------------------------------------
    // each lane owns a partial row sum over its 8 key slots per tile: fold the 4 lanes of a row
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        l_run[mb] += __shfl_xor(l_run[mb], 16);
        l_run[mb] += __shfl_xor(l_run[mb], 32);
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
