// Fused attention-JVP forward kernel (gfx950).
//
// Computes what semicat/jvp_utils/ryu_triton.py:73-291 computes - O, TO, M (= lse), MU, LI in one
// online-softmax pass - with a different decomposition: a workgroup of four wavefronts owns 128
// query rows of one (batch, head); each wavefront owns 32 of them as MFMA columns and walks over
// the keys in tiles of 32 staged in LDS (K, K_dot, V, V_dot row-major, shared by the four waves).
// Scores are produced transposed (S^T = K Q^T) so that the running maximum, the exp-sum and mu are
// per-lane scalars and the probability tile is directly the B operand of O^T += V^T P^T.
#pragma once
#include "sjvp_device.hpp"

namespace sjvp {

struct FwdParams {
    TensorView q, k, v, tq, tk, tv;
    elem_t* o;
    int64_t o_sb, o_sh, o_sl;
    elem_t* to;
    int64_t to_sb, to_sh, to_sl;
    float* lse;
    float* mu;
    float* li;
    int H, Lq, Lk, D, Lr;
    int q_blocks;  // ceil(Lq / 128)
    float scale;
    int vec;  // all tensors 16-byte aligned, strides % 8 == 0, D % 8 == 0
};

template <int HD, int BN, bool JVP>
struct FwdSmem {
    static constexpr int tile = BN * Pitch<HD>::value;          // elements per staged tensor
    static constexpr int bytes = (JVP ? 4 : 2) * tile * (int)sizeof(elem_t);
};

template <typename T, int HD, int BN, bool JVP>
__global__ __launch_bounds__(kThreads) void fwd_kernel(const FwdParams p) {
    extern __shared__ __align__(16) unsigned char smem_raw[];
    elem_t* sK = reinterpret_cast<elem_t*>(smem_raw);
    elem_t* sV = sK + FwdSmem<HD, BN, JVP>::tile;
    elem_t* sTK = sV + FwdSmem<HD, BN, JVP>::tile;
    elem_t* sTV = sTK + FwdSmem<HD, BN, JVP>::tile;

    constexpr int KC = HD / 16;  // k-chunks of the score contraction
    constexpr int DT = HD / 32;  // 32-wide tiles of the head dimension

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int x = lane & 31;
    const int hf = lane >> 5;

    const int bh = blockIdx.x / p.q_blocks;
    const int qb = blockIdx.x % p.q_blocks;
    const int b = bh / p.H, h = bh % p.H;
    const bool vec = p.vec != 0;

    const int qrow = qb * kOwned + wave * 32 + x;  // the query this lane owns
    const bool qvalid = qrow < p.Lq;
    const bool wave_active = (qb * kOwned + wave * 32) < p.Lq;

    // Owned-side operands (B of S^T = K Q^T), kept in registers for the whole pass.
    u32x4 qB[KC], tqB[KC];
    {
        const elem_t* qp = p.q.head(b, h) + (int64_t)qrow * p.q.sl;
#pragma unroll
        for (int c = 0; c < KC; ++c) qB[c] = load8(qp, 16 * c + 8 * hf, p.D, qvalid, vec);
        if constexpr (JVP) {
            const elem_t* tqp = p.tq.head(b, h) + (int64_t)qrow * p.tq.sl;
#pragma unroll
            for (int c = 0; c < KC; ++c) tqB[c] = load8(tqp, 16 * c + 8 * hf, p.D, qvalid, vec);
        }
    }

    const elem_t* kg = p.k.head(b, h);
    const elem_t* vg = p.v.head(b, h);
    const elem_t* tkg = JVP ? p.tk.head(b, h) : nullptr;
    const elem_t* tvg = JVP ? p.tv.head(b, h) : nullptr;

    // log2-domain softmax: s2 = S * scale * log2(e)
    const float sl2 = p.scale * kLog2e;
    float m_i = -INFINITY;  // running max (same in both half-lanes of a query)
    float l_i = 0.f;        // exp-sum over the keys this half-lane has seen
    float mu_i = 0.f;       // sum of p * S_dot over the same keys
    f32x16 acc[DT], gacc[DT], pacc[DT];
#pragma unroll
    for (int t = 0; t < DT; ++t) {
        acc[t] = f32x16{0};
        if constexpr (JVP) {
            gacc[t] = f32x16{0};
            pacc[t] = f32x16{0};
        }
    }

    for (int k0 = 0; k0 < p.Lk; k0 += BN) {
        __syncthreads();  // previous stage fully consumed
        stage_rows<HD, BN>(sK, kg, p.k.sl, k0, p.Lk, p.D, vec, tid);
        stage_rows<HD, BN>(sV, vg, p.v.sl, k0, p.Lk, p.D, vec, tid);
        if constexpr (JVP) {
            stage_rows<HD, BN>(sTK, tkg, p.tk.sl, k0, p.Lk, p.D, vec, tid);
            stage_rows<HD, BN>(sTV, tvg, p.tv.sl, k0, p.Lk, p.D, vec, tid);
        }
        __syncthreads();
        if (!wave_active) continue;

#pragma unroll
        for (int t = 0; t < BN / 32; ++t) {
            const int y0 = 32 * t;
            if (k0 + y0 >= p.Lk) break;
            f32x16 s = {0}, ts = {0};
#pragma unroll
            for (int c = 0; c < KC; ++c) {
                u32x4 a = lds_a_rows<HD>(sK, y0, c, x, hf);
                s = T::mfma(a, qB[c], s);
                if constexpr (JVP) {
                    ts = T::mfma(a, tqB[c], ts);
                    u32x4 at = lds_a_rows<HD>(sTK, y0, c, x, hf);
                    ts = T::mfma(at, qB[c], ts);
                }
            }
            const bool ragged = (k0 + y0 + 32 > p.Lk);
            float mloc = -INFINITY;
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                float sv = s[j] * sl2;
                if (ragged) {
                    int key = k0 + y0 + 8 * (j >> 2) + 4 * hf + (j & 3);
                    if (key >= p.Lk) {
                        sv = -INFINITY;
                        if constexpr (JVP) ts[j] = 0.f;
                    }
                }
                s[j] = sv;
                mloc = fmaxf(mloc, sv);
            }
            mloc = fmaxf(mloc, other_half(mloc));
            const float m_new = fmaxf(m_i, mloc);
            const float alpha = fast_exp2(m_i - m_new);
            m_i = m_new;
            float lsum = 0.f, musum = 0.f;
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                float pj = fast_exp2(s[j] - m_new);
                s[j] = pj;
                lsum += pj;
                if constexpr (JVP) {
                    float pt = pj * (ts[j] * p.scale);
                    ts[j] = pt;
                    musum += pt;
                }
            }
            l_i = l_i * alpha + lsum;
            if constexpr (JVP) mu_i = mu_i * alpha + musum;
#pragma unroll
            for (int d = 0; d < DT; ++d) {
                acc[d] *= alpha;
                if constexpr (JVP) {
                    gacc[d] *= alpha;
                    pacc[d] *= alpha;
                }
            }
#pragma unroll
            for (int c = 0; c < 2; ++c) {
                u32x4 pb = pack_b<T>(s, c);
                u32x4 ptb;
                if constexpr (JVP) ptb = pack_b<T>(ts, c);
#pragma unroll
                for (int d = 0; d < DT; ++d) {
                    u32x4 av = lds_a_transposed<HD>(sV, y0, c, 32 * d, lane);
                    acc[d] = T::mfma(av, pb, acc[d]);
                    if constexpr (JVP) {
                        gacc[d] = T::mfma(av, ptb, gacc[d]);
                        u32x4 atv = lds_a_transposed<HD>(sTV, y0, c, 32 * d, lane);
                        pacc[d] = T::mfma(atv, pb, pacc[d]);
                    }
                }
            }
        }
    }

    if (!wave_active) {
        // All 32 rows of this wave lie beyond Lq: their statistic rows get the values a zero
        // query row produces (and the reference initialises them with): log(Lk), 0, Lk.
        if (hf == 0) {
            const int64_t so = (int64_t)bh * p.Lr + qrow;
            p.lse[so] = fast_log2((float)p.Lk) * kLn2;
            if constexpr (JVP) p.mu[so] = 0.f;
            if (p.li) p.li[so] = (float)p.Lk;
        }
        return;
    }

    // Combine the two half-lanes' partial sums (they cover disjoint keys of the same query).
    const float l = l_i + other_half(l_i);
    const float inv_l = 1.0f / l;
    float mu_un = 0.f;
    if constexpr (JVP) mu_un = mu_i + other_half(mu_i);

    if (hf == 0) {
        // Statistic rows up to Lr are all written: a padded query row (all-zero q, q_dot) yields
        // exactly the values the reference initialises them with: log(Lk), 0, Lk.
        const int64_t so = (int64_t)bh * p.Lr + qrow;
        p.lse[so] = (m_i + fast_log2(l)) * kLn2;
        if constexpr (JVP) p.mu[so] = mu_un * inv_l;
        if (p.li) p.li[so] = l;
    }
    if (!qvalid) return;

    elem_t* orow = p.o + b * p.o_sb + h * p.o_sh + (int64_t)qrow * p.o_sl;
#pragma unroll
    for (int d = 0; d < DT; ++d) store_acc<T>(orow, 32 * d, hf, p.D, acc[d], inv_l, vec);
    if constexpr (JVP) {
        // TO = (g_acc - mu_un * O + p_tv_acc) / l     (ryu_triton.py:274-275)
        elem_t* trow = p.to + b * p.to_sb + h * p.to_sh + (int64_t)qrow * p.to_sl;
        const float cmu = mu_un * inv_l;
#pragma unroll
        for (int d = 0; d < DT; ++d) {
            f32x16 t;
#pragma unroll
            for (int j = 0; j < 16; ++j) t[j] = gacc[d][j] - cmu * acc[d][j] + pacc[d][j];
            store_acc<T>(trow, 32 * d, hf, p.D, t, inv_l, vec);
        }
    }
}

}  // namespace sjvp
