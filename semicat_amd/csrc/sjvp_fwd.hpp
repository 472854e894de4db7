// Fused attention-JVP forward kernel, 32-wide form for inputs of any alignment (gfx950).
//
// Computes what semicat/jvp_utils/ryu_triton.py:73-291 computes - O, TO, M (= lse), MU, LI in one
// online-softmax pass - with a different decomposition: a workgroup of four wavefronts owns 128
// query rows of one (batch, head); each wavefront owns 32 of them as MFMA columns and walks over
// the keys in stages of 32 copied through registers into one LDS stage (K, V, K_dot, V_dot; shared
// by the four waves).  Scores are produced transposed (S^T = K Q^T) so that the running maximum,
// the exp-sum and mu are per-lane scalars and the probability tile is directly the B operand of
// O^T += V^T P^T.  Inputs whose rows are 16-byte aligned take the 16-wide kernel of sjvp_fwd16.hpp
// instead; this one serves the rest (odd head dimensions, misaligned pointers or strides).
#pragma once
#include <type_traits>

#include "sjvp_device.hpp"

namespace sjvp {

struct FwdParams {
    TensorView q, k, v, tq, tk, tv;
    OutView o, to;
    float* lse;
    float* mu;
    float* li;
    int H, Lq, Lk, D, Lr;
    int q_blocks;  // workgroups per (batch, head): Lr / (32 * waves per workgroup)
    float scale;
    int vec;  // all tensors 16-byte aligned, strides % 8 == 0, D % 8 == 0
    RopeTables rope;  // rotation of q, k (and their tangents) as they are loaded; cos == null: none
};

// LDS layout: one stage of K, V (, K_dot, V_dot) slabs.
template <int HD, bool JVP>
struct FwdSmem {
    static constexpr int nt = JVP ? 4 : 2;             // tensors per stage
    static constexpr int slot = nt * Slab<HD>::elems;  // elements of the stage
    static constexpr int bytes = slot * (int)sizeof(elem_t);
};

// The reference maximum of the online softmax is only raised when a new tile exceeds it by more
// than this many log2 units.  Any reference point is valid as long as exp2 stays in range: the
// unnormalised probabilities are then bounded by 2^kMaxSlack instead of 1 and the final division
// by the exp-sum is unaffected.  This keeps the accumulator rescale out of almost every tile.
constexpr float kMaxSlack = 6.0f;

template <typename T, int HD, bool JVP, bool F32IO = false>
__global__ __launch_bounds__(kThreads, 1) void fwd_kernel(const FwdParams p) {
    extern __shared__ __align__(16) unsigned char smem_raw[];
    elem_t* stage = reinterpret_cast<elem_t*>(smem_raw);

    constexpr int KC = HD / 16;  // k-chunks of the score contraction
    constexpr int DT = HD / 32;  // 32-wide tiles of the head dimension

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int x = lane & 31;
    const int hf = lane >> 5;

    const int bh = blockIdx.x / p.q_blocks;
    const int qb = blockIdx.x % p.q_blocks;
    const int b = bh / p.H, h = bh % p.H;
    const bool vec = p.vec != 0;
    SlabLane<HD> ln;
    ln.init(tid);
    const int qrow = qb * kOwned + wave * 32 + x;  // the query this lane owns
    const bool qvalid = qrow < p.Lq;
    const bool wave_active = (qb * kOwned + wave * 32) < p.Lq;

    // Owned-side operands (B of S^T = K Q^T), kept in registers for the whole pass.
    u32x4 qB[KC], tqB[KC];
    {
        const elem_t* qp = p.q.head(b, h) + (int64_t)qrow * p.q.sl;
#pragma unroll
        for (int c = 0; c < KC; ++c) qB[c] = load8_io<T, F32IO>(qp, 16 * c + 8 * hf, p.D, qvalid, vec);
        if constexpr (JVP) {
            const elem_t* tqp = p.tq.head(b, h) + (int64_t)qrow * p.tq.sl;
#pragma unroll
            for (int c = 0; c < KC; ++c) tqB[c] = load8_io<T, F32IO>(tqp, 16 * c + 8 * hf, p.D, qvalid, vec);
        }
    }
    const elem_t* kg = p.k.head(b, h);
    const elem_t* vg = p.v.head(b, h);
    const elem_t* tkg = JVP ? p.tk.head(b, h) : nullptr;
    const elem_t* tvg = JVP ? p.tv.head(b, h) : nullptr;

    auto fill = [&](int st) {
        const int row0 = st * kStageRows;
        fill_slab<HD, T, F32IO>(ln, stage, kg, p.k.sl, row0, p.Lk, p.D, vec);
        fill_slab<HD, T, F32IO>(ln, stage + Slab<HD>::elems, vg, p.v.sl, row0, p.Lk, p.D, vec);
        if constexpr (JVP) {
            fill_slab<HD, T, F32IO>(ln, stage + 2 * Slab<HD>::elems, tkg, p.tk.sl, row0, p.Lk, p.D, vec);
            fill_slab<HD, T, F32IO>(ln, stage + 3 * Slab<HD>::elems, tvg, p.tv.sl, row0, p.Lk, p.D, vec);
        }
    };

    // log2-domain softmax: exponent = S * (scale*log2 e) - m
    const float sl2 = p.scale * kLog2e;
    float m_i = -INFINITY;    // reference maximum (same in both half-lanes of a query)
    float m_true = -INFINITY; // true running maximum (only needed to report LI)
    float l_i = 0.f;          // exp-sum over the keys this half-lane has seen
    float mu_i = 0.f;         // sum of p * S_dot over the same keys
    // acc = sum P~ V;  tacc = sum (P~ * S_dot) V + P~ V_dot  (the reference's g_acc + p_tv_acc, which
    // only ever appear added together, ryu_triton.py:274-275)
    f32x16 acc[DT], tacc[DT];
#pragma unroll
    for (int t = 0; t < DT; ++t) {
        acc[t] = f32x16{0};
        if constexpr (JVP) tacc[t] = f32x16{0};
    }

    // One online-softmax step over the stage in LDS (keys k0 .. k0+31).
    auto compute = [&](int k0, auto ragged_tag) {
        constexpr int NS = 1;
        constexpr bool RAGGED = decltype(ragged_tag)::value;
        const elem_t* slots[1] = {stage};
        f32x16 s[NS], ts[NS];
#pragma unroll
        for (int g = 0; g < NS; ++g) {
            s[g] = f32x16{0};
            ts[g] = f32x16{0};
        }
#pragma unroll
        for (int c = 0; c < KC; ++c) {
#pragma unroll
            for (int g = 0; g < NS; ++g) {
                u32x4 a = lds_a_rows<HD>(slots[g], c, x, hf);
                s[g] = T::mfma(a, qB[c], s[g]);
                if constexpr (JVP) {
                    ts[g] = T::mfma(a, tqB[c], ts[g]);
                    u32x4 at = lds_a_rows<HD>(slots[g] + 2 * Slab<HD>::elems, c, x, hf);
                    ts[g] = T::mfma(at, qB[c], ts[g]);
                }
            }
        }
        if constexpr (RAGGED) {
            // keys beyond Lk are zero rows in LDS (their S_dot is already 0)
            const int kl = k0 + (NS - 1) * kStageRows;
#pragma unroll
            for (int j = 0; j < 16; ++j)
                if (kl + 8 * (j >> 2) + 4 * hf + (j & 3) >= p.Lk) s[NS - 1][j] = -INFINITY;
        }
        float mloc = -INFINITY;
#pragma unroll
        for (int g = 0; g < NS; ++g)
#pragma unroll
            for (int j = 0; j < 16; j += 4)
                mloc = fmaxf(mloc, fmaxf(fmaxf(s[g][j], s[g][j + 1]), fmaxf(s[g][j + 2], s[g][j + 3])));
        mloc = fmaxf(mloc, other_half(mloc)) * sl2;
        m_true = fmaxf(m_true, mloc);
        if (__builtin_amdgcn_ballot_w64(mloc > m_i + kMaxSlack) != 0) {  // wave-uniform branch
            const float m_new = fmaxf(m_i, mloc);
            const float alpha = fast_exp2(m_i - m_new);  // 0 on the first tile
            m_i = m_new;
            l_i *= alpha;
            if constexpr (JVP) mu_i *= alpha;
#pragma unroll
            for (int d = 0; d < DT; ++d) {
                acc[d] *= alpha;
                if constexpr (JVP) tacc[d] *= alpha;
            }
        }
        float lsum = 0.f, musum = 0.f;
#pragma unroll
        for (int g = 0; g < NS; ++g) {
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                const float pj = fast_exp2(fmaf(s[g][j], sl2, -m_i));
                s[g][j] = pj;
                lsum += pj;
                if constexpr (JVP) {
                    const float pt = pj * (ts[g][j] * p.scale);
                    ts[g][j] = pt;
                    musum += pt;
                }
            }
        }
        l_i += lsum;
        if constexpr (JVP) mu_i += musum;
#pragma unroll
        for (int c = 0; c < 2; ++c) {
#pragma unroll
            for (int g = 0; g < NS; ++g) {
                const elem_t* sV = slots[g] + Slab<HD>::elems;
                const elem_t* sTV = slots[g] + 3 * Slab<HD>::elems;
                u32x4 pb = pack_b<T>(s[g], c);
                u32x4 ptb;
                if constexpr (JVP) ptb = pack_b<T>(ts[g], c);
#pragma unroll
                for (int d = 0; d < DT; ++d) {
                    u32x4 av = lds_a_transposed<HD>(sV, c, 32 * d, lane);
                    acc[d] = T::mfma(av, pb, acc[d]);
                    if constexpr (JVP) {
                        tacc[d] = T::mfma(av, ptb, tacc[d]);
                        u32x4 atv = lds_a_transposed<HD>(sTV, c, 32 * d, lane);
                        tacc[d] = T::mfma(atv, pb, tacc[d]);
                    }
                }
            }
        }
    };

    const int n = (p.Lk + kStageRows - 1) / kStageRows;
    for (int i = 0; i < n; ++i) {
        workgroup_barrier();  // the previous stage is fully consumed
        fill(i);
        workgroup_barrier();
        if (!wave_active) continue;
        const int k0 = i * kStageRows;
        if (k0 + kStageRows > p.Lk) compute(k0, std::true_type{});
        else compute(k0, std::false_type{});
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
        // LI is the exp-sum relative to the true row maximum (ryu_triton.py:291); l is relative
        // to m_i, which may lag behind it by up to kMaxSlack.
        if (p.li) p.li[so] = l * fast_exp2(m_i - m_true);
    }
    const float cmu = mu_un * inv_l;
    if constexpr (JVP) {
        // TO = (g_acc + p_tv_acc - mu_un * O) / l     (ryu_triton.py:274-275)
#pragma unroll
        for (int d = 0; d < DT; ++d)
#pragma unroll
            for (int j = 0; j < 16; ++j) tacc[d][j] -= cmu * acc[d][j];
    }
    if (!qvalid) return;
    elem_t* orow = p.o.head(b, h) + (int64_t)qrow * p.o.sl;
#pragma unroll
    for (int d = 0; d < DT; ++d) store_acc<T, F32IO>(orow, 32 * d, hf, p.D, acc[d], inv_l, vec);
    if constexpr (JVP) {
        elem_t* trow = p.to.head(b, h) + (int64_t)qrow * p.to.sl;
#pragma unroll
        for (int d = 0; d < DT; ++d) store_acc<T, F32IO>(trow, 32 * d, hf, p.D, tacc[d], inv_l, vec);
    }
}

}  // namespace sjvp
