// Fused attention-JVP forward, 16-wide form (gfx950; inputs with 16-byte aligned rows).
//
// Same mathematics and outputs as fwd_kernel (semicat/jvp_utils/ryu_triton.py:73-291: O, TO, M = lse,
// MU, LI in one online-softmax pass), decomposed for occupancy: a workgroup of eight wavefronts owns
// 128 queries of one (batch, head), 16 per wavefront as MFMA columns, and walks over the keys in
// stages of 32 streamed through an LDS ring by LDS-DMA.  A wavefront needs fewer than 128 registers,
// so several wavefronts per SIMD overlap their MFMA chains, exponentials and LDS reads, and two
// workgroups per CU overlap one's copies with the other's arithmetic.
#pragma once
#include "sjvp_fwd.hpp"
#include "sjvp_w16.hpp"

namespace sjvp {

// LDS layout, SPB = 1 (one stage per barrier): [own: Q (, Q_dot) rows of the workgroup, four slabs
// each][ring: R slots of K, V (, K_dot, V_dot) stage slabs][sink].  SPB = 2 (long key axes: two stages
// per barrier, half as many barriers): [ring of four slots][sink]; the own rows, which every wave
// moves into registers before the first stage is consumed, land in slots 2 and 3 (exactly their
// size), which then join the ring.  After the last stage the ring doubles as the per-wave staging
// tiles of the output stores.
template <int HD, int R, bool JVP, int SPB = 1>
struct Fwd16Smem {
    static constexpr int nt = JVP ? 4 : 2;
    static constexpr int slot = nt * Slab<HD>::elems;
    static constexpr int own = (JVP ? 2 : 1) * 4 * Slab<HD>::elems;
    static_assert(SPB == 1 || (SPB == 2 && R == 4 && own == 2 * slot), "SPB = 2 needs a ring of four slots");
    static constexpr int own_off = SPB == 2 ? 2 * slot : 0;
    static constexpr int ring_off = SPB == 2 ? 0 : own;
    static constexpr int sink = (SPB == 2 ? R * slot : own + R * slot) * (int)sizeof(elem_t);
    static constexpr int bytes = sink + kSink16;
    static_assert(R * slot >= kWaves16 * StoreStage16<HD>::elems, "ring too small to stage stores");
};

// ROPE: q, k and their tangents are rotated by p.rope as they are loaded (head dimension 64, one
// stage per barrier): the own rows in registers, each stage's K (, K_dot) slab in place in LDS.  Meant
// for key axes that one workgroup per (batch, head) walks once (every workgroup rotates the K rows it
// streams).
template <typename T, int HD, int R, bool JVP, int OCC, int SPB = 1, bool ROPE = false>
__global__ __launch_bounds__(kThreads16, OCC) void fwd16_kernel(const FwdParams p) {
    static_assert(!ROPE || (HD == 64 && SPB == 1), "the folded rotation covers HD = 64, one stage per barrier");
    extern __shared__ __align__(16) unsigned char smem_raw[];
    using SM = Fwd16Smem<HD, R, JVP, SPB>;
    elem_t* own = reinterpret_cast<elem_t*>(smem_raw) + SM::own_off;
    elem_t* ring = reinterpret_cast<elem_t*>(smem_raw) + SM::ring_off;
    constexpr int SE = Slab<HD>::elems;
    constexpr int KC = HD / 32;  // k-chunks of the score contraction
    constexpr int DT = HD / 16;  // 16-wide tiles of the head dimension

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 15;  // owned query within the wave
    const int g = lane >> 4;  // lane group
    // with one workgroup per (batch, head) the identity is kept: the fused backward relies on head i
    // having run on XCD i % 8
    const int bid = p.q_blocks > 1 ? xcd_linear_id((int)blockIdx.x, (int)gridDim.x) : (int)blockIdx.x;
    const int bh = bid / p.q_blocks;
    const int qb = bid % p.q_blocks;
    const int b = bh / p.H, h = bh % p.H;
    const int q0 = qb * kOwned16;
    const int qrow = q0 + wave * 16 + n;
    const bool wave_active = (q0 + wave * 16) < p.Lq;

    // own rows first (issued before the stages, so they land first), then the ring
    {
        CopyPlan<HD, JVP ? 8 : 4, 4> own_plan;
        if constexpr (JVP)
            own_plan.init(tid, q0, p.D, smem_raw + SM::sink, Src{p.q.head(b, h), p.q.sl},
                          Src{p.tq.head(b, h), p.tq.sl});
        else
            own_plan.init(tid, q0, p.D, smem_raw + SM::sink, Src{p.q.head(b, h), p.q.sl});
        own_plan.issue(own, p.Lq - q0, p.D == HD && q0 + kOwned16 <= p.Lq);
    }
    using StagePlan = CopyPlan<HD, SM::nt, 1>;
    constexpr int SPT = StagePlan::N;
    StagePlan plan;
    // slot layout K | V | K_dot | V_dot (primal only: K | V)
    if constexpr (JVP)
        plan.init(tid, 0, p.D, smem_raw + SM::sink, Src{p.k.head(b, h), p.k.sl}, Src{p.v.head(b, h), p.v.sl},
                  Src{p.tk.head(b, h), p.tk.sl}, Src{p.tv.head(b, h), p.tv.sl});
    else
        plan.init(tid, 0, p.D, smem_raw + SM::sink, Src{p.k.head(b, h), p.k.sl}, Src{p.v.head(b, h), p.v.sl});
    const int ns = (p.Lk + kStageRows - 1) / kStageRows;
    int issued = 0;
    auto issue_next = [&]() {
        plan.issue(ring + (issued % R) * SM::slot, p.Lk - issued * kStageRows,
                   p.D == HD && (issued + 1) * kStageRows <= p.Lk);
        ++issued;
    };
    while (issued < (SPB == 2 ? 2 : R) && issued < ns) issue_next();

    const float sl2 = p.scale * kLog2e;
    float m_i = -INFINITY;     // reference maximum (same in the four lanes of a query)
    float m_true = -INFINITY;  // maximum over the keys this lane has seen (for LI)
    float l_i = 0.f;           // exp-sum over the keys this lane has seen
    float mu_i = 0.f;          // sum of p * S_dot over the same keys
    // acc = sum P~ V;  tacc = sum (P~ * S_dot) V + P~ V_dot  (the reference's g_acc + p_tv_acc, which
    // only ever appear added together, ryu_triton.py:274-275)
    f32x4 acc[DT], tacc[DT];
#pragma unroll
    for (int t = 0; t < DT; ++t) {
        acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
        tacc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

    // SPB = 1: the own rows and stage 0 were issued before the other stages; SPB = 2: everything
    wait_stages<SPT>(SPB == 2 ? 0 : issued - 1);
    workgroup_barrier();
    u32x4 qB[KC], tqB[KC];
    {
        const int r = 16 * (wave & 1) + n;
        read_b_operands16<HD>(qB, own + (wave >> 1) * SE, r, g);
        if constexpr (JVP) read_b_operands16<HD>(tqB, own + (4 + (wave >> 1)) * SE, r, g);
        if constexpr (ROPE) {
            // the lane's two operands are columns 8g.. and 32 + 8g.. of its query: a rotation pair
            rope8<T>(qB[0], qB[1], p.rope, qrow, g, 1.0f);
            if constexpr (JVP) rope8<T>(tqB[0], tqB[1], p.rope, qrow, g, 1.0f);
        }
    }
    // ROPE: rotate the K (, K_dot) slab of a landed stage in place; 128 items per slab
    auto rotate_stage = [&](elem_t* slot, int k0) {
        if constexpr (ROPE) {
            if (tid < 128) rope_slab_item<T>(slot, tid, p.rope, k0, 1.0f);
            else if (JVP && tid < 256) rope_slab_item<T>(slot + 2 * SE, tid - 128, p.rope, k0, 1.0f);
            workgroup_barrier();
        }
    };
    rotate_stage(ring, 0);
    if constexpr (SPB == 2) {
        // the operands must have arrived in registers before the copies below overwrite their slots
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        workgroup_barrier();
        while (issued < R && issued < ns) issue_next();
    }

    auto compute = [&](const elem_t* slot, int k0) {
        const elem_t* sK = slot;
        const elem_t* sV = slot + SE;
        const elem_t* sTK = slot + 2 * SE;
        const elem_t* sTV = slot + 3 * SE;
        f32x4 s[2], ts[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            s[t] = f32x4{0.f, 0.f, 0.f, 0.f};
            ts[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < KC; ++c) {
                const u32x4 a = lds_a_rows16<HD>(sK, t, c, n, g);
                s[t] = T::mfma16(a, qB[c], s[t]);
                if constexpr (JVP) {
                    ts[t] = T::mfma16(a, tqB[c], ts[t]);
                    const u32x4 at = lds_a_rows16<HD>(sTK, t, c, n, g);
                    ts[t] = T::mfma16(at, qB[c], ts[t]);
                }
            }
        }
        if (k0 + kStageRows > p.Lk) {  // wave-uniform: only the last stage can be ragged
            // keys beyond Lk are zero rows in LDS (their S_dot is already 0)
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    if (k0 + 16 * t + 4 * g + j >= p.Lk) s[t][j] = -INFINITY;
        }
        float mloc = fmaxf(fmaxf(fmaxf(s[0][0], s[0][1]), fmaxf(s[0][2], s[0][3])),
                           fmaxf(fmaxf(s[1][0], s[1][1]), fmaxf(s[1][2], s[1][3]))) * sl2;
        m_true = fmaxf(m_true, mloc);
        if (__builtin_amdgcn_ballot_w64(mloc > m_i + kMaxSlack) != 0) {  // wave-uniform branch
            const float m_new = fmaxf(m_i, group_max(mloc));
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
#pragma unroll
        for (int t = 0; t < 2; ++t) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float pj = fast_exp2(fmaf(s[t][j], sl2, -m_i));
                s[t][j] = pj;
                l_i += pj;
                if constexpr (JVP) {
                    const float pt = pj * (ts[t][j] * p.scale);
                    ts[t][j] = pt;
                    mu_i += pt;
                }
            }
        }
        const u32x4 pb = pack_b16<T>(s[0], s[1]);
        u32x4 ptb;
        if constexpr (JVP) ptb = pack_b16<T>(ts[0], ts[1]);
#pragma unroll
        for (int d = 0; d < DT; ++d) {
            const u32x4 av = lds_a_tr16<HD>(sV, 16 * d, lane);
            acc[d] = T::mfma16(av, pb, acc[d]);
            if constexpr (JVP) {
                tacc[d] = T::mfma16(av, ptb, tacc[d]);
                const u32x4 atv = lds_a_tr16<HD>(sTV, 16 * d, lane);
                tacc[d] = T::mfma16(atv, pb, tacc[d]);
            }
        }
    };

    // One trip of the outer loop goes once round the ring, so that every LDS address of the
    // unrolled body is a per-lane constant plus an immediate offset.
    static_assert(R % SPB == 0, "a step must not wrap the ring");
    for (int i0 = 0; i0 < ns; i0 += R) {
#pragma unroll
        for (int h = 0; h < R; h += SPB) {
            const int i = i0 + h;
            if (i >= ns) break;
            if (i > 0) {
                // the stages of this step have landed for every wave; those of the last step are consumed
                wait_stages<SPT>(SPB == 2 ? 0 : issued - 1 - i);
                workgroup_barrier();
#pragma unroll
                for (int u = 0; u < SPB; ++u)
                    if (issued < ns) issue_next();
                rotate_stage(ring + h * SM::slot, i * kStageRows);
            }
            if (!wave_active) continue;
#pragma unroll
            for (int u = 0; u < SPB; ++u)
                if (i + u < ns) compute(ring + (h + u) * SM::slot, (i + u) * kStageRows);
        }
    }
    workgroup_barrier();  // every wave is done reading the ring: it becomes the store staging area
    const int64_t so = (int64_t)bh * p.Lr + qrow;
    if (!wave_active) {
        // All 16 rows of this wave lie beyond Lq: their statistic rows get the values a zero query
        // row produces (and the reference initialises them with): log(Lk), 0, Lk.
        if (g == 0) {
            p.lse[so] = fast_log2((float)p.Lk) * kLn2;
            if constexpr (JVP) p.mu[so] = 0.f;
            if (p.li) p.li[so] = (float)p.Lk;
        }
        return;
    }
    // Combine the four lanes' partial sums (they cover disjoint keys of the same query).
    const float l = group_sum(l_i);
    const float inv_l = 1.0f / l;
    float mu_un = 0.f;
    if constexpr (JVP) mu_un = group_sum(mu_i);
    if (p.li) m_true = group_max(m_true);
    if (g == 0) {
        // Statistic rows up to Lr are all written: a padded query row (all-zero q, q_dot) yields
        // exactly the values the reference initialises them with: log(Lk), 0, Lk.
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
        for (int d = 0; d < DT; ++d) tacc[d] -= cmu * acc[d];
    }
    elem_t* stage_tile = ring + wave * StoreStage16<HD>::elems;
    const int row0 = q0 + wave * 16;
    store_tile16<T, HD>(stage_tile, p.o.head(b, h), p.o.sl, row0, p.Lq, p.D, acc, inv_l, lane);
    if constexpr (JVP)
        store_tile16<T, HD>(stage_tile, p.to.head(b, h), p.to.sl, row0, p.Lq, p.D, tacc, inv_l, lane);
}

}  // namespace sjvp
