// Attention-JVP backward kernels (gfx950): gradients of q, k, v, q_dot, k_dot, v_dot for
// cotangents dO (on O) and G = dTO (on the tangent output), either of which may be absent.
//
// With P = exp(S - lse), N = S_dot - mu, W = G V^T, XY = G V_dot^T + dO V^T and the row sums
// s4 = rowsum(G*O), s7d = rowsum(G*TO) + rowsum(dO*O):
//     dS_dot = P*(W - s4)                    (semicat/jvp_utils/flash_jvp_backward.py:251-257)
//     dS     = dS_dot*N + P*(XY - s7d)       (flash_jvp_backward.py:1364-1407 plus the primal term
//                                             of semicat/jvp_utils/flash_attn_triton.py:606)
//     P_dot  = P*N                           (flash_jvp_backward.py:947-954)
//     dV_dot = P^T G            dV = P_dot^T G + P^T dO
//     dK_dot = s dS_dot^T Q     dK = s (dS^T Q + dS_dot^T Q_dot)
//     dQ_dot = s dS_dot K       dQ = s (dS K + dS_dot K_dot)
// The reference spends eight launches and 35 tile contractions on this.  This file holds the 32-wide
// pair for inputs of any alignment (the streamed side is copied through registers into one LDS
// stage); inputs with 16-byte aligned rows take the 16-wide kernels of sjvp_bwd16.hpp (one launch,
// short key axes) and sjvp_bwd16x.hpp (the same pair as here).  Two launches:
//   bwd_row_kernel   a wavefront owns 32 queries -> dQ, dQ_dot; it also forms s4 and s7d for its
//                    rows from O, TO, dO, G (O(L*D) work instead of five contractions) and leaves
//                    them, with lse in log2 units, in the workspace for
//   bwd_col_kernel   a wavefront owns 32 keys  -> dK, dV, dK_dot, dV_dot,
// each gradient accumulated in fp32 registers by exactly one wavefront and written once, so the
// result is deterministic and never round-trips through 16-bit partial sums.
#pragma once
#include <type_traits>

#include "sjvp_device.hpp"

namespace sjvp {

struct BwdParams {
    TensorView q, k, v, tq, tk, tv, o, to, dO, dTO;
    OutView dq, dk, dv, dtq, dtk, dtv;
    const float* lse;
    const float* mu;
    float* lse2;  // workspace [B*H][Lr]  lse * log2(e)
    float* s4;    // workspace [B*H][Lr]  rowsum(G*O)
    float* s7d;   // workspace [B*H][Lr]  rowsum(G*TO) + rowsum(dO*O)
    int H, Lq, Lk, D, Lr;
    int q_blocks, k_blocks;  // workgroups per (batch, head) along the owned axis
    // Set by the host where every query-side input (q, q_dot, o, o_dot, dO, dO_dot as present) has q's strides,
    // resp. every key-side input k's, and a row's byte offset inside its (batch, head) slice fits 31 bits: the
    // 16-wide row-owned and column-owned kernels then address their own rows from one offset.
    int q_side_uniform, k_side_uniform;
    int col_workgroups;  // workgroups of the column-owned pass in a launch that also holds others (set by its launcher)
    float scale;
    int vec;
    RopeTables rope;  // q, k (and tangents) are rotated as they are loaded, their gradients rotated back
    int* flags;        // workspace [B*H][Lr/64]: row-owned workgroups whose rows need the second launch
    int rowfix;        // second launch of the row-owned kernel: 0 never, 1 flagged workgroups, 2 always
    float rowfix_tau;  // a residue counts once it exceeds this fraction of the row's absolute tile sum
};

// ---------------------------------------------------------------------------------------------
// Row-owned kernel: dQ (and dQ_dot).  Tiles are transposed (rows = keys in registers, columns =
// this wave's queries in lanes), so the row statistics are per-lane scalars.
// LDS layout: one stage of K, V (, K_dot, V_dot) slabs.
template <int HD, bool HAS_G>
struct RowSmem {
    static constexpr int nt = HAS_G ? 4 : 2;
    static constexpr int slot = nt * Slab<HD>::elems;
    static constexpr int bytes = slot * (int)sizeof(elem_t);
};

// PASS: 0 the first (or only) launch; 1 the first launch of the "always" mode, which only measures the
// residues; 2 the second launch of the residue repair described in sjvp_bwd16x.hpp (sums from the
// workspace; workgroups that were not flagged leave at once).
template <typename T, int HD, bool HAS_DO, bool HAS_G, bool F32IO = false, int PASS = 0>
__global__ __launch_bounds__(kThreads, 1) void bwd_row_kernel(const BwdParams p) {
    constexpr bool SECOND = PASS == 2;   // second launch: sums from the workspace, flagged workgroups only
    constexpr bool MEASURE = PASS == 1;  // first launch of "always": residues and sums only, no gradients
    extern __shared__ __align__(16) unsigned char smem_raw[];
    elem_t* stage = reinterpret_cast<elem_t*>(smem_raw);

    constexpr int KC = HD / 16;
    constexpr int DT = HD / 32;
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
    const int qrow = qb * kOwned + wave * 32 + x;
    const bool qvalid = qrow < p.Lq;
    const bool wave_active = (qb * kOwned + wave * 32) < p.Lq;
    if constexpr (SECOND) {
        if (p.rowfix == 1 && p.flags[blockIdx.x] == 0) return;  // nothing to repair in this workgroup's rows
    }

    u32x4 qB[KC], tqB[KC], gB[KC], doB[KC], oR[KC], toR[KC];
    float lse2 = 0.f, mu = 0.f;
    const int64_t so = (int64_t)bh * p.Lr + qrow;
    {
        const elem_t* qp = p.q.head(b, h) + (int64_t)qrow * p.q.sl;
        const elem_t* op = p.o.head(b, h) + (int64_t)qrow * p.o.sl;
#pragma unroll
        for (int c = 0; c < KC; ++c) {
            qB[c] = load8_io<T, F32IO>(qp, 16 * c + 8 * hf, p.D, qvalid, vec);
            if constexpr (!SECOND) oR[c] = load8_io<T, F32IO>(op, 16 * c + 8 * hf, p.D, qvalid, vec);
        }
        if constexpr (HAS_G) {
            const elem_t* tqp = p.tq.head(b, h) + (int64_t)qrow * p.tq.sl;
            const elem_t* gp = p.dTO.head(b, h) + (int64_t)qrow * p.dTO.sl;
            const elem_t* top = p.to.head(b, h) + (int64_t)qrow * p.to.sl;
#pragma unroll
            for (int c = 0; c < KC; ++c) {
                tqB[c] = load8_io<T, F32IO>(tqp, 16 * c + 8 * hf, p.D, qvalid, vec);
                gB[c] = load8_io<T, F32IO>(gp, 16 * c + 8 * hf, p.D, qvalid, vec);
                if constexpr (!SECOND) toR[c] = load8_io<T, F32IO>(top, 16 * c + 8 * hf, p.D, qvalid, vec);
            }
        }
        if constexpr (HAS_DO) {
            const elem_t* dop = p.dO.head(b, h) + (int64_t)qrow * p.dO.sl;
#pragma unroll
            for (int c = 0; c < KC; ++c) doB[c] = load8_io<T, F32IO>(dop, 16 * c + 8 * hf, p.D, qvalid, vec);
        }
        // Per-lane row statistics; an invalid query lane uses zeros (finite P, results discarded).
        lse2 = qvalid ? p.lse[so] * kLog2e : 0.f;
        mu = (qvalid && HAS_G) ? p.mu[so] : 0.f;
    }

    // s4 = rowsum(G*O), s7d = rowsum(G*TO) + rowsum(dO*O): each half-lane holds half of the row's
    // columns (those of its B operands); the two halves are added across the wave.
    float s4 = 0.f, s7d = 0.f;
    auto row_sums = [&]() {
#pragma unroll
        for (int c = 0; c < KC; ++c) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float o0 = T::to_float((elem_t)(oR[c][i] & 0xffffu));
                const float o1 = T::to_float((elem_t)(oR[c][i] >> 16));
                if constexpr (HAS_G) {
                    const float g0 = T::to_float((elem_t)(gB[c][i] & 0xffffu));
                    const float g1 = T::to_float((elem_t)(gB[c][i] >> 16));
                    const float t0 = T::to_float((elem_t)(toR[c][i] & 0xffffu));
                    const float t1 = T::to_float((elem_t)(toR[c][i] >> 16));
                    s4 += g0 * o0 + g1 * o1;
                    s7d += g0 * t0 + g1 * t1;
                }
                if constexpr (HAS_DO) {
                    const float d0 = T::to_float((elem_t)(doB[c][i] & 0xffffu));
                    const float d1 = T::to_float((elem_t)(doB[c][i] >> 16));
                    s7d += d0 * o0 + d1 * o1;
                }
            }
        }
        s4 += other_half(s4);
        s7d += other_half(s7d);
    };
    if constexpr (SECOND) {
        // the corrected sums the first launch left in the workspace
        s4 = p.s4[so];
        s7d = p.s7d[so];
    } else {
        row_sums();
    }
    const elem_t* kg = p.k.head(b, h);
    const elem_t* vg = p.v.head(b, h);
    const elem_t* tkg = HAS_G ? p.tk.head(b, h) : nullptr;
    const elem_t* tvg = HAS_G ? p.tv.head(b, h) : nullptr;
    const float sl2 = p.scale * kLog2e;

    auto fill = [&](int st) {
        const int row0 = st * kStageRows;
        fill_slab<HD, T, F32IO>(ln, stage, kg, p.k.sl, row0, p.Lk, p.D, vec);
        fill_slab<HD, T, F32IO>(ln, stage + Slab<HD>::elems, vg, p.v.sl, row0, p.Lk, p.D, vec);
        if constexpr (HAS_G) {
            fill_slab<HD, T, F32IO>(ln, stage + 2 * Slab<HD>::elems, tkg, p.tk.sl, row0, p.Lk, p.D, vec);
            fill_slab<HD, T, F32IO>(ln, stage + 3 * Slab<HD>::elems, tvg, p.tv.sl, row0, p.Lk, p.D, vec);
        }
    };

    f32x16 dq[DT], dtq[DT];
#pragma unroll
    for (int t = 0; t < DT; ++t) {
        dq[t] = f32x16{0};
        if constexpr (HAS_G) dtq[t] = f32x16{0};
    }
    // First launch: this lane's part of sum_j dS_dot_ij and sum_j dS_ij, which are zero with exact row
    // sums and equal minus the rounding error of s4, s7d otherwise, and of their absolute sums (sampled
    // on every fourth key: they only set the scale of a threshold).
    float r4 = 0.f, r7 = 0.f, a4 = 0.f, a7 = 0.f;

    auto compute = [&](int k0, auto ragged_tag) {
        constexpr bool RAGGED = decltype(ragged_tag)::value;
        const elem_t* sK = stage;
        const elem_t* sV = stage + Slab<HD>::elems;
        const elem_t* sTK = stage + 2 * Slab<HD>::elems;
        const elem_t* sTV = stage + 3 * Slab<HD>::elems;
        f32x16 s = {0}, ts = {0}, w = {0}, xy = {0};
#pragma unroll
        for (int c = 0; c < KC; ++c) {
            u32x4 ak = lds_a_rows<HD>(sK, c, x, hf);
            u32x4 av = lds_a_rows<HD>(sV, c, x, hf);
            s = T::mfma(ak, qB[c], s);
            if constexpr (HAS_G) {
                ts = T::mfma(ak, tqB[c], ts);
                u32x4 atk = lds_a_rows<HD>(sTK, c, x, hf);
                ts = T::mfma(atk, qB[c], ts);
                w = T::mfma(av, gB[c], w);
                u32x4 atv = lds_a_rows<HD>(sTV, c, x, hf);
                xy = T::mfma(atv, gB[c], xy);
            }
            if constexpr (HAS_DO) xy = T::mfma(av, doB[c], xy);
        }
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            float pj = fast_exp2(fmaf(s[j], sl2, -lse2));
            if constexpr (RAGGED) {
                // keys beyond Lk are zero rows; exp(-lse) may overflow when every real score is
                // very negative, so their P is forced to zero
                if (k0 + 8 * (j >> 2) + 4 * hf + (j & 3) >= p.Lk) pj = 0.f;
            }
            if constexpr (HAS_G) {
                const float n = fmaf(ts[j], p.scale, -mu);
                const float dts = pj * (w[j] - s4);
                w[j] = dts;
                xy[j] = fmaf(dts, n, pj * (xy[j] - s7d));
                if constexpr (!SECOND) {
                    r4 += dts;
                    if ((j & 3) == 0) a4 += fabsf(dts);
                }
            } else {
                xy[j] = pj * (xy[j] - s7d);
            }
            if constexpr (!SECOND) {
                r7 += xy[j];
                if ((j & 3) == 0) a7 += fabsf(xy[j]);
            }
        }
        if constexpr (MEASURE) return;  // a launch that only measures the residues
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            const u32x4 dsB = pack_b<T>(xy, c);
            u32x4 dtsB;
            if constexpr (HAS_G) dtsB = pack_b<T>(w, c);
#pragma unroll
            for (int d = 0; d < DT; ++d) {
                const u32x4 ak = lds_a_transposed<HD>(sK, c, 32 * d, lane);
                dq[d] = T::mfma(ak, dsB, dq[d]);
                if constexpr (HAS_G) {
                    dtq[d] = T::mfma(ak, dtsB, dtq[d]);
                    const u32x4 atk = lds_a_transposed<HD>(sTK, c, 32 * d, lane);
                    dq[d] = T::mfma(atk, dtsB, dq[d]);
                }
            }
        }
    };

    const int n = (p.Lk + kStageRows - 1) / kStageRows;
    // every row below Lr gets its workspace entries (zeros beyond Lq): the column-owned kernel, which
    // runs after this one, stages 32-row groups
    if constexpr (!SECOND) {
        if (hf == 0) p.lse2[so] = lse2;
    }
    for (int i = 0; i < n; ++i) {
        workgroup_barrier();  // the previous stage is fully consumed
        fill(i);
        workgroup_barrier();
        if (!wave_active) continue;
        const int k0 = i * kStageRows;
        if (k0 + kStageRows > p.Lk) compute(k0, std::true_type{});
        else compute(k0, std::false_type{});
    }
    if constexpr (!SECOND) {
        // the residues of the row sums: corrected sums for the column-owned kernel and for the second
        // launch, which the workgroup asks for where a residue is not small against the rounding of the
        // tiles it is spread over
        r4 += other_half(r4);
        r7 += other_half(r7);
        a4 = 4.0f * (a4 + other_half(a4));
        a7 = 4.0f * (a7 + other_half(a7));
        if (hf == 0) {
            p.s4[so] = s4 + r4;
            p.s7d[so] = s7d + r7;
        }
        const bool wanted = qvalid && (fabsf(r4) > p.rowfix_tau * a4 || fabsf(r7) > p.rowfix_tau * a7);
        if (p.rowfix == 1) {
            const bool any = workgroup_barrier_or(wanted);
            if (tid == 0) p.flags[blockIdx.x] = any ? 1 : 0;
        }
        if constexpr (MEASURE) return;  // the second launch writes dQ, dQ_dot
    }
    if (!qvalid) return;
    elem_t* dqrow = p.dq.head(b, h) + (int64_t)qrow * p.dq.sl;
#pragma unroll
    for (int d = 0; d < DT; ++d) store_acc<T, F32IO>(dqrow, 32 * d, hf, p.D, dq[d], p.scale, vec);
    if constexpr (HAS_G) {
        elem_t* dtqrow = p.dtq.head(b, h) + (int64_t)qrow * p.dtq.sl;
#pragma unroll
        for (int d = 0; d < DT; ++d) store_acc<T, F32IO>(dtqrow, 32 * d, hf, p.D, dtq[d], p.scale, vec);
    }
}

// ---------------------------------------------------------------------------------------------
// Column-owned kernel: a wavefront owns 32 keys and streams the queries.  DO_K selects dK (and
// dK_dot), DO_V selects dV (and dV_dot); DT0/NDT select the 32-wide head-dimension tiles that are
// accumulated (at HD = 128 the work is split to stay inside the register file).
// LDS layout: one stage of Q (, Q_dot, G) (, dO) slabs followed by the stage's row statistics
// (lse2, mu, s4, s7d).
template <int HD, bool HAS_DO, bool HAS_G>
struct ColSmem {
    static constexpr int nt = 1 + (HAS_G ? 2 : 0) + (HAS_DO ? 1 : 0);
    static constexpr int stat_elems = 4 * kStageRows * 2;  // 4 float arrays of 32, in elem_t units
    static constexpr int slot = nt * Slab<HD>::elems + stat_elems;
    static constexpr int bytes = slot * (int)sizeof(elem_t);
};

template <typename T, int HD, bool HAS_DO, bool HAS_G, bool DO_K, bool DO_V, int DT0, int NDT, bool F32IO = false>
__global__ __launch_bounds__(kThreads, (DO_K && DO_V && HAS_G) ? 1 : 2) void bwd_col_kernel(
    const BwdParams p) {
    extern __shared__ __align__(16) unsigned char smem_raw[];
    using SM = ColSmem<HD, HAS_DO, HAS_G>;
    elem_t* stage = reinterpret_cast<elem_t*>(smem_raw);
    // stage layout: Q | [Q_dot | G] | [dO] | stats(lse2, mu, s4, s7d)
    constexpr int oTQ = Slab<HD>::elems;
    constexpr int oG = 2 * Slab<HD>::elems;
    constexpr int oDO = (HAS_G ? 3 : 1) * Slab<HD>::elems;
    constexpr int oST = SM::nt * Slab<HD>::elems;

    constexpr int KC = HD / 16;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int x = lane & 31;
    const int hf = lane >> 5;
    const int bh = blockIdx.x / p.k_blocks;
    const int kb = blockIdx.x % p.k_blocks;
    const int b = bh / p.H, h = bh % p.H;
    const bool vec = p.vec != 0;
    SlabLane<HD> ln;
    ln.init(tid);
    const int krow = kb * kOwned + wave * 32 + x;  // the key this lane owns
    const bool kvalid = krow < p.Lk;
    const bool wave_active = (kb * kOwned + wave * 32) < p.Lk;

    u32x4 kB[KC], vB[KC], tkB[KC], tvB[KC];
    {
        const elem_t* kp = p.k.head(b, h) + (int64_t)krow * p.k.sl;
        const elem_t* vp = p.v.head(b, h) + (int64_t)krow * p.v.sl;
#pragma unroll
        for (int c = 0; c < KC; ++c) {
            kB[c] = load8_io<T, F32IO>(kp, 16 * c + 8 * hf, p.D, kvalid, vec);
            if constexpr (DO_K) vB[c] = load8_io<T, F32IO>(vp, 16 * c + 8 * hf, p.D, kvalid, vec);
        }
        if constexpr (HAS_G) {
            const elem_t* tkp = p.tk.head(b, h) + (int64_t)krow * p.tk.sl;
            const elem_t* tvp = p.tv.head(b, h) + (int64_t)krow * p.tv.sl;
#pragma unroll
            for (int c = 0; c < KC; ++c) {
                tkB[c] = load8_io<T, F32IO>(tkp, 16 * c + 8 * hf, p.D, kvalid, vec);
                if constexpr (DO_K) tvB[c] = load8_io<T, F32IO>(tvp, 16 * c + 8 * hf, p.D, kvalid, vec);
            }
        }
    }
    const elem_t* qg = p.q.head(b, h);
    const elem_t* tqg = HAS_G ? p.tq.head(b, h) : nullptr;
    const elem_t* gg = HAS_G ? p.dTO.head(b, h) : nullptr;
    const elem_t* dog = HAS_DO ? p.dO.head(b, h) : nullptr;
    const float sl2 = p.scale * kLog2e;

    auto fill = [&](int st) {
        const int row0 = st * kStageRows;
        fill_slab<HD, T, F32IO>(ln, stage, qg, p.q.sl, row0, p.Lq, p.D, vec);
        if constexpr (HAS_G) {
            fill_slab<HD, T, F32IO>(ln, stage + oTQ, tqg, p.tq.sl, row0, p.Lq, p.D, vec);
            fill_slab<HD, T, F32IO>(ln, stage + oG, gg, p.dTO.sl, row0, p.Lq, p.D, vec);
        }
        if constexpr (HAS_DO) fill_slab<HD, T, F32IO>(ln, stage + oDO, dog, p.dO.sl, row0, p.Lq, p.D, vec);
        // Row statistics of the stage (rows < Lr are defined in all four arrays; rows beyond Lq
        // hold finite values and multiply zero rows of Q, Q_dot, G, dO below): the four arrays are
        // dealt to the waves, 32 lanes each.
        float* st_lds = reinterpret_cast<float*>(stage + oST);
        const int64_t so = (int64_t)bh * p.Lr + row0 + (lane & 31);
        constexpr int APW = 4 / kWaves;  // arrays per wave
        const int arr = wave * APW + hf;
        if (hf < APW) {
            const float* src = arr == 0 ? p.lse2 : arr == 1 ? p.mu : arr == 2 ? p.s4 : p.s7d;
            if (arr == 1 && !HAS_G) src = p.s4;  // mu is not used without the tangent cotangent
            st_lds[arr * 32 + (lane & 31)] = src[so];
        }
    };

    f32x16 dk[NDT], dv[NDT], dtk[NDT], dtv[NDT];
#pragma unroll
    for (int t = 0; t < NDT; ++t) {
        if constexpr (DO_K) dk[t] = f32x16{0};
        if constexpr (DO_V) dv[t] = f32x16{0};
        if constexpr (HAS_G) {
            if constexpr (DO_K) dtk[t] = f32x16{0};
            if constexpr (DO_V) dtv[t] = f32x16{0};
        }
    }

    auto compute = [&]() {
        const elem_t* sQ = stage;
        const elem_t* sTQ = stage + oTQ;
        const elem_t* sG = stage + oG;
        const elem_t* sDO = stage + oDO;
        const float* sStat = reinterpret_cast<const float*>(stage + oST);
        // tiles: rows = queries (registers), columns = this wave's keys (lanes)
        f32x16 s = {0}, ts = {0}, w = {0}, xy = {0};
#pragma unroll
        for (int c = 0; c < KC; ++c) {
            u32x4 aq = lds_a_rows<HD>(sQ, c, x, hf);
            s = T::mfma(aq, kB[c], s);
            if constexpr (HAS_G) {
                ts = T::mfma(aq, tkB[c], ts);
                u32x4 atq = lds_a_rows<HD>(sTQ, c, x, hf);
                ts = T::mfma(atq, kB[c], ts);
                if constexpr (DO_K) {
                    u32x4 ag = lds_a_rows<HD>(sG, c, x, hf);
                    w = T::mfma(ag, vB[c], w);
                    xy = T::mfma(ag, tvB[c], xy);
                }
            }
            if constexpr (HAS_DO && DO_K) {
                u32x4 ado = lds_a_rows<HD>(sDO, c, x, hf);
                xy = T::mfma(ado, vB[c], xy);
            }
        }
        // in place: s -> P, ts -> P_dot, w -> dS_dot, xy -> dS
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
            const int r0 = 8 * jj + 4 * hf;
            const f32x4 lse4 = *reinterpret_cast<const f32x4*>(sStat + 0 * kStageRows + r0);
            const f32x4 mu4 = *reinterpret_cast<const f32x4*>(sStat + 1 * kStageRows + r0);
            const f32x4 s44 = *reinterpret_cast<const f32x4*>(sStat + 2 * kStageRows + r0);
            const f32x4 s74 = *reinterpret_cast<const f32x4*>(sStat + 3 * kStageRows + r0);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int j = 4 * jj + i;
                const float pj = fast_exp2(fmaf(s[j], sl2, -lse4[i]));
                s[j] = pj;
                if constexpr (HAS_G) {
                    const float n = fmaf(ts[j], p.scale, -mu4[i]);
                    if constexpr (DO_K) {
                        const float dts = pj * (w[j] - s44[i]);
                        w[j] = dts;
                        xy[j] = fmaf(dts, n, pj * (xy[j] - s74[i]));
                    }
                    if constexpr (DO_V) ts[j] = pj * n;
                } else if constexpr (DO_K) {
                    xy[j] = pj * (xy[j] - s74[i]);
                }
            }
        }
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            u32x4 pB, dsB, pdB, dtsB;
            if constexpr (DO_V) pB = pack_b<T>(s, c);
            if constexpr (DO_K) dsB = pack_b<T>(xy, c);
            if constexpr (HAS_G) {
                if constexpr (DO_V) pdB = pack_b<T>(ts, c);
                if constexpr (DO_K) dtsB = pack_b<T>(w, c);
            }
#pragma unroll
            for (int d = 0; d < NDT; ++d) {
                const int d0 = 32 * (DT0 + d);
                if constexpr (DO_K) {
                    const u32x4 aq = lds_a_transposed<HD>(sQ, c, d0, lane);
                    dk[d] = T::mfma(aq, dsB, dk[d]);
                    if constexpr (HAS_G) {
                        dtk[d] = T::mfma(aq, dtsB, dtk[d]);
                        const u32x4 atq = lds_a_transposed<HD>(sTQ, c, d0, lane);
                        dk[d] = T::mfma(atq, dtsB, dk[d]);
                    }
                }
                if constexpr (DO_V) {
                    if constexpr (HAS_G) {
                        const u32x4 ag = lds_a_transposed<HD>(sG, c, d0, lane);
                        dtv[d] = T::mfma(ag, pB, dtv[d]);
                        dv[d] = T::mfma(ag, pdB, dv[d]);
                    }
                    if constexpr (HAS_DO) {
                        const u32x4 ado = lds_a_transposed<HD>(sDO, c, d0, lane);
                        dv[d] = T::mfma(ado, pB, dv[d]);
                    }
                }
            }
        }
    };

    const int n = (p.Lq + kStageRows - 1) / kStageRows;
    for (int i = 0; i < n; ++i) {
        workgroup_barrier();  // the previous stage is fully consumed
        fill(i);
        workgroup_barrier();
        if (wave_active) compute();
    }
    {
        if (!kvalid) return;
        if constexpr (DO_K) {
            elem_t* dkrow = p.dk.head(b, h) + (int64_t)krow * p.dk.sl;
#pragma unroll
            for (int d = 0; d < NDT; ++d)
                store_acc<T, F32IO>(dkrow, 32 * (DT0 + d), hf, p.D, dk[d], p.scale, vec);
            if constexpr (HAS_G) {
                elem_t* dtkrow = p.dtk.head(b, h) + (int64_t)krow * p.dtk.sl;
#pragma unroll
                for (int d = 0; d < NDT; ++d)
                    store_acc<T, F32IO>(dtkrow, 32 * (DT0 + d), hf, p.D, dtk[d], p.scale, vec);
            }
        }
        if constexpr (DO_V) {
            elem_t* dvrow = p.dv.head(b, h) + (int64_t)krow * p.dv.sl;
#pragma unroll
            for (int d = 0; d < NDT; ++d)
                store_acc<T, F32IO>(dvrow, 32 * (DT0 + d), hf, p.D, dv[d], 1.0f, vec);
            if constexpr (HAS_G) {
                elem_t* dtvrow = p.dtv.head(b, h) + (int64_t)krow * p.dtv.sl;
#pragma unroll
                for (int d = 0; d < NDT; ++d)
                    store_acc<T, F32IO>(dtvrow, 32 * (DT0 + d), hf, p.D, dtv[d], 1.0f, vec);
            }
        }
    }
}

}  // namespace sjvp
