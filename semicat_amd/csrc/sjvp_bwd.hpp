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
// The reference spends eight launches and 35 tile contractions on this; here it is three launches:
//   bwd_rowstats_kernel  s4, s7d from O, TO, dO, G (O(L*D) work instead of five contractions),
//   bwd_col_kernel       a wavefront owns 32 keys  -> dK, dV, dK_dot, dV_dot,
//   bwd_row_kernel       a wavefront owns 32 queries -> dQ, dQ_dot,
// each gradient accumulated in fp32 registers by exactly one wavefront and written once, so the
// result is deterministic and never round-trips through 16-bit partial sums.
#pragma once
#include "sjvp_device.hpp"

namespace sjvp {

struct OutView {
    elem_t* ptr;
    int64_t sb, sh, sl;
    __device__ __forceinline__ elem_t* head(int b, int h) const { return ptr + b * sb + h * sh; }
};

struct BwdParams {
    TensorView q, k, v, tq, tk, tv, o, to, dO, dTO;
    OutView dq, dk, dv, dtq, dtk, dtv;
    const float* lse;
    const float* mu;
    float* s4;   // [B*H][Lr]  rowsum(G*O)
    float* s7d;  // [B*H][Lr]  rowsum(G*TO) + rowsum(dO*O)
    int H, Lq, Lk, D, Lr;
    int q_blocks, k_blocks;  // ceil(L / 128)
    float scale;
    int vec;
};

// ---------------------------------------------------------------------------------------------
// Row sums.  Eight lanes per query row, 32 rows per workgroup.
template <typename T, bool HAS_DO, bool HAS_G>
__global__ __launch_bounds__(kThreads) void bwd_rowstats_kernel(const BwdParams p) {
    const int tid = threadIdx.x;
    const int sub = tid & 7;
    const int blocks_per_head = p.Lr / 32;
    const int bh = blockIdx.x / blocks_per_head;
    const int row = (blockIdx.x % blocks_per_head) * 32 + (tid >> 3);
    const int b = bh / p.H, h = bh % p.H;
    const bool valid = row < p.Lq;
    const bool vec = p.vec != 0;
    float a4 = 0.f, a7 = 0.f;
    if (valid) {
        const elem_t* orow = p.o.head(b, h) + (int64_t)row * p.o.sl;
        const elem_t* torow = HAS_G ? p.to.head(b, h) + (int64_t)row * p.to.sl : nullptr;
        const elem_t* grow = HAS_G ? p.dTO.head(b, h) + (int64_t)row * p.dTO.sl : nullptr;
        const elem_t* drow = HAS_DO ? p.dO.head(b, h) + (int64_t)row * p.dO.sl : nullptr;
        for (int d = 8 * sub; d < p.D; d += 64) {
            u32x4 ov = load8(orow, d, p.D, true, vec);
            u32x4 tov, gv, dv;
            if constexpr (HAS_G) {
                tov = load8(torow, d, p.D, true, vec);
                gv = load8(grow, d, p.D, true, vec);
            }
            if constexpr (HAS_DO) dv = load8(drow, d, p.D, true, vec);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int sh = 16 * (i & 1);
                float of = T::to_float((elem_t)((ov[i >> 1] >> sh) & 0xffffu));
                if constexpr (HAS_G) {
                    float gf = T::to_float((elem_t)((gv[i >> 1] >> sh) & 0xffffu));
                    float tf = T::to_float((elem_t)((tov[i >> 1] >> sh) & 0xffffu));
                    a4 += gf * of;
                    a7 += gf * tf;
                }
                if constexpr (HAS_DO) {
                    float df = T::to_float((elem_t)((dv[i >> 1] >> sh) & 0xffffu));
                    a7 += df * of;
                }
            }
        }
    }
#pragma unroll
    for (int m = 1; m < 8; m <<= 1) {
        a4 += __shfl_xor(a4, m, 64);
        a7 += __shfl_xor(a7, m, 64);
    }
    if (sub == 0) {
        p.s4[(int64_t)bh * p.Lr + row] = a4;
        p.s7d[(int64_t)bh * p.Lr + row] = a7;
    }
}

// ---------------------------------------------------------------------------------------------
// Column-owned kernel: dK, dV (and dK_dot, dV_dot).  Accumulates head-dimension tiles
// [DT0, DT0 + NDT) only; at HD = 128 it is launched twice to stay inside the register file.
template <int HD, int BM, bool HAS_DO, bool HAS_G>
struct ColSmem {
    static constexpr int tile = BM * Pitch<HD>::value;
    static constexpr int ntiles = 1 + (HAS_G ? 2 : 0) + (HAS_DO ? 1 : 0);
    static constexpr int bytes = ntiles * tile * (int)sizeof(elem_t) + 4 * BM * (int)sizeof(float);
};

template <typename T, int HD, int BM, bool HAS_DO, bool HAS_G, int DT0, int NDT>
__global__ __launch_bounds__(kThreads) void bwd_col_kernel(const BwdParams p) {
    extern __shared__ __align__(16) unsigned char smem_raw[];
    using SM = ColSmem<HD, BM, HAS_DO, HAS_G>;
    float* sStat = reinterpret_cast<float*>(smem_raw);  // [4][BM]: lse*log2e, mu, s4, s7d
    elem_t* sQ = reinterpret_cast<elem_t*>(smem_raw + 4 * BM * sizeof(float));
    elem_t* sTQ = sQ + SM::tile;                 // HAS_G
    elem_t* sG = sTQ + SM::tile;                 // HAS_G
    elem_t* sDO = HAS_G ? sG + SM::tile : sQ + SM::tile;  // HAS_DO

    constexpr int KC = HD / 16;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int x = lane & 31;
    const int hf = lane >> 5;
    const int bh = blockIdx.x / p.k_blocks;
    const int kb = blockIdx.x % p.k_blocks;
    const int b = bh / p.H, h = bh % p.H;
    const bool vec = p.vec != 0;

    const int krow = kb * kOwned + wave * 32 + x;  // the key this lane owns
    const bool kvalid = krow < p.Lk;
    const bool wave_active = (kb * kOwned + wave * 32) < p.Lk;

    u32x4 kB[KC], vB[KC], tkB[KC], tvB[KC];
    {
        const elem_t* kp = p.k.head(b, h) + (int64_t)krow * p.k.sl;
        const elem_t* vp = p.v.head(b, h) + (int64_t)krow * p.v.sl;
#pragma unroll
        for (int c = 0; c < KC; ++c) {
            kB[c] = load8(kp, 16 * c + 8 * hf, p.D, kvalid, vec);
            vB[c] = load8(vp, 16 * c + 8 * hf, p.D, kvalid, vec);
        }
        if constexpr (HAS_G) {
            const elem_t* tkp = p.tk.head(b, h) + (int64_t)krow * p.tk.sl;
            const elem_t* tvp = p.tv.head(b, h) + (int64_t)krow * p.tv.sl;
#pragma unroll
            for (int c = 0; c < KC; ++c) {
                tkB[c] = load8(tkp, 16 * c + 8 * hf, p.D, kvalid, vec);
                tvB[c] = load8(tvp, 16 * c + 8 * hf, p.D, kvalid, vec);
            }
        }
    }

    const elem_t* qg = p.q.head(b, h);
    const elem_t* tqg = HAS_G ? p.tq.head(b, h) : nullptr;
    const elem_t* gg = HAS_G ? p.dTO.head(b, h) : nullptr;
    const elem_t* dog = HAS_DO ? p.dO.head(b, h) : nullptr;
    const float sl2 = p.scale * kLog2e;

    f32x16 dk[NDT], dv[NDT], dtk[NDT], dtv[NDT];
#pragma unroll
    for (int t = 0; t < NDT; ++t) {
        dk[t] = f32x16{0};
        dv[t] = f32x16{0};
        if constexpr (HAS_G) {
            dtk[t] = f32x16{0};
            dtv[t] = f32x16{0};
        }
    }

    for (int q0 = 0; q0 < p.Lq; q0 += BM) {
        __syncthreads();
        stage_rows<HD, BM>(sQ, qg, p.q.sl, q0, p.Lq, p.D, vec, tid);
        if constexpr (HAS_G) {
            stage_rows<HD, BM>(sTQ, tqg, p.tq.sl, q0, p.Lq, p.D, vec, tid);
            stage_rows<HD, BM>(sG, gg, p.dTO.sl, q0, p.Lq, p.D, vec, tid);
        }
        if constexpr (HAS_DO) stage_rows<HD, BM>(sDO, dog, p.dO.sl, q0, p.Lq, p.D, vec, tid);
        if (tid < BM) {
            // Rows beyond Lq are staged as zeros everywhere: their P is finite (= 1) and multiplies
            // zero rows of Q, Q_dot, G, dO in every contraction below.
            const int row = q0 + tid;
            const bool rv = row < p.Lq;
            const int64_t so = (int64_t)bh * p.Lr + row;
            sStat[0 * BM + tid] = rv ? p.lse[so] * kLog2e : 0.f;
            sStat[1 * BM + tid] = (rv && HAS_G) ? p.mu[so] : 0.f;
            sStat[2 * BM + tid] = rv ? p.s4[so] : 0.f;
            sStat[3 * BM + tid] = rv ? p.s7d[so] : 0.f;
        }
        __syncthreads();
        if (!wave_active) continue;

#pragma unroll
        for (int t = 0; t < BM / 32; ++t) {
            const int y0 = 32 * t;
            if (q0 + y0 >= p.Lq) break;
            // tiles: rows = queries (registers), columns = this wave's keys (lanes)
            f32x16 s = {0}, ts = {0}, w = {0}, xy = {0};
#pragma unroll
            for (int c = 0; c < KC; ++c) {
                u32x4 aq = lds_a_rows<HD>(sQ, y0, c, x, hf);
                s = T::mfma(aq, kB[c], s);
                if constexpr (HAS_G) {
                    ts = T::mfma(aq, tkB[c], ts);
                    u32x4 atq = lds_a_rows<HD>(sTQ, y0, c, x, hf);
                    ts = T::mfma(atq, kB[c], ts);
                    u32x4 ag = lds_a_rows<HD>(sG, y0, c, x, hf);
                    w = T::mfma(ag, vB[c], w);
                    xy = T::mfma(ag, tvB[c], xy);
                }
                if constexpr (HAS_DO) {
                    u32x4 ado = lds_a_rows<HD>(sDO, y0, c, x, hf);
                    xy = T::mfma(ado, vB[c], xy);
                }
            }
            // in place: s -> P, ts -> P_dot, w -> dS_dot, xy -> dS
#pragma unroll
            for (int jj = 0; jj < 4; ++jj) {
                const int r0 = y0 + 8 * jj + 4 * hf;
                const f32x4 lse4 = *reinterpret_cast<const f32x4*>(sStat + 0 * BM + r0);
                const f32x4 mu4 = *reinterpret_cast<const f32x4*>(sStat + 1 * BM + r0);
                const f32x4 s44 = *reinterpret_cast<const f32x4*>(sStat + 2 * BM + r0);
                const f32x4 s74 = *reinterpret_cast<const f32x4*>(sStat + 3 * BM + r0);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int j = 4 * jj + i;
                    const float pj = fast_exp2(s[j] * sl2 - lse4[i]);
                    s[j] = pj;
                    if constexpr (HAS_G) {
                        const float n = ts[j] * p.scale - mu4[i];
                        const float dts = pj * (w[j] - s44[i]);
                        w[j] = dts;
                        xy[j] = dts * n + pj * (xy[j] - s74[i]);
                        ts[j] = pj * n;
                    } else {
                        xy[j] = pj * (xy[j] - s74[i]);
                    }
                }
            }
#pragma unroll
            for (int c = 0; c < 2; ++c) {
                const u32x4 pB = pack_b<T>(s, c);
                const u32x4 dsB = pack_b<T>(xy, c);
                u32x4 pdB, dtsB;
                if constexpr (HAS_G) {
                    pdB = pack_b<T>(ts, c);
                    dtsB = pack_b<T>(w, c);
                }
#pragma unroll
                for (int d = 0; d < NDT; ++d) {
                    const int d0 = 32 * (DT0 + d);
                    const u32x4 aq = lds_a_transposed<HD>(sQ, y0, c, d0, lane);
                    dk[d] = T::mfma(aq, dsB, dk[d]);
                    if constexpr (HAS_G) {
                        dtk[d] = T::mfma(aq, dtsB, dtk[d]);
                        const u32x4 atq = lds_a_transposed<HD>(sTQ, y0, c, d0, lane);
                        dk[d] = T::mfma(atq, dtsB, dk[d]);
                        const u32x4 ag = lds_a_transposed<HD>(sG, y0, c, d0, lane);
                        dtv[d] = T::mfma(ag, pB, dtv[d]);
                        dv[d] = T::mfma(ag, pdB, dv[d]);
                    }
                    if constexpr (HAS_DO) {
                        const u32x4 ado = lds_a_transposed<HD>(sDO, y0, c, d0, lane);
                        dv[d] = T::mfma(ado, pB, dv[d]);
                    }
                }
            }
        }
    }

    if (!kvalid) return;
    elem_t* dkrow = p.dk.head(b, h) + (int64_t)krow * p.dk.sl;
    elem_t* dvrow = p.dv.head(b, h) + (int64_t)krow * p.dv.sl;
#pragma unroll
    for (int d = 0; d < NDT; ++d) {
        store_acc<T>(dkrow, 32 * (DT0 + d), hf, p.D, dk[d], p.scale, vec);
        store_acc<T>(dvrow, 32 * (DT0 + d), hf, p.D, dv[d], 1.0f, vec);
    }
    if constexpr (HAS_G) {
        elem_t* dtkrow = p.dtk.head(b, h) + (int64_t)krow * p.dtk.sl;
        elem_t* dtvrow = p.dtv.head(b, h) + (int64_t)krow * p.dtv.sl;
#pragma unroll
        for (int d = 0; d < NDT; ++d) {
            store_acc<T>(dtkrow, 32 * (DT0 + d), hf, p.D, dtk[d], p.scale, vec);
            store_acc<T>(dtvrow, 32 * (DT0 + d), hf, p.D, dtv[d], 1.0f, vec);
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Row-owned kernel: dQ (and dQ_dot).  Tiles are transposed (rows = keys in registers, columns =
// this wave's queries in lanes), so the row statistics are per-lane scalars.
template <int HD, int BN, bool HAS_G>
struct RowSmem {
    static constexpr int tile = BN * Pitch<HD>::value;
    static constexpr int bytes = (HAS_G ? 4 : 2) * tile * (int)sizeof(elem_t);
};

template <typename T, int HD, int BN, bool HAS_DO, bool HAS_G>
__global__ __launch_bounds__(kThreads) void bwd_row_kernel(const BwdParams p) {
    extern __shared__ __align__(16) unsigned char smem_raw[];
    using SM = RowSmem<HD, BN, HAS_G>;
    elem_t* sK = reinterpret_cast<elem_t*>(smem_raw);
    elem_t* sV = sK + SM::tile;
    elem_t* sTK = sV + SM::tile;   // HAS_G
    elem_t* sTV = sTK + SM::tile;  // HAS_G

    constexpr int KC = HD / 16;
    constexpr int DT = HD / 32;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int x = lane & 31;
    const int hf = lane >> 5;
    const int bh = blockIdx.x / p.q_blocks;
    const int qb = blockIdx.x % p.q_blocks;
    const int b = bh / p.H, h = bh % p.H;
    const bool vec = p.vec != 0;

    const int qrow = qb * kOwned + wave * 32 + x;
    const bool qvalid = qrow < p.Lq;
    const bool wave_active = (qb * kOwned + wave * 32) < p.Lq;

    u32x4 qB[KC], tqB[KC], gB[KC], doB[KC];
    {
        const elem_t* qp = p.q.head(b, h) + (int64_t)qrow * p.q.sl;
#pragma unroll
        for (int c = 0; c < KC; ++c) qB[c] = load8(qp, 16 * c + 8 * hf, p.D, qvalid, vec);
        if constexpr (HAS_G) {
            const elem_t* tqp = p.tq.head(b, h) + (int64_t)qrow * p.tq.sl;
            const elem_t* gp = p.dTO.head(b, h) + (int64_t)qrow * p.dTO.sl;
#pragma unroll
            for (int c = 0; c < KC; ++c) {
                tqB[c] = load8(tqp, 16 * c + 8 * hf, p.D, qvalid, vec);
                gB[c] = load8(gp, 16 * c + 8 * hf, p.D, qvalid, vec);
            }
        }
        if constexpr (HAS_DO) {
            const elem_t* dop = p.dO.head(b, h) + (int64_t)qrow * p.dO.sl;
#pragma unroll
            for (int c = 0; c < KC; ++c) doB[c] = load8(dop, 16 * c + 8 * hf, p.D, qvalid, vec);
        }
    }
    // Per-lane row statistics; an invalid query lane uses zeros (finite P, results discarded).
    const int64_t so = (int64_t)bh * p.Lr + qrow;
    const float lse2 = qvalid ? p.lse[so] * kLog2e : 0.f;
    const float mu = (qvalid && HAS_G) ? p.mu[so] : 0.f;
    const float s4 = qvalid ? p.s4[so] : 0.f;
    const float s7d = qvalid ? p.s7d[so] : 0.f;

    const elem_t* kg = p.k.head(b, h);
    const elem_t* vg = p.v.head(b, h);
    const elem_t* tkg = HAS_G ? p.tk.head(b, h) : nullptr;
    const elem_t* tvg = HAS_G ? p.tv.head(b, h) : nullptr;
    const float sl2 = p.scale * kLog2e;

    f32x16 dq[DT], dtq[DT];
#pragma unroll
    for (int t = 0; t < DT; ++t) {
        dq[t] = f32x16{0};
        if constexpr (HAS_G) dtq[t] = f32x16{0};
    }

    for (int k0 = 0; k0 < p.Lk; k0 += BN) {
        __syncthreads();
        stage_rows<HD, BN>(sK, kg, p.k.sl, k0, p.Lk, p.D, vec, tid);
        stage_rows<HD, BN>(sV, vg, p.v.sl, k0, p.Lk, p.D, vec, tid);
        if constexpr (HAS_G) {
            stage_rows<HD, BN>(sTK, tkg, p.tk.sl, k0, p.Lk, p.D, vec, tid);
            stage_rows<HD, BN>(sTV, tvg, p.tv.sl, k0, p.Lk, p.D, vec, tid);
        }
        __syncthreads();
        if (!wave_active) continue;

#pragma unroll
        for (int t = 0; t < BN / 32; ++t) {
            const int y0 = 32 * t;
            if (k0 + y0 >= p.Lk) break;
            // Keys beyond Lk are staged as zero rows of K, K_dot, V, V_dot and their P is forced
            // to zero below.
            f32x16 s = {0}, ts = {0}, w = {0}, xy = {0};
#pragma unroll
            for (int c = 0; c < KC; ++c) {
                u32x4 ak = lds_a_rows<HD>(sK, y0, c, x, hf);
                u32x4 av = lds_a_rows<HD>(sV, y0, c, x, hf);
                s = T::mfma(ak, qB[c], s);
                if constexpr (HAS_G) {
                    ts = T::mfma(ak, tqB[c], ts);
                    u32x4 atk = lds_a_rows<HD>(sTK, y0, c, x, hf);
                    ts = T::mfma(atk, qB[c], ts);
                    w = T::mfma(av, gB[c], w);
                    u32x4 atv = lds_a_rows<HD>(sTV, y0, c, x, hf);
                    xy = T::mfma(atv, gB[c], xy);
                }
                if constexpr (HAS_DO) xy = T::mfma(av, doB[c], xy);
            }
            const bool ragged = (k0 + y0 + 32 > p.Lk);
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                float pj = fast_exp2(s[j] * sl2 - lse2);
                // exp(-lse) of a padded key may overflow when every real score is very negative
                if (ragged && k0 + y0 + 8 * (j >> 2) + 4 * hf + (j & 3) >= p.Lk) pj = 0.f;
                if constexpr (HAS_G) {
                    const float n = ts[j] * p.scale - mu;
                    const float dts = pj * (w[j] - s4);
                    w[j] = dts;
                    xy[j] = dts * n + pj * (xy[j] - s7d);
                } else {
                    xy[j] = pj * (xy[j] - s7d);
                }
            }
#pragma unroll
            for (int c = 0; c < 2; ++c) {
                const u32x4 dsB = pack_b<T>(xy, c);
                u32x4 dtsB;
                if constexpr (HAS_G) dtsB = pack_b<T>(w, c);
#pragma unroll
                for (int d = 0; d < DT; ++d) {
                    const u32x4 ak = lds_a_transposed<HD>(sK, y0, c, 32 * d, lane);
                    dq[d] = T::mfma(ak, dsB, dq[d]);
                    if constexpr (HAS_G) {
                        dtq[d] = T::mfma(ak, dtsB, dtq[d]);
                        const u32x4 atk = lds_a_transposed<HD>(sTK, y0, c, 32 * d, lane);
                        dq[d] = T::mfma(atk, dtsB, dq[d]);
                    }
                }
            }
        }
    }

    if (!qvalid) return;
    elem_t* dqrow = p.dq.head(b, h) + (int64_t)qrow * p.dq.sl;
#pragma unroll
    for (int d = 0; d < DT; ++d) store_acc<T>(dqrow, 32 * d, hf, p.D, dq[d], p.scale, vec);
    if constexpr (HAS_G) {
        elem_t* dtqrow = p.dtq.head(b, h) + (int64_t)qrow * p.dtq.sl;
#pragma unroll
        for (int d = 0; d < DT; ++d) store_acc<T>(dtqrow, 32 * d, hf, p.D, dtq[d], p.scale, vec);
    }
}

}  // namespace sjvp
