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
// The reference spends eight launches and 35 tile contractions on this; here it is two launches:
//   bwd_row_kernel   a wavefront owns 32 queries -> dQ, dQ_dot; it also forms s4 and s7d for its
//                    rows from O, TO, dO, G (O(L*D) work instead of five contractions) and leaves
//                    them, with lse in log2 units, in the workspace for
//   bwd_col_kernel   a wavefront owns 32 keys  -> dK, dV, dK_dot, dV_dot,
// each gradient accumulated in fp32 registers by exactly one wavefront and written once, so the
// result is deterministic and never round-trips through 16-bit partial sums.
#pragma once
#include <type_traits>

#include "sjvp_device.hpp"
#include "sjvp_stream.hpp"

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
    float scale;
    int vec;
};

// ---------------------------------------------------------------------------------------------
// Row-owned kernel: dQ (and dQ_dot).  Tiles are transposed (rows = keys in registers, columns =
// this wave's queries in lanes), so the row statistics are per-lane scalars.
// LDS layout on the LDS-DMA path at HD <= 64: [own: the workgroup's rows of Q, O (, Q_dot, G, TO)
// (, dO), one slab per wave each][lse and mu of those rows][ring of K, V (, K_dot, V_dot) stages]; the ring
// doubles as store staging after the last stage.
template <int HD, int R, bool HAS_DO, bool HAS_G, bool DMA>
struct RowSmem {
    static constexpr bool own_lds = DMA && HD <= 64;
    static constexpr int nt = HAS_G ? 4 : 2;
    static constexpr int slot = nt * Slab<HD>::elems;
    static constexpr int n_own = 2 + (HAS_G ? 3 : 0) + (HAS_DO ? 1 : 0);
    static constexpr int own = own_lds ? n_own * kWaves * Slab<HD>::elems : 0;
    static constexpr int stat = own_lds ? 2 * kOwned * 2 : 0;  // two float arrays, in elem_t units
    static constexpr int sink = (own + stat + R * slot) * (int)sizeof(elem_t);
    static constexpr int bytes = sink + kSinkBytes;
};

template <typename T, int HD, int R, bool HAS_DO, bool HAS_G, bool DMA>
__global__ __launch_bounds__(kThreads, 1) void bwd_row_kernel(const BwdParams p) {
    extern __shared__ __align__(16) unsigned char smem_raw[];
    using SM = RowSmem<HD, R, HAS_DO, HAS_G, DMA>;
    constexpr bool OWN_LDS = SM::own_lds;
    elem_t* own = reinterpret_cast<elem_t*>(smem_raw);
    float* own_stat = reinterpret_cast<float*>(own + SM::own);
    elem_t* ring = own + SM::own + SM::stat;
    // own tensor order: Q, O, [Q_dot, G, TO], [dO]
    constexpr int oQ = 0, oO = kWaves * Slab<HD>::elems, oTQ = 2 * kWaves * Slab<HD>::elems,
                  oG = 3 * kWaves * Slab<HD>::elems, oTO = 4 * kWaves * Slab<HD>::elems,
                  oDO = (HAS_G ? 5 : 2) * kWaves * Slab<HD>::elems;

    constexpr int KC = HD / 16;
    constexpr int DT = HD / 32;
    constexpr int SPT = SM::nt * Slab<HD>::per_thread;
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
    ln.init(tid, smem_raw + SM::sink);
    const int qrow = qb * kOwned + wave * 32 + x;
    const bool qvalid = qrow < p.Lq;
    const bool wave_active = (qb * kOwned + wave * 32) < p.Lq;

    u32x4 qB[KC], tqB[KC], gB[KC], doB[KC], oR[KC], toR[KC];
    float lse2 = 0.f, mu = 0.f;
    const int64_t so = (int64_t)bh * p.Lr + qrow;
    if constexpr (OWN_LDS) {
        // coalesced LDS-DMA copies of the workgroup's own rows; they are read back as B operands
        // after the first ring stages have been issued
        const int r0 = qb * kOwned;
        auto own_fill = [&](int off, const TensorView& t) {
#pragma unroll
            for (int s4 = 0; s4 < kWaves; ++s4)
                fill_slab<HD, true>(ln, own + off + s4 * Slab<HD>::elems, t.head(b, h), t.sl, r0 + 32 * s4,
                                    p.Lq, p.D, true);
        };
        own_fill(oQ, p.q);
        own_fill(oO, p.o);
        if constexpr (HAS_G) {
            own_fill(oTQ, p.tq);
            own_fill(oG, p.dTO);
            own_fill(oTO, p.to);
        }
        if constexpr (HAS_DO) own_fill(oDO, p.dO);
        // lse (lanes 0-31) and mu (lanes 32-63) of this wave's 32 rows; rows < Lr exist in both
        const float* src = hf == 0 ? p.lse : p.mu;
        if (HAS_G || hf == 0) dma4(src + so, lds_addr(own_stat) + (uint32_t)(wave * 64 * 4));
    } else {
        const elem_t* qp = p.q.head(b, h) + (int64_t)qrow * p.q.sl;
        const elem_t* op = p.o.head(b, h) + (int64_t)qrow * p.o.sl;
#pragma unroll
        for (int c = 0; c < KC; ++c) {
            qB[c] = load8(qp, 16 * c + 8 * hf, p.D, qvalid, vec);
            oR[c] = load8(op, 16 * c + 8 * hf, p.D, qvalid, vec);
        }
        if constexpr (HAS_G) {
            const elem_t* tqp = p.tq.head(b, h) + (int64_t)qrow * p.tq.sl;
            const elem_t* gp = p.dTO.head(b, h) + (int64_t)qrow * p.dTO.sl;
            const elem_t* top = p.to.head(b, h) + (int64_t)qrow * p.to.sl;
#pragma unroll
            for (int c = 0; c < KC; ++c) {
                tqB[c] = load8(tqp, 16 * c + 8 * hf, p.D, qvalid, vec);
                gB[c] = load8(gp, 16 * c + 8 * hf, p.D, qvalid, vec);
                toR[c] = load8(top, 16 * c + 8 * hf, p.D, qvalid, vec);
            }
        }
        if constexpr (HAS_DO) {
            const elem_t* dop = p.dO.head(b, h) + (int64_t)qrow * p.dO.sl;
#pragma unroll
            for (int c = 0; c < KC; ++c) doB[c] = load8(dop, 16 * c + 8 * hf, p.D, qvalid, vec);
        }
        // Per-lane row statistics; an invalid query lane uses zeros (finite P, results discarded).
        lse2 = qvalid ? p.lse[so] * kLog2e : 0.f;
        mu = (qvalid && HAS_G) ? p.mu[so] : 0.f;
        if constexpr (DMA) {
            // retire these loads before the first LDS-DMA copy so that wait_stages() only has the
            // ring's traffic to count
            asm volatile("" : "+v"(lse2), "+v"(mu));
#pragma unroll
            for (int c = 0; c < KC; ++c) {
                asm volatile("" : "+v"(qB[c]), "+v"(oR[c]));
                if constexpr (HAS_G) asm volatile("" : "+v"(tqB[c]), "+v"(gB[c]), "+v"(toR[c]));
                if constexpr (HAS_DO) asm volatile("" : "+v"(doB[c]));
            }
        }
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
    if constexpr (!OWN_LDS) row_sums();
    const elem_t* kg = p.k.head(b, h);
    const elem_t* vg = p.v.head(b, h);
    const elem_t* tkg = HAS_G ? p.tk.head(b, h) : nullptr;
    const elem_t* tvg = HAS_G ? p.tv.head(b, h) : nullptr;
    const float sl2 = p.scale * kLog2e;

    auto issue = [&](int stage) {
        elem_t* slot = ring + (stage % R) * SM::slot;
        const int row0 = stage * kStageRows;
        fill_slab<HD, DMA>(ln, slot, kg, p.k.sl, row0, p.Lk, p.D, vec);
        fill_slab<HD, DMA>(ln, slot + Slab<HD>::elems, vg, p.v.sl, row0, p.Lk, p.D, vec);
        if constexpr (HAS_G) {
            fill_slab<HD, DMA>(ln, slot + 2 * Slab<HD>::elems, tkg, p.tk.sl, row0, p.Lk, p.D, vec);
            fill_slab<HD, DMA>(ln, slot + 3 * Slab<HD>::elems, tvg, p.tv.sl, row0, p.Lk, p.D, vec);
        }
    };

    f32x16 dq[DT], dtq[DT];
#pragma unroll
    for (int t = 0; t < DT; ++t) {
        dq[t] = f32x16{0};
        if constexpr (HAS_G) dtq[t] = f32x16{0};
    }

    auto compute = [&](const elem_t* slot, int k0, auto ragged_tag) {
        constexpr bool RAGGED = decltype(ragged_tag)::value;
        const elem_t* sK = slot;
        const elem_t* sV = slot + Slab<HD>::elems;
        const elem_t* sTK = slot + 2 * Slab<HD>::elems;
        const elem_t* sTV = slot + 3 * Slab<HD>::elems;
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
    if constexpr (DMA) {
        int issued = 0;
        for (int s = 0; s < R && s < n; ++s, ++issued) issue(s);
        if constexpr (OWN_LDS) {
            wait_stages<SPT>(issued);  // the own rows were issued before these stages
            __syncthreads();
            const int sw = wave * Slab<HD>::elems;
            read_b_operands<HD>(qB, own + oQ + sw, x, hf);
            read_b_operands<HD>(oR, own + oO + sw, x, hf);
            if constexpr (HAS_G) {
                read_b_operands<HD>(tqB, own + oTQ + sw, x, hf);
                read_b_operands<HD>(gB, own + oG + sw, x, hf);
                read_b_operands<HD>(toR, own + oTO + sw, x, hf);
            }
            if constexpr (HAS_DO) read_b_operands<HD>(doB, own + oDO + sw, x, hf);
            lse2 = own_stat[wave * 64 + x] * kLog2e;
            if constexpr (HAS_G) mu = own_stat[wave * 64 + 32 + x];
            row_sums();
        }
    }
    if (hf == 0) {  // every row below Lr is written (zeros beyond Lq except lse2, which is finite):
                    // the column-owned kernel, which runs after this one, stages 32-row groups
        p.lse2[so] = lse2;
        p.s4[so] = s4;
        p.s7d[so] = s7d;
    }
    for (int i = 0; i < n; ++i) {
        if constexpr (DMA) {
            wait_stages<SPT>(ring_issued_before(i, R, n) - 1 - i);
            __syncthreads();
            if (i >= 1 && i - 1 + R < n) issue(i - 1 + R);
        } else {
            __syncthreads();
            issue(i);
            __syncthreads();
        }
        if (!wave_active) continue;
        const elem_t* slot = ring + (i % R) * SM::slot;
        const int k0 = i * kStageRows;
        if (k0 + kStageRows > p.Lk) {
            compute(slot, k0, std::true_type{});
        } else {
            compute(slot, k0, std::false_type{});
        }
    }
    if constexpr (DMA) {
        __syncthreads();  // every wave is done reading the ring: it becomes the store staging area
        if (!wave_active) return;
        elem_t* stage_tile = ring + wave * StoreStage<HD>::elems;
        const int row0 = qb * kOwned + wave * 32;
        store_tile_coalesced<T, HD>(stage_tile, p.dq.head(b, h), p.dq.sl, row0, p.Lq, p.D, dq, p.scale,
                                    lane);
        if constexpr (HAS_G)
            store_tile_coalesced<T, HD>(stage_tile, p.dtq.head(b, h), p.dtq.sl, row0, p.Lq, p.D, dtq,
                                        p.scale, lane);
    } else {
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
}

// ---------------------------------------------------------------------------------------------
// Column-owned kernel: a wavefront owns 32 keys and streams the queries.  DO_K selects dK (and
// dK_dot), DO_V selects dV (and dV_dot); DT0/NDT select the 32-wide head-dimension tiles that are
// accumulated (at HD = 128 the work is split to stay inside the register file).
// LDS layout on the LDS-DMA path at HD <= 64: [own: the workgroup's rows of K, V (, K_dot, V_dot),
// one slab per wave each][ring of Q (, Q_dot, G) (, dO) stages, each followed by its row statistics]; the
// ring doubles as store staging after the last stage.
template <int HD, int R, bool HAS_DO, bool HAS_G, bool DMA>
struct ColSmem {
    static constexpr bool own_lds = DMA && HD <= 64;
    static constexpr int nt = 1 + (HAS_G ? 2 : 0) + (HAS_DO ? 1 : 0);
    static constexpr int stat_elems = 4 * kStageRows * 2;  // 4 float arrays of 32, in elem_t units
    static constexpr int slot = nt * Slab<HD>::elems + stat_elems;
    static constexpr int own = own_lds ? (HAS_G ? 4 : 2) * kWaves * Slab<HD>::elems : 0;
    static constexpr int sink = (own + R * slot) * (int)sizeof(elem_t);
    static constexpr int bytes = sink + kSinkBytes;
};

template <typename T, int HD, int R, bool HAS_DO, bool HAS_G, bool DO_K, bool DO_V, int DT0, int NDT,
          bool DMA>
__global__ __launch_bounds__(kThreads, (DO_K && DO_V && HAS_G) ? 1 : 2) void bwd_col_kernel(
    const BwdParams p) {
    extern __shared__ __align__(16) unsigned char smem_raw[];
    using SM = ColSmem<HD, R, HAS_DO, HAS_G, DMA>;
    constexpr bool OWN_LDS = SM::own_lds;
    elem_t* own = reinterpret_cast<elem_t*>(smem_raw);
    elem_t* ring = own + SM::own;
    // own tensor order: K, V, [K_dot, V_dot];  slot layout: Q | [Q_dot | G] | [dO] | stats(lse2, mu, s4, s7d)
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
    ln.init(tid, smem_raw + SM::sink);
    // LDS-DMA instructions per stage issued by every wave: the tensors plus one 4-byte copy of
    // statistics
    constexpr int SPT = SM::nt * Slab<HD>::per_thread + 1;
    const int krow = kb * kOwned + wave * 32 + x;  // the key this lane owns
    const bool kvalid = krow < p.Lk;
    const bool wave_active = (kb * kOwned + wave * 32) < p.Lk;

    u32x4 kB[KC], vB[KC], tkB[KC], tvB[KC];
    if constexpr (OWN_LDS) {
        const int r0 = kb * kOwned;
        auto own_fill = [&](int idx, const TensorView& t) {
#pragma unroll
            for (int s4 = 0; s4 < kWaves; ++s4)
                fill_slab<HD, true>(ln, own + (kWaves * idx + s4) * Slab<HD>::elems, t.head(b, h), t.sl,
                                    r0 + 32 * s4, p.Lk, p.D, true);
        };
        own_fill(0, p.k);
        own_fill(1, p.v);
        if constexpr (HAS_G) {
            own_fill(2, p.tk);
            own_fill(3, p.tv);
        }
    } else {
        const elem_t* kp = p.k.head(b, h) + (int64_t)krow * p.k.sl;
        const elem_t* vp = p.v.head(b, h) + (int64_t)krow * p.v.sl;
#pragma unroll
        for (int c = 0; c < KC; ++c) {
            kB[c] = load8(kp, 16 * c + 8 * hf, p.D, kvalid, vec);
            if constexpr (DO_K) vB[c] = load8(vp, 16 * c + 8 * hf, p.D, kvalid, vec);
        }
        if constexpr (HAS_G) {
            const elem_t* tkp = p.tk.head(b, h) + (int64_t)krow * p.tk.sl;
            const elem_t* tvp = p.tv.head(b, h) + (int64_t)krow * p.tv.sl;
#pragma unroll
            for (int c = 0; c < KC; ++c) {
                tkB[c] = load8(tkp, 16 * c + 8 * hf, p.D, kvalid, vec);
                if constexpr (DO_K) tvB[c] = load8(tvp, 16 * c + 8 * hf, p.D, kvalid, vec);
            }
        }
        if constexpr (DMA) {
#pragma unroll
            for (int c = 0; c < KC; ++c) {
                asm volatile("" : "+v"(kB[c]));
                if constexpr (DO_K) asm volatile("" : "+v"(vB[c]));
                if constexpr (HAS_G) {
                    asm volatile("" : "+v"(tkB[c]));
                    if constexpr (DO_K) asm volatile("" : "+v"(tvB[c]));
                }
            }
        }
    }
    const elem_t* qg = p.q.head(b, h);
    const elem_t* tqg = HAS_G ? p.tq.head(b, h) : nullptr;
    const elem_t* gg = HAS_G ? p.dTO.head(b, h) : nullptr;
    const elem_t* dog = HAS_DO ? p.dO.head(b, h) : nullptr;
    const float sl2 = p.scale * kLog2e;

    auto issue = [&](int stage) {
        elem_t* slot = ring + (stage % R) * SM::slot;
        const int row0 = stage * kStageRows;
        fill_slab<HD, DMA>(ln, slot, qg, p.q.sl, row0, p.Lq, p.D, vec);
        if constexpr (HAS_G) {
            fill_slab<HD, DMA>(ln, slot + oTQ, tqg, p.tq.sl, row0, p.Lq, p.D, vec);
            fill_slab<HD, DMA>(ln, slot + oG, gg, p.dTO.sl, row0, p.Lq, p.D, vec);
        }
        if constexpr (HAS_DO) fill_slab<HD, DMA>(ln, slot + oDO, dog, p.dO.sl, row0, p.Lq, p.D, vec);
        // Row statistics of the stage (rows < Lr are defined in all four arrays; rows beyond Lq
        // hold finite values and multiply zero rows of Q, Q_dot, G, dO below).
        float* st = reinterpret_cast<float*>(slot + oST);
        const int64_t so = (int64_t)bh * p.Lr + row0 + (lane & 31);
        // the four arrays (lse2, mu, s4, s7d) are dealt to the waves, 32 lanes each; every wave
        // issues exactly one 4-byte LDS-DMA instruction
        constexpr int APW = 4 / kWaves;  // arrays per wave
        const int arr = wave * APW + hf;
        if (hf < APW) {
            const float* src = arr == 0 ? p.lse2 : arr == 1 ? p.mu : arr == 2 ? p.s4 : p.s7d;
            if (arr == 1 && !HAS_G) src = p.s4;  // mu is not used without the tangent cotangent
            if constexpr (DMA) {
                dma4(src + so, lds_addr(st) + (uint32_t)(wave * APW * 32 * 4));
            } else {
                st[arr * 32 + (lane & 31)] = src[so];
            }
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

    auto compute = [&](const elem_t* slot) {
        const elem_t* sQ = slot;
        const elem_t* sTQ = slot + oTQ;
        const elem_t* sG = slot + oG;
        const elem_t* sDO = slot + oDO;
        const float* sStat = reinterpret_cast<const float*>(slot + oST);
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
    if constexpr (DMA) {
        int issued = 0;
        for (int s = 0; s < R && s < n; ++s, ++issued) issue(s);
        if constexpr (OWN_LDS) {
            wait_stages<SPT>(issued);  // the own rows were issued before these stages
            __syncthreads();
            read_b_operands<HD>(kB, own + wave * Slab<HD>::elems, x, hf);
            if constexpr (DO_K) read_b_operands<HD>(vB, own + (kWaves + wave) * Slab<HD>::elems, x, hf);
            if constexpr (HAS_G) {
                read_b_operands<HD>(tkB, own + (2 * kWaves + wave) * Slab<HD>::elems, x, hf);
                if constexpr (DO_K)
                    read_b_operands<HD>(tvB, own + (3 * kWaves + wave) * Slab<HD>::elems, x, hf);
            }
        }
    }
    for (int i = 0; i < n; ++i) {
        if constexpr (DMA) {
            wait_stages<SPT>(ring_issued_before(i, R, n) - 1 - i);
            __syncthreads();
            if (i >= 1 && i - 1 + R < n) issue(i - 1 + R);
        } else {
            __syncthreads();
            issue(i);
            __syncthreads();
        }
        if (!wave_active) continue;
        compute(ring + (i % R) * SM::slot);
    }
    if constexpr (DMA) {
        __syncthreads();  // every wave is done reading the ring: it becomes the store staging area
        if (!wave_active) return;
        elem_t* stage_tile = ring + wave * StoreStage<HD>::elems;
        const int row0 = kb * kOwned + wave * 32;
        // NDT tiles starting at head-dimension tile DT0: the staging tile and the row pointers are
        // offset by 32*DT0 columns, and the column bound is reduced accordingly
        const int dcol = 32 * DT0;
        auto put = [&](const OutView& t, const f32x16* acc, float mul) {
            store_tile_coalesced<T, 32 * NDT>(stage_tile, t.head(b, h) + dcol, t.sl, row0, p.Lk,
                                              p.D - dcol, acc, mul, lane);
        };
        if constexpr (DO_K) {
            put(p.dk, dk, p.scale);
            if constexpr (HAS_G) put(p.dtk, dtk, p.scale);
        }
        if constexpr (DO_V) {
            put(p.dv, dv, 1.0f);
            if constexpr (HAS_G) put(p.dtv, dtv, 1.0f);
        }
    } else {
        if (!kvalid) return;
        if constexpr (DO_K) {
            elem_t* dkrow = p.dk.head(b, h) + (int64_t)krow * p.dk.sl;
#pragma unroll
            for (int d = 0; d < NDT; ++d)
                store_acc<T>(dkrow, 32 * (DT0 + d), hf, p.D, dk[d], p.scale, vec);
            if constexpr (HAS_G) {
                elem_t* dtkrow = p.dtk.head(b, h) + (int64_t)krow * p.dtk.sl;
#pragma unroll
                for (int d = 0; d < NDT; ++d)
                    store_acc<T>(dtkrow, 32 * (DT0 + d), hf, p.D, dtk[d], p.scale, vec);
            }
        }
        if constexpr (DO_V) {
            elem_t* dvrow = p.dv.head(b, h) + (int64_t)krow * p.dv.sl;
#pragma unroll
            for (int d = 0; d < NDT; ++d)
                store_acc<T>(dvrow, 32 * (DT0 + d), hf, p.D, dv[d], 1.0f, vec);
            if constexpr (HAS_G) {
                elem_t* dtvrow = p.dtv.head(b, h) + (int64_t)krow * p.dtv.sl;
#pragma unroll
                for (int d = 0; d < NDT; ++d)
                    store_acc<T>(dtvrow, 32 * (DT0 + d), hf, p.D, dtv[d], 1.0f, vec);
            }
        }
    }
}

}  // namespace sjvp
