// Single-launch attention-JVP backward, 16-wide form, for short key axes (Lk <= 128, head dimension
// <= 64, 16-byte aligned rows): one workgroup of eight wavefronts per (batch, head) owns every key
// (16 per wavefront), streams the queries once in stages of 32 and produces all six gradients, so
// each of the sixteen tensors crosses HBM exactly once and every score-side tile is computed once.
//
// Mathematics as in sjvp_bwd.hpp.  Per stage of 32 queries:
//   1. threads 0..255: row sums s4, s7d of the NEXT stage from its G, dO, O, TO slabs (8 per row);
//   2. wave w (keys 16w..16w+15): tiles S, S_dot, W, XY -> P, P_dot, dS_dot, dS (queries in
//      registers, keys in lanes); dK, dV, dK_dot, dV_dot accumulate in registers; dS and dS_dot go
//      as 16-bit into an LDS bounce tile [key][query];
//   3. after a barrier, wave w forms one 16x16 tile of dQ and one of dQ_dot for the stage from the
//      bounce tile and the own rows of K, K_dot (both through transposing LDS reads) and puts them
//      into a staging tile, from where 512 threads send the stage's dQ / dQ_dot rows out as whole
//      rows after the next barrier: a stage's dQ rows are complete after one pass over the keys, so
//      nothing is accumulated across stages and no atomics or partial sums are needed.
// Results are deterministic.
#pragma once
#include "sjvp_bwd.hpp"
#include "sjvp_w16.hpp"

namespace sjvp {

// LDS layout: [own K, K_dot: four slabs each][own V, V_dot: four slabs each; once they have been
// read into registers the same memory is the bounce tile dS (, dS_dot): [128 keys][32 queries + pad]]
// [ring of query stages: Q | [Q_dot | G] | [dO] | O | [TO] | raw lse, mu | lse2, mu, s4, s7d]
// [staging tile of a stage's dQ (, dQ_dot)][sink]
// In the last stage the two ring slots that no stage uses again hold the per-wave staging tiles of the
// output stores.
template <int HD, int R, bool HAS_DO, bool HAS_G>
struct Fused16Smem {
    static constexpr int nt = 2 + (HAS_G ? 3 : 0) + (HAS_DO ? 1 : 0);
    static constexpr int stat_elems = 6 * kStageRows * 2;  // 6 float arrays of 32, in elem_t units
    static constexpr int slot = nt * Slab<HD>::elems + stat_elems;
    static constexpr int own_k = (HAS_G ? 2 : 1) * 4 * Slab<HD>::elems;  // K (, K_dot)
    static constexpr int own_v = own_k;                                  // V (, V_dot)
    // bounce tile [128 keys][32 queries], 64 bytes per key: eight units of four queries, unit u of key y at
    // position u ^ bounce_swz(y).  Two buffers (even and odd stages) of one tile per kind (dS, dS_dot).
    static constexpr int bounce_one = kOwned16 * kStageRows;
    static constexpr int bounce = 2 * (HAS_G ? 2 : 1) * bounce_one;
    static constexpr int vregion = own_v > bounce ? own_v : bounce;
    // staging of a stage's dQ (, dQ_dot) tiles, [32 queries][HD + 8], so that they leave as whole rows;
    // two buffers (even and odd stages)
    static constexpr int qpitch = HD + 8;
    static constexpr int qstage_one = (HAS_G ? 2 : 1) * kStageRows * qpitch;
    static constexpr int qstage = 2 * qstage_one;
    static constexpr int sink = (own_k + vregion + R * slot + qstage) * (int)sizeof(elem_t);
    static constexpr int bytes = sink + kSink16;
};

// Position of unit u (four queries, 8 bytes) of key y in its 64-byte row of a bounce tile: with it the
// 8-byte writes of a wave (16 keys x 4 units per instruction) and the transposing reads (4 keys x 4 units
// per group of 16 lanes, groups 4 keys apart) spread over all banks.
__device__ __forceinline__ int bounce_swz(int key) { return 4 * ((key >> 2) & 1) + 2 * ((key >> 3) & 1); }

// ROPE: q, k and their tangents are rotated by p.rope once they are in LDS (own K, K_dot rows in the
// prologue, each stage's Q, Q_dot slabs by the threads that do not form row sums), and the gradients
// dQ, dQ_dot, dK, dK_dot go back through the inverse rotation on their way out (head dimension 64).
template <typename T, int HD, int R, bool HAS_DO, bool HAS_G, bool ROPE = false>
__global__ __launch_bounds__(kThreads16, HAS_G ? 2 : 4) void bwd_fused16_kernel(const BwdParams p) {
    static_assert(HD <= 64, "the accumulators of four gradients must fit the register file");
    static_assert(!ROPE || HD == 64, "the folded rotation covers a head dimension of 64");
    extern __shared__ __align__(16) unsigned char smem_raw[];
    using SM = Fused16Smem<HD, R, HAS_DO, HAS_G>;
    constexpr int SE = Slab<HD>::elems;
    elem_t* ownK = reinterpret_cast<elem_t*>(smem_raw);  // K slabs 0..3, then K_dot slabs 0..3
    elem_t* ownV = ownK + SM::own_k;                      // V slabs 0..3, then V_dot slabs 0..3
    elem_t* bounce0 = ownV;  // aliases V, V_dot after the prologue: [buffer][dS | dS_dot][key][query]
    constexpr int oBT = SM::bounce_one, BBUF = (HAS_G ? 2 : 1) * SM::bounce_one;
    elem_t* ring = ownV + SM::vregion;
    elem_t* qstage = ring + R * SM::slot;                 // dQ (, dQ_dot) tiles of one stage on their way out
    // slot layout
    constexpr int oTQ = SE, oG = 2 * SE, oDO = (HAS_G ? 3 : 1) * SE;
    constexpr int oO = oDO + (HAS_DO ? SE : 0), oTO = oO + SE;
    constexpr int oST = SM::nt * SE;
    constexpr int BP = kStageRows;  // elements per key row of a bounce tile
    constexpr int KC = HD / 32;
    constexpr int DT = HD / 16;

    const int tid = threadIdx.x;
    if (tid == 0) *reinterpret_cast<unsigned*>(smem_raw + SM::sink + 8) = 0u;  // see `announced` below
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 15;
    const int g = lane >> 4;
    // Heads are taken in descending order, groups of eight kept together (workgroups are dealt to
    // the eight XCDs round-robin, and the forward takes head i in workgroup i): when the backward
    // directly follows the forward, the heads the forward touched last are still in their XCD's L2.
    const int groups = (int)gridDim.x >> 3;
    const int bh = (int)blockIdx.x < 8 * groups ? 8 * (groups - 1 - ((int)blockIdx.x >> 3)) + ((int)blockIdx.x & 7)
                                                : (int)blockIdx.x;
    const int b = bh / p.H, h = bh % p.H;
    const int key_slabs = (p.Lk + 31) >> 5;           // 32-key slabs that hold at least one key
    const bool wave_active = (wave >> 1) < key_slabs;  // waves of a partly filled slab all take part
    // Keys beyond Lk are zero rows: their score is 0 and exp(-lse) overflows once every real score of
    // a row is very negative, so their P is forced to zero (they would reach dQ, dQ_dot of valid
    // queries through the bounce tile as 0 * inf otherwise).  Wave-uniform flag, per-lane predicate.
    const bool ragged_keys = wave * 16 + 16 > p.Lk;
    const bool key_padded = wave * 16 + n >= p.Lk;
    // Without the cotangent on TO a wave needs few enough registers for two workgroups per compute unit
    // (four waves per SIMD, 128 registers), if the lane geometry of the steps outside step 2 is formed where
    // it is used instead of being carried through the stage loop: there it comes from a lane id the
    // compiler cannot see through.
    auto lane_now = [&]() {
        int v = lane;
        if constexpr (!HAS_G) asm volatile("" : "+v"(v));
        return v;
    };

    using StagePlan = CopyPlan<HD, SM::nt, 1>;
    constexpr int SPT = StagePlan::N + 1;  // plus one 4-byte copy of statistics
    StagePlan plan;
    {
        const Src q{p.q.head(b, h), p.q.sl}, o{p.o.head(b, h), p.o.sl};
        if constexpr (HAS_G && HAS_DO)
            plan.init(tid, 0, p.D, smem_raw + SM::sink, q, Src{p.tq.head(b, h), p.tq.sl},
                      Src{p.dTO.head(b, h), p.dTO.sl}, Src{p.dO.head(b, h), p.dO.sl}, o,
                      Src{p.to.head(b, h), p.to.sl});
        else if constexpr (HAS_G)
            plan.init(tid, 0, p.D, smem_raw + SM::sink, q, Src{p.tq.head(b, h), p.tq.sl},
                      Src{p.dTO.head(b, h), p.dTO.sl}, o, Src{p.to.head(b, h), p.to.sl});
        else
            plan.init(tid, 0, p.D, smem_raw + SM::sink, q, Src{p.dO.head(b, h), p.dO.sl}, o);
    }
    const int ns = (p.Lq + kStageRows - 1) / kStageRows;
    int issued = 0;
    auto issue_next = [&]() {
        elem_t* slot = ring + (issued % R) * SM::slot;
        const int row0 = issued * kStageRows;
        plan.issue(slot, p.Lq - row0, p.D == HD && row0 + kStageRows <= p.Lq);
        // raw lse (wave 0) and mu (wave 1) of the stage's rows (rows < Lr exist); every wave issues
        // exactly one 4-byte LDS-DMA instruction, the others as a placeholder into the sink
        float* raw = reinterpret_cast<float*>(slot + oST);
        if (wave < 2) {
            const float* src = (wave == 1 && HAS_G) ? p.mu : p.lse;
            if (lane < 32) dma4(src + (int64_t)bh * p.Lr + row0 + lane, lds_addr(raw) + (uint32_t)(wave * 32 * 4));
        } else {
            if (lane == 0) dma4(plan.any, plan.sink);
        }
        ++issued;
    };
    issue_next();
    // The first stage is issued before the own rows: it lands first and its row sums are formed while the
    // own rows (four times its size) are still on their way.
    constexpr int OWN = (HAS_G ? 16 : 8) * Slab<HD>::chunks / kThreads16;  // own-row copies per wave
    {
        CopyPlan<HD, HAS_G ? 16 : 8, 4> own_plan;
        if constexpr (HAS_G)
            own_plan.init(tid, 0, p.D, smem_raw + SM::sink, Src{p.k.head(b, h), p.k.sl},
                          Src{p.tk.head(b, h), p.tk.sl}, Src{p.v.head(b, h), p.v.sl},
                          Src{p.tv.head(b, h), p.tv.sl});
        else
            own_plan.init(tid, 0, p.D, smem_raw + SM::sink, Src{p.k.head(b, h), p.k.sl},
                          Src{p.v.head(b, h), p.v.sl});
        own_plan.issue(ownK, p.Lk, p.D == HD && p.Lk == kOwned16);
    }
    const float sl2 = p.scale * kLog2e;

    // Row sums of a landed stage: thread t < 256 handles row t/8, columns 8*(t%8) .. +7; the eight
    // partial sums meet through DPP moves and the thread of column 0 writes the row's statistics.
    auto row_sums = [&](elem_t* slot) {
        if (tid >= 256) return;
        const int tid_l = wave * 64 + lane_now();
        const int r = tid_l >> 3, part = tid_l & 7;
        float s4 = 0.f, s7d = 0.f;
        if (part < HD / 8) {
            const int off = r * HD + ((part ^ swz<HD>(r)) << 3);
            const u32x4 o4 = *reinterpret_cast<const u32x4*>(slot + oO + off);
            u32x4 g4, t4, d4;
            if constexpr (HAS_G) {
                g4 = *reinterpret_cast<const u32x4*>(slot + oG + off);
                t4 = *reinterpret_cast<const u32x4*>(slot + oTO + off);
            }
            if constexpr (HAS_DO) d4 = *reinterpret_cast<const u32x4*>(slot + oDO + off);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if constexpr (HAS_G) {
                    s4 = T::dot2(g4[i], o4[i], s4);
                    s7d = T::dot2(g4[i], t4[i], s7d);
                }
                if constexpr (HAS_DO) s7d = T::dot2(d4[i], o4[i], s7d);
            }
        }
        s4 = sum8(s4);
        s7d = sum8(s7d);
        if (part == 0) {
            float* raw = reinterpret_cast<float*>(slot + oST);
            float* fin = raw + 2 * kStageRows;
            fin[0 * kStageRows + r] = raw[r] * kLog2e;
            fin[1 * kStageRows + r] = HAS_G ? raw[kStageRows + r] : 0.f;
            fin[2 * kStageRows + r] = -s4;  // the W and XY tiles start from these instead of subtracting them
            fin[3 * kStageRows + r] = -s7d;
        }
    };

    u32x4 kB[KC], vB[KC], tkB[KC], tvB[KC];
    f32x4 dk[DT], dv[DT], dtk[DT], dtv[DT];
#pragma unroll
    for (int t = 0; t < DT; ++t) {
        dk[t] = f32x4{0.f, 0.f, 0.f, 0.f};
        dv[t] = f32x4{0.f, 0.f, 0.f, 0.f};
        dtk[t] = f32x4{0.f, 0.f, 0.f, 0.f};
        dtv[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

    // Step 2: this wave's 32 x 16 tiles of one stage.
    auto tile = [&](const elem_t* slot, elem_t* bounceS) {
        const elem_t* sQ = slot;
        const elem_t* sTQ = slot + oTQ;
        const elem_t* sG = slot + oG;
        const elem_t* sDO = slot + oDO;
        const float* sStat = reinterpret_cast<const float*>(slot + oST) + 2 * kStageRows;
        f32x4 s[2], ts[2], w[2], xy[2];
        auto scores = [&](int t) __attribute__((always_inline)) {
            s[t] = f32x4{0.f, 0.f, 0.f, 0.f};
            ts[t] = f32x4{0.f, 0.f, 0.f, 0.f};
            // W - s4 and XY - s7d: the accumulators start at the negated row sums (register j of tile t is
            // query 16t + 4g + j)
            w[t] = *reinterpret_cast<const f32x4*>(sStat + 2 * kStageRows + 16 * t + 4 * g);
            xy[t] = *reinterpret_cast<const f32x4*>(sStat + 3 * kStageRows + 16 * t + 4 * g);
#pragma unroll
            for (int c = 0; c < KC; ++c) {
                const u32x4 aq = lds_a_rows16<HD>(sQ, t, c, n, g);
                s[t] = T::mfma16(aq, kB[c], s[t]);
                if constexpr (HAS_G) {
                    ts[t] = T::mfma16(aq, tkB[c], ts[t]);
                    const u32x4 atq = lds_a_rows16<HD>(sTQ, t, c, n, g);
                    ts[t] = T::mfma16(atq, kB[c], ts[t]);
                    const u32x4 ag = lds_a_rows16<HD>(sG, t, c, n, g);
                    w[t] = T::mfma16(ag, vB[c], w[t]);
                    xy[t] = T::mfma16(ag, tvB[c], xy[t]);
                }
                if constexpr (HAS_DO) {
                    const u32x4 ado = lds_a_rows16<HD>(sDO, t, c, n, g);
                    xy[t] = T::mfma16(ado, vB[c], xy[t]);
                }
            }
        };
        // in place: s -> P, ts -> P_dot, w -> dS_dot, xy -> dS  (register j of tile t is query 16t + 4g + j)
        auto pointwise_of = [&](int t, auto ragged_tag) __attribute__((always_inline)) {
            const int r0 = 16 * t + 4 * g;
            const f32x4 lse4 = *reinterpret_cast<const f32x4*>(sStat + 0 * kStageRows + r0);
            const f32x4 mu4 = *reinterpret_cast<const f32x4*>(sStat + 1 * kStageRows + r0);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                float pj = fast_exp2(fmaf(s[t][j], sl2, -lse4[j]));
                if (decltype(ragged_tag)::value && key_padded) pj = 0.f;
                s[t][j] = pj;
                if constexpr (HAS_G) {
                    const float nn = fmaf(ts[t][j], p.scale, -mu4[j]);
                    const float dts = pj * w[t][j];
                    w[t][j] = dts;
                    xy[t][j] = fmaf(dts, nn, pj * xy[t][j]);
                    ts[t][j] = pj * nn;
                } else {
                    xy[t][j] = pj * xy[t][j];
                }
            }
        };
        // a wave whose sixteen keys all exist (wave-uniform) skips the selects of the padded keys
        auto pointwise = [&](int t) __attribute__((always_inline)) {
            if (ragged_keys) pointwise_of(t, std::true_type{});
            else pointwise_of(t, std::false_type{});
        };
        // the second tile's MFMA chains run under the first tile's pointwise arithmetic
        scores(0);
        __builtin_amdgcn_sched_barrier(0);
        scores(1);
        pointwise(0);
        __builtin_amdgcn_sched_barrier(0);
        // the first transposed operands of the output contractions are fetched under the second
        // tile's pointwise arithmetic
        const u32x4 aq0 = lds_a_tr16<HD>(sQ, 0, lane);
        u32x4 atq0, ag0, ado0;
        if constexpr (HAS_G) {
            atq0 = lds_a_tr16<HD>(sTQ, 0, lane);
            ag0 = lds_a_tr16<HD>(sG, 0, lane);
        }
        if constexpr (HAS_DO) ado0 = lds_a_tr16<HD>(sDO, 0, lane);
        __builtin_amdgcn_sched_barrier(0);
        pointwise(1);
        const u32x4 pB = pack_b16<T>(s[0], s[1]);
        const u32x4 dsB = pack_b16<T>(xy[0], xy[1]);
        u32x4 pdB, dtsB;
        if constexpr (HAS_G) {
            pdB = pack_b16<T>(ts[0], ts[1]);
            dtsB = pack_b16<T>(w[0], w[1]);
        }
        // bounce[key][query]: the packed registers 2t, 2t+1 are queries 16t + 4g .. + 3, i.e. unit 4t + g, of
        // key 16w + n
        {
            const int key = wave * 16 + n;
            elem_t* row = bounceS + key * BP;
            const int u0 = (g ^ bounce_swz(key)) << 2, u1 = ((4 + g) ^ bounce_swz(key)) << 2;
            *reinterpret_cast<u32x2*>(row + u0) = u32x2{dsB[0], dsB[1]};
            *reinterpret_cast<u32x2*>(row + u1) = u32x2{dsB[2], dsB[3]};
            if constexpr (HAS_G) {
                *reinterpret_cast<u32x2*>(row + oBT + u0) = u32x2{dtsB[0], dtsB[1]};
                *reinterpret_cast<u32x2*>(row + oBT + u1) = u32x2{dtsB[2], dtsB[3]};
            }
        }
#pragma unroll
        for (int d = 0; d < DT; ++d) {
            const u32x4 aq = d == 0 ? aq0 : lds_a_tr16<HD>(sQ, 16 * d, lane);
            dk[d] = T::mfma16(aq, dsB, dk[d]);
            if constexpr (HAS_G) {
                dtk[d] = T::mfma16(aq, dtsB, dtk[d]);
                const u32x4 atq = d == 0 ? atq0 : lds_a_tr16<HD>(sTQ, 16 * d, lane);
                dk[d] = T::mfma16(atq, dtsB, dk[d]);
                const u32x4 ag = d == 0 ? ag0 : lds_a_tr16<HD>(sG, 16 * d, lane);
                dtv[d] = T::mfma16(ag, pB, dtv[d]);
                dv[d] = T::mfma16(ag, pdB, dv[d]);
            }
            if constexpr (HAS_DO) {
                const u32x4 ado = d == 0 ? ado0 : lds_a_tr16<HD>(sDO, 16 * d, lane);
                dv[d] = T::mfma16(ado, pB, dv[d]);
            }
        }
    };

    // B operand of step 3: Tile[k = key][x = query 16*qt + n] from a bounce tile, keys of slab kk in
    // the k numbering of lds_a_tr16 (rows 4g..4g+3 and 16+4g..16+4g+3 of the slab).
    auto bounce_b = [&](const elem_t* bounce, int kk, int qt, int lane_l) {
        const int i16 = lane_l & 15, g = lane_l >> 4;
        const int row = 32 * kk + 4 * g + (i16 >> 2);  // rows row and row + 16 share their swizzle
        const elem_t* p0 = bounce + row * BP + (((4 * qt + (i16 & 3)) ^ bounce_swz(row)) << 2);
        typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
        s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p0));
        s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p0 + 16 * BP));
        u32x2 l2 = __builtin_bit_cast(u32x2, lo);
        u32x2 h2 = __builtin_bit_cast(u32x2, hi);
        return u32x4{l2[0], l2[1], h2[0], h2[1]};
    };

    // Step 3: 16 x 16 tiles (head-dimension tile dt, query tile qt) of dQ and dQ_dot for the stage.
    // HD = 64: wave w forms tile w of both; HD = 32: waves 0..3 form dQ, waves 4..7 dQ_dot.
    constexpr int NTILES = 2 * DT;
    auto row_outputs = [&](const elem_t* bounceS, elem_t* qstage_i, auto full_tag) {
        const elem_t* bounceT = bounceS + oBT;
        constexpr bool FULL = decltype(full_tag)::value;  // all four key slabs hold keys
        const int tq = wave;                           // dQ tile of this wave
        const int tt = NTILES == 8 ? wave : wave - 4;      // dQ_dot tile of this wave
        const bool do_q = tq < NTILES;
        const bool do_t = HAS_G && tt >= 0 && tt < NTILES;
        const int tile_id = do_q ? tq : tt;
        if (!do_q && !do_t) return;
        const int dt = tile_id % DT, qt = tile_id / DT;
        const int lane_l = lane_now();
        // three independent chains: dS K, dS_dot K_dot (both into dQ) and dS_dot K (dQ_dot)
        f32x4 a0 = {0.f, 0.f, 0.f, 0.f}, a1 = {0.f, 0.f, 0.f, 0.f}, a2 = {0.f, 0.f, 0.f, 0.f};
        auto step = [&](int kk) {
            const u32x4 ak = lds_a_tr16<HD>(ownK + kk * SE, 16 * dt, lane_l);
            if (do_q) {
                a0 = T::mfma16(ak, bounce_b(bounceS, kk, qt, lane_l), a0);
                if constexpr (HAS_G) {
                    const u32x4 bt = bounce_b(bounceT, kk, qt, lane_l);
                    const u32x4 atk = lds_a_tr16<HD>(ownK + (4 + kk) * SE, 16 * dt, lane_l);
                    a1 = T::mfma16(atk, bt, a1);
                    if (do_t) a2 = T::mfma16(ak, bt, a2);
                }
            } else {
                a2 = T::mfma16(ak, bounce_b(bounceT, kk, qt, lane_l), a2);
            }
        };
        if constexpr (FULL) {
#pragma unroll
            for (int kk = 0; kk < 4; ++kk) step(kk);
        } else {
            for (int kk = 0; kk < key_slabs; ++kk) step(kk);
        }
        // lane = query 16*qt + n, registers = columns 16*dt + 4g .. + 3: into the staging tile, from
        // where flush_rows() sends whole rows after the next barrier
        elem_t* st = qstage_i + (16 * qt + (lane_l & 15)) * SM::qpitch + 16 * dt + 4 * (lane_l >> 4);
        if (do_q) {
            a0 += a1;
            *reinterpret_cast<u32x2*>(st) =
                u32x2{T::pack2(a0[0] * p.scale, a0[1] * p.scale), T::pack2(a0[2] * p.scale, a0[3] * p.scale)};
        }
        if (do_t) {
            *reinterpret_cast<u32x2*>(st + kStageRows * SM::qpitch) =
                u32x2{T::pack2(a2[0] * p.scale, a2[1] * p.scale), T::pack2(a2[2] * p.scale, a2[3] * p.scale)};
        }
    };
    // dQ (threads 0..255) and dQ_dot (256..511) of the stage that starts at row0: one 16-byte piece
    // of a row per thread (HD / 8 pieces per row).  Issued before the stage copy of the iteration, so
    // the stores are older than every copy a later wait_stages() still allows to be outstanding.
    auto flush_rows = [&](int row0, const elem_t* qstage_i) {
        constexpr int CH = HD / 8;
        const int tid_l = wave * 64 + lane_now();
        const int half = tid_l >> 8, t = tid_l & 255;
        if (half == 1 && !HAS_G) return;
        const int r = t / CH, c = t % CH;
        if (r < kStageRows && row0 + r < p.Lq && 8 * c < p.D) {
            const elem_t* srow = qstage_i + half * kStageRows * SM::qpitch + r * SM::qpitch;
            u32x4 v = *reinterpret_cast<const u32x4*>(srow + 8 * c);
            if constexpr (ROPE)
                v = rope8_inverse_chunk<T>(v, *reinterpret_cast<const u32x4*>(srow + 8 * (c ^ 4)), p.rope, row0 + r, c);
            elem_t* dst = (half == 0 ? p.dq.head(b, h) + (int64_t)(row0 + r) * p.dq.sl
                                     : p.dtq.head(b, h) + (int64_t)(row0 + r) * p.dtq.sl) + 8 * c;
            __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(dst));
        }
    };

    // Only stage 0 and the own rows are waited for here; the later stages are issued once these
    // have landed, so that their copies run under the arithmetic instead of ahead of it.
    wait_stages<OWN>(1);  // everything but the OWN youngest copies of this wave: stage 0
    workgroup_barrier();
    row_sums(ring);
    wait_stages<SPT>(0);
    workgroup_barrier();
    if (issued < ns) issue_next();
    // ROPE: Q (, Q_dot) of a landed stage, one item per thread of the upper half of the workgroup
    auto rotate_stage = [&](elem_t* slot, int row0) {
        if constexpr (ROPE) {
            const int it = tid - 256;
            if (it >= 0 && it < 128) rope_slab_item<T>(slot, it, p.rope, row0, 1.0f);
            else if (HAS_G && it >= 128) rope_slab_item<T>(slot + oTQ, it - 128, p.rope, row0, 1.0f);
        }
    };
    if constexpr (ROPE) {
        // own K (, K_dot): slabs of 32 keys, 128 items each
        constexpr int items = (HAS_G ? 8 : 4) * 128;
#pragma unroll
        for (int it = tid; it < items; it += kThreads16) {
            const int slab = it >> 7;
            rope_slab_item<T>(ownK + slab * SE, it & 127, p.rope, 32 * (slab & 3), 1.0f);
        }
        workgroup_barrier();
    }
    {
        const int r = 16 * (wave & 1) + n;
        const int sidx = wave >> 1;
        read_b_operands16<HD>(kB, ownK + sidx * SE, r, g);
        read_b_operands16<HD>(vB, ownV + sidx * SE, r, g);
        if constexpr (HAS_G) {
            read_b_operands16<HD>(tkB, ownK + (4 + sidx) * SE, r, g);
            read_b_operands16<HD>(tvB, ownV + (4 + sidx) * SE, r, g);
        }
    }
    rotate_stage(ring, 0);
    // dK, dV (, dK_dot, dV_dot) of this wave's sixteen keys through its staging tile
    auto key_gradients = [&](elem_t* stage_tile) {
        const int row0 = wave * 16;
        store_tile16<T, HD, ROPE>(stage_tile, p.dk.head(b, h), p.dk.sl, row0, p.Lk, p.D, dk, p.scale, lane, &p.rope);
        if constexpr (HAS_G)
            store_tile16<T, HD, ROPE>(stage_tile, p.dtk.head(b, h), p.dtk.sl, row0, p.Lk, p.D, dtk, p.scale, lane,
                                      &p.rope);
        store_tile16<T, HD>(stage_tile, p.dv.head(b, h), p.dv.sl, row0, p.Lk, p.D, dv, 1.0f, lane);
        if constexpr (HAS_G)
            store_tile16<T, HD>(stage_tile, p.dtv.head(b, h), p.dtv.sl, row0, p.Lk, p.D, dtv, 1.0f, lane);
    };
    // One workgroup barrier per stage.  Iteration i: step 2 of stage i (tiles into bounce buffer i % 2), the
    // barrier, then the row sums of stage i+1, step 3 of stage i (bounce buffer i % 2 -> staging buffer i % 2)
    // and the rows of stage i-1 on their way out (staging buffer (i-1) % 2).  Step 2 of stage i+1 follows
    // without a barrier: it writes the other bounce buffer, and what it needs from other waves, the
    // statistics (and rotated rows) of stage i+1, is announced through a counter in LDS that the waves
    // forming them raise (SIG waves per stage), which a wave polls before its step 2.
    constexpr unsigned SIG = ROPE ? 8 : 4;
    unsigned* announced = reinterpret_cast<unsigned*>(smem_raw + SM::sink + 8);
    auto announce = [&]() {
        __builtin_amdgcn_s_waitcnt(0xC07F);  // this wave's LDS writes are done
        if (lane == 0) __hip_atomic_fetch_add(announced, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    };
    auto await_announced = [&](unsigned target) {
        // the announcing waves get there without waiting for anyone behind this point; the bound only
        // keeps a mistake from hanging the machine
        typedef __attribute__((address_space(3))) volatile unsigned lds_counter;  // an LDS read, not a flat one
        lds_counter* flag = (lds_counter*)announced;
        for (int spins = 0; *flag < target && spins < (1 << 22); ++spins) __builtin_amdgcn_s_sleep(1);
        asm volatile("" ::: "memory");
    };
    workgroup_barrier();  // every wave has read V, V_dot, whose memory the bounce tiles take over
    for (int i = 0; i < ns; ++i) {
        if (issued < ns && issued < i + R) issue_next();  // into the slot of stage issued - R <= i - 1
        elem_t* slot = ring + (i % R) * SM::slot;
        elem_t* bounce_i = bounce0 + (i & 1) * BBUF;
        if (i >= 1) await_announced(SIG * (unsigned)i);
        if (wave_active) tile(slot, bounce_i);
        if (!ROPE && i == ns - 1 && wave_active) {
            // The gradients of this wave's keys are complete.  They leave now, while step 3 of the last stage
            // is still to come, through per-wave staging tiles in the two ring slots that no stage uses again
            // (waves 0..3 in one, 4..7 in the other): the stores drain under the remaining arithmetic
            // instead of after it.  (With the folded rotation the stores need registers that the stage loop
            // cannot spare; they follow the loop there.)
            static_assert(R >= 3 && SM::slot >= 4 * StoreStage16<HD>::elems, "two spare slots hold the staging tiles");
            key_gradients(ring + ((i + 1 + (wave >> 2)) % R) * SM::slot + (wave & 3) * StoreStage16<HD>::elems);
        }
        if (i + 1 < ns) wait_stages<SPT>(issued - 2 - i);  // stage i+1 has landed (this wave's part)
        workgroup_barrier();  // bounce buffer i % 2 is complete; stage i+1 is in LDS; stage i's slot is free
        if (i >= 1) flush_rows((i - 1) * kStageRows, qstage + ((i - 1) & 1) * SM::qstage_one);
        if (i + 1 < ns) {
            row_sums(ring + ((i + 1) % R) * SM::slot);
            rotate_stage(ring + ((i + 1) % R) * SM::slot, (i + 1) * kStageRows);
            if (ROPE || tid < 256) announce();
        }
        elem_t* qstage_i = qstage + (i & 1) * SM::qstage_one;
        if (key_slabs == 4) row_outputs(bounce_i, qstage_i, std::true_type{});
        else row_outputs(bounce_i, qstage_i, std::false_type{});
    }
    workgroup_barrier();  // the last stage's dQ (, dQ_dot) tiles are in their staging tile; the ring is free
    flush_rows((ns - 1) * kStageRows, qstage + ((ns - 1) & 1) * SM::qstage_one);
    if constexpr (ROPE) {
        static_assert(R * SM::slot >= kWaves16 * StoreStage16<HD>::elems, "ring too small to stage stores");
        if (wave_active) key_gradients(ring + wave * StoreStage16<HD>::elems);
    }
}

}  // namespace sjvp
