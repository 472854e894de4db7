// Attention-JVP backward for key axes beyond one workgroup, 16-wide form (gfx950; inputs with 16-byte
// aligned rows): the row-owned and column-owned pair of sjvp_bwd.hpp (same mathematics, the same
// workspace arrays lse*log2e, s4, s7d, the two sums negated here) with 16 owned positions per wavefront,
// so that several wavefronts share a SIMD and a workgroup's copies overlap another's arithmetic.
//   bwd_row16_kernel   4 waves x 16 queries; streams K, V (, K_dot, V_dot)        -> dQ (, dQ_dot)
//   bwd_col16_kernel   4 waves x 16 keys;    streams Q (, Q_dot, G) (, dO) + stats -> dK, dV (, dK_dot, dV_dot)
// (workgroups of four waves: at 160-200 registers two or three of them share a CU)
// The owned rows are loaded straight into registers (each lane its own 16-byte pieces), the streamed
// side goes through an LDS ring filled by LDS-DMA.  Each gradient is accumulated in fp32 registers by
// exactly one wavefront and written once: deterministic, no atomics.
//
// Row sums.  The row-owned kernel starts from s4' = rowsum(G*O), s7d' = rowsum(G*TO) + rowsum(dO*O),
// formed from the 16-bit outputs, whose rounding leaves s4' = s4 + e4, s7d' = s7d + e7.  With the exact
// sums, sum_j dS_dot_ij = sum_j dS_ij = 0 for every query i; with the rounded ones the sums over the
// keys come out as rho4 = -e4 and rho7 = -e7.  A wave owns whole query rows, so it accumulates both
// residues in fp32 beside its tiles (per-lane adds) and
//   - leaves the corrected sums s4' + rho4 = sum_j P W, s7d' + rho7 = sum_j P (N W + XY) in the
//     workspace: the column-owned kernel works with the sums the reference's preprocess kernel forms
//     from the probabilities (semicat/jvp_utils/flash_jvp_backward.py:2266-2287).  They are stored
//     negated: both kernels start the accumulators of W and XY from minus the sums, so that W - s4 and
//     XY - s7d come out of the matrix cores and cost no vector instruction;
//   - flags its workgroup where a residue is not small against the row's |dS_dot| / |dS| mass (sharp
//     rows, gradients formed by cancellation).  A second launch of the same kernel (PASS = 2) runs the
//     flagged workgroups again with the corrected sums, so that their dQ, dQ_dot are formed from tiles
//     that were rounded without the residue in them; the others leave at once.
// BwdParams::rowfix: 0 no second launch; 1 as described; 2 every workgroup runs twice and the first
// launch (PASS = 1) only measures (the reference's preprocess + backward structure).
#pragma once
#include "sjvp_bwd.hpp"
#include "sjvp_w16.hpp"

namespace sjvp {

constexpr int kXWaves16 = 4;
constexpr int kXThreads16 = 64 * kXWaves16;
constexpr int kXOwned16 = 16 * kXWaves16;  // owned positions per workgroup

// B operands (all head-dimension chunks of 32) of one owned row, straight from global memory.
template <int HD>
__device__ __forceinline__ void load_b_operands16(u32x4* out, const elem_t* row, int g, int D, bool valid) {
#pragma unroll
    for (int c = 0; c < HD / 32; ++c) out[c] = load8(row, 32 * c + 8 * g, D, valid, true);
}

// The same from a uniform slice pointer and the lane's byte offset in the slice: whole rows of HD elements
// that all exist, no predicates, one 32-bit offset for every tensor of equal strides.
template <int HD>
__device__ __forceinline__ void load_b_operands16_at(u32x4* out, const elem_t* slice, uint32_t lane_bytes) {
    const char* base = reinterpret_cast<const char*>(slice);
#pragma unroll
    for (int c = 0; c < HD / 32; ++c) out[c] = *reinterpret_cast<const u32x4*>(base + lane_bytes + 64 * c);
}

// sum over the 16-bit pairs of a[i]*b[i]
template <typename T>
__device__ __forceinline__ float dot8(const u32x4& a, const u32x4& b) {
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) s = T::dot2(a[i], b[i], s);
    return s;
}

// ---------------------------------------------------------------------------------------------
// Row-owned kernel.  LDS: [ring of K | V (| K_dot | V_dot) stages][sink]; the ring doubles as store
// staging after the last stage.
template <int HD, int R, bool HAS_G>
struct Row16Smem {
    static constexpr int nt = HAS_G ? 4 : 2;
    static constexpr int slot = nt * Slab<HD>::elems;
    static constexpr int sink = R * slot * (int)sizeof(elem_t);
    static constexpr int bytes = sink + kSink16;
    static_assert(R * slot >= kXWaves16 * StoreStage16<HD>::elems, "ring too small to stage stores");
};

// (the body of the kernel as a function of the workgroup's index and the number of workgroups, so that the
// second launch can also ride at the end of the column-owned launch, see bwd_col16_repair_kernel)
template <typename T, int HD, int R, bool HAS_DO, bool HAS_G, int PASS>
__device__ __forceinline__ void bwd_row16_body(const BwdParams p, const int block, const int blocks) {
    constexpr bool SECOND = PASS == 2;   // second launch: sums from the workspace, flagged workgroups only
    constexpr bool MEASURE = PASS == 1;  // first launch of "always": residues and sums only, no gradients
    extern __shared__ __align__(16) unsigned char smem_raw[];
    using SM = Row16Smem<HD, R, HAS_G>;
    elem_t* ring = reinterpret_cast<elem_t*>(smem_raw);
    constexpr int SE = Slab<HD>::elems;
    constexpr int KC = HD / 32;
    constexpr int DT = HD / 16;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 15;
    const int g = lane >> 4;
    const int q_blocks = p.Lr / kXOwned16;  // statistic rows up to Lr are all covered
    // Workgroups run through the heads in descending order: this launch follows the forward, which
    // ran through them in ascending order, so it starts on what the caches still hold (the
    // column-owned launch after it ascends again).
    const int bid = blocks - 1 - xcd_linear_id(block, blocks);
    const int bh = bid / q_blocks;
    const int qb = bid % q_blocks;
    const int b = bh / p.H, h = bh % p.H;
    const int q0 = qb * kXOwned16;
    const int qrow = q0 + wave * 16 + n;
    const bool qvalid = qrow < p.Lq;
    const bool wave_active = (q0 + wave * 16) < p.Lq;
    if constexpr (SECOND) {
        if (p.rowfix == 1 && p.flags[bid] == 0) return;  // nothing to repair in this workgroup's rows
    }

    // The own rows are requested first, as B operands; the set-up of the stage copies runs while they travel.
    u32x4 qB[KC], tqB[KC], gB[KC], doB[KC];
    u32x4 oR[KC], toR[KC];
    float s4 = 0.f, s7d = 0.f;
    const int64_t so = (int64_t)bh * p.Lr + qrow;  // rows below Lr exist in every statistic
    if (p.q_side_uniform && p.D == HD && q0 + kXOwned16 <= p.Lq) {
        // the common case: whole rows that all exist, every tensor with q's strides
        const int64_t slice = b * p.q.sb + h * p.q.sh;
        const uint32_t at = ((uint32_t)qrow * (uint32_t)p.q.sl + 8u * (uint32_t)g) * (uint32_t)sizeof(elem_t);
        load_b_operands16_at<HD>(qB, p.q.ptr + slice, at);
        if constexpr (!SECOND) load_b_operands16_at<HD>(oR, p.o.ptr + slice, at);
        if constexpr (HAS_G) {
            load_b_operands16_at<HD>(tqB, p.tq.ptr + slice, at);
            load_b_operands16_at<HD>(gB, p.dTO.ptr + slice, at);
            if constexpr (!SECOND) load_b_operands16_at<HD>(toR, p.to.ptr + slice, at);
        }
        if constexpr (HAS_DO) load_b_operands16_at<HD>(doB, p.dO.ptr + slice, at);
    } else {
        load_b_operands16<HD>(qB, p.q.head(b, h) + (int64_t)qrow * p.q.sl, g, p.D, qvalid);
        if constexpr (!SECOND) load_b_operands16<HD>(oR, p.o.head(b, h) + (int64_t)qrow * p.o.sl, g, p.D, qvalid);
        if constexpr (HAS_G) {
            load_b_operands16<HD>(tqB, p.tq.head(b, h) + (int64_t)qrow * p.tq.sl, g, p.D, qvalid);
            load_b_operands16<HD>(gB, p.dTO.head(b, h) + (int64_t)qrow * p.dTO.sl, g, p.D, qvalid);
            if constexpr (!SECOND) load_b_operands16<HD>(toR, p.to.head(b, h) + (int64_t)qrow * p.to.sl, g, p.D, qvalid);
        }
        if constexpr (HAS_DO) load_b_operands16<HD>(doB, p.dO.head(b, h) + (int64_t)qrow * p.dO.sl, g, p.D, qvalid);
    }
    float lse_in = p.lse[so];  // requested with the rows: they are awaited together
    float mu_in = HAS_G ? p.mu[so] : 0.f;

    using StagePlan = CopyPlan<HD, SM::nt, 1, kXThreads16>;
    constexpr int SPT = StagePlan::N;
    StagePlan plan;
    if constexpr (HAS_G)
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
    // Stage 0 only for now: the loads of the own rows are awaited by a wait for everything this wave has
    // outstanding (the compiler cannot tell them from the stage copies), so the later stages are issued once
    // the own rows are in registers and land under the first stage's arithmetic.
    issue_next();

    // row sums s4 = rowsum(G*O), s7d = rowsum(G*TO) + rowsum(dO*O) from the lane's 16-byte pieces, combined
    // over the four lanes of a query
    {
        if constexpr (SECOND) {
            // the corrected sums the first launch left in the workspace (negated there)
            s4 = -p.s4[so];
            s7d = -p.s7d[so];
        } else {
#pragma unroll
            for (int c = 0; c < KC; ++c) {
                if constexpr (HAS_G) {
                    s4 += dot8<T>(gB[c], oR[c]);
                    s7d += dot8<T>(gB[c], toR[c]);
                }
                if constexpr (HAS_DO) s7d += dot8<T>(doB[c], oR[c]);
            }
            s4 = group_sum(s4);
            s7d = group_sum(s7d);
        }
    }
    asm volatile("" : "+v"(lse_in), "+v"(mu_in));  // not before the copies of stage 0 are under way
    float lse2 = lse_in * kLog2e;
    float mu = HAS_G ? mu_in : 0.f;
    // The tiles W and XY are accumulated on top of -s4 and -s7d, so that W - s4 and XY - s7d leave the matrix
    // cores ready for use.
    float n4 = -s4, n7 = -s7d;
    asm volatile("" : "+v"(lse2), "+v"(mu), "+v"(n4), "+v"(n7));  // every load so far is awaited here
    while (issued < R && issued < ns) issue_next();
    // every row below Lr gets its workspace entries (zeros beyond Lq except lse2, which is finite): the
    // column-owned kernel, which runs after this one, stages 32-row groups
    if constexpr (!SECOND) {
        if (g == 0) p.lse2[so] = lse2;
    }
    const float sl2 = p.scale * kLog2e;
    f32x4 dq[DT], dtq[DT];
#pragma unroll
    for (int t = 0; t < DT; ++t) {
        dq[t] = f32x4{0.f, 0.f, 0.f, 0.f};
        dtq[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    // First launch: this lane's part of sum_j dS_dot_ij, sum_j dS_ij (zero in exact arithmetic), and of
    // their absolute sums, which only set the scale of a threshold and are sampled on every fourth key.
    float r4 = 0.f, r7 = 0.f, a4 = 0.f, a7 = 0.f;

    auto compute = [&](const elem_t* slot, int k0, auto ragged_tag) {
        const elem_t* sK = slot;
        const elem_t* sV = slot + SE;
        const elem_t* sTK = slot + 2 * SE;
        const elem_t* sTV = slot + 3 * SE;
        // tiles: rows = keys (registers), columns = this wave's queries (lanes)
        f32x4 s[2], ts[2], w[2], xy[2];
        auto scores = [&](int t) __attribute__((always_inline)) {
            s[t] = f32x4{0.f, 0.f, 0.f, 0.f};
            ts[t] = f32x4{0.f, 0.f, 0.f, 0.f};
            w[t] = f32x4{n4, n4, n4, n4};
            xy[t] = f32x4{n7, n7, n7, n7};
#pragma unroll
            for (int c = 0; c < KC; ++c) {
                const u32x4 ak = lds_a_rows16<HD>(sK, t, c, n, g);
                const u32x4 av = lds_a_rows16<HD>(sV, t, c, n, g);
                s[t] = T::mfma16(ak, qB[c], s[t]);
                if constexpr (HAS_G) {
                    ts[t] = T::mfma16(ak, tqB[c], ts[t]);
                    const u32x4 atk = lds_a_rows16<HD>(sTK, t, c, n, g);
                    ts[t] = T::mfma16(atk, qB[c], ts[t]);
                    w[t] = T::mfma16(av, gB[c], w[t]);
                    const u32x4 atv = lds_a_rows16<HD>(sTV, t, c, n, g);
                    xy[t] = T::mfma16(atv, gB[c], xy[t]);
                }
                if constexpr (HAS_DO) xy[t] = T::mfma16(av, doB[c], xy[t]);
            }
        };
        constexpr bool ragged = decltype(ragged_tag)::value;  // the stage reaches beyond Lk (only the last one can)
        // in place: w -> dS_dot, xy -> dS
        auto pointwise = [&](int t) __attribute__((always_inline)) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                float pj = fast_exp2(fmaf(s[t][j], sl2, -lse2));
                // keys beyond Lk are zero rows; exp(-lse) may overflow when every real score is very
                // negative, so their P is forced to zero
                if constexpr (ragged) {
                    if (k0 + 16 * t + 4 * g + j >= p.Lk) pj = 0.f;
                }
                if constexpr (HAS_G) {
                    const float nn = fmaf(ts[t][j], p.scale, -mu);
                    const float dts = pj * w[t][j];
                    w[t][j] = dts;
                    xy[t][j] = fmaf(dts, nn, pj * xy[t][j]);
                    if constexpr (!SECOND) {
                        r4 += dts;
                        if (j == 0) a4 += fabsf(dts);
                    }
                } else {
                    xy[t][j] = pj * xy[t][j];
                }
                if constexpr (!SECOND) {
                    r7 += xy[t][j];
                    if (j == 0) a7 += fabsf(xy[t][j]);
                }
            }
        };
        // the second key tile's MFMA chains run under the first tile's element-wise arithmetic
        scores(0);
        __builtin_amdgcn_sched_barrier(0);
        scores(1);
        pointwise(0);
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (MEASURE) {  // a launch that only measures the residues
            pointwise(1);
            return;
        }
        // the transposed operands of the output contractions are read one step ahead, the first ones
        // under the second tile's element-wise arithmetic
        u32x4 ak = lds_a_tr16<HD>(sK, 0, lane), atk;
        if constexpr (HAS_G) atk = lds_a_tr16<HD>(sTK, 0, lane);
        __builtin_amdgcn_sched_barrier(0);
        pointwise(1);
        const u32x4 dsB = pack_b16<T>(xy[0], xy[1]);
        u32x4 dtsB;
        if constexpr (HAS_G) dtsB = pack_b16<T>(w[0], w[1]);
#pragma unroll
        for (int d = 0; d < DT; ++d) {
            u32x4 nk, ntk;
            if (d + 1 < DT) {
                nk = lds_a_tr16<HD>(sK, 16 * (d + 1), lane);
                if constexpr (HAS_G) ntk = lds_a_tr16<HD>(sTK, 16 * (d + 1), lane);
            }
            __builtin_amdgcn_sched_barrier(0);
            dq[d] = T::mfma16(ak, dsB, dq[d]);
            if constexpr (HAS_G) {
                dtq[d] = T::mfma16(ak, dtsB, dtq[d]);
                dq[d] = T::mfma16(atk, dtsB, dq[d]);
            }
            __builtin_amdgcn_sched_barrier(0);
            ak = nk;
            if constexpr (HAS_G) atk = ntk;
        }
    };

    // The last stage, the only one that can reach beyond Lk, runs behind the loop in a form of its own: the
    // selects of its padded keys (a compare and two selects per tile element) stay out of the loop.
    auto stage = [&](int i, auto ragged_tag) {
        // copies issued after stage i: the later stages; anything else in flight (the own rows'
        // loads, the statistics) only makes the wait stricter
        wait_stages<SPT>(issued - 1 - i);
        workgroup_barrier();  // stage i has landed for every wave; stage i-1 is fully consumed
        if (i > 0 && issued < ns) issue_next();
        if (wave_active) compute(ring + (i % R) * SM::slot, i * kStageRows, ragged_tag);
    };
    for (int i = 0; i < ns - 1; ++i) stage(i, std::false_type{});
    stage(ns - 1, std::true_type{});
    if constexpr (!SECOND) {
        // the residues of the row sums (see the top of the file); the four lanes of a query hold its keys
        r4 = group_sum(r4);
        r7 = group_sum(r7);
        a4 = 4.0f * group_sum(a4);
        a7 = 4.0f * group_sum(a7);
        if (g == 0) {
            p.s4[so] = n4 - r4;  // minus the corrected sums: the column-owned kernel starts its tiles from them
            p.s7d[so] = n7 - r7;
        }
        // A residue matters where it is not small against the rounding of the tiles it is spread over:
        // |rho| against tau * sum_j |tile_ij|, tau = the unit roundoff of the 16-bit format.  NaN compares false.
        const bool wanted = qvalid && (fabsf(r4) > p.rowfix_tau * a4 || fabsf(r7) > p.rowfix_tau * a7);
        if (p.rowfix == 1) {
            const bool any = workgroup_barrier_or(wanted);
            if (tid == 0) p.flags[bid] = any ? 1 : 0;
        }
        if constexpr (MEASURE) return;  // the second launch writes dQ, dQ_dot
    }
    workgroup_barrier();  // every wave is done reading the ring: it becomes the store staging area
    if (!wave_active) return;
    elem_t* stage_tile = ring + wave * StoreStage16<HD>::elems;
    const int row0 = q0 + wave * 16;
    store_tile16<T, HD>(stage_tile, p.dq.head(b, h), p.dq.sl, row0, p.Lq, p.D, dq, p.scale, lane);
    if constexpr (HAS_G)
        store_tile16<T, HD>(stage_tile, p.dtq.head(b, h), p.dtq.sl, row0, p.Lq, p.D, dtq, p.scale, lane);
}

template <typename T, int HD, int R, bool HAS_DO, bool HAS_G, int OCC, int PASS = 0>
__global__ __launch_bounds__(kXThreads16, OCC) void bwd_row16_kernel(const BwdParams p) {
    bwd_row16_body<T, HD, R, HAS_DO, HAS_G, PASS>(p, (int)blockIdx.x, (int)gridDim.x);
}

// ---------------------------------------------------------------------------------------------
// Column-owned kernel: a workgroup of four waves owns 64 keys.  PART selects the gradients that are
// accumulated: 3 all four (HD <= 64), 1 dK (, dK_dot), 2 dV (, dV_dot) (HD = 128 runs as two launches
// to stay inside the register file).  LDS: [ring of Q | [Q_dot | G] | [dO] | lse2, mu, s4, s7d stages]
// [sink]; the ring doubles as store staging after the last stage.
template <int HD, int R, bool HAS_DO, bool HAS_G>
struct Col16Smem {
    static constexpr int nt = 1 + (HAS_G ? 2 : 0) + (HAS_DO ? 1 : 0);
    static constexpr int stat_elems = 4 * kStageRows * 2;  // 4 float arrays of 32, in elem_t units
    static constexpr int slot = nt * Slab<HD>::elems + stat_elems;
    static constexpr int sink = R * slot * (int)sizeof(elem_t);
    static constexpr int bytes = sink + kSink16;
    static_assert(R * slot >= kXWaves16 * StoreStage16<HD>::elems, "ring too small to stage stores");
};

template <typename T, int HD, int R, bool HAS_DO, bool HAS_G, int PART>
__device__ __forceinline__ void bwd_col16_body(const BwdParams p, const int block, const int blocks) {
    extern __shared__ __align__(16) unsigned char smem_raw[];
    using SM = Col16Smem<HD, R, HAS_DO, HAS_G>;
    constexpr bool DO_K = (PART & 1) != 0, DO_V = (PART & 2) != 0;
    elem_t* ring = reinterpret_cast<elem_t*>(smem_raw);
    constexpr int SE = Slab<HD>::elems;
    constexpr int oTQ = SE, oG = 2 * SE, oDO = (HAS_G ? 3 : 1) * SE, oST = SM::nt * SE;
    constexpr int KC = HD / 32;
    constexpr int DT = HD / 16;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 15;
    const int g = lane >> 4;
    const int k_blocks = (p.Lk + kXOwned16 - 1) / kXOwned16;
    const int bid = xcd_linear_id(block, blocks);
    const int bh = bid / k_blocks;
    const int kb = bid % k_blocks;
    const int b = bh / p.H, h = bh % p.H;
    const int key0 = kb * kXOwned16;
    const int krow = key0 + wave * 16 + n;
    const bool kvalid = krow < p.Lk;
    const bool wave_active = (key0 + wave * 16) < p.Lk;

    using StagePlan = CopyPlan<HD, SM::nt, 1, kXThreads16>;
    constexpr int SPT = StagePlan::N + 1;  // plus one 4-byte copy of statistics
    StagePlan plan;
    const int ns = (p.Lq + kStageRows - 1) / kStageRows;
    int issued = 0;
    auto issue_next = [&]() {
        elem_t* slot = ring + (issued % R) * SM::slot;
        const int row0 = issued * kStageRows;
        plan.issue(slot, p.Lq - row0, p.D == HD && row0 + kStageRows <= p.Lq);
        // the four statistic arrays (lse2, mu, s4, s7d) of the stage's rows, one per wave, 32 lanes
        // each (rows < Lr exist in all of them); every wave issues exactly one 4-byte LDS-DMA
        // (the three workspace arrays lie one behind the other: chosen by arithmetic, which stays in scalar
        // registers, where a choice among four pointers becomes a table in memory)
        const int64_t plane = p.s4 - p.lse2;
        const float* src = p.lse2 + (wave == 0 ? 0 : wave == 3 ? 2 : 1) * plane;  // lse2 | s4 | s4 | s7d
        if (HAS_G && wave == 1) src = p.mu;
        float* st = reinterpret_cast<float*>(slot + oST);
        if (lane < 32) dma4(src + (int64_t)bh * p.Lr + row0 + lane, lds_addr(st) + (uint32_t)(wave * 32 * 4));
        ++issued;
    };
    // called behind the requests for the own rows on both paths below (see bwd_row16_kernel): set-up of the
    // stage copies, and stage 0 only for now
    auto begin_copies = [&]() __attribute__((always_inline)) {
        {
            const Src q{p.q.head(b, h), p.q.sl};
            if constexpr (HAS_G && HAS_DO)
                plan.init(tid, 0, p.D, smem_raw + SM::sink, q, Src{p.tq.head(b, h), p.tq.sl},
                          Src{p.dTO.head(b, h), p.dTO.sl}, Src{p.dO.head(b, h), p.dO.sl});
            else if constexpr (HAS_G)
                plan.init(tid, 0, p.D, smem_raw + SM::sink, q, Src{p.tq.head(b, h), p.tq.sl},
                          Src{p.dTO.head(b, h), p.dTO.sl});
            else
                plan.init(tid, 0, p.D, smem_raw + SM::sink, q, Src{p.dO.head(b, h), p.dO.sl});
        }
        issue_next();
    };
    // the own rows are requested first; the set-up of the stage copies runs while they travel
    u32x4 kB[KC], vB[KC], tkB[KC], tvB[KC];
    if (p.k_side_uniform && p.D == HD && key0 + kXOwned16 <= p.Lk) {
        // the common case: whole rows that all exist, every tensor with k's strides
        const int64_t slice = b * p.k.sb + h * p.k.sh;
        const uint32_t at = ((uint32_t)krow * (uint32_t)p.k.sl + 8u * (uint32_t)g) * (uint32_t)sizeof(elem_t);
        load_b_operands16_at<HD>(kB, p.k.ptr + slice, at);
        if constexpr (DO_K) load_b_operands16_at<HD>(vB, p.v.ptr + slice, at);
        if constexpr (HAS_G) {
            load_b_operands16_at<HD>(tkB, p.tk.ptr + slice, at);
            if constexpr (DO_K) load_b_operands16_at<HD>(tvB, p.tv.ptr + slice, at);
        }
        begin_copies();
    } else {
        load_b_operands16<HD>(kB, p.k.head(b, h) + (int64_t)krow * p.k.sl, g, p.D, kvalid);
        if constexpr (DO_K) load_b_operands16<HD>(vB, p.v.head(b, h) + (int64_t)krow * p.v.sl, g, p.D, kvalid);
        if constexpr (HAS_G) {
            load_b_operands16<HD>(tkB, p.tk.head(b, h) + (int64_t)krow * p.tk.sl, g, p.D, kvalid);
            if constexpr (DO_K) load_b_operands16<HD>(tvB, p.tv.head(b, h) + (int64_t)krow * p.tv.sl, g, p.D, kvalid);
        }
        begin_copies();
    }
#pragma unroll
    for (int c = 0; c < KC; ++c) {  // the own rows are awaited here
        asm volatile("" : "+v"(kB[c]));
        if constexpr (DO_K) asm volatile("" : "+v"(vB[c]));
        if constexpr (HAS_G) {
            asm volatile("" : "+v"(tkB[c]));
            if constexpr (DO_K) asm volatile("" : "+v"(tvB[c]));
        }
    }
    while (issued < R && issued < ns) issue_next();
    const float sl2 = p.scale * kLog2e;
    f32x4 dk[DT], dv[DT], dtk[DT], dtv[DT];
#pragma unroll
    for (int t = 0; t < DT; ++t) {
        dk[t] = f32x4{0.f, 0.f, 0.f, 0.f};
        dv[t] = f32x4{0.f, 0.f, 0.f, 0.f};
        dtk[t] = f32x4{0.f, 0.f, 0.f, 0.f};
        dtv[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

    auto compute = [&](const elem_t* slot) {
        const elem_t* sQ = slot;
        const elem_t* sTQ = slot + oTQ;
        const elem_t* sG = slot + oG;
        const elem_t* sDO = slot + oDO;
        const float* sStat = reinterpret_cast<const float*>(slot + oST);
        // tiles: rows = queries (registers), columns = this wave's keys (lanes).
        // The A operands of every contraction step are read from LDS one step ahead of the MFMAs
        // that use them (two register sets), so that a wave's matrix pipe does not sit out an LDS
        // round trip per step; the first operands of the gradient phase and the row statistics are
        // requested before the last score step and arrive during the element-wise work.
        struct AOps {
            u32x4 q, tq, g, d;
        };
        auto load_score = [&](int t, int c) {
            AOps a;
            a.q = lds_a_rows16<HD>(sQ, t, c, n, g);
            if constexpr (HAS_G) {
                a.tq = lds_a_rows16<HD>(sTQ, t, c, n, g);
                if constexpr (DO_K) a.g = lds_a_rows16<HD>(sG, t, c, n, g);
            }
            if constexpr (HAS_DO && DO_K) a.d = lds_a_rows16<HD>(sDO, t, c, n, g);
            return a;
        };
        auto load_grad = [&](int d) {
            AOps a;
            if constexpr (DO_K) {
                a.q = lds_a_tr16<HD>(sQ, 16 * d, lane);
                if constexpr (HAS_G) a.tq = lds_a_tr16<HD>(sTQ, 16 * d, lane);
            }
            if constexpr (DO_V) {
                if constexpr (HAS_G) a.g = lds_a_tr16<HD>(sG, 16 * d, lane);
                if constexpr (HAS_DO) a.d = lds_a_tr16<HD>(sDO, 16 * d, lane);
            }
            return a;
        };
        f32x4 s[2], ts[2], w[2], xy[2];
        f32x4 lse4[2], mu4[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            s[t] = f32x4{0.f, 0.f, 0.f, 0.f};
            ts[t] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
        // The workspace holds -s4 and -s7d: W and XY are accumulated on top of them, so that W - s4 and
        // XY - s7d leave the matrix cores ready for use.
        auto load_sums = [&](int u) __attribute__((always_inline)) {
            const int r0 = 16 * u + 4 * g;  // register j of tile u is query 16 u + 4 g + j
            if constexpr (HAS_G && DO_K) w[u] = *reinterpret_cast<const f32x4*>(sStat + 2 * kStageRows + r0);
            if constexpr (DO_K) xy[u] = *reinterpret_cast<const f32x4*>(sStat + 3 * kStageRows + r0);
        };
        auto load_stats = [&](int u) __attribute__((always_inline)) {
            const int r0 = 16 * u + 4 * g;
            lse4[u] = *reinterpret_cast<const f32x4*>(sStat + 0 * kStageRows + r0);
            if constexpr (HAS_G) mu4[u] = *reinterpret_cast<const f32x4*>(sStat + 1 * kStageRows + r0);
        };
        auto score_step = [&](int t, int c, const AOps& a) __attribute__((always_inline)) {
            s[t] = T::mfma16(a.q, kB[c], s[t]);
            if constexpr (HAS_G) {
                ts[t] = T::mfma16(a.q, tkB[c], ts[t]);
                ts[t] = T::mfma16(a.tq, kB[c], ts[t]);
                if constexpr (DO_K) {
                    w[t] = T::mfma16(a.g, vB[c], w[t]);
                    xy[t] = T::mfma16(a.g, tvB[c], xy[t]);
                }
            }
            if constexpr (HAS_DO && DO_K) xy[t] = T::mfma16(a.d, vB[c], xy[t]);
        };
        // in place: s -> P, ts -> P_dot, w -> dS_dot, xy -> dS  (rows beyond Lq are zero rows of Q,
        // Q_dot, G, dO with finite statistics: they contribute nothing)
        auto pointwise = [&](int t) __attribute__((always_inline)) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float pj = fast_exp2(fmaf(s[t][j], sl2, -lse4[t][j]));
                s[t][j] = pj;
                if constexpr (HAS_G) {
                    const float nn = fmaf(ts[t][j], p.scale, -mu4[t][j]);
                    if constexpr (DO_K) {
                        const float dts = pj * w[t][j];
                        w[t][j] = dts;
                        xy[t][j] = fmaf(dts, nn, pj * xy[t][j]);
                    }
                    if constexpr (DO_V) ts[t][j] = pj * nn;
                } else if constexpr (DO_K) {
                    xy[t][j] = pj * xy[t][j];
                }
            }
        };
        load_sums(0);
        AOps cur = load_score(0, 0);
        load_stats(0);
#pragma unroll
        for (int c = 0; c < KC; ++c) {
            AOps nxt;
            if (c + 1 < KC) {
                nxt = load_score(0, c + 1);
            } else {
                load_sums(1);
                nxt = load_score(1, 0);
            }
            __builtin_amdgcn_sched_barrier(0);  // keep the reads ahead of this step's MFMAs
            score_step(0, c, cur);
            __builtin_amdgcn_sched_barrier(0);
            cur = nxt;
        }
        // the second tile's MFMA chains run under the first tile's element-wise arithmetic
#pragma unroll
        for (int c = 0; c < KC; ++c) {
            AOps nxt;
            if (c + 1 < KC) {
                nxt = load_score(1, c + 1);
            } else {
                load_stats(1);
                nxt = load_grad(0);
            }
            score_step(1, c, cur);
            cur = nxt;
        }
        pointwise(0);
        __builtin_amdgcn_sched_barrier(0);
        pointwise(1);
        u32x4 pB, dsB, pdB, dtsB;
        if constexpr (DO_V) pB = pack_b16<T>(s[0], s[1]);
        if constexpr (DO_K) dsB = pack_b16<T>(xy[0], xy[1]);
        if constexpr (HAS_G) {
            if constexpr (DO_V) pdB = pack_b16<T>(ts[0], ts[1]);
            if constexpr (DO_K) dtsB = pack_b16<T>(w[0], w[1]);
        }
#pragma unroll
        for (int d = 0; d < DT; ++d) {
            AOps nxt;
            if (d + 1 < DT) nxt = load_grad(d + 1);
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (DO_K) {
                dk[d] = T::mfma16(cur.q, dsB, dk[d]);
                if constexpr (HAS_G) {
                    dtk[d] = T::mfma16(cur.q, dtsB, dtk[d]);
                    dk[d] = T::mfma16(cur.tq, dtsB, dk[d]);
                }
            }
            if constexpr (DO_V) {
                if constexpr (HAS_G) {
                    dtv[d] = T::mfma16(cur.g, pB, dtv[d]);
                    dv[d] = T::mfma16(cur.g, pdB, dv[d]);
                }
                if constexpr (HAS_DO) dv[d] = T::mfma16(cur.d, pB, dv[d]);
            }
            __builtin_amdgcn_sched_barrier(0);
            cur = nxt;
        }
    };

    for (int i = 0; i < ns; ++i) {
        wait_stages<SPT>(issued - 1 - i);
        workgroup_barrier();  // stage i has landed for every wave; stage i-1 is fully consumed
        if (i > 0 && issued < ns) issue_next();
        if (wave_active) compute(ring + (i % R) * SM::slot);
    }
    workgroup_barrier();  // every wave is done reading the ring: it becomes the store staging area
    if (!wave_active) return;
    elem_t* stage_tile = ring + wave * StoreStage16<HD>::elems;
    const int row0 = key0 + wave * 16;
    if constexpr (DO_K) {
        store_tile16<T, HD>(stage_tile, p.dk.head(b, h), p.dk.sl, row0, p.Lk, p.D, dk, p.scale, lane);
        if constexpr (HAS_G)
            store_tile16<T, HD>(stage_tile, p.dtk.head(b, h), p.dtk.sl, row0, p.Lk, p.D, dtk, p.scale, lane);
    }
    if constexpr (DO_V) {
        store_tile16<T, HD>(stage_tile, p.dv.head(b, h), p.dv.sl, row0, p.Lk, p.D, dv, 1.0f, lane);
        if constexpr (HAS_G)
            store_tile16<T, HD>(stage_tile, p.dtv.head(b, h), p.dtv.sl, row0, p.Lk, p.D, dtv, 1.0f, lane);
    }
}

template <typename T, int HD, int R, bool HAS_DO, bool HAS_G, int PART, int OCC>
__global__ __launch_bounds__(kXThreads16, OCC) void bwd_col16_kernel(const BwdParams p) {
    bwd_col16_body<T, HD, R, HAS_DO, HAS_G, PART>(p, (int)blockIdx.x, (int)gridDim.x);
}

// The column-owned launch with the second launch of the row-owned kernel at its end: workgroups
// 0 .. col_blocks - 1 are the column-owned kernel's, the rest the row-owned kernel's second pass, which does
// not depend on the column pass (it rewrites dQ, dQ_dot of flagged workgroups from the sums the first pass
// left).  Nearly all of those workgroups leave at once; dealt out behind the column pass they fill the time in
// which its last workgroups run alone, where a launch of their own costs a few microseconds.
template <typename T, int HD, int R, bool HAS_DO, bool HAS_G, int OCC>
__global__ __launch_bounds__(kXThreads16, OCC) void bwd_col16_repair_kernel(const BwdParams p) {
    const int col_blocks = p.col_workgroups;
    if ((int)blockIdx.x < col_blocks)
        bwd_col16_body<T, HD, R, HAS_DO, HAS_G, 3>(p, (int)blockIdx.x, col_blocks);
    else
        bwd_row16_body<T, HD, R, HAS_DO, HAS_G, 2>(p, (int)blockIdx.x - col_blocks, (int)gridDim.x - col_blocks);
}

// ---------------------------------------------------------------------------------------------
// Column-owned kernel for the head dimension 128: a workgroup of eight waves owns 64 keys; waves
// 2 r and 2 r + 1 share keys 16 r .. 16 r + 15.  Four gradients of 16 x 128 do not fit one wave's
// registers beside the operands, so the pair splits the work without repeating any of it: member m
// forms the score-side tiles (S, S_dot, W, XY -> P, P_dot, dS_dot, dS) of the stage's query tile m
// (16 queries), the two exchange their packed tiles through LDS, and member m accumulates all four
// gradients for head-dimension columns 64 m .. 64 m + 63 over the stage's 32 queries.  One launch,
// 12 tile contractions (6 + 6), the query side streamed once.
// LDS: [ring of Q | [Q_dot | G] | [dO] | lse2, mu, s4, s7d stages][exchange: 8 waves x 4 tiles][sink];
// the ring doubles as store staging after the last stage.
template <int HD, int R, bool HAS_DO, bool HAS_G>
struct Col16pSmem {
    static constexpr int nt = 1 + (HAS_G ? 2 : 0) + (HAS_DO ? 1 : 0);
    static constexpr int stat_elems = 4 * kStageRows * 2;
    static constexpr int slot = nt * Slab<HD>::elems + stat_elems;
    static constexpr int xch = kWaves16 * 4 * 64 * 4;  // u32x2 per lane, tile and wave, in elem_t units
    static constexpr int sink = (R * slot + xch) * (int)sizeof(elem_t);
    static constexpr int bytes = sink + kSink16;
    static_assert(R * slot >= kWaves16 * StoreStage16<64>::elems, "ring too small to stage stores");
};

template <typename T, int HD, int R, bool HAS_DO, bool HAS_G>
__device__ __forceinline__ void bwd_col16p_body(const BwdParams p, const int block, const int blocks) {
    static_assert(HD == 128, "the paired form exists for the head dimension that needs it");
    extern __shared__ __align__(16) unsigned char smem_raw[];
    using SM = Col16pSmem<HD, R, HAS_DO, HAS_G>;
    elem_t* ring = reinterpret_cast<elem_t*>(smem_raw);
    u32x2* xch = reinterpret_cast<u32x2*>(ring + R * SM::slot);  // [wave][tile 0..3][lane]
    constexpr int SE = Slab<HD>::elems;
    constexpr int oTQ = SE, oG = 2 * SE, oDO = (HAS_G ? 3 : 1) * SE, oST = SM::nt * SE;
    constexpr int KC = HD / 32;
    constexpr int DH = HD / 32;  // 16-wide head-dimension tiles per member (half of HD / 16)
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int pr = wave >> 1, m = wave & 1;  // pair, member
    const int n = lane & 15;
    const int g = lane >> 4;
    const int k_blocks = (p.Lk + kXOwned16 - 1) / kXOwned16;
    const int bid = xcd_linear_id(block, blocks);
    const int bh = bid / k_blocks;
    const int kb = bid % k_blocks;
    const int b = bh / p.H, h = bh % p.H;
    const int key0 = kb * kXOwned16;
    const int krow = key0 + pr * 16 + n;
    const bool kvalid = krow < p.Lk;
    const bool pair_active = (key0 + pr * 16) < p.Lk;

    using StagePlan = CopyPlan<HD, SM::nt, 1, kThreads16>;
    constexpr int SPT = StagePlan::N + 1;  // plus one 4-byte copy of statistics (or its placeholder)
    StagePlan plan;
    const int ns = (p.Lq + kStageRows - 1) / kStageRows;
    int issued = 0;
    auto issue_next = [&]() {
        elem_t* slot = ring + (issued % R) * SM::slot;
        const int row0 = issued * kStageRows;
        plan.issue(slot, p.Lq - row0, p.D == HD && row0 + kStageRows <= p.Lq);
        // the four statistic arrays of the stage's rows by waves 0..3; the others issue a placeholder
        if (wave < 4) {
            const int64_t plane = p.s4 - p.lse2;  // see bwd_col16_body
            const float* src = p.lse2 + (wave == 0 ? 0 : wave == 3 ? 2 : 1) * plane;  // lse2 | s4 | s4 | s7d
            if (HAS_G && wave == 1) src = p.mu;
            float* st = reinterpret_cast<float*>(slot + oST);
            if (lane < 32) dma4(src + (int64_t)bh * p.Lr + row0 + lane, lds_addr(st) + (uint32_t)(wave * 32 * 4));
        } else {
            if (lane == 0) dma4(plan.any, plan.sink);
        }
        ++issued;
    };
    // called behind the requests for the own rows on both paths below (see bwd_row16_kernel): set-up of the
    // stage copies, and stage 0 only for now
    auto begin_copies = [&]() __attribute__((always_inline)) {
        const Src q{p.q.head(b, h), p.q.sl};
        if constexpr (HAS_G && HAS_DO)
            plan.init(tid, 0, p.D, smem_raw + SM::sink, q, Src{p.tq.head(b, h), p.tq.sl},
                      Src{p.dTO.head(b, h), p.dTO.sl}, Src{p.dO.head(b, h), p.dO.sl});
        else if constexpr (HAS_G)
            plan.init(tid, 0, p.D, smem_raw + SM::sink, q, Src{p.tq.head(b, h), p.tq.sl},
                      Src{p.dTO.head(b, h), p.dTO.sl});
        else
            plan.init(tid, 0, p.D, smem_raw + SM::sink, q, Src{p.dO.head(b, h), p.dO.sl});
        issue_next();
    };
    // the own rows are requested first; the set-up of the stage copies runs while they travel
    u32x4 kB[KC], vB[KC], tkB[KC], tvB[KC];
    if (p.k_side_uniform && p.D == HD && key0 + kXOwned16 <= p.Lk) {
        // the common case: whole rows that all exist, every tensor with k's strides
        const int64_t slice = b * p.k.sb + h * p.k.sh;
        const uint32_t at = ((uint32_t)krow * (uint32_t)p.k.sl + 8u * (uint32_t)g) * (uint32_t)sizeof(elem_t);
        load_b_operands16_at<HD>(kB, p.k.ptr + slice, at);
        load_b_operands16_at<HD>(vB, p.v.ptr + slice, at);
        if constexpr (HAS_G) {
            load_b_operands16_at<HD>(tkB, p.tk.ptr + slice, at);
            load_b_operands16_at<HD>(tvB, p.tv.ptr + slice, at);
        }
        begin_copies();
    } else {
        load_b_operands16<HD>(kB, p.k.head(b, h) + (int64_t)krow * p.k.sl, g, p.D, kvalid);
        load_b_operands16<HD>(vB, p.v.head(b, h) + (int64_t)krow * p.v.sl, g, p.D, kvalid);
        if constexpr (HAS_G) {
            load_b_operands16<HD>(tkB, p.tk.head(b, h) + (int64_t)krow * p.tk.sl, g, p.D, kvalid);
            load_b_operands16<HD>(tvB, p.tv.head(b, h) + (int64_t)krow * p.tv.sl, g, p.D, kvalid);
        }
        begin_copies();
    }
#pragma unroll
    for (int c = 0; c < KC; ++c) {  // the own rows are awaited here
        asm volatile("" : "+v"(kB[c]), "+v"(vB[c]));
        if constexpr (HAS_G) asm volatile("" : "+v"(tkB[c]), "+v"(tvB[c]));
    }
    while (issued < R && issued < ns) issue_next();
    const float sl2 = p.scale * kLog2e;
    f32x4 dk[DH], dv[DH], dtk[DH], dtv[DH];
#pragma unroll
    for (int t = 0; t < DH; ++t) {
        dk[t] = f32x4{0.f, 0.f, 0.f, 0.f};
        dv[t] = f32x4{0.f, 0.f, 0.f, 0.f};
        dtk[t] = f32x4{0.f, 0.f, 0.f, 0.f};
        dtv[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    // packed tiles of this member's query tile: P, P_dot, dS, dS_dot (register j = query 16 m + 4 g + j)
    u32x2 mine[4];
    u32x2* my_x = xch + (wave * 4) * 64 + lane;
    const u32x2* other_x = xch + ((wave ^ 1) * 4) * 64 + lane;

    auto scores = [&](const elem_t* slot) {
        const elem_t* sQ = slot;
        const elem_t* sTQ = slot + oTQ;
        const elem_t* sG = slot + oG;
        const elem_t* sDO = slot + oDO;
        const float* sStat = reinterpret_cast<const float*>(slot + oST);
        // the workspace holds -s4 and -s7d: W and XY are accumulated on top of them
        const int r0 = 16 * m + 4 * g;
        f32x4 s = {0.f, 0.f, 0.f, 0.f}, ts = {0.f, 0.f, 0.f, 0.f};
        f32x4 w = *reinterpret_cast<const f32x4*>(sStat + 2 * kStageRows + r0);
        f32x4 xy = *reinterpret_cast<const f32x4*>(sStat + 3 * kStageRows + r0);
#pragma unroll
        for (int c = 0; c < KC; ++c) {
            const u32x4 aq = lds_a_rows16<HD>(sQ, m, c, n, g);
            s = T::mfma16(aq, kB[c], s);
            if constexpr (HAS_G) {
                ts = T::mfma16(aq, tkB[c], ts);
                const u32x4 atq = lds_a_rows16<HD>(sTQ, m, c, n, g);
                ts = T::mfma16(atq, kB[c], ts);
                const u32x4 ag = lds_a_rows16<HD>(sG, m, c, n, g);
                w = T::mfma16(ag, vB[c], w);
                xy = T::mfma16(ag, tvB[c], xy);
            }
            if constexpr (HAS_DO) {
                const u32x4 ado = lds_a_rows16<HD>(sDO, m, c, n, g);
                xy = T::mfma16(ado, vB[c], xy);
            }
        }
        // rows beyond Lq are zero rows of Q, Q_dot, G, dO with finite statistics: they contribute nothing
        const f32x4 lse4 = *reinterpret_cast<const f32x4*>(sStat + 0 * kStageRows + r0);
        const f32x4 mu4 = *reinterpret_cast<const f32x4*>(sStat + 1 * kStageRows + r0);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float pj = fast_exp2(fmaf(s[j], sl2, -lse4[j]));
            s[j] = pj;
            if constexpr (HAS_G) {
                const float nn = fmaf(ts[j], p.scale, -mu4[j]);
                const float dts = pj * w[j];
                w[j] = dts;
                xy[j] = fmaf(dts, nn, pj * xy[j]);
                ts[j] = pj * nn;
            } else {
                xy[j] = pj * xy[j];
            }
        }
        mine[0] = u32x2{T::pack2(s[0], s[1]), T::pack2(s[2], s[3])};
        mine[2] = u32x2{T::pack2(xy[0], xy[1]), T::pack2(xy[2], xy[3])};
        my_x[0 * 64] = mine[0];
        my_x[2 * 64] = mine[2];
        if constexpr (HAS_G) {
            mine[1] = u32x2{T::pack2(ts[0], ts[1]), T::pack2(ts[2], ts[3])};
            mine[3] = u32x2{T::pack2(w[0], w[1]), T::pack2(w[2], w[3])};
            my_x[1 * 64] = mine[1];
            my_x[3 * 64] = mine[3];
        }
    };
    // B operand over the stage's 32 queries from the pair's two packed tiles (query tile 0 first)
    auto both = [&](int which) {
        const u32x2 o = other_x[which * 64];
        return m == 0 ? u32x4{mine[which][0], mine[which][1], o[0], o[1]}
                      : u32x4{o[0], o[1], mine[which][0], mine[which][1]};
    };
    auto outputs = [&](const elem_t* slot) {
        const elem_t* sQ = slot;
        const elem_t* sTQ = slot + oTQ;
        const elem_t* sG = slot + oG;
        const elem_t* sDO = slot + oDO;
        const u32x4 pB = both(0), dsB = both(2);
        u32x4 pdB, dtsB;
        if constexpr (HAS_G) {
            pdB = both(1);
            dtsB = both(3);
        }
#pragma unroll
        for (int d = 0; d < DH; ++d) {
            const int d0 = 64 * m + 16 * d;
            const u32x4 aq = lds_a_tr16<HD>(sQ, d0, lane);
            dk[d] = T::mfma16(aq, dsB, dk[d]);
            if constexpr (HAS_G) {
                dtk[d] = T::mfma16(aq, dtsB, dtk[d]);
                const u32x4 atq = lds_a_tr16<HD>(sTQ, d0, lane);
                dk[d] = T::mfma16(atq, dtsB, dk[d]);
                const u32x4 ag = lds_a_tr16<HD>(sG, d0, lane);
                dtv[d] = T::mfma16(ag, pB, dtv[d]);
                dv[d] = T::mfma16(ag, pdB, dv[d]);
            }
            if constexpr (HAS_DO) {
                const u32x4 ado = lds_a_tr16<HD>(sDO, d0, lane);
                dv[d] = T::mfma16(ado, pB, dv[d]);
            }
        }
    };

    for (int i = 0; i < ns; ++i) {
        wait_stages<SPT>(issued - 1 - i);
        workgroup_barrier();  // stage i has landed for every wave; stage i-1 and the exchange area are free
        if (i > 0 && issued < ns) issue_next();
        const elem_t* slot = ring + (i % R) * SM::slot;
        if (pair_active) scores(slot);
        workgroup_barrier();  // the partner's tiles are visible
        if (pair_active) outputs(slot);
    }
    workgroup_barrier();  // every wave is done reading the ring: it becomes the store staging area
    if (!pair_active) return;
    elem_t* stage_tile = ring + wave * StoreStage16<64>::elems;
    const int row0 = key0 + pr * 16;
    const int dcol = 64 * m;
    const int Dm = p.D - dcol;  // columns of this member's half that exist (may be <= 0)
    store_tile16<T, 64>(stage_tile, p.dk.head(b, h) + dcol, p.dk.sl, row0, p.Lk, Dm, dk, p.scale, lane);
    if constexpr (HAS_G)
        store_tile16<T, 64>(stage_tile, p.dtk.head(b, h) + dcol, p.dtk.sl, row0, p.Lk, Dm, dtk, p.scale, lane);
    store_tile16<T, 64>(stage_tile, p.dv.head(b, h) + dcol, p.dv.sl, row0, p.Lk, Dm, dv, 1.0f, lane);
    if constexpr (HAS_G)
        store_tile16<T, 64>(stage_tile, p.dtv.head(b, h) + dcol, p.dtv.sl, row0, p.Lk, Dm, dtv, 1.0f, lane);
}

template <typename T, int HD, int R, bool HAS_DO, bool HAS_G>
__global__ __launch_bounds__(kThreads16, 2) void bwd_col16p_kernel(const BwdParams p) {
    bwd_col16p_body<T, HD, R, HAS_DO, HAS_G>(p, (int)blockIdx.x, (int)gridDim.x);
}

// The paired column-owned launch with the second pass of the row-owned kernel at its end (see
// bwd_col16_repair_kernel).  The row-owned kernel's workgroups have four waves, these eight: in a workgroup that
// takes a row item the upper four leave at once, and the barriers of the others count the waves that are left.
template <typename T, int HD, int R, int RROW, bool HAS_DO, bool HAS_G>
__global__ __launch_bounds__(kThreads16, 2) void bwd_col16p_repair_kernel(const BwdParams p) {
    const int col_blocks = p.col_workgroups;
    if ((int)blockIdx.x < col_blocks) {
        bwd_col16p_body<T, HD, R, HAS_DO, HAS_G>(p, (int)blockIdx.x, col_blocks);
    } else {
        if ((int)threadIdx.x >= kXThreads16) return;
        bwd_row16_body<T, HD, RROW, HAS_DO, HAS_G, 2>(p, (int)blockIdx.x - col_blocks, (int)gridDim.x - col_blocks);
    }
}

}  // namespace sjvp
