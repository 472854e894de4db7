// Single-launch attention-JVP backward for short key axes (Lk <= 128, head dimension <= 64,
// 16-byte aligned rows): one workgroup per (batch, head) owns every key, streams the queries once
// and produces all six gradients, so each of the sixteen tensors crosses HBM exactly once and the
// score-side tiles are computed once (the two-launch form recomputes them and re-reads the inputs).
//
// The mathematics is that of sjvp_bwd.hpp.  Per stage of 32 queries:
//   1. (all threads) row sums s4, s7d of the NEXT stage from its G, dO, O, TO slabs, 8 threads per row;
//   2. (wave w = keys 32w..32w+31) tiles S, S_dot, W, XY -> P, P_dot, dS_dot, dS with queries in
//      registers and keys in lanes; dK, dV, dK_dot, dV_dot accumulate in registers as in
//      bwd_col_kernel; dS and dS_dot are also written as 16-bit to an LDS bounce tile [query][key];
//   3. after a barrier, wave w forms one 32-column tile of dQ (w < 2) or dQ_dot (w >= 2) for the
//      stage from the bounce tile (B operand, row-major) and the transposed own rows of K, K_dot
//      (A operand), and stores it; a stage's dQ rows are complete after one pass over the keys, so
//      nothing is accumulated across stages and no atomics or partial sums are needed.
// Results are deterministic.
#pragma once
#include "sjvp_bwd.hpp"

namespace sjvp {

// LDS layout: [own K, V (, K_dot, V_dot): one slab per wave each][ring of query stages:
// Q | [Q_dot | G] | [dO] | O | [TO] | raw lse, mu (one copy pair per two waves) | lse2, mu, s4, s7d]
// [bounce: dS (, dS_dot) as [32 queries][128 keys + pad]][sink]
template <int HD, int R, bool HAS_DO, bool HAS_G>
struct FusedSmem {
    static constexpr int nt = 2 + (HAS_G ? 3 : 0) + (HAS_DO ? 1 : 0);
    static constexpr int stat_elems = 8 * kStageRows * 2;  // 8 float arrays of 32, in elem_t units
    static constexpr int slot = nt * Slab<HD>::elems + stat_elems;
    static constexpr int own = (HAS_G ? 4 : 2) * kWaves * Slab<HD>::elems;
    static constexpr int bpitch = kOwned + 8;  // 272 bytes: 16-byte row reads of 8 lanes cover all banks
    static constexpr int bounce_one = kStageRows * bpitch;
    static constexpr int bounce = (HAS_G ? 2 : 1) * bounce_one;
    static constexpr int sink = (own + R * slot + bounce) * (int)sizeof(elem_t);
    static constexpr int bytes = sink + kSinkBytes;
};

template <typename T, int HD, int R, bool HAS_DO, bool HAS_G>
__global__ __launch_bounds__(kThreads, 1) void bwd_fused_kernel(const BwdParams p) {
    static_assert(kWaves == 4 && HD <= 64, "one workgroup covers 128 keys with four waves");
    extern __shared__ __align__(16) unsigned char smem_raw[];
    using SM = FusedSmem<HD, R, HAS_DO, HAS_G>;
    elem_t* own = reinterpret_cast<elem_t*>(smem_raw);
    elem_t* ring = own + SM::own;
    elem_t* bounceS = ring + R * SM::slot;
    elem_t* bounceT = bounceS + SM::bounce_one;
    constexpr int SE = Slab<HD>::elems;
    constexpr int oTQ = SE, oG = 2 * SE, oDO = (HAS_G ? 3 : 1) * SE;
    constexpr int oO = oDO + (HAS_DO ? SE : 0), oTO = oO + SE;
    constexpr int oST = SM::nt * SE;
    constexpr int BP = SM::bpitch;

    constexpr int KC = HD / 16;
    constexpr int NDT = HD / 32;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int x = lane & 31;
    const int hf = lane >> 5;
    const int bh = blockIdx.x;
    const int b = bh / p.H, h = bh % p.H;
    SlabLane<HD> ln;
    ln.init(tid, smem_raw + SM::sink);
    // LDS-DMA instructions per stage issued by every wave: the tensors plus one 4-byte copy of
    // statistics
    constexpr int SPT = SM::nt * Slab<HD>::per_thread + 1;
    const bool wave_active = wave * 32 < p.Lk;
    const int key_waves = (p.Lk + 31) >> 5;  // waves that own at least one key

    {
        auto own_fill = [&](int idx, const TensorView& t) {
#pragma unroll
            for (int s4 = 0; s4 < kWaves; ++s4)
                fill_slab<HD, true>(ln, own + (kWaves * idx + s4) * SE, t.head(b, h), t.sl, 32 * s4, p.Lk,
                                    p.D, true);
        };
        own_fill(0, p.k);
        own_fill(1, p.v);
        if constexpr (HAS_G) {
            own_fill(2, p.tk);
            own_fill(3, p.tv);
        }
    }
    const elem_t* qg = p.q.head(b, h);
    const elem_t* tqg = HAS_G ? p.tq.head(b, h) : nullptr;
    const elem_t* gg = HAS_G ? p.dTO.head(b, h) : nullptr;
    const elem_t* dog = HAS_DO ? p.dO.head(b, h) : nullptr;
    const elem_t* og = p.o.head(b, h);
    const elem_t* tog = HAS_G ? p.to.head(b, h) : nullptr;
    const float sl2 = p.scale * kLog2e;

    auto issue = [&](int stage) {
        elem_t* slot = ring + (stage % R) * SM::slot;
        const int row0 = stage * kStageRows;
        fill_slab<HD, true>(ln, slot, qg, p.q.sl, row0, p.Lq, p.D, true);
        if constexpr (HAS_G) {
            fill_slab<HD, true>(ln, slot + oTQ, tqg, p.tq.sl, row0, p.Lq, p.D, true);
            fill_slab<HD, true>(ln, slot + oG, gg, p.dTO.sl, row0, p.Lq, p.D, true);
        }
        if constexpr (HAS_DO) fill_slab<HD, true>(ln, slot + oDO, dog, p.dO.sl, row0, p.Lq, p.D, true);
        fill_slab<HD, true>(ln, slot + oO, og, p.o.sl, row0, p.Lq, p.D, true);
        if constexpr (HAS_G) fill_slab<HD, true>(ln, slot + oTO, tog, p.to.sl, row0, p.Lq, p.D, true);
        // raw lse (even waves) and mu (odd waves) of the stage's rows, 32 lanes each (rows < Lr exist);
        // every wave issues exactly one 4-byte LDS-DMA instruction
        float* raw = reinterpret_cast<float*>(slot + oST);
        const float* src = ((wave & 1) && HAS_G) ? p.mu : p.lse;
        if (hf == 0) dma4(src + (int64_t)bh * p.Lr + row0 + x, lds_addr(raw) + (uint32_t)(wave * 32 * 4));
    };

    // Row sums of a landed stage: thread t handles row t/8, columns 8*(t%8) .. +7; the eight partial
    // sums meet through lane shuffles and the thread of column 0 writes the row's four statistics.
    auto row_sums = [&](elem_t* slot) {
        const int r = tid >> 3, part = tid & 7;
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
                const float o0 = T::to_float((elem_t)(o4[i] & 0xffffu));
                const float o1 = T::to_float((elem_t)(o4[i] >> 16));
                if constexpr (HAS_G) {
                    const float g0 = T::to_float((elem_t)(g4[i] & 0xffffu));
                    const float g1 = T::to_float((elem_t)(g4[i] >> 16));
                    const float t0 = T::to_float((elem_t)(t4[i] & 0xffffu));
                    const float t1 = T::to_float((elem_t)(t4[i] >> 16));
                    s4 += g0 * o0 + g1 * o1;
                    s7d += g0 * t0 + g1 * t1;
                }
                if constexpr (HAS_DO) {
                    const float d0 = T::to_float((elem_t)(d4[i] & 0xffffu));
                    const float d1 = T::to_float((elem_t)(d4[i] >> 16));
                    s7d += d0 * o0 + d1 * o1;
                }
            }
        }
#pragma unroll
        for (int m = 1; m < 8; m <<= 1) {
            s4 += __shfl_xor(s4, m, 64);
            s7d += __shfl_xor(s7d, m, 64);
        }
        if (part == 0) {
            float* raw = reinterpret_cast<float*>(slot + oST);
            float* fin = raw + 4 * kStageRows;
            fin[0 * kStageRows + r] = raw[r] * kLog2e;
            fin[1 * kStageRows + r] = HAS_G ? raw[kStageRows + r] : 0.f;
            fin[2 * kStageRows + r] = s4;
            fin[3 * kStageRows + r] = s7d;
        }
    };

    u32x4 kB[KC], vB[KC], tkB[KC], tvB[KC];
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

    // Step 2: the column-owned tile of one stage.
    auto tile = [&](const elem_t* slot) {
        const elem_t* sQ = slot;
        const elem_t* sTQ = slot + oTQ;
        const elem_t* sG = slot + oG;
        const elem_t* sDO = slot + oDO;
        const float* sStat = reinterpret_cast<const float*>(slot + oST) + 4 * kStageRows;
        f32x16 s = {0}, ts = {0}, w = {0}, xy = {0};
#pragma unroll
        for (int c = 0; c < KC; ++c) {
            u32x4 aq = lds_a_rows<HD>(sQ, c, x, hf);
            s = T::mfma(aq, kB[c], s);
            if constexpr (HAS_G) {
                ts = T::mfma(aq, tkB[c], ts);
                u32x4 atq = lds_a_rows<HD>(sTQ, c, x, hf);
                ts = T::mfma(atq, kB[c], ts);
                u32x4 ag = lds_a_rows<HD>(sG, c, x, hf);
                w = T::mfma(ag, vB[c], w);
                xy = T::mfma(ag, tvB[c], xy);
            }
            if constexpr (HAS_DO) {
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
                    const float dts = pj * (w[j] - s44[i]);
                    w[j] = dts;
                    xy[j] = fmaf(dts, n, pj * (xy[j] - s74[i]));
                    ts[j] = pj * n;
                } else {
                    xy[j] = pj * (xy[j] - s74[i]);
                }
            }
        }
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            u32x4 pB, dsB, pdB, dtsB;
            pB = pack_b<T>(s, c);
            dsB = pack_b<T>(xy, c);
            if constexpr (HAS_G) {
                pdB = pack_b<T>(ts, c);
                dtsB = pack_b<T>(w, c);
            }
            // bounce[query][key]: register 8c + 2i (+1) of the tile is query 16c + 4hf + 8(i/2) + 2(i%2) (+1)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int qr = 16 * c + 4 * hf + 8 * (i >> 1) + 2 * (i & 1);
                elem_t* d0 = bounceS + qr * BP + wave * 32 + x;
                d0[0] = (elem_t)(dsB[i] & 0xffffu);
                d0[BP] = (elem_t)(dsB[i] >> 16);
                if constexpr (HAS_G) {
                    elem_t* d1 = bounceT + qr * BP + wave * 32 + x;
                    d1[0] = (elem_t)(dtsB[i] & 0xffffu);
                    d1[BP] = (elem_t)(dtsB[i] >> 16);
                }
            }
#pragma unroll
            for (int d = 0; d < NDT; ++d) {
                const int d0 = 32 * d;
                const u32x4 aq = lds_a_transposed<HD>(sQ, c, d0, lane);
                dk[d] = T::mfma(aq, dsB, dk[d]);
                if constexpr (HAS_G) {
                    dtk[d] = T::mfma(aq, dtsB, dtk[d]);
                    const u32x4 atq = lds_a_transposed<HD>(sTQ, c, d0, lane);
                    dk[d] = T::mfma(atq, dtsB, dk[d]);
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
    };

    // Step 3: this wave's tile of dQ or dQ_dot for the stage's 32 queries.
    const int out_t = wave >> 1;  // 0: dQ, 1: dQ_dot
    const int out_d = wave & 1;   // 32-column tile of the head dimension
    const bool out_active = out_d < NDT && (out_t == 0 || HAS_G);
    auto row_outputs = [&](int row0) {
        if (!out_active) return;
        f32x16 acc = {0};
        const int d0 = 32 * out_d;
        const int nkc = 2 * key_waves;
        for (int kc = 0; kc < nkc; ++kc) {
            const elem_t* kslab = own + (kc >> 1) * SE;
            const u32x4 ak = lds_a_transposed_nat<HD>(kslab, kc & 1, d0, lane);
            const u32x4 bs = *reinterpret_cast<const u32x4*>(bounceS + x * BP + 16 * kc + 8 * hf);
            if constexpr (HAS_G) {
                const u32x4 bt = *reinterpret_cast<const u32x4*>(bounceT + x * BP + 16 * kc + 8 * hf);
                if (out_t == 0) {
                    const u32x4 atk = lds_a_transposed_nat<HD>(kslab + 2 * kWaves * SE, kc & 1, d0, lane);
                    acc = T::mfma(ak, bs, acc);
                    acc = T::mfma(atk, bt, acc);
                } else {
                    acc = T::mfma(ak, bt, acc);
                }
            } else {
                acc = T::mfma(ak, bs, acc);
            }
        }
        const int qrow = row0 + x;
        if (qrow < p.Lq) {
            const OutView& t = out_t == 0 ? p.dq : p.dtq;
            store_acc<T>(t.head(b, h) + (int64_t)qrow * t.sl, d0, hf, p.D, acc, p.scale, true);
        }
    };

#ifdef SJVP_X_STAMP
    int n_st = 0;
    const unsigned long long t_0 = __builtin_amdgcn_s_memtime();
    auto stamp = [&]() {
        if (tid == SJVP_X_STAMP * 64) p.lse2[(int64_t)bh * p.Lr + 1 + n_st] = (float)(long long)(__builtin_amdgcn_s_memtime() - t_0);
        ++n_st;
    };
    if (tid == 0) p.lse2[(int64_t)bh * p.Lr] = (float)(t_0 & 0xffffffull);
#else
    auto stamp = [&]() {};
#endif
    const int n = (p.Lq + kStageRows - 1) / kStageRows;
    int issued = 0;
    for (; issued < R && issued < n; ++issued) issue(issued);
    wait_stages<SPT>(issued - 1);  // the own rows and stage 0 were issued before the others
    __syncthreads();
    read_b_operands<HD>(kB, own + wave * SE, x, hf);
    read_b_operands<HD>(vB, own + (kWaves + wave) * SE, x, hf);
    if constexpr (HAS_G) {
        read_b_operands<HD>(tkB, own + (2 * kWaves + wave) * SE, x, hf);
        read_b_operands<HD>(tvB, own + (3 * kWaves + wave) * SE, x, hf);
    }
    stamp();
    row_sums(ring);
    for (int i = 0; i < n; ++i) {
        __syncthreads();  // stage i and its statistics are visible; stage i-1 and the bounce tile are free
        stamp();
        if (i >= 1 && issued < n) issue(issued++);
        elem_t* slot = ring + (i % R) * SM::slot;
        stamp();
        if (wave_active) tile(slot);
        stamp();
        if (i + 1 < n) wait_stages<SPT>(issued - 2 - i);  // stage i+1 has landed (this wave's part)
        __syncthreads();
        stamp();
        if (i + 1 < n) row_sums(ring + ((i + 1) % R) * SM::slot);
        stamp();
        row_outputs(i * kStageRows);
        stamp();
    }
    __syncthreads();  // every wave is done reading the ring: it becomes the store staging area
    stamp();
    if (!wave_active) return;
    elem_t* stage_tile = ring + wave * StoreStage<HD>::elems;
    const int row0 = wave * 32;
    auto put = [&](const OutView& t, const f32x16* acc, float mul) {
        store_tile_coalesced<T, HD>(stage_tile, t.head(b, h), t.sl, row0, p.Lk, p.D, acc, mul, lane);
    };
    put(p.dk, dk, p.scale);
    if constexpr (HAS_G) put(p.dtk, dtk, p.scale);
    put(p.dv, dv, 1.0f);
    if constexpr (HAS_G) put(p.dtv, dtv, 1.0f);
    stamp();
#ifdef SJVP_X_STAMP
    __builtin_amdgcn_s_waitcnt(0);
    stamp();
#endif
}

}  // namespace sjvp
