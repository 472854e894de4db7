// fp32 mode of the attention-JVP path (gfx950): fp32 tensors in and out, every product, sum and
// exponential in fp32 on the vector ALUs.  This is the correctness mode of the library (the
// reference's fp32 math path, semicat/jvp_utils/ryu_triton.py:426-454, meets 1e-5 against fp64; the
// 16-bit MFMA kernels cannot): it is not tuned for speed and uses no matrix instructions.
//
// Decomposition: a group of eight lanes owns one row of the owned axis (a query in fwd_f32_kernel and
// bwd_row_f32_kernel, a key in bwd_col_f32_kernel) and splits the head dimension: lane c of the group
// holds columns 32 m + 4 c + e (m < HD/32, e < 4), so that the eight lanes read one 128-byte piece
// of an LDS row per instruction.  The other axis is streamed through LDS in tiles of 16 rows; per
// streamed row every dot product is a per-lane partial sum combined over the eight lanes by DPP
// moves.  A workgroup of 256 threads owns 32 rows.  Same mathematics, statistics (lse, mu, li rows up
// to Lr) and workspace hand-over (lse * log2 e, s4, s7d) as the 16-bit kernels.
#pragma once
#include "sjvp_w16.hpp"

namespace sjvp {

constexpr int kF32Threads = 256;
constexpr int kF32Owned = 32;  // owned rows per workgroup
constexpr int kF32Tile = 16;   // streamed rows per LDS tile

struct F32In {
    const float* ptr;
    int64_t sb, sh, sl;
    __device__ __forceinline__ const float* head(int b, int h) const { return ptr + b * sb + h * sh; }
};
struct F32Out {
    float* ptr;
    int64_t sb, sh, sl;
    __device__ __forceinline__ float* head(int b, int h) const { return ptr + b * sb + h * sh; }
};

struct FwdParamsF32 {
    F32In q, k, v, tq, tk, tv;
    F32Out o, to;
    float* lse;
    float* mu;
    float* li;  // may be null
    int H, Lq, Lk, D, Lr;
    float scale;
};

struct BwdParamsF32 {
    F32In q, k, v, tq, tk, tv, o, to, dO, dTO;
    F32Out dq, dk, dv, dtq, dtk, dtv;
    const float* lse;
    const float* mu;
    float* lse2;  // workspace [B*H][Lr]
    float* s4;
    float* s7d;
    int H, Lq, Lk, D, Lr;
    float scale;
};

// column of element (m, e) of lane c (c = lane % 8)
__device__ __forceinline__ int f32_col(int c, int m, int e) { return 32 * m + 4 * c + e; }

// This lane's columns of one global row; zero where the row is invalid or the column is >= D.
template <int HD>
__device__ __forceinline__ void f32_load_own(float* x, const float* row, int c, int D, bool valid) {
#pragma unroll
    for (int m = 0; m < HD / 32; ++m)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int col = f32_col(c, m, e);
            x[4 * m + e] = (valid && col < D) ? row[col] : 0.f;
        }
}

template <int HD>
__device__ __forceinline__ void f32_store_own(float* row, const float* x, float mul, int c, int D) {
#pragma unroll
    for (int m = 0; m < HD / 32; ++m)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int col = f32_col(c, m, e);
            if (col < D) row[col] = x[4 * m + e] * mul;
        }
}

// Rows row0 .. row0+15 of one [L][D] head slice into an LDS tile [16][HD], zero-filled beyond L, D.
template <int HD>
__device__ __forceinline__ void f32_fill_tile(float* tile, const float* g, int64_t sl, int row0, int L, int D,
                                              int tid) {
#pragma unroll
    for (int it = 0; it < kF32Tile * HD / kF32Threads; ++it) {
        const int idx = tid + it * kF32Threads;
        const int r = idx / HD, col = idx % HD;
        const int row = row0 + r;
        tile[idx] = (row < L && col < D) ? g[(int64_t)row * sl + col] : 0.f;
    }
}

// This lane's four columns (m) of tile row r.
template <int HD>
__device__ __forceinline__ f32x4 f32_tile4(const float* tile, int r, int c, int m) {
    return *reinterpret_cast<const f32x4*>(tile + r * HD + 32 * m + 4 * c);
}

template <int HD>
__device__ __forceinline__ float f32_dot(const float* x, const float* tile, int r, int c) {
    float s = 0.f;
#pragma unroll
    for (int m = 0; m < HD / 32; ++m) {
        const f32x4 t = f32_tile4<HD>(tile, r, c, m);
#pragma unroll
        for (int e = 0; e < 4; ++e) s = fmaf(x[4 * m + e], t[e], s);
    }
    return s;
}

template <int HD>
__device__ __forceinline__ void f32_axpy(float* acc, float a, const float* tile, int r, int c) {
#pragma unroll
    for (int m = 0; m < HD / 32; ++m) {
        const f32x4 t = f32_tile4<HD>(tile, r, c, m);
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[4 * m + e] = fmaf(a, t[e], acc[4 * m + e]);
    }
}

// ---------------------------------------------------------------------------------------------
// Forward (ryu_triton.py:188-291 in fp32): O, TO, lse, mu, li.  LDS: K | V | K_dot | V_dot tiles.
template <int HD, bool JVP>
__global__ __launch_bounds__(kF32Threads) void fwd_f32_kernel(const FwdParamsF32 p) {
    __shared__ __align__(16) float tiles[(JVP ? 4 : 2) * kF32Tile * HD];
    float* sK = tiles;
    float* sV = tiles + kF32Tile * HD;
    float* sTK = tiles + 2 * kF32Tile * HD;
    float* sTV = tiles + 3 * kF32Tile * HD;
    constexpr int C = HD / 8;
    const int tid = threadIdx.x;
    const int c = tid & 7;
    const int q_blocks = p.Lr / kF32Owned;
    const int bh = blockIdx.x / q_blocks, qb = blockIdx.x % q_blocks;
    const int b = bh / p.H, h = bh % p.H;
    const int qrow = qb * kF32Owned + (tid >> 3);
    const bool qvalid = qrow < p.Lq;

    float q[C], tq[C], acc[C], tacc[C];
    f32_load_own<HD>(q, p.q.head(b, h) + (int64_t)qrow * p.q.sl, c, p.D, qvalid);
    if constexpr (JVP) f32_load_own<HD>(tq, p.tq.head(b, h) + (int64_t)qrow * p.tq.sl, c, p.D, qvalid);
#pragma unroll
    for (int i = 0; i < C; ++i) {
        acc[i] = 0.f;
        tacc[i] = 0.f;
    }
    const float sl2 = p.scale * kLog2e;
    float m_i = -INFINITY, l_i = 0.f, mu_i = 0.f;  // running maximum (log2 units), exp-sum, sum p * S_dot

    for (int k0 = 0; k0 < p.Lk; k0 += kF32Tile) {
        workgroup_barrier();
        f32_fill_tile<HD>(sK, p.k.head(b, h), p.k.sl, k0, p.Lk, p.D, tid);
        f32_fill_tile<HD>(sV, p.v.head(b, h), p.v.sl, k0, p.Lk, p.D, tid);
        if constexpr (JVP) {
            f32_fill_tile<HD>(sTK, p.tk.head(b, h), p.tk.sl, k0, p.Lk, p.D, tid);
            f32_fill_tile<HD>(sTV, p.tv.head(b, h), p.tv.sl, k0, p.Lk, p.D, tid);
        }
        workgroup_barrier();
        float s[kF32Tile], ts[kF32Tile];
        float mloc = -INFINITY;
#pragma unroll
        for (int j = 0; j < kF32Tile; ++j) {
            s[j] = sum8(f32_dot<HD>(q, sK, j, c)) * sl2;
            if constexpr (JVP) ts[j] = sum8(f32_dot<HD>(tq, sK, j, c) + f32_dot<HD>(q, sTK, j, c)) * p.scale;
            if (k0 + j >= p.Lk) s[j] = -INFINITY;
            mloc = fmaxf(mloc, s[j]);
        }
        const float m_new = fmaxf(m_i, mloc);  // finite: every tile holds at least one key
        const float alpha = fast_exp2(m_i - m_new);
        m_i = m_new;
        l_i *= alpha;
        mu_i *= alpha;
#pragma unroll
        for (int i = 0; i < C; ++i) {
            acc[i] *= alpha;
            tacc[i] *= alpha;
        }
#pragma unroll
        for (int j = 0; j < kF32Tile; ++j) {
            const float pj = fast_exp2(s[j] - m_i);
            l_i += pj;
            f32_axpy<HD>(acc, pj, sV, j, c);
            if constexpr (JVP) {
                const float pt = pj * ts[j];
                mu_i += pt;
                f32_axpy<HD>(tacc, pt, sV, j, c);
                f32_axpy<HD>(tacc, pj, sTV, j, c);
            }
        }
    }
    const float inv_l = 1.0f / l_i;
    const float mu = mu_i * inv_l;
    const int64_t so = (int64_t)bh * p.Lr + qrow;  // rows below Lr exist
    if (c == 0) {
        // a padded query row (all-zero q, q_dot) yields log(Lk), 0, Lk by itself
        p.lse[so] = (m_i + fast_log2(l_i)) * kLn2;
        if constexpr (JVP) p.mu[so] = mu;
        if (p.li) p.li[so] = l_i;
    }
    if (!qvalid) return;
    f32_store_own<HD>(p.o.head(b, h) + (int64_t)qrow * p.o.sl, acc, inv_l, c, p.D);
    if constexpr (JVP) {
        // TO = (sum (p S_dot) v + sum p v_dot - mu_un O_un) / l   (ryu_triton.py:274-275)
#pragma unroll
        for (int i = 0; i < C; ++i) tacc[i] -= mu * acc[i];
        f32_store_own<HD>(p.to.head(b, h) + (int64_t)qrow * p.to.sl, tacc, inv_l, c, p.D);
    }
}

// ---------------------------------------------------------------------------------------------
// Row-owned backward: dQ (, dQ_dot) and the row sums for the column-owned kernel.
template <int HD, bool HAS_DO, bool HAS_G>
__global__ __launch_bounds__(kF32Threads) void bwd_row_f32_kernel(const BwdParamsF32 p) {
    __shared__ __align__(16) float tiles[(HAS_G ? 4 : 2) * kF32Tile * HD];
    float* sK = tiles;
    float* sV = tiles + kF32Tile * HD;
    float* sTK = tiles + 2 * kF32Tile * HD;
    float* sTV = tiles + 3 * kF32Tile * HD;
    constexpr int C = HD / 8;
    const int tid = threadIdx.x;
    const int c = tid & 7;
    const int q_blocks = p.Lr / kF32Owned;
    const int bh = blockIdx.x / q_blocks, qb = blockIdx.x % q_blocks;
    const int b = bh / p.H, h = bh % p.H;
    const int qrow = qb * kF32Owned + (tid >> 3);
    const bool qvalid = qrow < p.Lq;

    float q[C], tq[C], g[C], dO[C], dq[C], dtq[C];
    float s4 = 0.f, s7d = 0.f;
    {
        float o[C], to[C];
        f32_load_own<HD>(q, p.q.head(b, h) + (int64_t)qrow * p.q.sl, c, p.D, qvalid);
        f32_load_own<HD>(o, p.o.head(b, h) + (int64_t)qrow * p.o.sl, c, p.D, qvalid);
        if constexpr (HAS_G) {
            f32_load_own<HD>(tq, p.tq.head(b, h) + (int64_t)qrow * p.tq.sl, c, p.D, qvalid);
            f32_load_own<HD>(g, p.dTO.head(b, h) + (int64_t)qrow * p.dTO.sl, c, p.D, qvalid);
            f32_load_own<HD>(to, p.to.head(b, h) + (int64_t)qrow * p.to.sl, c, p.D, qvalid);
        }
        if constexpr (HAS_DO) f32_load_own<HD>(dO, p.dO.head(b, h) + (int64_t)qrow * p.dO.sl, c, p.D, qvalid);
#pragma unroll
        for (int i = 0; i < C; ++i) {
            if constexpr (HAS_G) {
                s4 = fmaf(g[i], o[i], s4);
                s7d = fmaf(g[i], to[i], s7d);
            }
            if constexpr (HAS_DO) s7d = fmaf(dO[i], o[i], s7d);
            dq[i] = 0.f;
            dtq[i] = 0.f;
        }
        s4 = sum8(s4);
        s7d = sum8(s7d);
    }
    const int64_t so = (int64_t)bh * p.Lr + qrow;
    const float lse2 = p.lse[so] * kLog2e;
    const float mu = HAS_G ? p.mu[so] : 0.f;
    if (c == 0) {
        p.lse2[so] = lse2;
        p.s4[so] = s4;
        p.s7d[so] = s7d;
    }
    const float sl2 = p.scale * kLog2e;
    for (int k0 = 0; k0 < p.Lk; k0 += kF32Tile) {
        workgroup_barrier();
        f32_fill_tile<HD>(sK, p.k.head(b, h), p.k.sl, k0, p.Lk, p.D, tid);
        f32_fill_tile<HD>(sV, p.v.head(b, h), p.v.sl, k0, p.Lk, p.D, tid);
        if constexpr (HAS_G) {
            f32_fill_tile<HD>(sTK, p.tk.head(b, h), p.tk.sl, k0, p.Lk, p.D, tid);
            f32_fill_tile<HD>(sTV, p.tv.head(b, h), p.tv.sl, k0, p.Lk, p.D, tid);
        }
        workgroup_barrier();
#pragma unroll 4
        for (int j = 0; j < kF32Tile; ++j) {
            const float s = sum8(f32_dot<HD>(q, sK, j, c));
            float pj = fast_exp2(fmaf(s, sl2, -lse2));
            if (k0 + j >= p.Lk) pj = 0.f;  // a zero-padded key: exp(-lse) may overflow
            float xy = 0.f;
            if constexpr (HAS_DO) xy += f32_dot<HD>(dO, sV, j, c);
            if constexpr (HAS_G) {
                xy += f32_dot<HD>(g, sTV, j, c);
                xy = sum8(xy);
                const float ts = sum8(f32_dot<HD>(tq, sK, j, c) + f32_dot<HD>(q, sTK, j, c));
                const float w = sum8(f32_dot<HD>(g, sV, j, c));
                const float nn = fmaf(ts, p.scale, -mu);
                const float dts = pj * (w - s4);
                const float ds = fmaf(dts, nn, pj * (xy - s7d));
                f32_axpy<HD>(dq, ds, sK, j, c);
                f32_axpy<HD>(dq, dts, sTK, j, c);
                f32_axpy<HD>(dtq, dts, sK, j, c);
            } else {
                xy = sum8(xy);
                f32_axpy<HD>(dq, pj * (xy - s7d), sK, j, c);
            }
        }
    }
    if (!qvalid) return;
    f32_store_own<HD>(p.dq.head(b, h) + (int64_t)qrow * p.dq.sl, dq, p.scale, c, p.D);
    if constexpr (HAS_G) f32_store_own<HD>(p.dtq.head(b, h) + (int64_t)qrow * p.dtq.sl, dtq, p.scale, c, p.D);
}

// ---------------------------------------------------------------------------------------------
// Column-owned backward: dK, dV (, dK_dot, dV_dot).  LDS: Q | [Q_dot | G] | [dO] tiles and the four
// statistics of the tile's rows.
template <int HD, bool HAS_DO, bool HAS_G>
__global__ __launch_bounds__(kF32Threads) void bwd_col_f32_kernel(const BwdParamsF32 p) {
    constexpr int NT = 1 + (HAS_G ? 2 : 0) + (HAS_DO ? 1 : 0);
    __shared__ __align__(16) float tiles[NT * kF32Tile * HD + 4 * kF32Tile];
    float* sQ = tiles;
    float* sTQ = tiles + kF32Tile * HD;
    float* sG = tiles + 2 * kF32Tile * HD;
    float* sDO = tiles + (HAS_G ? 3 : 1) * kF32Tile * HD;
    float* sStat = tiles + NT * kF32Tile * HD;  // lse2 | mu | s4 | s7d
    constexpr int C = HD / 8;
    const int tid = threadIdx.x;
    const int c = tid & 7;
    const int k_blocks = (p.Lk + kF32Owned - 1) / kF32Owned;
    const int bh = blockIdx.x / k_blocks, kb = blockIdx.x % k_blocks;
    const int b = bh / p.H, h = bh % p.H;
    const int krow = kb * kF32Owned + (tid >> 3);
    const bool kvalid = krow < p.Lk;

    float k[C], v[C], tk[C], tv[C], dk[C], dv[C], dtk[C], dtv[C];
    f32_load_own<HD>(k, p.k.head(b, h) + (int64_t)krow * p.k.sl, c, p.D, kvalid);
    f32_load_own<HD>(v, p.v.head(b, h) + (int64_t)krow * p.v.sl, c, p.D, kvalid);
    if constexpr (HAS_G) {
        f32_load_own<HD>(tk, p.tk.head(b, h) + (int64_t)krow * p.tk.sl, c, p.D, kvalid);
        f32_load_own<HD>(tv, p.tv.head(b, h) + (int64_t)krow * p.tv.sl, c, p.D, kvalid);
    }
#pragma unroll
    for (int i = 0; i < C; ++i) {
        dk[i] = 0.f;
        dv[i] = 0.f;
        dtk[i] = 0.f;
        dtv[i] = 0.f;
    }
    const float sl2 = p.scale * kLog2e;
    for (int q0 = 0; q0 < p.Lq; q0 += kF32Tile) {
        workgroup_barrier();
        f32_fill_tile<HD>(sQ, p.q.head(b, h), p.q.sl, q0, p.Lq, p.D, tid);
        if constexpr (HAS_G) {
            f32_fill_tile<HD>(sTQ, p.tq.head(b, h), p.tq.sl, q0, p.Lq, p.D, tid);
            f32_fill_tile<HD>(sG, p.dTO.head(b, h), p.dTO.sl, q0, p.Lq, p.D, tid);
        }
        if constexpr (HAS_DO) f32_fill_tile<HD>(sDO, p.dO.head(b, h), p.dO.sl, q0, p.Lq, p.D, tid);
        if (tid < 4 * kF32Tile) {
            const int which = tid / kF32Tile, r = tid % kF32Tile;
            const float* src = which == 0 ? p.lse2 : which == 1 ? p.mu : which == 2 ? p.s4 : p.s7d;
            // rows below Lr exist in every statistic; mu is absent without a cotangent on TO
            sStat[tid] = (which == 1 && !HAS_G) ? 0.f : src[(int64_t)bh * p.Lr + q0 + r];
        }
        workgroup_barrier();
#pragma unroll 4
        for (int i = 0; i < kF32Tile; ++i) {
            const float s = sum8(f32_dot<HD>(k, sQ, i, c));
            float pi = fast_exp2(fmaf(s, sl2, -sStat[i]));
            if (q0 + i >= p.Lq || !kvalid) pi = 0.f;  // padded query rows and padded keys contribute nothing
            float xy = 0.f;
            if constexpr (HAS_DO) xy += f32_dot<HD>(v, sDO, i, c);
            if constexpr (HAS_G) {
                xy += f32_dot<HD>(tv, sG, i, c);
                xy = sum8(xy);
                const float ts = sum8(f32_dot<HD>(k, sTQ, i, c) + f32_dot<HD>(tk, sQ, i, c));
                const float w = sum8(f32_dot<HD>(v, sG, i, c));
                const float nn = fmaf(ts, p.scale, -sStat[kF32Tile + i]);
                const float dts = pi * (w - sStat[2 * kF32Tile + i]);
                const float ds = fmaf(dts, nn, pi * (xy - sStat[3 * kF32Tile + i]));
                f32_axpy<HD>(dk, ds, sQ, i, c);
                f32_axpy<HD>(dk, dts, sTQ, i, c);
                f32_axpy<HD>(dtk, dts, sQ, i, c);
                f32_axpy<HD>(dv, pi * nn, sG, i, c);
                f32_axpy<HD>(dtv, pi, sG, i, c);
                if constexpr (HAS_DO) f32_axpy<HD>(dv, pi, sDO, i, c);
            } else {
                xy = sum8(xy);
                f32_axpy<HD>(dk, pi * (xy - sStat[3 * kF32Tile + i]), sQ, i, c);
                f32_axpy<HD>(dv, pi, sDO, i, c);
            }
        }
    }
    if (!kvalid) return;
    f32_store_own<HD>(p.dk.head(b, h) + (int64_t)krow * p.dk.sl, dk, p.scale, c, p.D);
    f32_store_own<HD>(p.dv.head(b, h) + (int64_t)krow * p.dv.sl, dv, 1.0f, c, p.D);
    if constexpr (HAS_G) {
        f32_store_own<HD>(p.dtk.head(b, h) + (int64_t)krow * p.dtk.sl, dtk, p.scale, c, p.D);
        f32_store_own<HD>(p.dtv.head(b, h) + (int64_t)krow * p.dtv.sl, dtv, 1.0f, c, p.D);
    }
}

}  // namespace sjvp
