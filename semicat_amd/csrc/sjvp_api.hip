// C ABI of the attention-JVP library (declared in include/sjvp.h): argument validation, kernel
// selection and launches.  No device memory is allocated or freed here and no state is kept.
#include "../../include/sjvp.h"

#include <hip/hip_runtime.h>
#include <math.h>

#include "sjvp_bwd.hpp"
#include "sjvp_bwd16.hpp"
#include "sjvp_bwd16x.hpp"
#include "sjvp_fwd.hpp"
#include "sjvp_fwd16.hpp"
#include "sjvp_rope.hpp"

using namespace sjvp;

namespace {

inline int round_up(int x, int m) { return (x + m - 1) / m * m; }

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

struct VecCheck {
    bool ok = true;
    void add(const void* p, const int64_t* s) {
        if (!p) return;
        ok = ok && aligned16(p) && (s[0] % 8 == 0) && (s[1] % 8 == 0) && (s[2] % 8 == 0);
    }
};

inline TensorView view(const void* p, const int64_t* s) {
    return TensorView{static_cast<const elem_t*>(p), s[0], s[1], s[2]};
}
inline OutView out_view(void* p, const int64_t* s) {
    return OutView{static_cast<elem_t*>(p), s[0], s[1], s[2]};
}

int check_common(int B, int H, int Lq, int Lk, int D, int dtype) {
    if (dtype != SJVP_BF16 && dtype != SJVP_FP16) return SJVP_ERR_DTYPE;
    if (B < 1 || H < 1 || Lq < 1 || Lk < 1) return SJVP_ERR_SHAPE;
    if (D < 16 || D > 128) return SJVP_ERR_HEAD_DIM;
    const int64_t blocks = (int64_t)B * H * ((int64_t)round_up(Lq > Lk ? Lq : Lk, 32) / 32);
    if (blocks > 0x7fffffffLL) return SJVP_ERR_SHAPE;
    return SJVP_OK;
}

template <typename K, typename... Extra>
int launch(K kernel, int grid, int smem_bytes, hipStream_t stream, const auto& params, int threads,
           Extra... extra) {
    if (smem_bytes > 64 * 1024) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                hipFuncAttributeMaxDynamicSharedMemorySize,
                                smem_bytes) != hipSuccess) {
            (void)hipGetLastError();
            return SJVP_ERR_LAUNCH;
        }
    }
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(threads), smem_bytes, stream, params, extra...);
    return hipGetLastError() == hipSuccess ? SJVP_OK : SJVP_ERR_LAUNCH;
}

template <typename K>
int launch(K kernel, int grid, int smem_bytes, hipStream_t stream, const auto& params) {
    return launch(kernel, grid, smem_bytes, stream, params, kThreads);
}

// Ring depths (stages of 32 rows in flight) of the 16-wide kernels per head-dimension class, sized
// to the LDS a workgroup may take when several of them are to share the 160 KB of a CU.
template <int HD>
struct Ring {
    static constexpr int fwd16 = 2;                    // with tangents (four slabs per stage)
    static constexpr int fwd16_primal = 4;             // primal only (two slabs per stage)
    static constexpr int fused = 3;
    static constexpr int pair = HD == 128 ? 2 : 3;     // row-owned / column-owned backward pair
};

// key-axis length from which the forward takes two stages per barrier
constexpr int kFwdPairedFrom = 256;

// 32-wide forward for inputs of any alignment (register-staged copies, one stage in LDS)
template <typename T, int HD>
int fwd_hd(const FwdParams& p, int grid, bool jvp, hipStream_t stream) {
    if (jvp) return launch(fwd_kernel<T, HD, true>, grid, FwdSmem<HD, true>::bytes, stream, p);
    return launch(fwd_kernel<T, HD, false>, grid, FwdSmem<HD, false>::bytes, stream, p);
}

template <typename T, int HD>
int fwd16_hd(const FwdParams& p, int grid, bool jvp, hipStream_t stream) {
    // two stages in flight and at most 128 registers: two workgroups (sixteen waves) share a CU, which
    // overlaps one's copies with the other's arithmetic; HD = 128 needs the whole register budget
    constexpr int R = Ring<HD>::fwd16;
    constexpr int RP = Ring<HD>::fwd16_primal;
    constexpr int OCC = HD == 128 ? 2 : 4;
    if (p.Lk >= kFwdPairedFrom) {
        // long key axes: two stages per barrier over a ring of four slots in the same LDS footprint
        if (jvp)
            return launch(fwd16_kernel<T, HD, 4, true, OCC, 2>, grid, Fwd16Smem<HD, 4, true, 2>::bytes, stream,
                          p, kThreads16);
        return launch(fwd16_kernel<T, HD, 4, false, OCC, 2>, grid, Fwd16Smem<HD, 4, false, 2>::bytes, stream,
                      p, kThreads16);
    }
    if (jvp)
        return launch(fwd16_kernel<T, HD, R, true, OCC>, grid, Fwd16Smem<HD, R, true>::bytes, stream, p,
                      kThreads16);
    return launch(fwd16_kernel<T, HD, RP, false, OCC>, grid, Fwd16Smem<HD, RP, false>::bytes, stream, p,
                  kThreads16);
}

template <typename T>
int fwd_dtype(const FwdParams& p, int grid, bool jvp, hipStream_t stream) {
    // LDS-DMA streaming needs 16-byte aligned rows; anything else takes the register-staged path
    if (p.vec) {
        if (p.D <= 32) return fwd16_hd<T, 32>(p, grid, jvp, stream);
        if (p.D <= 64) return fwd16_hd<T, 64>(p, grid, jvp, stream);
        return fwd16_hd<T, 128>(p, grid, jvp, stream);
    }
    if (p.D <= 32) return fwd_hd<T, 32>(p, grid, jvp, stream);
    if (p.D <= 64) return fwd_hd<T, 64>(p, grid, jvp, stream);
    return fwd_hd<T, 128>(p, grid, jvp, stream);
}

template <typename T, int HD, bool HAS_DO, bool HAS_G, bool DMA>
int bwd_mode(const BwdParams& p, int BH, int parts, hipStream_t stream) {
    if constexpr (DMA) {
        if constexpr (HD <= 64) {
            // short key axis: one launch, one workgroup per (batch, head)
            if (parts == SJVP_BWD_ALL && p.Lk <= kOwned16) {
                constexpr int FR = Ring<HD>::fused;
                return launch(bwd_fused16_kernel<T, HD, FR, HAS_DO, HAS_G>, BH,
                              Fused16Smem<HD, FR, HAS_DO, HAS_G>::bytes, stream, p, kThreads16);
            }
        }
        // 16-wide pair: the row-owned kernel first (besides dQ, dQ_dot it leaves the row sums in the
        // workspace), then the column-owned one; workgroups of four waves own 64 positions
        constexpr int XR = Ring<HD>::pair;
        int rc = SJVP_OK;
        if (parts & SJVP_BWD_ROW)
            rc = launch(bwd_row16_kernel<T, HD, XR, HAS_DO, HAS_G, (HD == 128 ? 2 : 3)>,
                        BH * (p.Lr / kXOwned16), Row16Smem<HD, XR, HAS_G>::bytes, stream, p, kXThreads16);
        if (rc != SJVP_OK || !(parts & SJVP_BWD_COL)) return rc;
        const int grid = BH * ((p.Lk + kXOwned16 - 1) / kXOwned16);
        using CS = Col16Smem<HD, XR, HAS_DO, HAS_G>;
        if constexpr (HD == 128) {
            // two launches, each accumulating two of the four gradients (register budget)
            rc = launch(bwd_col16_kernel<T, HD, XR, HAS_DO, HAS_G, 1, 2>, grid, CS::bytes, stream, p, kXThreads16);
            if (rc != SJVP_OK) return rc;
            return launch(bwd_col16_kernel<T, HD, XR, HAS_DO, HAS_G, 2, 2>, grid, CS::bytes, stream, p, kXThreads16);
        } else {
            return launch(bwd_col16_kernel<T, HD, XR, HAS_DO, HAS_G, 3, 2>, grid, CS::bytes, stream, p, kXThreads16);
        }
    } else {
        // 32-wide pair for inputs of any alignment, same order
        int rc = SJVP_OK;
        if (parts & SJVP_BWD_ROW)
            rc = launch(bwd_row_kernel<T, HD, HAS_DO, HAS_G>, BH * p.q_blocks, RowSmem<HD, HAS_G>::bytes, stream, p);
        if (rc != SJVP_OK || !(parts & SJVP_BWD_COL)) return rc;
        const int col_grid = BH * p.k_blocks;
        using SM = ColSmem<HD, HAS_DO, HAS_G>;
        if constexpr (HD == 128) {
            // two launches, each accumulating half of the head dimension (register budget)
            rc = launch(bwd_col_kernel<T, HD, HAS_DO, HAS_G, true, true, 0, 2>, col_grid, SM::bytes, stream, p);
            if (rc != SJVP_OK) return rc;
            return launch(bwd_col_kernel<T, HD, HAS_DO, HAS_G, true, true, 2, 2>, col_grid, SM::bytes, stream, p);
        } else {
            return launch(bwd_col_kernel<T, HD, HAS_DO, HAS_G, true, true, 0, HD / 32>, col_grid, SM::bytes,
                          stream, p);
        }
    }
}

template <typename T, int HD, bool DMA>
int bwd_hd(const BwdParams& p, int BH, bool has_do, bool has_g, int parts, hipStream_t stream) {
    if (has_do && has_g) return bwd_mode<T, HD, true, true, DMA>(p, BH, parts, stream);
    if (has_g) return bwd_mode<T, HD, false, true, DMA>(p, BH, parts, stream);
    return bwd_mode<T, HD, true, false, DMA>(p, BH, parts, stream);
}

template <typename T>
int bwd_dtype(const BwdParams& p, int BH, bool has_do, bool has_g, int parts, hipStream_t stream) {
    if (p.vec) {
        if (p.D <= 32) return bwd_hd<T, 32, true>(p, BH, has_do, has_g, parts, stream);
        if (p.D <= 64) return bwd_hd<T, 64, true>(p, BH, has_do, has_g, parts, stream);
        return bwd_hd<T, 128, true>(p, BH, has_do, has_g, parts, stream);
    }
    if (p.D <= 32) return bwd_hd<T, 32, false>(p, BH, has_do, has_g, parts, stream);
    if (p.D <= 64) return bwd_hd<T, 64, false>(p, BH, has_do, has_g, parts, stream);
    return bwd_hd<T, 128, false>(p, BH, has_do, has_g, parts, stream);
}

}  // namespace

extern "C" {

int sjvp_fwd(const void* q, const void* k, const void* v, const void* tq, const void* tk,
             const void* tv, void* o, void* to, float* lse, float* mu, float* li, int B, int H,
             int Lq, int Lk, int D, const int64_t* strides, float scale, int dtype, void* stream) {
    if (!q || !k || !v || !o || !lse || !strides) return SJVP_ERR_NULL;
    const bool jvp = tq || tk || tv || to || mu;
    if (jvp && (!tq || !tk || !tv || !to || !mu)) return SJVP_ERR_NULL;
    int rc = check_common(B, H, Lq, Lk, D, dtype);
    if (rc != SJVP_OK) return rc;

    const void* ptrs[SJVP_F_COUNT] = {q, k, v, tq, tk, tv, o, to};
    VecCheck vc;
    for (int i = 0; i < SJVP_F_COUNT; ++i) vc.add(ptrs[i], strides + 3 * i);

    FwdParams p{};
    p.q = view(q, strides + 3 * SJVP_F_Q);
    p.k = view(k, strides + 3 * SJVP_F_K);
    p.v = view(v, strides + 3 * SJVP_F_V);
    if (jvp) {
        p.tq = view(tq, strides + 3 * SJVP_F_TQ);
        p.tk = view(tk, strides + 3 * SJVP_F_TK);
        p.tv = view(tv, strides + 3 * SJVP_F_TV);
        p.to = out_view(to, strides + 3 * SJVP_F_TO);
    }
    p.o = out_view(o, strides + 3 * SJVP_F_O);
    p.lse = lse;
    p.mu = mu;
    p.li = li;
    p.H = H;
    p.Lq = Lq;
    p.Lk = Lk;
    p.D = D;
    p.Lr = round_up(Lq, 128);
    p.q_blocks = p.Lr / kOwned;  // covers every statistic row below Lr
    p.scale = scale > 0.f ? scale : 1.0f / sqrtf((float)D);
    p.vec = (vc.ok && D % 8 == 0) ? 1 : 0;

    const int grid = B * H * p.q_blocks;
    hipStream_t s = static_cast<hipStream_t>(stream);
    return dtype == SJVP_BF16 ? fwd_dtype<Bf16>(p, grid, jvp, s) : fwd_dtype<Fp16>(p, grid, jvp, s);
}

size_t sjvp_bwd_workspace_bytes(int B, int H, int Lq, int Lk, int D, int dtype) {
    (void)Lk;
    (void)D;
    (void)dtype;
    if (B < 1 || H < 1 || Lq < 1) return 0;
    return (size_t)3 * (size_t)B * (size_t)H * (size_t)round_up(Lq, 128) * sizeof(float);
}

int sjvp_bwd(const void* q, const void* k, const void* v, const void* tq, const void* tk,
             const void* tv, const void* o, const void* to, const void* dO, const void* dTO,
             const float* lse, const float* mu, void* dq, void* dk, void* dv, void* dtq, void* dtk,
             void* dtv, void* workspace, size_t workspace_bytes, int B, int H, int Lq, int Lk, int D,
             const int64_t* strides, float scale, int dtype, void* stream) {
    return sjvp_bwd_parts(SJVP_BWD_ALL, q, k, v, tq, tk, tv, o, to, dO, dTO, lse, mu, dq, dk, dv, dtq, dtk,
                          dtv, workspace, workspace_bytes, B, H, Lq, Lk, D, strides, scale, dtype, stream);
}

int sjvp_bwd_parts(int parts, const void* q, const void* k, const void* v, const void* tq,
                   const void* tk, const void* tv, const void* o, const void* to, const void* dO,
                   const void* dTO, const float* lse, const float* mu, void* dq, void* dk, void* dv,
                   void* dtq, void* dtk, void* dtv, void* workspace, size_t workspace_bytes, int B,
                   int H, int Lq, int Lk, int D, const int64_t* strides, float scale, int dtype,
                   void* stream) {
    if (parts < SJVP_BWD_ROW || parts > SJVP_BWD_ALL) return SJVP_ERR_PARTS;
    if (!dO && !dTO) return SJVP_ERR_COTANGENT;
    const bool has_do = dO != nullptr, has_g = dTO != nullptr;
    if (!q || !k || !v || !o || !lse || !dq || !dk || !dv || !strides) return SJVP_ERR_NULL;
    if (has_g && (!tq || !tk || !tv || !to || !mu || !dtq || !dtk || !dtv)) return SJVP_ERR_NULL;
    int rc = check_common(B, H, Lq, Lk, D, dtype);
    if (rc != SJVP_OK) return rc;
    if (!workspace || workspace_bytes < sjvp_bwd_workspace_bytes(B, H, Lq, Lk, D, dtype) ||
        (reinterpret_cast<uintptr_t>(workspace) & 3u))
        return SJVP_ERR_WORKSPACE;

    const void* ptrs[SJVP_B_COUNT] = {q, k, v, has_g ? tq : nullptr, has_g ? tk : nullptr,
                                      has_g ? tv : nullptr, o, has_g ? to : nullptr, dO, dTO, dq, dk,
                                      dv, has_g ? dtq : nullptr, has_g ? dtk : nullptr,
                                      has_g ? dtv : nullptr};
    VecCheck vc;
    for (int i = 0; i < SJVP_B_COUNT; ++i) vc.add(ptrs[i], strides + 3 * i);

    BwdParams p{};
    p.q = view(q, strides + 3 * SJVP_B_Q);
    p.k = view(k, strides + 3 * SJVP_B_K);
    p.v = view(v, strides + 3 * SJVP_B_V);
    p.o = view(o, strides + 3 * SJVP_B_O);
    if (has_do) p.dO = view(dO, strides + 3 * SJVP_B_DO);
    p.dq = out_view(dq, strides + 3 * SJVP_B_DQ);
    p.dk = out_view(dk, strides + 3 * SJVP_B_DK);
    p.dv = out_view(dv, strides + 3 * SJVP_B_DV);
    if (has_g) {
        p.tq = view(tq, strides + 3 * SJVP_B_TQ);
        p.tk = view(tk, strides + 3 * SJVP_B_TK);
        p.tv = view(tv, strides + 3 * SJVP_B_TV);
        p.to = view(to, strides + 3 * SJVP_B_TO);
        p.dTO = view(dTO, strides + 3 * SJVP_B_DTO);
        p.dtq = out_view(dtq, strides + 3 * SJVP_B_DTQ);
        p.dtk = out_view(dtk, strides + 3 * SJVP_B_DTK);
        p.dtv = out_view(dtv, strides + 3 * SJVP_B_DTV);
    }
    p.lse = lse;
    p.mu = mu;
    p.H = H;
    p.Lq = Lq;
    p.Lk = Lk;
    p.D = D;
    p.Lr = round_up(Lq, 128);
    p.q_blocks = p.Lr / kOwned;
    p.k_blocks = round_up(Lk, kOwned) / kOwned;
    p.lse2 = static_cast<float*>(workspace);
    p.s4 = p.lse2 + (size_t)B * H * p.Lr;
    p.s7d = p.s4 + (size_t)B * H * p.Lr;
    p.scale = scale > 0.f ? scale : 1.0f / sqrtf((float)D);
    p.vec = (vc.ok && D % 8 == 0) ? 1 : 0;

    hipStream_t s = static_cast<hipStream_t>(stream);
    return dtype == SJVP_BF16 ? bwd_dtype<Bf16>(p, B * H, has_do, has_g, parts, s)
                              : bwd_dtype<Fp16>(p, B * H, has_do, has_g, parts, s);
}

int sjvp_rope(int n, const void* const* x, void* const* y, const int64_t* strides, const float* cos,
              const float* sin, int64_t cs_stride, int B, int H, int L, int D, int rot_dim, int in_dtype,
              int out_dtype, int inverse, void* stream) {
    if (!x || !y || !strides || !cos || !sin) return SJVP_ERR_NULL;
    if (n < 1 || n > kRopeMaxTensors) return SJVP_ERR_ROTARY;
    if (B < 1 || H < 1 || L < 1 || D < 1) return SJVP_ERR_SHAPE;
    if (rot_dim < 2 || rot_dim > D || (rot_dim & 1)) return SJVP_ERR_ROTARY;
    auto known = [](int d) { return d == SJVP_BF16 || d == SJVP_FP16 || d == SJVP_FP32; };
    if (!known(in_dtype) || !known(out_dtype)) return SJVP_ERR_DTYPE;
    if (in_dtype != SJVP_FP32 && out_dtype != SJVP_FP32 && in_dtype != out_dtype) return SJVP_ERR_ROTARY;
    const int half = rot_dim / 2;
    const int in_bytes = in_dtype == SJVP_FP32 ? 4 : 2, out_bytes = out_dtype == SJVP_FP32 ? 4 : 2;

    RopeParams p;
    // eight columns per thread need every row start and the second half of a pair 16-byte aligned
    bool vec = half % 8 == 0 && (D - rot_dim) % 8 == 0 && aligned16(cos) && aligned16(sin) && cs_stride % 4 == 0;
    for (int i = 0; i < kRopeMaxTensors; ++i) {
        const int j = i < n ? i : 0;  // unused slots repeat tensor 0 (never dereferenced: grid.y = n)
        if (!x[j] || !y[j]) return SJVP_ERR_NULL;
        p.x[i] = x[j];
        p.y[i] = y[j];
        for (int d = 0; d < 3; ++d) {
            p.xs[i][d] = strides[6 * j + d];
            p.ys[i][d] = strides[6 * j + 3 + d];
            vec = vec && (p.xs[i][d] * in_bytes) % 16 == 0 && (p.ys[i][d] * out_bytes) % 16 == 0;
        }
        vec = vec && aligned16(x[j]) && aligned16(y[j]);
    }
    p.cos = cos;
    p.sin = sin;
    p.cs = cs_stride;
    p.H = H;
    p.L = L;
    p.D = D;
    p.half = half;
    const int w = vec ? 8 : 1;
    p.units = half / w + (D - rot_dim) / w;
    p.total = (int64_t)B * H * L * p.units;
    p.sign = inverse ? -1.0f : 1.0f;
    p.h_fast = p.ys[0][1] < p.ys[0][2] ? 1 : 0;  // follow the output's memory order
    const int64_t blocks = (p.total + kRopeThreads - 1) / kRopeThreads;
    if (blocks > 0x7fffffffLL) return SJVP_ERR_SHAPE;

    auto go = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, dim3((unsigned)blocks, (unsigned)n), dim3(kRopeThreads), 0,
                           static_cast<hipStream_t>(stream), p);
        return hipGetLastError() == hipSuccess ? SJVP_OK : SJVP_ERR_LAUNCH;
    };
    auto by_out = [&](auto in_tag) {
        using IN = decltype(in_tag);
        if (out_dtype == SJVP_FP32) return vec ? go(rope_kernel<IN, F32, true>) : go(rope_kernel<IN, F32, false>);
        if (out_dtype == SJVP_BF16) return vec ? go(rope_kernel<IN, Bf16, true>) : go(rope_kernel<IN, Bf16, false>);
        return vec ? go(rope_kernel<IN, Fp16, true>) : go(rope_kernel<IN, Fp16, false>);
    };
    if (in_dtype == SJVP_FP32) return by_out(F32{});
    if (in_dtype == SJVP_BF16) return by_out(Bf16{});
    return by_out(Fp16{});
}

const char* sjvp_strerror(int status) {
    switch (status) {
        case SJVP_OK: return "ok";
        case SJVP_ERR_NULL: return "a required pointer is NULL";
        case SJVP_ERR_SHAPE: return "B, H, Lq and Lk must be >= 1 and within the index range";
        case SJVP_ERR_HEAD_DIM: return "head dimension must satisfy 16 <= D <= 128";
        case SJVP_ERR_DTYPE: return "dtype must be SJVP_BF16 or SJVP_FP16";
        case SJVP_ERR_WORKSPACE: return "workspace is NULL, misaligned or smaller than sjvp_bwd_workspace_bytes()";
        case SJVP_ERR_LAUNCH: return "HIP kernel launch failed";
        case SJVP_ERR_COTANGENT: return "at least one of dO and dTO must be given";
        case SJVP_ERR_PARTS: return "parts must be SJVP_BWD_ROW, SJVP_BWD_COL or SJVP_BWD_ALL";
        case SJVP_ERR_ROTARY: return "sjvp_rope: n must be 1..4, rot_dim even and 2 <= rot_dim <= D, and bf16 / fp16 must not be mixed";
        default: return "unknown sjvp status";
    }
}

int sjvp_version(void) { return SJVP_VERSION; }

}  // extern "C"
