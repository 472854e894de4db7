// C ABI of the attention-JVP library (declared in include/sjvp.h): argument validation, kernel
// selection and launches.  No device memory is allocated or freed here; the only state kept is the
// per-device address of the static scratch array that sjvp_bwd_noalloc() works in.
#include "../../include/sjvp.h"

#include <hip/hip_runtime.h>
#include <math.h>

#include <atomic>
#include <mutex>

#include "sjvp_launch.hpp"
#include "sjvp_rope.hpp"
#include "sjvp_w16.hpp"

using namespace sjvp;

namespace {

inline int round_up(int x, int m) { return (x + m - 1) / m * m; }

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Whether every row of every tensor starts on a 16-byte boundary (`unit` elements of the tensors'
// storage type make 16 bytes: 8 for 16-bit storage, 4 for fp32).
struct VecCheck {
    int unit = 8;
    bool ok = true;
    void add(const void* p, const int64_t* s) {
        if (!p) return;
        ok = ok && aligned16(p) && (s[0] % unit == 0) && (s[1] % unit == 0) && (s[2] % unit == 0);
    }
};

// Views of the 16-bit kernels.  `m` = 2 for fp32 storage: the kernels address rows in 2-byte units.
inline TensorView view(const void* p, const int64_t* s, int m = 1) {
    return TensorView{static_cast<const elem_t*>(p), m * s[0], m * s[1], m * s[2]};
}
inline OutView out_view(void* p, const int64_t* s, int m = 1) {
    return OutView{static_cast<elem_t*>(p), m * s[0], m * s[1], m * s[2]};
}

inline F32In view32(const void* p, const int64_t* s) {
    return F32In{static_cast<const float*>(p), s[0], s[1], s[2]};
}
inline F32Out out_view32(void* p, const int64_t* s) { return F32Out{static_cast<float*>(p), s[0], s[1], s[2]}; }

int check_common(int B, int H, int Lq, int Lk, int D, int dtype, float scale) {
    if (dtype < SJVP_BF16 || dtype > SJVP_FP32_BF16) return SJVP_ERR_DTYPE;
    if (B < 1 || H < 1 || Lq < 1 || Lk < 1) return SJVP_ERR_SHAPE;
    if (D < 16 || D > 128) return SJVP_ERR_HEAD_DIM;
    // the finest launch takes one workgroup per 32 rows of the longer axis rounded up to 128 (the
    // statistic rows): that grid, in 64 bits, has to fit the 31 bits of a launch dimension
    const int64_t longer = Lq > Lk ? Lq : Lk;
    if (longer > (1LL << 30)) return SJVP_ERR_SHAPE;  // keeps the 32-bit round-ups below exact
    const int64_t blocks = (int64_t)B * H * ((longer + 127) / 128 * 4);
    if (blocks > 0x7fffffffLL) return SJVP_ERR_SHAPE;
    if (!(scale >= 0.f) || isinf(scale)) return SJVP_ERR_SCALE;  // 0 selects the default; NaN fails too
    return SJVP_OK;
}

// The folded rotary embedding serves the shapes of the single-workgroup kernels: head dimension 64
// rotated as a whole, a key axis of at most 128, 16-bit tensors with 16-byte aligned rows.
int check_rotary(const float* cos, const float* sin, int64_t cs_stride, int table_rows, int Lq, int Lk, int D,
                 int dtype) {
    if (!cos || !sin) return SJVP_ERR_NULL;
    if (dtype != SJVP_BF16 && dtype != SJVP_FP16) return SJVP_ERR_ROTARY;
    if (D != 64 || Lk > kOwned16 || table_rows < (Lq > Lk ? Lq : Lk)) return SJVP_ERR_ROTARY;
    if (!aligned16(cos) || !aligned16(sin) || cs_stride % 4 != 0 || cs_stride < 32) return SJVP_ERR_ROTARY;
    return SJVP_OK;
}

inline float resolve_scale(float scale, int D) { return scale > 0.f ? scale : 1.0f / sqrtf((float)D); }

constexpr int kMaxDevices = 64;

// Process-wide setting of sjvp_set_row_sum_repair().
std::atomic<int> g_row_sum_repair{SJVP_REPAIR_AUTO};

// Compute units of the current device (looked up once per device).
int compute_units() {
    static std::atomic<int> cached[kMaxDevices] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 256;
    int n = cached[dev].load(std::memory_order_relaxed);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n < 1) n = 256;
        cached[dev].store(n, std::memory_order_relaxed);
    }
    return n;
}

// Kernel selection of the backward: the single launch where it fits, else the row + column pair.
template <typename T>
int bwd_select(const BwdParams& p, int BH, bool has_do, bool has_g, int parts, hipStream_t stream) {
    if (!p.vec) return bwd_pair_any<T>(p, BH, has_do, has_g, parts, stream);
    // the single launch takes its row sums from the 16-bit outputs and cannot repair them: a caller who
    // asked for the repair everywhere gets the pair (the folded rotation exists in the single launch only)
    const bool single = parts == SJVP_BWD_ALL && p.Lk <= kOwned16 && p.D <= 64;
    // The single launch is one workgroup per (batch, head) pair walking the whole query axis: a few
    // pairs with a long query axis would leave most of the chip idle, while the row-owned launch of the
    // pair spreads the queries over Lq / 64 workgroups per pair.
    const bool few_long = 2 * BH <= compute_units() && p.Lq >= 4 * kOwned16 && !p.rope.cos;
    if (single && !few_long && (p.rowfix != SJVP_REPAIR_ALWAYS || p.rope.cos))
        return bwd_fused<T>(p, BH, has_do, has_g, stream);
    return bwd_pair_vec<T>(p, BH, has_do, has_g, parts, stream);
}

// The backward's tensors as they arrive through the C ABI.
struct BwdTensors {
    const void *q, *k, *v, *tq, *tk, *tv, *o, *to, *dO, *dTO;
    const float *lse, *mu;
    void *dq, *dk, *dv, *dtq, *dtk, *dtv;
};

int check_bwd(int parts, const BwdTensors& t, int B, int H, int Lq, int Lk, int D, const int64_t* strides,
              float scale, int dtype) {
    if (parts < SJVP_BWD_ROW || parts > SJVP_BWD_ALL) return SJVP_ERR_PARTS;
    if (!t.dO && !t.dTO) return SJVP_ERR_COTANGENT;
    if (!t.q || !t.k || !t.v || !t.o || !t.lse || !t.dq || !t.dk || !t.dv || !strides) return SJVP_ERR_NULL;
    if (t.dTO && (!t.tq || !t.tk || !t.tv || !t.to || !t.mu || !t.dtq || !t.dtk || !t.dtv)) return SJVP_ERR_NULL;
    return check_common(B, H, Lq, Lk, D, dtype, scale);
}

// Launches of the backward on a validated problem; `ws` holds sjvp_bwd_workspace_bytes(): 3 * B * H * Lr
// floats and, behind them, B * H * Lr / 64 flags.
int run_bwd(int parts, const BwdTensors& t, float* ws, int B, int H, int Lq, int Lk, int D,
            const int64_t* strides, float scale, int dtype, void* stream,
            RopeTables rope = RopeTables{nullptr, nullptr, 0, 0}) {
    const bool has_do = t.dO != nullptr, has_g = t.dTO != nullptr;
    if (dtype == SJVP_FP32) {
        BwdParamsF32 f{};
        f.q = view32(t.q, strides + 3 * SJVP_B_Q);
        f.k = view32(t.k, strides + 3 * SJVP_B_K);
        f.v = view32(t.v, strides + 3 * SJVP_B_V);
        f.o = view32(t.o, strides + 3 * SJVP_B_O);
        if (has_do) f.dO = view32(t.dO, strides + 3 * SJVP_B_DO);
        f.dq = out_view32(t.dq, strides + 3 * SJVP_B_DQ);
        f.dk = out_view32(t.dk, strides + 3 * SJVP_B_DK);
        f.dv = out_view32(t.dv, strides + 3 * SJVP_B_DV);
        if (has_g) {
            f.tq = view32(t.tq, strides + 3 * SJVP_B_TQ);
            f.tk = view32(t.tk, strides + 3 * SJVP_B_TK);
            f.tv = view32(t.tv, strides + 3 * SJVP_B_TV);
            f.to = view32(t.to, strides + 3 * SJVP_B_TO);
            f.dTO = view32(t.dTO, strides + 3 * SJVP_B_DTO);
            f.dtq = out_view32(t.dtq, strides + 3 * SJVP_B_DTQ);
            f.dtk = out_view32(t.dtk, strides + 3 * SJVP_B_DTK);
            f.dtv = out_view32(t.dtv, strides + 3 * SJVP_B_DTV);
        }
        f.lse = t.lse;
        f.mu = t.mu;
        f.H = H;
        f.Lq = Lq;
        f.Lk = Lk;
        f.D = D;
        f.Lr = round_up(Lq, 128);
        f.lse2 = ws;
        f.s4 = f.lse2 + (size_t)B * H * f.Lr;
        f.s7d = f.s4 + (size_t)B * H * f.Lr;
        f.scale = resolve_scale(scale, D);
        return bwd_f32(f, B * H, has_do, has_g, parts, static_cast<hipStream_t>(stream));
    }
    const void* ptrs[SJVP_B_COUNT] = {t.q, t.k, t.v, has_g ? t.tq : nullptr, has_g ? t.tk : nullptr,
                                      has_g ? t.tv : nullptr, t.o, has_g ? t.to : nullptr, t.dO, t.dTO,
                                      t.dq, t.dk, t.dv, has_g ? t.dtq : nullptr, has_g ? t.dtk : nullptr,
                                      has_g ? t.dtv : nullptr};
    const bool f32io = dtype == SJVP_FP32_BF16;
    const int m = f32io ? 2 : 1;
    VecCheck vc;
    vc.unit = f32io ? 4 : 8;
    for (int i = 0; i < SJVP_B_COUNT; ++i) vc.add(ptrs[i], strides + 3 * i);

    BwdParams p{};
    p.q = view(t.q, strides + 3 * SJVP_B_Q, m);
    p.k = view(t.k, strides + 3 * SJVP_B_K, m);
    p.v = view(t.v, strides + 3 * SJVP_B_V, m);
    p.o = view(t.o, strides + 3 * SJVP_B_O, m);
    if (has_do) p.dO = view(t.dO, strides + 3 * SJVP_B_DO, m);
    p.dq = out_view(t.dq, strides + 3 * SJVP_B_DQ, m);
    p.dk = out_view(t.dk, strides + 3 * SJVP_B_DK, m);
    p.dv = out_view(t.dv, strides + 3 * SJVP_B_DV, m);
    if (has_g) {
        p.tq = view(t.tq, strides + 3 * SJVP_B_TQ, m);
        p.tk = view(t.tk, strides + 3 * SJVP_B_TK, m);
        p.tv = view(t.tv, strides + 3 * SJVP_B_TV, m);
        p.to = view(t.to, strides + 3 * SJVP_B_TO, m);
        p.dTO = view(t.dTO, strides + 3 * SJVP_B_DTO, m);
        p.dtq = out_view(t.dtq, strides + 3 * SJVP_B_DTQ, m);
        p.dtk = out_view(t.dtk, strides + 3 * SJVP_B_DTK, m);
        p.dtv = out_view(t.dtv, strides + 3 * SJVP_B_DTV, m);
    }
    p.lse = t.lse;
    p.mu = t.mu;
    p.H = H;
    p.Lq = Lq;
    p.Lk = Lk;
    p.D = D;
    p.Lr = round_up(Lq, 128);
    p.q_blocks = p.Lr / kOwned;
    p.k_blocks = round_up(Lk, kOwned) / kOwned;
    p.lse2 = ws;
    p.s4 = p.lse2 + (size_t)B * H * p.Lr;
    p.s7d = p.s4 + (size_t)B * H * p.Lr;
    p.flags = reinterpret_cast<int*>(p.s7d + (size_t)B * H * p.Lr);  // one per 64 statistic rows
    p.scale = resolve_scale(scale, D);
    p.vec = (vc.ok && D % 8 == 0) ? 1 : 0;
    p.rope = rope;
    {
        auto same = [&](int a, int b) {
            return !ptrs[b] || (strides[3 * a] == strides[3 * b] && strides[3 * a + 1] == strides[3 * b + 1] &&
                                strides[3 * a + 2] == strides[3 * b + 2]);
        };
        auto fits = [&](int a, int rows) {
            return strides[3 * a + 2] >= 0 && (int64_t)rows * strides[3 * a + 2] + D < (int64_t(1) << 29);
        };
        p.q_side_uniform = !f32io && fits(SJVP_B_Q, p.Lr) && same(SJVP_B_Q, SJVP_B_TQ) && same(SJVP_B_Q, SJVP_B_O) &&
                           same(SJVP_B_Q, SJVP_B_TO) && (!has_do || same(SJVP_B_Q, SJVP_B_DO)) &&
                           (!has_g || same(SJVP_B_Q, SJVP_B_DTO));
        p.k_side_uniform = !f32io && fits(SJVP_B_K, round_up(Lk, kOwned)) && same(SJVP_B_K, SJVP_B_V) &&
                           same(SJVP_B_K, SJVP_B_TK) && same(SJVP_B_K, SJVP_B_TV);
    }
    p.rowfix = g_row_sum_repair.load(std::memory_order_relaxed);
    p.rowfix_tau = dtype == SJVP_FP16 ? 0x1p-11f : 0x1p-8f;  // unit roundoff of the tiles' 16-bit format
    if (rope.cos && (!p.vec || parts != SJVP_BWD_ALL)) return SJVP_ERR_ROTARY;  // the single launch only

    hipStream_t s = static_cast<hipStream_t>(stream);
    if (f32io) return bwd_f32io(p, B * H, has_do, has_g, parts, s);
    return dtype == SJVP_BF16 ? bwd_select<Bf16>(p, B * H, has_do, has_g, parts, s)
                              : bwd_select<Fp16>(p, B * H, has_do, has_g, parts, s);
}

// Scratch of sjvp_bwd_noalloc(): the backward's workspace (lse in log2 units and the two row sums,
// 3 floats per statistic row, and one flag per 64 rows) for up to SJVP_NOALLOC_MAX_ROWS rows, resident in every GPU the library
// runs on from the moment its code is loaded until the process ends.  In host code the array's name
// is only a handle for hipGetSymbolAddress(); its device address differs from GPU to GPU and is
// looked up once per device, with that device current.
static __device__ __align__(256) __attribute__((used)) float scratch[3 * (size_t)SJVP_NOALLOC_MAX_ROWS +
                                                                    SJVP_NOALLOC_MAX_ROWS / 64];

std::mutex g_scratch_mutex;
float* g_scratch_ptr[kMaxDevices] = {};

int fwd_impl(const void* q, const void* k, const void* v, const void* tq, const void* tk, const void* tv,
             void* o, void* to, float* lse, float* mu, float* li, int B, int H, int Lq, int Lk, int D,
             const int64_t* strides, float scale, int dtype, RopeTables rope, void* stream);

int static_scratch(float** out) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return SJVP_ERR_SCRATCH;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* ptr = nullptr;
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) return SJVP_ERR_SCRATCH;
        g_scratch_ptr[dev] = static_cast<float*>(ptr);
    }
    *out = g_scratch_ptr[dev];
    return SJVP_OK;
}

}  // namespace

extern "C" {

int sjvp_fwd(const void* q, const void* k, const void* v, const void* tq, const void* tk,
             const void* tv, void* o, void* to, float* lse, float* mu, float* li, int B, int H,
             int Lq, int Lk, int D, const int64_t* strides, float scale, int dtype, void* stream) {
    return fwd_impl(q, k, v, tq, tk, tv, o, to, lse, mu, li, B, H, Lq, Lk, D, strides, scale, dtype,
                    RopeTables{nullptr, nullptr, 0, 0}, stream);
}

int sjvp_fwd_rotary(const void* q, const void* k, const void* v, const void* tq, const void* tk,
                    const void* tv, void* o, void* to, float* lse, float* mu, float* li, int B, int H,
                    int Lq, int Lk, int D, const int64_t* strides, float scale, int dtype,
                    const float* cos, const float* sin, int64_t cs_stride, int table_rows, void* stream) {
    const int rc = check_rotary(cos, sin, cs_stride, table_rows, Lq, Lk, D, dtype);
    if (rc != SJVP_OK) return rc;
    return fwd_impl(q, k, v, tq, tk, tv, o, to, lse, mu, li, B, H, Lq, Lk, D, strides, scale, dtype,
                    RopeTables{cos, sin, cs_stride, table_rows}, stream);
}

}  // extern "C"

namespace {

int fwd_impl(const void* q, const void* k, const void* v, const void* tq, const void* tk, const void* tv,
             void* o, void* to, float* lse, float* mu, float* li, int B, int H, int Lq, int Lk, int D,
             const int64_t* strides, float scale, int dtype, RopeTables rope, void* stream) {
    if (!q || !k || !v || !o || !lse || !strides) return SJVP_ERR_NULL;
    const bool jvp = tq || tk || tv || to || mu;
    if (jvp && (!tq || !tk || !tv || !to || !mu)) return SJVP_ERR_NULL;
    int rc = check_common(B, H, Lq, Lk, D, dtype, scale);
    if (rc != SJVP_OK) return rc;

    if (dtype == SJVP_FP32) {
        FwdParamsF32 f{};
        f.q = view32(q, strides + 3 * SJVP_F_Q);
        f.k = view32(k, strides + 3 * SJVP_F_K);
        f.v = view32(v, strides + 3 * SJVP_F_V);
        if (jvp) {
            f.tq = view32(tq, strides + 3 * SJVP_F_TQ);
            f.tk = view32(tk, strides + 3 * SJVP_F_TK);
            f.tv = view32(tv, strides + 3 * SJVP_F_TV);
            f.to = out_view32(to, strides + 3 * SJVP_F_TO);
        }
        f.o = out_view32(o, strides + 3 * SJVP_F_O);
        f.lse = lse;
        f.mu = mu;
        f.li = li;
        f.H = H;
        f.Lq = Lq;
        f.Lk = Lk;
        f.D = D;
        f.Lr = round_up(Lq, 128);
        f.scale = resolve_scale(scale, D);
        return fwd_f32(f, B * H, jvp, static_cast<hipStream_t>(stream));
    }
    const void* ptrs[SJVP_F_COUNT] = {q, k, v, tq, tk, tv, o, to};
    const bool f32io = dtype == SJVP_FP32_BF16;
    const int m = f32io ? 2 : 1;
    VecCheck vc;
    vc.unit = f32io ? 4 : 8;
    for (int i = 0; i < SJVP_F_COUNT; ++i) vc.add(ptrs[i], strides + 3 * i);

    FwdParams p{};
    p.q = view(q, strides + 3 * SJVP_F_Q, m);
    p.k = view(k, strides + 3 * SJVP_F_K, m);
    p.v = view(v, strides + 3 * SJVP_F_V, m);
    if (jvp) {
        p.tq = view(tq, strides + 3 * SJVP_F_TQ, m);
        p.tk = view(tk, strides + 3 * SJVP_F_TK, m);
        p.tv = view(tv, strides + 3 * SJVP_F_TV, m);
        p.to = out_view(to, strides + 3 * SJVP_F_TO, m);
    }
    p.o = out_view(o, strides + 3 * SJVP_F_O, m);
    p.lse = lse;
    p.mu = mu;
    p.li = li;
    p.H = H;
    p.Lq = Lq;
    p.Lk = Lk;
    p.D = D;
    p.Lr = round_up(Lq, 128);
    p.q_blocks = p.Lr / kOwned;  // covers every statistic row below Lr
    p.scale = resolve_scale(scale, D);
    p.vec = (vc.ok && D % 8 == 0) ? 1 : 0;
    p.rope = rope;
    if (rope.cos && !p.vec) return SJVP_ERR_ROTARY;

    const int grid = B * H * p.q_blocks;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (f32io) return fwd_f32io(p, grid, jvp, s);
    // LDS-DMA streaming needs 16-byte aligned rows; anything else takes the register-staged path
    if (p.vec) return dtype == SJVP_BF16 ? fwd_vec<Bf16>(p, grid, jvp, s) : fwd_vec<Fp16>(p, grid, jvp, s);
    return dtype == SJVP_BF16 ? fwd_any<Bf16>(p, grid, jvp, s) : fwd_any<Fp16>(p, grid, jvp, s);
}

}  // namespace

extern "C" {

size_t sjvp_bwd_workspace_bytes(int B, int H, int Lq, int Lk, int D, int dtype) {
    (void)Lk;
    (void)D;
    (void)dtype;
    if (B < 1 || H < 1 || Lq < 1) return 0;
    // three floats per statistic row (lse in log2 units, the two row sums) and one flag per 64 rows
    const size_t rows = (size_t)B * (size_t)H * (size_t)round_up(Lq, 128);
    return 3 * rows * sizeof(float) + rows / 64 * sizeof(int);
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
    const BwdTensors t{q, k, v, tq, tk, tv, o, to, dO, dTO, lse, mu, dq, dk, dv, dtq, dtk, dtv};
    int rc = check_bwd(parts, t, B, H, Lq, Lk, D, strides, scale, dtype);
    if (rc != SJVP_OK) return rc;
    if (!workspace || workspace_bytes < sjvp_bwd_workspace_bytes(B, H, Lq, Lk, D, dtype) ||
        (reinterpret_cast<uintptr_t>(workspace) & 3u))
        return SJVP_ERR_WORKSPACE;
    return run_bwd(parts, t, static_cast<float*>(workspace), B, H, Lq, Lk, D, strides, scale, dtype, stream);
}

int sjvp_bwd_rotary(const void* q, const void* k, const void* v, const void* tq, const void* tk,
                    const void* tv, const void* o, const void* to, const void* dO, const void* dTO,
                    const float* lse, const float* mu, void* dq, void* dk, void* dv, void* dtq, void* dtk,
                    void* dtv, int B, int H, int Lq, int Lk, int D, const int64_t* strides, float scale,
                    int dtype, const float* cos, const float* sin, int64_t cs_stride, int table_rows,
                    void* stream) {
    const BwdTensors t{q, k, v, tq, tk, tv, o, to, dO, dTO, lse, mu, dq, dk, dv, dtq, dtk, dtv};
    int rc = check_bwd(SJVP_BWD_ALL, t, B, H, Lq, Lk, D, strides, scale, dtype);
    if (rc != SJVP_OK) return rc;
    rc = check_rotary(cos, sin, cs_stride, table_rows, Lq, Lk, D, dtype);
    if (rc != SJVP_OK) return rc;
    // the single-launch backward, which these shapes take, uses no workspace
    return run_bwd(SJVP_BWD_ALL, t, nullptr, B, H, Lq, Lk, D, strides, scale, dtype, stream,
                   RopeTables{cos, sin, cs_stride, table_rows});
}

int sjvp_bwd_noalloc(const void* q, const void* k, const void* v, const void* tq, const void* tk,
                     const void* tv, const void* o, const void* to, const void* dO, const void* dTO,
                     const float* lse, const float* mu, void* dq, void* dk, void* dv, void* dtq,
                     void* dtk, void* dtv, int B, int H, int Lq, int Lk, int D, const int64_t* strides,
                     float scale, int dtype, void* stream) {
    const BwdTensors t{q, k, v, tq, tk, tv, o, to, dO, dTO, lse, mu, dq, dk, dv, dtq, dtk, dtv};
    int rc = check_bwd(SJVP_BWD_ALL, t, B, H, Lq, Lk, D, strides, scale, dtype);
    if (rc != SJVP_OK) return rc;
    if ((int64_t)B * H * round_up(Lq, 128) > (int64_t)SJVP_NOALLOC_MAX_ROWS) return SJVP_ERR_SCRATCH;
    float* ws = nullptr;
    rc = static_scratch(&ws);
    if (rc != SJVP_OK) return rc;
    return run_bwd(SJVP_BWD_ALL, t, ws, B, H, Lq, Lk, D, strides, scale, dtype, stream);
}

int sjvp_rope(int n, const void* const* x, void* const* y, const int64_t* strides, const float* cos,
              const float* sin, int64_t cs_stride, int B, int H, int L, int D, int rot_dim, int in_dtype,
              int out_dtype, int inverse, void* stream) {
    if (!x || !y || !strides) return SJVP_ERR_NULL;
    if (rot_dim != 0 && (!cos || !sin)) return SJVP_ERR_NULL;  // rot_dim 0: cast / layout change only
    if (n < 1 || n > kRopeMaxTensors) return SJVP_ERR_ROTARY;
    if (B < 1 || H < 1 || L < 1 || D < 1) return SJVP_ERR_SHAPE;
    if (rot_dim < 0 || rot_dim > D || (rot_dim & 1)) return SJVP_ERR_ROTARY;
    auto known = [](int d) { return d == SJVP_BF16 || d == SJVP_FP16 || d == SJVP_FP32; };
    if (!known(in_dtype) || !known(out_dtype)) return SJVP_ERR_DTYPE;
    if (in_dtype != SJVP_FP32 && out_dtype != SJVP_FP32 && in_dtype != out_dtype) return SJVP_ERR_ROTARY;
    const int half = rot_dim / 2;
    const int in_bytes = in_dtype == SJVP_FP32 ? 4 : 2, out_bytes = out_dtype == SJVP_FP32 ? 4 : 2;

    RopeParams p;
    // eight columns per thread need every row start and the second half of a pair 16-byte aligned
    bool vec = half % 8 == 0 && (D - rot_dim) % 8 == 0 &&
               (rot_dim == 0 || (aligned16(cos) && aligned16(sin) && cs_stride % 4 == 0));
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
        RopeParams copy = p;
        void* args[] = {&copy};
        return hipLaunchKernel(reinterpret_cast<const void*>(kernel), dim3((unsigned)blocks, (unsigned)n),
                               dim3(kRopeThreads), args, 0, static_cast<hipStream_t>(stream)) == hipSuccess
                   ? SJVP_OK
                   : SJVP_ERR_LAUNCH;
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

int sjvp_set_row_sum_repair(int mode) {
    if (mode < SJVP_REPAIR_OFF || mode > SJVP_REPAIR_ALWAYS) return SJVP_ERR_PARTS;
    return g_row_sum_repair.exchange(mode);
}

const char* sjvp_strerror(int status) {
    switch (status) {
        case SJVP_OK: return "ok";
        case SJVP_ERR_NULL: return "a required pointer is NULL";
        case SJVP_ERR_SHAPE: return "B, H, Lq and Lk must be >= 1 and within the index range";
        case SJVP_ERR_HEAD_DIM: return "head dimension must satisfy 16 <= D <= 128";
        case SJVP_ERR_DTYPE: return "dtype must be SJVP_BF16, SJVP_FP16, SJVP_FP32 or SJVP_FP32_BF16";
        case SJVP_ERR_WORKSPACE: return "workspace is NULL, misaligned or smaller than sjvp_bwd_workspace_bytes()";
        case SJVP_ERR_LAUNCH: return "HIP kernel launch failed";
        case SJVP_ERR_COTANGENT: return "at least one of dO and dTO must be given";
        case SJVP_ERR_PARTS: return "parts must be SJVP_BWD_ROW, SJVP_BWD_COL or SJVP_BWD_ALL (sjvp_set_row_sum_repair: mode must be SJVP_REPAIR_OFF, _AUTO or _ALWAYS)";
        case SJVP_ERR_SCALE: return "scale must be finite and >= 0 (0 selects 1/sqrt(D))";
        case SJVP_ERR_SCRATCH: return "sjvp_bwd_noalloc: B * H * ceil(Lq/128)*128 exceeds SJVP_NOALLOC_MAX_ROWS, or the static scratch could not be located on this device";
        case SJVP_ERR_ROTARY: return "rotary embedding: sjvp_rope needs n in 1..4, rot_dim even with 0 <= rot_dim <= D, and no mix of bf16 and fp16; sjvp_fwd_rotary / sjvp_bwd_rotary need D = 64, Lk <= 128, bf16 or fp16 tensors with 16-byte aligned rows, and 16-byte aligned fp32 tables of at least max(Lq, Lk) rows with a row stride that is a multiple of 4";
        default: return "unknown sjvp status";
    }
}

int sjvp_version(void) { return SJVP_VERSION; }

#ifndef SJVP_BUILD_ID
#define SJVP_BUILD_ID "SJVP_BUILD_ID=unknown"
#endif
const char* sjvp_build_id(void) { return SJVP_BUILD_ID; }

}  // extern "C"
