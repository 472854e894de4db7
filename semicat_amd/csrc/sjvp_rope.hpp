// Rotary position embedding of up to four [B,H,L,D] tensors in one launch, with the dtype cast and
// the layout change folded in: y[..., i]        = x[..., i] cos[l, i] - x[..., i + half] sin[l, i]
//                              y[..., i + half] = x[..., i + half] cos[l, i] + x[..., i] sin[l, i]
// for i < half = rot_dim / 2 and position l; elements from rot_dim on are copied.  This is the
// non-interleaved form that semicat/net/duo.py:45-55 applies to q and k through
// flash_attn.layers.rotary.apply_rotary_emb_torch.  The map is linear in x, so the same launch
// rotates forward-mode tangents, and with `sign` = -1 (the inverse rotation, which is also the
// transpose) it back-propagates cotangents.
//
// Pure streaming work: one thread moves eight pairs (two 16-byte loads and stores for 16-bit data),
// adjacent threads adjacent columns; the arithmetic is fp32 and each output is rounded once.
#pragma once
#include "sjvp_device.hpp"

namespace sjvp {

constexpr int kRopeMaxTensors = 4;
constexpr int kRopeThreads = 256;

struct RopeParams {
    const void* x[kRopeMaxTensors];
    void* y[kRopeMaxTensors];
    int64_t xs[kRopeMaxTensors][3];  // batch, head, sequence strides in elements
    int64_t ys[kRopeMaxTensors][3];
    const float* cos;  // [L][half], row stride cs
    const float* sin;
    int64_t cs;
    int H, L, D, half;
    int units;      // work items per row
    int64_t total;  // rows * units
    float sign;     // +1 rotation, -1 inverse rotation
    int h_fast;     // rows are enumerated head-first (sequence-major memory) instead of position-first
};

struct F32 {};  // tag for fp32 storage (Bf16 / Fp16 are the 16-bit traits)

template <typename T>
struct RopeIo {
    using elem = elem_t;
    static __device__ __forceinline__ float get(const elem* p) { return T::to_float(*p); }
    static __device__ __forceinline__ void put(elem* p, float v) { *p = (elem_t)(T::pack2(v, 0.f) & 0xffffu); }
    static __device__ __forceinline__ void get8(const elem* p, float* v) {
        const u32x4 r = *reinterpret_cast<const u32x4*>(p);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[2 * i] = T::to_float((elem_t)(r[i] & 0xffffu));
            v[2 * i + 1] = T::to_float((elem_t)(r[i] >> 16));
        }
    }
    static __device__ __forceinline__ void put8(elem* p, const float* v) {
        u32x4 r;
#pragma unroll
        for (int i = 0; i < 4; ++i) r[i] = T::pack2(v[2 * i], v[2 * i + 1]);
        *reinterpret_cast<u32x4*>(p) = r;
    }
};

template <>
struct RopeIo<F32> {
    using elem = float;
    static __device__ __forceinline__ float get(const float* p) { return *p; }
    static __device__ __forceinline__ void put(float* p, float v) { *p = v; }
    static __device__ __forceinline__ void get8(const float* p, float* v) {
        const f32x4 a = *reinterpret_cast<const f32x4*>(p);
        const f32x4 b = *reinterpret_cast<const f32x4*>(p + 4);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[i] = a[i];
            v[4 + i] = b[i];
        }
    }
    static __device__ __forceinline__ void put8(float* p, const float* v) {
        *reinterpret_cast<f32x4*>(p) = f32x4{v[0], v[1], v[2], v[3]};
        *reinterpret_cast<f32x4*>(p + 4) = f32x4{v[4], v[5], v[6], v[7]};
    }
};

// VEC: eight columns per work item (every row start 16-byte aligned, half and D - 2 half multiples
// of 8); otherwise one column (pair) per work item.
template <typename IN, typename OUT, bool VEC>
__global__ __launch_bounds__(kRopeThreads) void rope_kernel(const RopeParams p) {
    using In = RopeIo<IN>;
    using Out = RopeIo<OUT>;
    const int64_t idx = (int64_t)blockIdx.x * kRopeThreads + threadIdx.x;
    if (idx >= p.total) return;
    const int t = blockIdx.y;
    const int unit = (int)(idx % p.units);
    const int64_t row = idx / p.units;
    // consecutive rows follow the axis that is closer in memory
    const int l = p.h_fast ? (int)((row / p.H) % p.L) : (int)(row % p.L);
    const int h = p.h_fast ? (int)(row % p.H) : (int)((row / p.L) % p.H);
    const int64_t b = row / ((int64_t)p.L * p.H);
    const typename In::elem* x =
        reinterpret_cast<const typename In::elem*>(p.x[t]) + b * p.xs[t][0] + h * p.xs[t][1] + l * p.xs[t][2];
    typename Out::elem* y =
        reinterpret_cast<typename Out::elem*>(p.y[t]) + b * p.ys[t][0] + h * p.ys[t][1] + l * p.ys[t][2];
    constexpr int W = VEC ? 8 : 1;
    const int pair_units = p.half / W;
    if (unit < pair_units) {
        const int i0 = unit * W;
        float a[W], c[W], co[W], si[W];
        if constexpr (VEC) {
            In::get8(x + i0, a);
            In::get8(x + p.half + i0, c);
            const f32x4* cp = reinterpret_cast<const f32x4*>(p.cos + (int64_t)l * p.cs + i0);
            const f32x4* sp = reinterpret_cast<const f32x4*>(p.sin + (int64_t)l * p.cs + i0);
            const f32x4 c0 = cp[0], c1 = cp[1], s0 = sp[0], s1 = sp[1];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                co[i] = c0[i];
                co[4 + i] = c1[i];
                si[i] = s0[i];
                si[4 + i] = s1[i];
            }
        } else {
            a[0] = In::get(x + i0);
            c[0] = In::get(x + p.half + i0);
            co[0] = p.cos[(int64_t)l * p.cs + i0];
            si[0] = p.sin[(int64_t)l * p.cs + i0];
        }
        float lo[W], hi[W];
#pragma unroll
        for (int i = 0; i < W; ++i) {
            const float s = p.sign * si[i];
            lo[i] = a[i] * co[i] - c[i] * s;
            hi[i] = c[i] * co[i] + a[i] * s;
        }
        if constexpr (VEC) {
            Out::put8(y + i0, lo);
            Out::put8(y + p.half + i0, hi);
        } else {
            Out::put(y + i0, lo[0]);
            Out::put(y + p.half + i0, hi[0]);
        }
    } else {
        // columns from rot_dim on pass through (cast only)
        const int i0 = 2 * p.half + (unit - pair_units) * W;
        if constexpr (VEC) {
            float v[8];
            In::get8(x + i0, v);
            Out::put8(y + i0, v);
        } else {
            Out::put(y + i0, In::get(x + i0));
        }
    }
}

}  // namespace sjvp
