// Device-side building blocks shared by the attention-JVP kernels (gfx950 / CDNA4 only).
//
// Tile algebra used everywhere in this library
// --------------------------------------------
// One wavefront (64 lanes) owns 32 positions of one sequence axis ("owned" axis X: queries in the
// forward and in the dQ kernel, keys in the dK/dV kernel) and walks over the other axis ("looped"
// axis Y) in tiles of 32.  Every score-like 32x32 tile is produced by
//     v_mfma_f32_32x32x16_{bf16,f16}:  C[y][x] += sum_d A[y][d] * B[d][x]
// with A read row-major from LDS (the looped side) and B held in registers (the owned side), so
// that in the accumulator lane l holds column x = l % 32 and, in register j, row
//     y = 8*(j/4) + 4*(l/32) + (j%4).
// Per-x quantities (softmax max/sum, row statistics) are then per-lane scalars, and the tile,
// converted to 16-bit in place, is already the B operand (k = y) of the next contraction
//     OUT^T[d][x] += sum_y A'[d][y] * Tile[y][x],
// whose A' = (looped-side tensor)^T is fetched from the same row-major LDS tile with the
// transposing LDS read ds_read_b64_tr_b16.  No tile ever goes through LDS or shuffles.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace sjvp {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef uint16_t elem_t;  // storage type of one 16-bit element, whatever its format

constexpr int kThreads = 256;  // 4 wavefronts per workgroup
constexpr int kWaves = 4;
constexpr int kOwned = 32 * kWaves;  // positions of the owned axis per workgroup
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

struct Bf16 {
    static __device__ __forceinline__ f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                      __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
        bf16x2 v = {(__bf16)lo, (__bf16)hi};
        return __builtin_bit_cast(uint32_t, v);
    }
    static __device__ __forceinline__ float to_float(elem_t x) {
        return __builtin_bit_cast(float, (uint32_t)x << 16);
    }
};

struct Fp16 {
    static __device__ __forceinline__ f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                     __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
        f16x2 v = {(_Float16)lo, (_Float16)hi};
        return __builtin_bit_cast(uint32_t, v);
    }
    static __device__ __forceinline__ float to_float(elem_t x) {
        return (float)__builtin_bit_cast(_Float16, x);
    }
};

// A [B,H,L,D] view: base pointer and element strides; the last dimension has unit stride.
struct TensorView {
    const elem_t* ptr;
    int64_t sb, sh, sl;
    __device__ __forceinline__ const elem_t* head(int b, int h) const {
        return ptr + b * sb + h * sh;
    }
};

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

__device__ __forceinline__ float other_half(float x) { return __shfl_xor(x, 32, 64); }

// Eight consecutive elements starting at column d of one row; zero where the row is invalid or
// the column is >= D.  `vec` (uniform) promises 16-byte alignment and D % 8 == 0.
__device__ __forceinline__ u32x4 load8(const elem_t* row, int d, int D, bool valid, bool vec) {
    u32x4 r = {0u, 0u, 0u, 0u};
    if (valid) {
        if (vec) {
            if (d < D) r = *reinterpret_cast<const u32x4*>(row + d);
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                uint32_t lo = (d + 2 * i < D) ? row[d + 2 * i] : 0u;
                uint32_t hi = (d + 2 * i + 1 < D) ? row[d + 2 * i + 1] : 0u;
                r[i] = lo | (hi << 16);
            }
        }
    }
    return r;
}

// Four consecutive elements (packed in two dwords) to columns d..d+3 of one row, masked at D.
__device__ __forceinline__ void store4(elem_t* row, int d, int D, u32x2 val, bool vec) {
    if (vec) {
        if (d < D) *reinterpret_cast<u32x2*>(row + d) = val;
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (d + i < D) row[d + i] = (elem_t)((val[i >> 1] >> (16 * (i & 1))) & 0xffffu);
    }
}

// LDS row pitch (elements) of a staged [rows][HD] tile.  The 16-element pad makes the pitch
// 8 banks (mod 32) so that the four rows touched by one 16-lane group of a transposing read fall
// into disjoint banks.
template <int HD>
struct Pitch {
    static constexpr int value = HD + 16;
};

// Cooperative global -> LDS copy of ROWS rows (row0 .. row0+ROWS-1 of a [L][D] head slice) into a
// row-major LDS tile, zero-filled beyond L and beyond D.
template <int HD, int ROWS>
__device__ __forceinline__ void stage_rows(elem_t* lds, const elem_t* g, int64_t sl, int row0,
                                           int L, int D, bool vec, int tid) {
    constexpr int CH = HD / 8;
    constexpr int P = Pitch<HD>::value;
#pragma unroll
    for (int id = tid; id < ROWS * CH; id += kThreads) {
        int r = id / CH, c = id % CH;
        int row = row0 + r;
        u32x4 val = load8(g + (int64_t)row * sl, c * 8, D, row < L, vec);
        *reinterpret_cast<u32x4*>(lds + r * P + c * 8) = val;
    }
}

// A operand (32 rows y0..y0+31 of the looped side, k = d chunk c) read row-major from LDS.
template <int HD>
__device__ __forceinline__ u32x4 lds_a_rows(const elem_t* lds, int y0, int c, int x, int hf) {
    return *reinterpret_cast<const u32x4*>(lds + (y0 + x) * Pitch<HD>::value + 16 * c + 8 * hf);
}

// A operand of the transposed use: A'[d][y] for d = d0 + x and the eight looped positions that the
// lane's half owns in k-chunk c of a score tile, i.e. y0 + 16c + 4hf + {0..3} and + 8 more.  Read
// with two ds_read_b64_tr_b16: within each group of 16 lanes, lane 4j+g supplies the address of row
// (k0 + j), columns 4g..4g+3, and lane i receives column i of those four rows.
template <int HD>
__device__ __forceinline__ u32x4 lds_a_transposed(const elem_t* lds, int y0, int c, int d0, int lane) {
    constexpr int P = Pitch<HD>::value;
    const int hf = lane >> 5;
    const int i16 = lane & 15;
    const int xb = lane & 16;  // 0 or 16: which half of the 32 output rows d this 16-lane group feeds
    const int krow = y0 + 16 * c + 4 * hf + (i16 >> 2);
    const elem_t* p0 = lds + krow * P + d0 + xb + 4 * (i16 & 3);
    typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
    s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p0));
    s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p0 + 8 * P));
    u32x2 l2 = __builtin_bit_cast(u32x2, lo);
    u32x2 h2 = __builtin_bit_cast(u32x2, hi);
    u32x4 r = {l2[0], l2[1], h2[0], h2[1]};
    return r;
}

// Convert k-chunk c (registers 8c .. 8c+7) of a score-like tile into a B operand.
template <typename T>
__device__ __forceinline__ u32x4 pack_b(const f32x16& t, int c) {
    u32x4 r;
#pragma unroll
    for (int i = 0; i < 4; ++i) r[i] = T::pack2(t[8 * c + 2 * i], t[8 * c + 2 * i + 1]);
    return r;
}

// Store one transposed accumulator tile (OUT^T[d][x]: lane = row x of the output tensor, register
// j = column d0 + 8*(j/4) + 4*hf + j%4) scaled by `mul`, as 16-bit, masked at D.
template <typename T>
__device__ __forceinline__ void store_acc(elem_t* row, int d0, int hf, int D, const f32x16& acc,
                                          float mul, bool vec) {
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) {
        u32x2 val = {T::pack2(acc[4 * jj] * mul, acc[4 * jj + 1] * mul),
                     T::pack2(acc[4 * jj + 2] * mul, acc[4 * jj + 3] * mul)};
        store4(row, d0 + 8 * jj + 4 * hf, D, val, vec);
    }
}

}  // namespace sjvp
