// Device-side building blocks shared by the attention-JVP kernels (gfx950 / CDNA4 only).
//
// Tile algebra used everywhere in this library (32-wide form; sjvp_w16.hpp has the 16-wide one)
// ------------------------------------------------------------------------------------------------
// One wavefront (64 lanes) owns 32 positions of one sequence axis ("owned" axis X: queries in the
// forward and in the dQ kernel, keys in the dK/dV kernel) and walks over the other axis ("looped"
// axis Y) in stages of 32 rows.  Every score-like 32x32 tile is produced by
//     v_mfma_f32_32x32x16_{bf16,f16}:  C[y][x] += sum_d A[y][d] * B[d][x]
// with A read row-major from LDS (the looped side) and B held in registers (the owned side), so
// that in the accumulator lane l holds column x = l % 32 and, in register j, row
//     y = 8*(j/4) + 4*(l/32) + (j%4).
// Per-x quantities (softmax max/sum, row statistics) are then per-lane scalars, and the tile,
// converted to 16-bit in place, is already the B operand (k = y) of the next contraction
//     OUT^T[d][x] += sum_y A'[d][y] * Tile[y][x],
// whose A' = (looped-side tensor)^T is fetched from the same row-major LDS stage with the
// transposing LDS read ds_read_b64_tr_b16.  No tile ever goes through LDS or shuffles.
//
// Streaming
// ---------
// The looped side lives in LDS stage slabs: unpadded [32][HD] 16-bit, XOR-swizzled in units of 16
// bytes, which keeps both LDS access patterns (row-major 16-byte reads, and the 4-row x 32-byte
// footprint of a transposing read) free of bank conflicts.  The 16-wide kernels fill a ring of such
// stages with the LDS-DMA form of the global load (global_load_lds_dwordx4: 16 bytes per lane
// straight into LDS, no registers), issued ahead of use and retired with explicit
// s_waitcnt vmcnt(n); because every lane of an LDS-DMA load supplies its own global address, the
// swizzle costs nothing at copy time.  The 32-wide kernels (inputs of any alignment) copy one
// stage at a time through registers.
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

#ifndef SJVP_WAVES
#define SJVP_WAVES 4
#endif
constexpr int kWaves = SJVP_WAVES;  // wavefronts per workgroup (2 or 4)
constexpr int kThreads = 64 * kWaves;
constexpr int kOwned = 32 * kWaves;  // positions of the owned axis per workgroup
constexpr int kStageRows = 32;       // rows of the looped axis per stage
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

struct Bf16 {
    static __device__ __forceinline__ f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                      __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ f32x4 mfma16(u32x4 a, u32x4 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a),
                                                      __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
        bf16x2 v = {(__bf16)lo, (__bf16)hi};
        return __builtin_bit_cast(uint32_t, v);
    }
    static __device__ __forceinline__ float to_float(elem_t x) {
        return __builtin_bit_cast(float, (uint32_t)x << 16);
    }
    // a.lo * b.lo + a.hi * b.hi + c on a packed pair, accumulated in fp32 (v_dot2c_f32_bf16)
    static __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a), __builtin_bit_cast(bf16x2, b), c,
                                               false);
    }
};

struct Fp16 {
    static __device__ __forceinline__ f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                     __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ f32x4 mfma16(u32x4 a, u32x4 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a),
                                                     __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
        f16x2 v = {(_Float16)lo, (_Float16)hi};
        return __builtin_bit_cast(uint32_t, v);
    }
    static __device__ __forceinline__ float to_float(elem_t x) {
        return (float)__builtin_bit_cast(_Float16, x);
    }
    static __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, a), __builtin_bit_cast(f16x2, b), c, false);
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

struct OutView {
    elem_t* ptr;
    int64_t sb, sh, sl;
    __device__ __forceinline__ elem_t* head(int b, int h) const { return ptr + b * sb + h * sh; }
};

// cos / sin tables of a rotary position embedding folded into a kernel (see sjvp_w16.hpp)
struct RopeTables {
    const float* cos;  // [rows][32] fp32, row stride cs (multiple of 4, 16-byte aligned base); null: no rotation
    const float* sin;
    int64_t cs;
    int rows;          // rows of the tables (positions beyond are clamped; their data is zero padding)
};

// Workgroup barrier.  __syncthreads() leaves the wait for this wave's own LDS writes to the compiler,
// and at the head of a loop the compiler has been seen to hoist that wait into the loop's preheader
// only, so that a wave reached the barrier with the LDS write that ends its loop body still queued
// and another wave read the old value behind the barrier (one 16 x 16 tile of dQ in one of some ten
// thousand).  The explicit s_waitcnt lgkmcnt(0) is kept by the compiler wherever the barrier goes.
__device__ __forceinline__ void workgroup_barrier() {
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0); vmcnt and expcnt untouched
    __syncthreads();
}
// The same with a vote: true if `pred` holds for any thread of the workgroup.
__device__ __forceinline__ bool workgroup_barrier_or(bool pred) {
    __builtin_amdgcn_s_waitcnt(0xC07F);
    return __syncthreads_or(pred) != 0;
}

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

// load8 for either storage: F32IO rows hold fp32 elements (the row pointer is passed as elem_t* with
// strides counted in 2-byte units, so that row addressing is the same for both storages); they are
// rounded to T's 16-bit format as they are loaded.  `vec` promises 16-byte alignment and D % 8 == 0.
template <typename T, bool F32IO>
__device__ __forceinline__ u32x4 load8_io(const elem_t* row, int d, int D, bool valid, bool vec) {
    if constexpr (!F32IO) {
        return load8(row, d, D, valid, vec);
    } else {
        const float* fr = reinterpret_cast<const float*>(row);
        float x[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        if (valid) {
            if (vec) {
                if (d < D) {
                    const f32x4 a = *reinterpret_cast<const f32x4*>(fr + d);
                    const f32x4 b = *reinterpret_cast<const f32x4*>(fr + d + 4);
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        x[i] = a[i];
                        x[4 + i] = b[i];
                    }
                }
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    if (d + i < D) x[i] = fr[d + i];
            }
        }
        return u32x4{T::pack2(x[0], x[1]), T::pack2(x[2], x[3]), T::pack2(x[4], x[5]), T::pack2(x[6], x[7])};
    }
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

// ---------------------------------------------------------------------------------------------
// LDS stage slab: [32 rows][HD] elements, 16-byte chunk c of row r stored at chunk position
// c ^ swz(r).  The LDS has 64 banks of 4 bytes, i.e. 256 bytes per bank row, and serves a 16-byte
// read of 16 lanes per cycle: swz is chosen so that 16 consecutive slab rows read at one logical
// chunk (the A operand of a score tile) land in 16 distinct 16-byte positions of a bank row
// (measured on gfx950: 546 bytes/clk per CU against 315 with a swizzle that repeats every 8 rows).
// The transposing reads (4 rows x 32 bytes per group of 16 lanes) run at their full rate with it too.
// (A variant that also separates the four rows of a transposing read into distinct 32-byte positions
// measured worse: more conflict cycles on the hardware counter and 2 % less throughput.)
// swz has period 16 in the row.
template <int HD>
__device__ __forceinline__ int swz(int row) {
    if constexpr (HD == 32) return (row >> 2) & 3;  // four 64-byte rows per bank row
    if constexpr (HD == 64) return (row >> 1) & 7;  // two 128-byte rows per bank row
    return row & 15;                                // one 256-byte row per bank row
}

template <int HD>
struct Slab {
    static constexpr int elems = kStageRows * HD;
    static constexpr int chunks = kStageRows * HD / 8;  // 16-byte chunks
    static constexpr int per_thread = (chunks + kThreads - 1) / kThreads;
};

// LDS byte address of a pointer into shared memory: the low half of its flat address.
__device__ __forceinline__ uint32_t lds_addr(const void* p) {
    return (uint32_t)(uintptr_t)p;
}

// LDS-DMA: each active lane copies 16 bytes from its global address to LDS byte address
// base + 16 * lane_id (base must be wave-uniform).  Completion is tracked by vmcnt only.  M0 carries
// the LDS base; nothing else in these kernels uses M0 (gfx9 LDS instructions do not need it).
__device__ __forceinline__ void dma16(const void* gptr, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off"
                 :
                 : "v"(gptr), "s"(__builtin_amdgcn_readfirstlane(lds_base))
                 : "memory");
}
// 4-byte form: LDS byte address base + 4 * lane_id.
__device__ __forceinline__ void dma4(const void* gptr, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dword %0, off"
                 :
                 : "v"(gptr), "s"(__builtin_amdgcn_readfirstlane(lds_base))
                 : "memory");
}

// s_waitcnt vmcnt(ahead * SPT + EXTRA): at most `ahead` later stages (SPT vector-memory instructions each,
// SPT a compile-time constant) of this wave's copies may still be outstanding afterwards.  Loads and
// LDS-DMA copies retire in issue order, so everything issued before those stages has landed.
// EXTRA counts other vector-memory instructions (stores) known to have been issued after them.
// `ahead` is wave-uniform and small (at most the ring depth); counts beyond the 6-bit field are
// clamped, which only makes the wait stricter.
template <int SPT, int EXTRA = 0>
__device__ __forceinline__ void wait_stages(int ahead) {
#define SJVP_VMCNT(n) __builtin_amdgcn_s_waitcnt((((n) > 63 ? 63 : (n)) & 15) | ((((n) > 63 ? 63 : (n)) >> 4) << 14) | 0x0F70)
    switch (ahead) {
        case 0: SJVP_VMCNT(EXTRA); break;
        case 1: SJVP_VMCNT(SPT + EXTRA); break;
        case 2: SJVP_VMCNT(2 * SPT + EXTRA); break;
        case 3: SJVP_VMCNT(3 * SPT + EXTRA); break;
        case 4: SJVP_VMCNT(4 * SPT + EXTRA); break;
        case 5: SJVP_VMCNT(5 * SPT + EXTRA); break;
        case 6: SJVP_VMCNT(6 * SPT + EXTRA); break;
        default: SJVP_VMCNT(7 * SPT + EXTRA); break;
    }
#undef SJVP_VMCNT
}

// Per-thread geometry of a synchronous slab copy by the kThreads threads of a 32-wide workgroup:
// which 16-byte chunk positions of a slab this thread fills and which (row, column) of the source
// they hold.  Computed once per kernel.
template <int HD>
struct SlabLane {
    static constexpr int N = Slab<HD>::per_thread;
    int r[N];     // slab row
    int c8[N];    // source column (elements) of the chunk
    int pos8[N];  // element offset of the chunk position inside the slab
    bool on[N];   // the position exists (slabs smaller than the workgroup)
    __device__ __forceinline__ void init(int tid) {
        constexpr int CH = HD / 8;
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const int pos = tid + i * kThreads;
            r[i] = pos / CH;
            c8[i] = 8 * ((pos % CH) ^ swz<HD>(r[i]));
            pos8[i] = pos * 8;
            on[i] = pos < Slab<HD>::chunks;
        }
    }
};

// Copy stage rows row0 .. row0+31 of one [L][D] head slice into a slab (swizzled), zero-filled
// beyond L and beyond D: a synchronous copy through registers that works for any alignment (`vec`
// selects 16-byte loads when the rows allow them).
template <int HD, typename T = Bf16, bool F32IO = false>
__device__ __forceinline__ void fill_slab(const SlabLane<HD>& ln, elem_t* slab, const elem_t* g,
                                          int64_t sl, int row0, int L, int D, bool vec) {
#pragma unroll
    for (int i = 0; i < SlabLane<HD>::N; ++i) {
        if (Slab<HD>::chunks % kThreads != 0 && !ln.on[i]) break;
        const int row = row0 + ln.r[i];
        *reinterpret_cast<u32x4*>(slab + ln.pos8[i]) =
            load8_io<T, F32IO>(g + (int64_t)row * sl, ln.c8[i], D, row < L, vec);
    }
}

// A operand (the 32 rows of a slab, k = d chunk cc of 16) read row-major.
template <int HD>
__device__ __forceinline__ u32x4 lds_a_rows(const elem_t* slab, int cc, int x, int hf) {
    return *reinterpret_cast<const u32x4*>(slab + x * HD + (((2 * cc + hf) ^ swz<HD>(x)) << 3));
}

// A operand of the transposed use: A'[d][y] for d = d0 + x and the eight slab rows that the lane's
// half owns in k-chunk c of a score tile, i.e. 16c + 4hf + {0..3} and + 8 more.  Read with two
// ds_read_b64_tr_b16: within each group of 16 lanes, lane 4j+g supplies the address of row
// (k0 + j), columns 4g..4g+3, and lane i receives column i of those four rows.
template <int HD>
__device__ __forceinline__ u32x4 lds_a_transposed(const elem_t* slab, int c, int d0, int lane) {
    const int hf = lane >> 5;
    const int i16 = lane & 15;
    const int xb = lane & 16;  // which half of the 32 output rows d this 16-lane group feeds
    const int krow = 16 * c + 4 * hf + (i16 >> 2);
    const int e = d0 + xb + 4 * (i16 & 3);  // logical element (column) offset, multiple of 4
    const elem_t* p0 = slab + krow * HD + (((e >> 3) ^ swz<HD>(krow)) << 3) + (e & 7);
    const elem_t* p1 = slab + (krow + 8) * HD + (((e >> 3) ^ swz<HD>(krow + 8)) << 3) + (e & 7);
    typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
    s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p0));
    s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p1));
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
template <typename T, bool F32IO = false>
__device__ __forceinline__ void store_acc(elem_t* row, int d0, int hf, int D, const f32x16& acc,
                                          float mul, bool vec) {
    if constexpr (F32IO) {
        // fp32 storage: the scaled accumulators leave unrounded
        float* fr = reinterpret_cast<float*>(row);
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
            const int d = d0 + 8 * jj + 4 * hf;
            const f32x4 val = {acc[4 * jj] * mul, acc[4 * jj + 1] * mul, acc[4 * jj + 2] * mul, acc[4 * jj + 3] * mul};
            if (vec) {
                if (d < D) *reinterpret_cast<f32x4*>(fr + d) = val;
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (d + i < D) fr[d + i] = val[i];
            }
        }
        return;
    }
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) {
        u32x2 val = {T::pack2(acc[4 * jj] * mul, acc[4 * jj + 1] * mul),
                     T::pack2(acc[4 * jj + 2] * mul, acc[4 * jj + 3] * mul)};
        store4(row, d0 + 8 * jj + 4 * hf, D, val, vec);
    }
}

}  // namespace sjvp
