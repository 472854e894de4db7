// Building blocks of the 16-wide kernels (gfx950): eight wavefronts per workgroup, each owning 16
// positions of the owned axis, so that a wavefront's accumulators and operands stay well below 128
// registers and two to four wavefronts share a SIMD (their MFMA, VALU and LDS phases overlap).
//
// Tile algebra (v_mfma_f32_16x16x32_{bf16,f16}): C[y][x] += sum_k A[y][k] B[k][x] with
//     A: lane l holds row y = l % 16, k = 8*(l/16) + i (i < 8);   B: column x = l % 16, same k;
//     C: lane l holds column x = l % 16 and, in register j < 4, row y = 4*(l/16) + j.
// The owned side is the B operand (registers), the looped side the A operand (row-major LDS reads).
// A stage of 32 looped rows gives two 16-row score tiles t = 0, 1; converted to 16-bit, their eight
// registers are directly the B operand of the next contraction OUT^T[d][x] += A'[d][y] Tile[y][x]
// under the k numbering  k = 8g + i  <->  y = 16*(i/4) + 4g + i%4  (g = l/16), and A' in that numbering
// is what two transposing LDS reads (rows 4g..4g+3 and 16+4g..16+4g+3, sixteen columns) deliver.
#pragma once
#include "sjvp_device.hpp"

namespace sjvp {

constexpr int kWaves16 = 8;
constexpr int kThreads16 = 64 * kWaves16;
constexpr int kOwned16 = 16 * kWaves16;  // owned positions per workgroup (== kOwned)
constexpr int kSink16 = 16;              // bytes of LDS that placeholder copies may overwrite
static_assert(kOwned16 == kOwned, "both kernel families use the same workgroup grid");

struct Src {
    const elem_t* ptr;  // [L][D] slice of one (batch, head)
    int64_t sl;         // row stride in elements
};

// Workgroups are dealt to the eight XCDs round-robin (workgroup i runs on XCD i % 8), each XCD with
// an L2 of its own.  Kernels in which several workgroups of a (batch, head) pair stream the same
// rows take their work item from this map: XCD x gets the contiguous range x * G/8 .. (x+1) * G/8 - 1
// of the linear order, so the workgroups of one pair run on one XCD, close in time, and find the
// streamed rows in its L2.  Grids that are not a multiple of eight keep the identity.
__device__ __forceinline__ int xcd_linear_id(int bid, int grid) {
    if (grid & 7) return bid;
    return (bid & 7) * (grid >> 3) + (bid >> 3);
}

// Per-thread geometry of an LDS-DMA copy of NS slabs that lie back to back in LDS: slab j holds rows
// 32*(j % SPTN) .. +31 (relative to the first row of the copy window) of tensor j / SPTN.  Successive
// calls of issue() copy successive windows (32*SPTN rows further down every tensor).  Every wave
// that takes part issues exactly N vector-memory instructions per call: a wave with no valid lane issues a 4-byte
// placeholder copy into the sink, which keeps the vmcnt arithmetic of wait_stages exact.
template <int HD, int NS, int SPTN, int NT = kThreads16>
struct CopyPlan {
    static constexpr int chunks = Slab<HD>::chunks;
    static constexpr int total = NS * chunks;
    static constexpr int N = (total + NT - 1) / NT;  // NT threads take part (tid = 0 .. NT-1)
    static constexpr int NTENS = NS / SPTN;
    static_assert(NS % SPTN == 0 && chunks % 64 == 0, "slabs are whole multiples of a wave's 64 chunks");
    const elem_t* src[N];  // global address of this thread's chunk in the next window
    int64_t adv[N];        // elements from one window to the next (wave-uniform)
    int row[N];            // row of the chunk relative to the window's first row
    uint32_t wbase[N];     // byte offset of the wave's first chunk position from the region base
    uint32_t pos[N];       // byte offset of this thread's chunk position
    bool ok[N];            // the column of the chunk is below D
    bool on[N];            // the position exists (wave-uniform)
    const elem_t* any;     // some valid global address (source of placeholder copies)
    uint32_t sink;

    // Tensors are passed one by one (not as an array) so that the wave-uniform choice among them
    // stays a chain of scalar selects.  NT and the chunks of a slab are powers of two, so a thread's
    // positions are the SAME chunk (row within the slab, column) of successive slabs (NT >= chunks) or
    // of successive parts of one slab (NT < chunks): the column and the swizzle are computed once and
    // the slab index is a scalar, which keeps this set-up to a few instructions per position (it runs
    // once per workgroup, and a workgroup with a short loop lives only some ten thousand cycles).
    __device__ __forceinline__ void init(int tid, int first_row, int D, const void* sink_lds, Src t0,
                                         Src t1 = Src{nullptr, 0}, Src t2 = Src{nullptr, 0},
                                         Src t3 = Src{nullptr, 0}, Src t4 = Src{nullptr, 0},
                                         Src t5 = Src{nullptr, 0}) {
        static_assert(NTENS <= 6, "at most six tensors per copy");
        static_assert(NT % chunks == 0 || chunks % NT == 0, "thread count and slab size are powers of two");
        constexpr int CH = HD / 8;
        any = t0.ptr;
        sink = lds_addr(sink_lds);
        const int q0 = tid % chunks;                      // position within its slab for i = 0
        const int c8 = 8 * ((q0 % CH) ^ swz<HD>(q0 / CH));  // rows r and r + 16 k share their swizzle
        static_assert(NT >= chunks || (NT / CH) % 16 == 0, "parts of a slab start at multiples of 16 rows");
        const int j0 = __builtin_amdgcn_readfirstlane(tid / chunks);  // slab of position i = 0 (wave-uniform)
        const bool col_ok = c8 < D;
#pragma unroll
        for (int i = 0; i < N; ++i) {
            int j, r;
            if constexpr (NT >= chunks) {
                j = j0 + (NT / chunks) * i;
                r = q0 / CH;
            } else {
                j = i / (chunks / NT);
                r = q0 / CH + (NT / CH) * (i % (chunks / NT));
            }
            on[i] = j < NS;
            // the tensor of slab j: known at compile time where a thread's slabs never straddle two tensors,
            // else one of NT / chunks neighbours, chosen by the (wave-uniform) slab of position 0
            const Src ts[6] = {t0, t1, t2, t3, t4, t5};
            const elem_t* ptr;
            int64_t sl;
            if constexpr (NT < chunks) {
                constexpr int PPS = chunks / NT;
                ptr = ts[(i / PPS) / SPTN < NTENS ? (i / PPS) / SPTN : 0].ptr;
                sl = ts[(i / PPS) / SPTN < NTENS ? (i / PPS) / SPTN : 0].sl;
            } else if constexpr (SPTN % (NT / chunks) == 0) {
                constexpr int SPI = NT / chunks;
                ptr = ts[(SPI * i) / SPTN < NTENS ? (SPI * i) / SPTN : 0].ptr;
                sl = ts[(SPI * i) / SPTN < NTENS ? (SPI * i) / SPTN : 0].sl;
            } else {
                static_assert(NT < chunks || SPTN % (NT / chunks) == 0 || SPTN == 1, "slabs per tensor");
                constexpr int SPI = NT / chunks;
                ptr = ts[SPI * i < NTENS ? SPI * i : 0].ptr;
                sl = ts[SPI * i < NTENS ? SPI * i : 0].sl;
#pragma unroll
                for (int k = 1; k < SPI; ++k) {
                    if (SPI * i + k < NTENS && j0 == k) {
                        ptr = ts[SPI * i + k < NTENS ? SPI * i + k : 0].ptr;
                        sl = ts[SPI * i + k < NTENS ? SPI * i + k : 0].sl;
                    }
                }
            }
            const int slab_row = 32 * (j % SPTN);  // scalar
            row[i] = slab_row + r;
            src[i] = (ptr + (int64_t)(first_row + slab_row) * sl) + ((int64_t)r * sl + c8);
            adv[i] = 32 * SPTN * sl;
            ok[i] = col_ok;
            wbase[i] = (uint32_t)(((tid & ~63) + i * NT) * 16);
            pos[i] = (uint32_t)((tid + i * NT) * 16);
        }
    }

    // Copy the next window into `region`; rows_left = rows of the window that exist (zero fill beyond).
    // `whole` (wave-uniform): the caller knows that every row of the window exists and that D covers every
    // chunk, so every lane copies and nothing is predicated (a few instructions per copy instead of the
    // forty of the general form, which matters in loops that are bound by instruction issue).
    __device__ __forceinline__ void issue(elem_t* region, int rows_left, bool whole = false) {
        const uint32_t base = lds_addr(region);
        if (total % NT == 0 && whole) {
#pragma unroll
            for (int i = 0; i < N; ++i) {
                dma16(src[i], base + wbase[i]);
                src[i] += adv[i];
            }
            return;
        }
#pragma unroll
        for (int i = 0; i < N; ++i) {
            bool valid = false;
            if (total % NT == 0 || on[i]) {
                valid = ok[i] && row[i] < rows_left;
                if (valid) {
                    dma16(src[i], base + wbase[i]);
                } else {
                    *reinterpret_cast<u32x4*>(reinterpret_cast<unsigned char*>(region) + pos[i]) =
                        u32x4{0u, 0u, 0u, 0u};
                }
                src[i] += adv[i];
            }
            if (__builtin_amdgcn_ballot_w64(valid) == 0) {
                if ((threadIdx.x & 63) == 0) dma4(any, sink);
            }
        }
    }
};

// A operand of a score tile: rows 16t .. 16t+15 of a slab, k = head-dimension chunk c of 32.
template <int HD>
__device__ __forceinline__ u32x4 lds_a_rows16(const elem_t* slab, int t, int c, int n, int g) {
    const int r = 16 * t + n;
    return *reinterpret_cast<const u32x4*>(slab + r * HD + (((4 * c + g) ^ swz<HD>(r)) << 3));
}

// B operands of one owned row (all head-dimension chunks of 32) from a landed slab.
template <int HD>
__device__ __forceinline__ void read_b_operands16(u32x4* out, const elem_t* slab, int r, int g) {
#pragma unroll
    for (int c = 0; c < HD / 32; ++c)
        out[c] = *reinterpret_cast<const u32x4*>(slab + r * HD + (((4 * c + g) ^ swz<HD>(r)) << 3));
}

// A' operand of an output contraction: A'[d0 + n][k] for the lane group's eight slab rows
// 4g..4g+3 and 16+4g..16+4g+3 (see the k numbering at the top).  Two ds_read_b64_tr_b16: within a
// group of 16 lanes, lane 4j+c supplies the address of row (first + j), columns 4c..4c+3, and lane i
// receives column i of those four rows.  Rows r and r+16 share their swizzle.
template <int HD>
__device__ __forceinline__ u32x4 lds_a_tr16(const elem_t* slab, int d0, int lane) {
    const int g = lane >> 4;
    const int i16 = lane & 15;
    const int r = 4 * g + (i16 >> 2);
    const int e = d0 + 4 * (i16 & 3);
    const elem_t* p0 = slab + r * HD + (((e >> 3) ^ swz<HD>(r)) << 3) + (e & 7);
    typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
    s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p0));
    s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p0 + 16 * HD));
    u32x2 l2 = __builtin_bit_cast(u32x2, lo);
    u32x2 h2 = __builtin_bit_cast(u32x2, hi);
    u32x4 out = {l2[0], l2[1], h2[0], h2[1]};
    return out;
}

// The two score-like tiles of a stage as the B operand of the next contraction.
template <typename T>
__device__ __forceinline__ u32x4 pack_b16(const f32x4& t0, const f32x4& t1) {
    u32x4 r = {T::pack2(t0[0], t0[1]), T::pack2(t0[2], t0[3]), T::pack2(t1[0], t1[1]),
               T::pack2(t1[2], t1[3])};
    return r;
}

// Sum / maximum over the four lanes (l, l^16, l^32, l^48) that share an owned position.
__device__ __forceinline__ float group_sum(float v) {
    v += __shfl_xor(v, 16, 64);
    v += __shfl_xor(v, 32, 64);
    return v;
}
__device__ __forceinline__ float group_max(float v) {
    v = fmaxf(v, __shfl_xor(v, 16, 64));
    v = fmaxf(v, __shfl_xor(v, 32, 64));
    return v;
}

// Sum over each aligned group of eight consecutive lanes, by DPP moves (no LDS traffic): the quad
// permutations [1,0,3,2] and [2,3,0,1], then row_half_mirror, which pairs lane i with lane 7 - i of
// its group of eight, i.e. with the other quad.
__device__ __forceinline__ float sum8(float v) {
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));
    return v;
}

// ---------------------------------------------------------------------------------------------
// Rotary position embedding folded into the attention kernels (head dimension 64, rotation over the
// whole head: column j < 32 of a row is paired with column j + 32, as semicat/net/duo.py:45-55 does
// through flash_attn's non-interleaved apply_rotary_emb_torch).  The rotation is linear, so tangents
// take the same rotation as their primals and cotangents the inverse (= transposed) one.
// Rotate eight column pairs: x0 holds columns j .. j+7 (j = 8 * chunk), x1 columns 32+j .. 32+j+7 of a
// row at position pos.  sign = +1: y0 = x0 c - x1 s, y1 = x1 c + x0 s; sign = -1: the inverse.
// fp32 arithmetic, one rounding per element.
template <typename T>
__device__ __forceinline__ void rope8(u32x4& x0, u32x4& x1, const RopeTables& rt, int pos, int chunk, float sign) {
    pos = pos < rt.rows ? pos : rt.rows - 1;
    const float* cr = rt.cos + (int64_t)pos * rt.cs + 8 * chunk;
    const float* sr = rt.sin + (int64_t)pos * rt.cs + 8 * chunk;
    const f32x4 c0 = *reinterpret_cast<const f32x4*>(cr), c1 = *reinterpret_cast<const f32x4*>(cr + 4);
    const f32x4 s0 = *reinterpret_cast<const f32x4*>(sr), s1 = *reinterpret_cast<const f32x4*>(sr + 4);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float ca = i < 2 ? c0[2 * i] : c1[2 * i - 4], cb = i < 2 ? c0[2 * i + 1] : c1[2 * i - 3];
        const float sa = sign * (i < 2 ? s0[2 * i] : s1[2 * i - 4]), sb = sign * (i < 2 ? s0[2 * i + 1] : s1[2 * i - 3]);
        const float a0 = T::to_float((elem_t)(x0[i] & 0xffffu)), a1 = T::to_float((elem_t)(x0[i] >> 16));
        const float b0 = T::to_float((elem_t)(x1[i] & 0xffffu)), b1 = T::to_float((elem_t)(x1[i] >> 16));
        x0[i] = T::pack2(fmaf(a0, ca, -b0 * sa), fmaf(a1, cb, -b1 * sb));
        x1[i] = T::pack2(fmaf(b0, ca, a0 * sa), fmaf(b1, cb, a1 * sb));
    }
}

// One output chunk of the inverse rotation from a row held in LDS as 16-byte chunks: chunk c of the
// result needs chunk c and its partner c ^ 4 of the input (`mine`, `other`).
template <typename T>
__device__ __forceinline__ u32x4 rope8_inverse_chunk(u32x4 mine, u32x4 other, const RopeTables& rt, int pos, int c) {
    u32x4 lo = c < 4 ? mine : other, hi = c < 4 ? other : mine;
    rope8<T>(lo, hi, rt, pos, c & 3, -1.0f);
    return c < 4 ? lo : hi;
}

// Rotate rows of a swizzled [32][64] slab in place: item it (0..127) is row it / 4, chunk pair it % 4.
template <typename T>
__device__ __forceinline__ void rope_slab_item(elem_t* slab, int it, const RopeTables& rt, int row0, float sign) {
    const int r = it >> 2, c = it & 3;
    u32x4* p0 = reinterpret_cast<u32x4*>(slab + r * 64 + ((c ^ swz<64>(r)) << 3));
    u32x4* p1 = reinterpret_cast<u32x4*>(slab + r * 64 + (((c + 4) ^ swz<64>(r)) << 3));
    u32x4 x0 = *p0, x1 = *p1;
    rope8<T>(x0, x1, rt, row0 + r, c, sign);
    *p0 = x0;
    *p1 = x1;
}

// Per-wave staging tile of the coalesced row stores: [16 rows][HD + 8] elements.
template <int HD>
struct StoreStage16 {
    static constexpr int pitch = HD + 8;
    static constexpr int elems = 16 * pitch;
};

// Store OUT[row0 + r][0..D) for r < 16 from transposed accumulator tiles acc[HD/16] (lane = row,
// registers = 4 consecutive columns 16*dt + 4g ..) scaled by mul: 8-byte writes into the wave's
// staging tile, 16-byte reads back row-major, 16-byte global stores (a 128-byte row per 8 lanes).
// Issues exactly max(1, HD / 32) global store instructions.
template <typename T, int HD, bool ROPE = false>
__device__ __forceinline__ void store_tile16(elem_t* stage, elem_t* gp, int64_t sl, int row0, int L, int D,
                                             const f32x4* acc, float mul, int lane,
                                             const RopeTables* rt = nullptr) {
    constexpr int P = StoreStage16<HD>::pitch;
    const int n = lane & 15, g = lane >> 4;
#pragma unroll
    for (int dt = 0; dt < HD / 16; ++dt) {
        u32x2 val = {T::pack2(acc[dt][0] * mul, acc[dt][1] * mul), T::pack2(acc[dt][2] * mul, acc[dt][3] * mul)};
        *reinterpret_cast<u32x2*>(stage + n * P + 16 * dt + 4 * g) = val;
    }
    constexpr int CH = HD / 8;    // 16-byte chunks per row
    constexpr int RPI = 64 / CH;  // rows per store instruction
#pragma unroll
    for (int it = 0; it < (16 + RPI - 1) / RPI; ++it) {
        const int r = it * RPI + lane / CH;
        const int c = lane % CH;
        if (RPI <= 16 || r < 16) {
            u32x4 v = *reinterpret_cast<const u32x4*>(stage + r * P + 8 * c);
            if constexpr (ROPE) {
                // a gradient of a rotated tensor goes back through the inverse rotation
                static_assert(!ROPE || HD == 64, "the folded rotation covers a head dimension of 64");
                const u32x4 other = *reinterpret_cast<const u32x4*>(stage + r * P + 8 * (c ^ 4));
                v = rope8_inverse_chunk<T>(v, other, *rt, row0 + r, c);
            }
            if (row0 + r < L && 8 * c < D) {
                u32x4* dst = reinterpret_cast<u32x4*>(gp + (int64_t)(row0 + r) * sl + 8 * c);
                __builtin_nontemporal_store(v, dst);  // written once, not read again by this launch
            }
        }
    }
}

}  // namespace sjvp
