// Helpers around the LDS stage slabs: reading a workgroup's own rows back as MFMA B operands, and
// turning the transposed accumulator layout into coalesced 16-byte row stores through a per-wave
// staging tile.
#pragma once
#include "sjvp_device.hpp"

namespace sjvp {

// Per-wave staging tile used to turn the transposed accumulator layout into coalesced 16-byte row
// stores: [32 rows][HD + 8] elements (the pad spreads the 8-byte column writes over the banks).
template <int HD>
struct StoreStage {
    static constexpr int pitch = HD + 8;
    static constexpr int elems = 32 * pitch;
};

// Store OUT[row0 + r][0..D) for r < 32 from transposed accumulator tiles acc[DT] (lane = row,
// registers = columns) scaled by mul: 8-byte writes into the wave's staging tile, 16-byte reads
// back row-major, 16-byte global stores (one 128-byte row per 8 lanes).  Issues exactly HD / 16
// global store instructions.  Needs D % 8 == 0 and 16-byte aligned rows.
template <typename T, int HD, typename Acc>
__device__ __forceinline__ void store_tile_coalesced(elem_t* stage, elem_t* g, int64_t sl, int row0,
                                                     int L, int D, const Acc& acc, float mul,
                                                     int lane) {
    constexpr int DT = HD / 32;
    constexpr int P = StoreStage<HD>::pitch;
    const int x = lane & 31, hf = lane >> 5;
#pragma unroll
    for (int d = 0; d < DT; ++d) {
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
            u32x2 val = {T::pack2(acc[d][4 * jj] * mul, acc[d][4 * jj + 1] * mul),
                         T::pack2(acc[d][4 * jj + 2] * mul, acc[d][4 * jj + 3] * mul)};
            *reinterpret_cast<u32x2*>(stage + x * P + 32 * d + 8 * jj + 4 * hf) = val;
        }
    }
    constexpr int CH = HD / 8;           // 16-byte chunks per row
    constexpr int RPI = 64 / CH;         // rows per store instruction
#pragma unroll
    for (int it = 0; it < 32 / RPI; ++it) {
        const int r = it * RPI + lane / CH;
        const int c = lane % CH;
        const u32x4 v = *reinterpret_cast<const u32x4*>(stage + r * P + 8 * c);
        if (row0 + r < L && 8 * c < D)
            *reinterpret_cast<u32x4*>(g + (int64_t)(row0 + r) * sl + 8 * c) = v;
    }
}

// B operands (k-chunks of 16 over the head dimension) of slab row `r`, read from a landed slab.
template <int HD>
__device__ __forceinline__ void read_b_operands(u32x4* out, const elem_t* slab, int r, int hf) {
#pragma unroll
    for (int c = 0; c < HD / 16; ++c)
        out[c] = *reinterpret_cast<const u32x4*>(slab + r * HD + (((2 * c + hf) ^ swz<HD>(r)) << 3));
}

}  // namespace sjvp
