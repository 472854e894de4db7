// Translation unit: 16-wide forward kernels for one element type (SJVP_T = Bf16 or Fp16).
#include "sjvp_fwd16.hpp"
#include "sjvp_launch.hpp"

namespace sjvp {
namespace {

// Ring depths (stages of 32 keys in flight) per head-dimension class, sized to the LDS a workgroup
// may take when two of them are to share the 160 KB of a CU.
constexpr int kRingJvp = 2;     // with tangents (four slabs per stage)
constexpr int kRingPrimal = 4;  // primal only (two slabs per stage)
// key-axis length from which the forward takes two stages per barrier
constexpr int kFwdPairedFrom = 256;

template <typename T, int HD>
int fwd16_hd(const FwdParams& p, int grid, bool jvp, hipStream_t stream) {
    // two stages in flight and at most 128 registers: two workgroups (sixteen waves) share a CU, which
    // overlaps one's copies with the other's arithmetic; HD = 128 needs the whole register budget
    constexpr int OCC = HD == 128 ? 2 : 4;
    if constexpr (HD == 64) {
        if (p.rope.cos) {  // rotary embedding folded in (short key axes only, checked by the caller)
            if (jvp)
                return launch(fwd16_kernel<T, HD, kRingJvp, true, OCC, 1, true>, grid,
                              Fwd16Smem<HD, kRingJvp, true>::bytes, stream, p, kThreads16);
            return launch(fwd16_kernel<T, HD, kRingPrimal, false, OCC, 1, true>, grid,
                          Fwd16Smem<HD, kRingPrimal, false>::bytes, stream, p, kThreads16);
        }
    }
    if (p.Lk >= kFwdPairedFrom) {
        // long key axes: two stages per barrier over a ring of four slots in the same LDS footprint
        if (jvp)
            return launch(fwd16_kernel<T, HD, 4, true, OCC, 2>, grid, Fwd16Smem<HD, 4, true, 2>::bytes, stream,
                          p, kThreads16);
        return launch(fwd16_kernel<T, HD, 4, false, OCC, 2>, grid, Fwd16Smem<HD, 4, false, 2>::bytes, stream,
                      p, kThreads16);
    }
    if (jvp)
        return launch(fwd16_kernel<T, HD, kRingJvp, true, OCC>, grid, Fwd16Smem<HD, kRingJvp, true>::bytes,
                      stream, p, kThreads16);
    return launch(fwd16_kernel<T, HD, kRingPrimal, false, OCC>, grid, Fwd16Smem<HD, kRingPrimal, false>::bytes,
                  stream, p, kThreads16);
}

}  // namespace

template <>
int fwd_vec<SJVP_T>(const FwdParams& p, int grid, bool jvp, hipStream_t stream) {
    if (p.D <= 32) return fwd16_hd<SJVP_T, 32>(p, grid, jvp, stream);
    if (p.D <= 64) return fwd16_hd<SJVP_T, 64>(p, grid, jvp, stream);
    return fwd16_hd<SJVP_T, 128>(p, grid, jvp, stream);
}

}  // namespace sjvp
