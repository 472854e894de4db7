// Translation unit: 16-wide row-owned + column-owned backward pair for one element type (SJVP_T).
#include "sjvp_bwd16x.hpp"
#include "sjvp_launch.hpp"

#ifndef SJVP_COL16P_RING
#define SJVP_COL16P_RING 2
#endif

namespace sjvp {
namespace {

template <typename T, int HD, bool HAS_DO, bool HAS_G>
int pair_mode(const BwdParams& p, int BH, int parts, hipStream_t stream) {
    // the row-owned kernel first (besides dQ, dQ_dot it leaves the row sums in the workspace), then
    // the column-owned one; workgroups of four waves own 64 positions
    constexpr int XR = HD == 128 ? 2 : 3;  // ring depth
    int rc = SJVP_OK;
    bool rides = false;
    if (parts & SJVP_BWD_ROW) {
        constexpr int OCC = HD == 128 ? 2 : 3;
        const int grid = BH * (p.Lr / kXOwned16);
        constexpr int smem = Row16Smem<HD, XR, HAS_G>::bytes;
        // "always": a launch that measures the row-sum residues, then one that computes with the corrected
        // sums; otherwise the pass itself and, unless switched off, a second launch in which the workgroups
        // whose residues call for it run again
        if (p.rowfix == 2) rc = launch(bwd_row16_kernel<T, HD, XR, HAS_DO, HAS_G, OCC, 1>, grid, smem, stream, p, kXThreads16);
        else rc = launch(bwd_row16_kernel<T, HD, XR, HAS_DO, HAS_G, OCC, 0>, grid, smem, stream, p, kXThreads16);
        // The second launch does not depend on the column-owned pass.  Where nearly all of its workgroups leave
        // at once (repair of flagged workgroups only), they ride at the end of that launch instead of paying for
        // one of their own.
        // (not at D = 128 with the cotangent on O only: the row-owned body needs more registers than that
        // column-owned kernel, which would lose a resident workgroup per compute unit to it)
        rides = p.rowfix == 1 && (parts & SJVP_BWD_COL) && (HD != 128 || HAS_G);
        if (rc == SJVP_OK && p.rowfix != 0 && !rides)
            rc = launch(bwd_row16_kernel<T, HD, XR, HAS_DO, HAS_G, OCC, 2>, grid, smem, stream, p, kXThreads16);
    }
    if (rc != SJVP_OK || !(parts & SJVP_BWD_COL)) return rc;
    const int grid = BH * ((p.Lk + kXOwned16 - 1) / kXOwned16);
    using CS = Col16Smem<HD, XR, HAS_DO, HAS_G>;
    if constexpr (HD == 128) {
        // eight waves: wave pairs share 16 keys, split the score-side tiles by query tile and the
        // gradients by head-dimension half (one launch, nothing computed twice)
        constexpr int PR = SJVP_COL16P_RING;  // ring depths 2, 3, 4 measure the same (the kernel is issue-bound)
        using PS = Col16pSmem<HD, PR, HAS_DO, HAS_G>;
        if (rides) {
            BwdParams pr = p;
            pr.col_workgroups = grid;
            constexpr int smem = PS::bytes > Row16Smem<HD, XR, HAS_G>::bytes ? PS::bytes : Row16Smem<HD, XR, HAS_G>::bytes;
            return launch(bwd_col16p_repair_kernel<T, HD, PR, XR, HAS_DO, HAS_G>, grid + BH * (p.Lr / kXOwned16), smem,
                          stream, pr, kThreads16);
        }
        return launch(bwd_col16p_kernel<T, HD, PR, HAS_DO, HAS_G>, grid, PS::bytes, stream, p, kThreads16);
    } else {
        if (rides) {
            BwdParams pr = p;
            pr.col_workgroups = grid;
            constexpr int smem = CS::bytes > Row16Smem<HD, XR, HAS_G>::bytes ? CS::bytes : Row16Smem<HD, XR, HAS_G>::bytes;
            return launch(bwd_col16_repair_kernel<T, HD, XR, HAS_DO, HAS_G, 2>, grid + BH * (p.Lr / kXOwned16), smem,
                          stream, pr, kXThreads16);
        }
        return launch(bwd_col16_kernel<T, HD, XR, HAS_DO, HAS_G, 3, 2>, grid, CS::bytes, stream, p, kXThreads16);
    }
}

template <typename T, int HD>
int pair_hd(const BwdParams& p, int BH, bool has_do, bool has_g, int parts, hipStream_t stream) {
    if (has_do && has_g) return pair_mode<T, HD, true, true>(p, BH, parts, stream);
    if (has_g) return pair_mode<T, HD, false, true>(p, BH, parts, stream);
    return pair_mode<T, HD, true, false>(p, BH, parts, stream);
}

}  // namespace

template <>
int bwd_pair_vec<SJVP_T>(const BwdParams& p, int BH, bool has_do, bool has_g, int parts, hipStream_t stream) {
    if (p.D <= 32) return pair_hd<SJVP_T, 32>(p, BH, has_do, has_g, parts, stream);
    if (p.D <= 64) return pair_hd<SJVP_T, 64>(p, BH, has_do, has_g, parts, stream);
    return pair_hd<SJVP_T, 128>(p, BH, has_do, has_g, parts, stream);
}

}  // namespace sjvp
