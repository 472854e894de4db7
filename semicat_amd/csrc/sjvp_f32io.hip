// Translation unit: the 32-wide register-staged kernels on fp32 tensors with bf16 arithmetic: inputs
// are rounded to bf16 as they are loaded and results are stored as fp32, which folds the casts that
// semicat/jvp_utils/functional.py:318-322,330-331 performs around the op for fp32 callers.
#include "sjvp_bwd.hpp"
#include "sjvp_fwd.hpp"
#include "sjvp_launch.hpp"

namespace sjvp {
namespace {

using T = Bf16;

template <int HD>
int fwd_hd(const FwdParams& p, int grid, bool jvp, hipStream_t stream) {
    if (jvp) return launch(fwd_kernel<T, HD, true, true>, grid, FwdSmem<HD, true>::bytes, stream, p, kThreads);
    return launch(fwd_kernel<T, HD, false, true>, grid, FwdSmem<HD, false>::bytes, stream, p, kThreads);
}

template <int HD, bool HAS_DO, bool HAS_G>
int pair_mode(const BwdParams& p, int BH, int parts, hipStream_t stream) {
    int rc = SJVP_OK;
    if (parts & SJVP_BWD_ROW) {
        const int grid = BH * p.q_blocks;
        constexpr int smem = RowSmem<HD, HAS_G>::bytes;
        // "always": measure the row-sum residues, then compute with the corrected sums; otherwise the pass
        // and, unless switched off, a second launch for the workgroups whose residues call for it
        if (p.rowfix == 2) rc = launch(bwd_row_kernel<T, HD, HAS_DO, HAS_G, true, 1>, grid, smem, stream, p, kThreads);
        else rc = launch(bwd_row_kernel<T, HD, HAS_DO, HAS_G, true, 0>, grid, smem, stream, p, kThreads);
        if (rc == SJVP_OK && p.rowfix != 0)
            rc = launch(bwd_row_kernel<T, HD, HAS_DO, HAS_G, true, 2>, grid, smem, stream, p, kThreads);
    }
    if (rc != SJVP_OK || !(parts & SJVP_BWD_COL)) return rc;
    const int col_grid = BH * p.k_blocks;
    using SM = ColSmem<HD, HAS_DO, HAS_G>;
    if constexpr (HD == 128) {
        rc = launch(bwd_col_kernel<T, HD, HAS_DO, HAS_G, true, true, 0, 2, true>, col_grid, SM::bytes, stream, p,
                    kThreads);
        if (rc != SJVP_OK) return rc;
        return launch(bwd_col_kernel<T, HD, HAS_DO, HAS_G, true, true, 2, 2, true>, col_grid, SM::bytes, stream, p,
                      kThreads);
    } else {
        return launch(bwd_col_kernel<T, HD, HAS_DO, HAS_G, true, true, 0, HD / 32, true>, col_grid, SM::bytes,
                      stream, p, kThreads);
    }
}

template <int HD>
int pair_hd(const BwdParams& p, int BH, bool has_do, bool has_g, int parts, hipStream_t stream) {
    if (has_do && has_g) return pair_mode<HD, true, true>(p, BH, parts, stream);
    if (has_g) return pair_mode<HD, false, true>(p, BH, parts, stream);
    return pair_mode<HD, true, false>(p, BH, parts, stream);
}

}  // namespace

int fwd_f32io(const FwdParams& p, int grid, bool jvp, hipStream_t stream) {
    if (p.D <= 32) return fwd_hd<32>(p, grid, jvp, stream);
    if (p.D <= 64) return fwd_hd<64>(p, grid, jvp, stream);
    return fwd_hd<128>(p, grid, jvp, stream);
}

int bwd_f32io(const BwdParams& p, int BH, bool has_do, bool has_g, int parts, hipStream_t stream) {
    if (p.D <= 32) return pair_hd<32>(p, BH, has_do, has_g, parts, stream);
    if (p.D <= 64) return pair_hd<64>(p, BH, has_do, has_g, parts, stream);
    return pair_hd<128>(p, BH, has_do, has_g, parts, stream);
}

}  // namespace sjvp
