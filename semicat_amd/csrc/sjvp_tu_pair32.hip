// Translation unit: 32-wide row-owned + column-owned backward pair (inputs of any alignment) for one
// element type (SJVP_T).
#include "sjvp_bwd.hpp"
#include "sjvp_launch.hpp"

namespace sjvp {
namespace {

template <typename T, int HD, bool HAS_DO, bool HAS_G>
int pair_mode(const BwdParams& p, int BH, int parts, hipStream_t stream) {
    int rc = SJVP_OK;
    if (parts & SJVP_BWD_ROW) {
        const int grid = BH * p.q_blocks;
        constexpr int smem = RowSmem<HD, HAS_G>::bytes;
        // "always": measure the row-sum residues, then compute with the corrected sums; otherwise the pass
        // and, unless switched off, a second launch for the workgroups whose residues call for it
        if (p.rowfix == 2) rc = launch(bwd_row_kernel<T, HD, HAS_DO, HAS_G, false, 1>, grid, smem, stream, p, kThreads);
        else rc = launch(bwd_row_kernel<T, HD, HAS_DO, HAS_G, false, 0>, grid, smem, stream, p, kThreads);
        if (rc == SJVP_OK && p.rowfix != 0)
            rc = launch(bwd_row_kernel<T, HD, HAS_DO, HAS_G, false, 2>, grid, smem, stream, p, kThreads);
    }
    if (rc != SJVP_OK || !(parts & SJVP_BWD_COL)) return rc;
    const int col_grid = BH * p.k_blocks;
    using SM = ColSmem<HD, HAS_DO, HAS_G>;
    if constexpr (HD == 128) {
        // two launches, each accumulating half of the head dimension (register budget)
        rc = launch(bwd_col_kernel<T, HD, HAS_DO, HAS_G, true, true, 0, 2>, col_grid, SM::bytes, stream, p,
                    kThreads);
        if (rc != SJVP_OK) return rc;
        return launch(bwd_col_kernel<T, HD, HAS_DO, HAS_G, true, true, 2, 2>, col_grid, SM::bytes, stream, p,
                      kThreads);
    } else {
        return launch(bwd_col_kernel<T, HD, HAS_DO, HAS_G, true, true, 0, HD / 32>, col_grid, SM::bytes, stream,
                      p, kThreads);
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
int bwd_pair_any<SJVP_T>(const BwdParams& p, int BH, bool has_do, bool has_g, int parts, hipStream_t stream) {
    if (p.D <= 32) return pair_hd<SJVP_T, 32>(p, BH, has_do, has_g, parts, stream);
    if (p.D <= 64) return pair_hd<SJVP_T, 64>(p, BH, has_do, has_g, parts, stream);
    return pair_hd<SJVP_T, 128>(p, BH, has_do, has_g, parts, stream);
}

}  // namespace sjvp
