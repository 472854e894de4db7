// Translation unit: the fp32 (vector-ALU) kernels of the correctness mode.
#include "sjvp_f32.hpp"
#include "sjvp_launch.hpp"

namespace sjvp {
namespace {

template <int HD>
int fwd_hd(const FwdParamsF32& p, int BH, bool jvp, hipStream_t stream) {
    const int grid = BH * (p.Lr / kF32Owned);
    if (jvp) return launch(fwd_f32_kernel<HD, true>, grid, 0, stream, p, kF32Threads);
    return launch(fwd_f32_kernel<HD, false>, grid, 0, stream, p, kF32Threads);
}

template <int HD, bool HAS_DO, bool HAS_G>
int bwd_mode(const BwdParamsF32& p, int BH, int parts, hipStream_t stream) {
    int rc = SJVP_OK;
    if (parts & SJVP_BWD_ROW)
        rc = launch(bwd_row_f32_kernel<HD, HAS_DO, HAS_G>, BH * (p.Lr / kF32Owned), 0, stream, p, kF32Threads);
    if (rc != SJVP_OK || !(parts & SJVP_BWD_COL)) return rc;
    return launch(bwd_col_f32_kernel<HD, HAS_DO, HAS_G>, BH * ((p.Lk + kF32Owned - 1) / kF32Owned), 0, stream, p,
                  kF32Threads);
}

template <int HD>
int bwd_hd(const BwdParamsF32& p, int BH, bool has_do, bool has_g, int parts, hipStream_t stream) {
    if (has_do && has_g) return bwd_mode<HD, true, true>(p, BH, parts, stream);
    if (has_g) return bwd_mode<HD, false, true>(p, BH, parts, stream);
    return bwd_mode<HD, true, false>(p, BH, parts, stream);
}

}  // namespace

int fwd_f32(const FwdParamsF32& p, int BH, bool jvp, hipStream_t stream) {
    if (p.D <= 32) return fwd_hd<32>(p, BH, jvp, stream);
    if (p.D <= 64) return fwd_hd<64>(p, BH, jvp, stream);
    return fwd_hd<128>(p, BH, jvp, stream);
}

int bwd_f32(const BwdParamsF32& p, int BH, bool has_do, bool has_g, int parts, hipStream_t stream) {
    if (p.D <= 32) return bwd_hd<32>(p, BH, has_do, has_g, parts, stream);
    if (p.D <= 64) return bwd_hd<64>(p, BH, has_do, has_g, parts, stream);
    return bwd_hd<128>(p, BH, has_do, has_g, parts, stream);
}

}  // namespace sjvp
