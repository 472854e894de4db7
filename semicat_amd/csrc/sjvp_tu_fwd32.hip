// Translation unit: 32-wide forward kernels (inputs of any alignment; register-staged copies, one
// stage in LDS) for one element type (SJVP_T = Bf16 or Fp16).
#include "sjvp_fwd.hpp"
#include "sjvp_launch.hpp"

namespace sjvp {
namespace {

template <typename T, int HD>
int fwd_hd(const FwdParams& p, int grid, bool jvp, hipStream_t stream) {
    if (jvp) return launch(fwd_kernel<T, HD, true>, grid, FwdSmem<HD, true>::bytes, stream, p, kThreads);
    return launch(fwd_kernel<T, HD, false>, grid, FwdSmem<HD, false>::bytes, stream, p, kThreads);
}

}  // namespace

template <>
int fwd_any<SJVP_T>(const FwdParams& p, int grid, bool jvp, hipStream_t stream) {
    if (p.D <= 32) return fwd_hd<SJVP_T, 32>(p, grid, jvp, stream);
    if (p.D <= 64) return fwd_hd<SJVP_T, 64>(p, grid, jvp, stream);
    return fwd_hd<SJVP_T, 128>(p, grid, jvp, stream);
}

}  // namespace sjvp
