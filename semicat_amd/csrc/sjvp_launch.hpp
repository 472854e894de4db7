// Host-side launch plumbing shared by the translation units of the library: the kernels are
// instantiated per element type in separate units (compiled in parallel), each exporting the
// selection functions declared here; sjvp_api.hip validates arguments and calls them.
#pragma once
#include <hip/hip_runtime.h>

#include "../../include/sjvp.h"
#include "sjvp_bwd.hpp"
#include "sjvp_f32.hpp"
#include "sjvp_fwd.hpp"

namespace sjvp {

// Launch with the status of this launch only (not the thread's sticky last error).
template <typename K, typename P>
int launch(K kernel, int grid, int smem_bytes, hipStream_t stream, const P& params, int threads) {
    if (smem_bytes > 64 * 1024) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                hipFuncAttributeMaxDynamicSharedMemorySize, smem_bytes) != hipSuccess)
            return SJVP_ERR_LAUNCH;
    }
    P copy = params;
    void* args[] = {&copy};
    const hipError_t rc = hipLaunchKernel(reinterpret_cast<const void*>(kernel), dim3(grid), dim3(threads), args,
                                          (size_t)smem_bytes, stream);
    return rc == hipSuccess ? SJVP_OK : SJVP_ERR_LAUNCH;
}

// Forward: 16-wide LDS-DMA kernels (16-byte aligned rows) and the 32-wide register-staged ones.
template <typename T> int fwd_vec(const FwdParams& p, int grid, bool jvp, hipStream_t stream);
template <typename T> int fwd_any(const FwdParams& p, int grid, bool jvp, hipStream_t stream);

// Backward: the single launch (short key axes, D <= 64), the 16-wide pair and the 32-wide pair.
template <typename T> int bwd_fused(const BwdParams& p, int BH, bool has_do, bool has_g, hipStream_t stream);
template <typename T> int bwd_pair_vec(const BwdParams& p, int BH, bool has_do, bool has_g, int parts, hipStream_t stream);
template <typename T> int bwd_pair_any(const BwdParams& p, int BH, bool has_do, bool has_g, int parts, hipStream_t stream);

// fp32 tensors with bf16 arithmetic (the cast folded into the loads and stores): 32-wide kernels.
// The views carry fp32 pointers cast to elem_t* and strides counted in 2-byte units.
int fwd_f32io(const FwdParams& p, int grid, bool jvp, hipStream_t stream);
int bwd_f32io(const BwdParams& p, int BH, bool has_do, bool has_g, int parts, hipStream_t stream);

// fp32 correctness mode (vector ALUs): forward, and the row-owned + column-owned backward pair.
int fwd_f32(const FwdParamsF32& p, int BH, bool jvp, hipStream_t stream);
int bwd_f32(const BwdParamsF32& p, int BH, bool has_do, bool has_g, int parts, hipStream_t stream);

}  // namespace sjvp
