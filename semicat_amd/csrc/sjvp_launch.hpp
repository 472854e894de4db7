// Host-side launch plumbing shared by the translation units of the library: the kernels are
// instantiated per element type in separate units (compiled in parallel), each exporting the
// selection functions declared here; sjvp_api.hip validates arguments and calls them.
#pragma once
#include <hip/hip_runtime.h>

#include <atomic>

#include "../../include/sjvp.h"
#include "sjvp_bwd.hpp"
#include "sjvp_f32.hpp"
#include "sjvp_fwd.hpp"

namespace sjvp {

// Launch with the status of this launch only (not the thread's sticky last error).
// A kernel that needs more than 64 KB of LDS has its limit raised first.  K is a function pointer
// type shared by many kernels, so the (kernel, device) pairs already served are remembered in a small
// table: the attribute call, which costs host time on every launch otherwise, runs once per pair.
inline bool lds_limit_raised(const void* kernel, int smem_bytes) {
    constexpr int kSlots = 512;
    struct Slot {
        std::atomic<const void*> kernel{nullptr};
        std::atomic<int> bytes{0};
    };
    static Slot table[kSlots][8];  // open addressing over kernels, by device (devices beyond 8 are not cached)
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return false;
    Slot* hit = nullptr;
    if (dev >= 0 && dev < 8) {
        size_t h = (reinterpret_cast<uintptr_t>(kernel) >> 4) % kSlots;
        for (int probe = 0; probe < kSlots; ++probe, h = (h + 1) % kSlots) {
            Slot& s = table[h][dev];
            const void* cur = s.kernel.load(std::memory_order_acquire);
            if (cur == kernel) {
                if (s.bytes.load(std::memory_order_acquire) >= smem_bytes) return true;
                hit = &s;
                break;
            }
            if (cur == nullptr) {
                const void* expected = nullptr;
                if (s.kernel.compare_exchange_strong(expected, kernel, std::memory_order_acq_rel) || expected == kernel) {
                    hit = &s;
                    break;
                }
            }
        }
    }
    if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, smem_bytes) != hipSuccess) return false;
    if (hit) hit->bytes.store(smem_bytes, std::memory_order_release);
    return true;
}

template <typename K, typename P>
int launch(K kernel, int grid, int smem_bytes, hipStream_t stream, const P& params, int threads) {
    if (smem_bytes > 64 * 1024 && !lds_limit_raised(reinterpret_cast<const void*>(kernel), smem_bytes))
        return SJVP_ERR_LAUNCH;
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
