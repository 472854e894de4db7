// Translation unit: single-launch backward (short key axes) for one element type (SJVP_T).
#include "sjvp_bwd16.hpp"
#include "sjvp_launch.hpp"

namespace sjvp {
namespace {

constexpr int kRingFused = 3;

template <typename T, int HD, bool HAS_DO, bool HAS_G>
int fused_mode(const BwdParams& p, int BH, hipStream_t stream) {
    if constexpr (HD == 64) {
        if (p.rope.cos)  // rotary embedding folded in
            return launch(bwd_fused16_kernel<T, HD, kRingFused, HAS_DO, HAS_G, true>, BH,
                          Fused16Smem<HD, kRingFused, HAS_DO, HAS_G>::bytes, stream, p, kThreads16);
    }
    return launch(bwd_fused16_kernel<T, HD, kRingFused, HAS_DO, HAS_G>, BH,
                  Fused16Smem<HD, kRingFused, HAS_DO, HAS_G>::bytes, stream, p, kThreads16);
}

template <typename T, int HD>
int fused_hd(const BwdParams& p, int BH, bool has_do, bool has_g, hipStream_t stream) {
    if (has_do && has_g) return fused_mode<T, HD, true, true>(p, BH, stream);
    if (has_g) return fused_mode<T, HD, false, true>(p, BH, stream);
    return fused_mode<T, HD, true, false>(p, BH, stream);
}

}  // namespace

template <>
int bwd_fused<SJVP_T>(const BwdParams& p, int BH, bool has_do, bool has_g, hipStream_t stream) {
    if (p.D <= 32) return fused_hd<SJVP_T, 32>(p, BH, has_do, has_g, stream);
    return fused_hd<SJVP_T, 64>(p, BH, has_do, has_g, stream);
}

}  // namespace sjvp
