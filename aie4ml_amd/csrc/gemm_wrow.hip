// Dispatch of the Dense kernel for short reductions that keeps weights in registers and streams 64-row pieces
// (gemm_wrow.hpp); its instances are compiled per rounding kind in gemm_wrow_*.hip.
#include "gemm_wrow.hpp"

namespace a4g {

// The shapes of wreg_applicable, with the weights also at hand in fragment order, in the rounding modes that have an
// instance (the two rarest keep the kernel of gemm_wreg.hip).
bool wrow_applicable(const GemmArgs& g) {
    return g.Wf != nullptr && aligned16(g.Wf) && g.mode != A4G_RND_SYMMETRIC_ZERO && g.mode != A4G_RND_CONV_ODD &&
           (static_cast<int64_t>(g.M) + 2 * WS_ROWS) * g.lda < (int64_t{1} << 31) && rowpacked_bytes(g.N + WS_BN, g.K) < (int64_t{1} << 31);
}

hipError_t launch_wrow(const GemmArgs& g, hipStream_t stream) {
    switch (g.mode) {
    case A4G_RND_SYMMETRIC_INF: return launch_wrow_sym_inf(g, stream);
    case A4G_RND_CONV_EVEN: return launch_wrow_conv_even(g, stream);
    default: return launch_wrow_plain(g, stream);
    }
}

}  // namespace a4g
