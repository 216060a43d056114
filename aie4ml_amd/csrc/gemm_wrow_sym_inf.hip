// gemm_wrow_kernel for one rounding kind (gemm_wrow.hpp).
#include "gemm_wrow.hpp"

namespace a4g {
hipError_t launch_wrow_sym_inf(const GemmArgs& g, hipStream_t stream) { return launch_wrow_kind<1>(g, stream); }
}  // namespace a4g
