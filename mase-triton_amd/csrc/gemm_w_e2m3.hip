// MXFP GEMM kernels for weights in E2M3; see gemm_impl.h.
#include "gemm_impl.h"

namespace mase {
int gemm_w_e2m3(const GemmArgs& g) { return gemm_for_weight_format<SFmt<2, 3>>(g); }
}  // namespace mase
