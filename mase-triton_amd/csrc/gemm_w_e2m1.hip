// MXFP GEMM kernels for weights in E2M1; see gemm_impl.h.
#include "gemm_impl.h"

namespace mase {
int gemm_w_e2m1(const GemmArgs& g) { return gemm_for_weight_format<SFmt<2, 1>>(g); }
}  // namespace mase
