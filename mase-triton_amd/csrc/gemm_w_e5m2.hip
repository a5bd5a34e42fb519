// MXFP GEMM kernels for weights in E5M2; see gemm_impl.h.
#include "gemm_impl.h"

namespace mase {
int gemm_w_e5m2(const GemmArgs& g) { return gemm_for_weight_format<SFmt<5, 2>>(g); }
}  // namespace mase
