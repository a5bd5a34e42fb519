// MXFP GEMM kernels for weights in E3M2; see gemm_impl.h.
#include "gemm_impl.h"

namespace mase {
int gemm_w_e3m2(const GemmArgs& g) { return gemm_for_weight_format<SFmt<3, 2>>(g); }
}  // namespace mase
