// The fp32-storage instantiations of the plain GEMM (kernels and launch logic in gemm_core.h), in a translation
// unit of their own so that they compile beside the bf16 ones of gemm.hip.
#include "gemm_core.h"

namespace ptj_gemm_detail {
int launch_plain_f32(const GemmArgs& g, int splits, hipStream_t st) { return gemm_impl<float>(g, splits, st); }
}  // namespace ptj_gemm_detail
