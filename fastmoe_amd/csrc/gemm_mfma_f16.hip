// The f16 instantiations of the matrix-core grouped GEMM (gemm_mfma_impl.h).
#include "gemm_mfma_impl.h"

namespace fmoe {
template int launch_gemm_mfma_typed<__half>(int, const GemmArgs&, hipStream_t);
template int launch_gemm_mfma_bwd_typed<__half>(const GemmArgs&, const GemmArgs&, hipStream_t);
}  // namespace fmoe
