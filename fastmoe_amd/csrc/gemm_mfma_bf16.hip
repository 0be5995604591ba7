// The bf16 instantiations of the matrix-core grouped GEMM (gemm_mfma_impl.h).
#include "gemm_mfma_impl.h"

namespace fmoe {
template int launch_gemm_mfma_typed<__hip_bfloat16>(int, const GemmArgs&, hipStream_t);
template int launch_gemm_mfma_bwd_typed<__hip_bfloat16>(const GemmArgs&, const GemmArgs&,
                                                        hipStream_t);
}  // namespace fmoe
