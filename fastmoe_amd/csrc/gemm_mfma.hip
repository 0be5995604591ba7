// Host-side dispatch of the bf16 / f16 matrix-core grouped GEMM: whether a call fits
// the kernels, and which element type's instantiations (gemm_mfma_bf16.hip,
// gemm_mfma_f16.hip, both from gemm_mfma_impl.h) run it.
#include "dma_desc.h"
#include "gemm.h"

namespace fmoe {

template <typename T> int launch_gemm_mfma_typed(int mode, const GemmArgs& g, hipStream_t s);
template <typename T>
int launch_gemm_mfma_bwd_typed(const GemmArgs& gd, const GemmArgs& gw, hipStream_t s);
extern template int launch_gemm_mfma_typed<__hip_bfloat16>(int, const GemmArgs&, hipStream_t);
extern template int launch_gemm_mfma_typed<__half>(int, const GemmArgs&, hipStream_t);
extern template int launch_gemm_mfma_bwd_typed<__hip_bfloat16>(const GemmArgs&, const GemmArgs&,
                                                               hipStream_t);
extern template int launch_gemm_mfma_bwd_typed<__half>(const GemmArgs&, const GemmArgs&,
                                                       hipStream_t);

bool gemm_mfma_supported(int mode, const GemmArgs& g, int dtype) {
  (void)mode;
  if (dtype != FMOE_BF16 && dtype != FMOE_F16) return false;
  if (g.in_feat % 8 != 0 || g.out_feat % 8 != 0) return false;
  // tile-relative byte offsets are 32-bit: 256 rows of either feature size
  if (!dma_ld_supported(g.in_feat) || !dma_ld_supported(g.out_feat)) return false;
  if (((uintptr_t)g.a | (uintptr_t)g.b | (uintptr_t)g.c) % 16 != 0) return false;
  return true;
}

int launch_gemm_mfma_bwd(const GemmArgs& gd, const GemmArgs& gw, int dtype, hipStream_t s) {
  if (!gemm_mfma_supported(GEMM_DGRAD, gd, dtype) || !gemm_mfma_supported(GEMM_WGRAD, gw, dtype))
    return set_error(FMOE_ERR_UNSUPPORTED, "grouped GEMM: shape not MFMA-aligned");
  if (dtype == FMOE_BF16) return launch_gemm_mfma_bwd_typed<__hip_bfloat16>(gd, gw, s);
  return launch_gemm_mfma_bwd_typed<__half>(gd, gw, s);
}

int launch_gemm_mfma(int mode, const GemmArgs& g, int dtype, hipStream_t s) {
  if (!gemm_mfma_supported(mode, g, dtype))
    return set_error(FMOE_ERR_UNSUPPORTED, "grouped GEMM: shape not MFMA-aligned");
  if (dtype == FMOE_BF16) return launch_gemm_mfma_typed<__hip_bfloat16>(mode, g, s);
  return launch_gemm_mfma_typed<__half>(mode, g, s);
}

}  // namespace fmoe
