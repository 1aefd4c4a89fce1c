// Large-M MFMA dequant-GEMM (placeholder until the tiled kernels land: reports unsupported so
// that callers take the shape-agnostic kernels).
#include "caifx_internal.hpp"

namespace caifx {

int mfma_forward(const GemmArgs &, hipStream_t) { return CAIFX_ERR_UNSUPPORTED; }
int mfma_backward(const GemmArgs &, hipStream_t) { return CAIFX_ERR_UNSUPPORTED; }
size_t mfma_workspace_bytes(const GemmArgs &, bool) { return 0; }

}  // namespace caifx
