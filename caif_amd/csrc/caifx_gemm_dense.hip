// The tiled matrix-core GEMM for a weight stored in the 16-bit compute type itself (the bf16 / bf16 and
// fp16 / fp16 cells of the FrozenLinear grid, src/caif_device_frozen_linear.cpp:301-318 same-dtype view +
// :465-509 GemmEx): the producers copy the stored values into the operand tiles, everything else is the kernel of
// caifx_gemm_tile.hpp.  A translation unit of its own so that it compiles beside the integer-code instantiations.
#include "caifx_gemm_tile.hpp"

namespace caifx {
namespace gemm_tile {

namespace {
template <typename CT, typename XT> int pick(const TileArgs &t, bool backward, bool grouped, hipStream_t s)
{
  return backward ? launch_tile<CT, XT, W_DENSE16, true>(t, grouped, s) : launch_tile<CT, XT, W_DENSE16, false>(t, grouped, s);
}
}  // namespace

int dense_launch(const TileArgs &t, int compute_dtype, int x_dtype, bool backward, bool grouped, hipStream_t s)
{
  if (compute_dtype == CAIFX_BF16)
    return x_dtype == CAIFX_F32 ? pick<bf16_t, float>(t, backward, grouped, s) : pick<bf16_t, bf16_t>(t, backward, grouped, s);
  if (compute_dtype == CAIFX_F16)
    return x_dtype == CAIFX_F32 ? pick<f16_t, float>(t, backward, grouped, s) : pick<f16_t, f16_t>(t, backward, grouped, s);
  return CAIFX_ERR_UNSUPPORTED;
}

}  // namespace gemm_tile
}  // namespace caifx
