// Instantiations of the block-descent kernel (general variant) for padded widths 52, 56.
#include "ops_solver_kernel.h"
namespace nkh {
namespace solver {
template __global__ void BlockDescentTileKernel<52, false>(ModelView, DataView, BlockDescentSolveParams, uint32_t, uint32_t, uint32_t, uint32_t);
template __global__ void BlockDescentTileKernel<56, false>(ModelView, DataView, BlockDescentSolveParams, uint32_t, uint32_t, uint32_t, uint32_t);
}  // namespace solver
}  // namespace nkh
