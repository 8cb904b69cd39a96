// Instantiations of the block-descent kernel (general variant) for padded widths 40, 44, 48.
#include "ops_solver_kernel.h"
namespace nkh {
namespace solver {
template __global__ void BlockDescentTileKernel<40, false>(ModelView, DataView, BlockDescentSolveParams, uint32_t, uint32_t, uint32_t, uint32_t);
template __global__ void BlockDescentTileKernel<44, false>(ModelView, DataView, BlockDescentSolveParams, uint32_t, uint32_t, uint32_t, uint32_t);
template __global__ void BlockDescentTileKernel<48, false>(ModelView, DataView, BlockDescentSolveParams, uint32_t, uint32_t, uint32_t, uint32_t);
}  // namespace solver
}  // namespace nkh
