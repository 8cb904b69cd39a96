// Instantiations of the block-descent kernel (general variant) for padded widths 4, 8, 12, 16, 20, 24.
#include "ops_solver_kernel.h"
namespace nkh {
namespace solver {
template __global__ void BlockDescentTileKernel<4, false>(ModelView, DataView, BlockDescentSolveParams, uint32_t, uint32_t, uint32_t, uint32_t);
template __global__ void BlockDescentTileKernel<8, false>(ModelView, DataView, BlockDescentSolveParams, uint32_t, uint32_t, uint32_t, uint32_t);
template __global__ void BlockDescentTileKernel<12, false>(ModelView, DataView, BlockDescentSolveParams, uint32_t, uint32_t, uint32_t, uint32_t);
template __global__ void BlockDescentTileKernel<16, false>(ModelView, DataView, BlockDescentSolveParams, uint32_t, uint32_t, uint32_t, uint32_t);
template __global__ void BlockDescentTileKernel<20, false>(ModelView, DataView, BlockDescentSolveParams, uint32_t, uint32_t, uint32_t, uint32_t);
template __global__ void BlockDescentTileKernel<24, false>(ModelView, DataView, BlockDescentSolveParams, uint32_t, uint32_t, uint32_t, uint32_t);
}  // namespace solver
}  // namespace nkh
