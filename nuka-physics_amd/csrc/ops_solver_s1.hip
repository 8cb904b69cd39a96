// Instantiations of the block-descent kernel (contacts-only variant) for padded widths 28, 32, 36.
#include "ops_solver_kernel.h"
namespace nkh {
namespace solver {
template __global__ void BlockDescentTileKernel<28, true>(ModelView, DataView, BlockDescentSolveParams, uint32_t, uint32_t, uint32_t, uint32_t);
template __global__ void BlockDescentTileKernel<32, true>(ModelView, DataView, BlockDescentSolveParams, uint32_t, uint32_t, uint32_t, uint32_t);
template __global__ void BlockDescentTileKernel<36, true>(ModelView, DataView, BlockDescentSolveParams, uint32_t, uint32_t, uint32_t, uint32_t);
}  // namespace solver
}  // namespace nkh
