// Instantiations of the block-descent kernel for reduced blocks (contact heads only; full width, width of the sweeps): 36/20, 44/24.
#include "ops_solver_kernel.h"
namespace nkh {
namespace solver {
template __global__ void BlockDescentTileKernel<36, true, 20>(ModelView, DataView, BlockDescentSolveParams, uint32_t, uint32_t, uint32_t, uint32_t);
template __global__ void BlockDescentTileKernel<44, true, 24>(ModelView, DataView, BlockDescentSolveParams, uint32_t, uint32_t, uint32_t, uint32_t);
}  // namespace solver
}  // namespace nkh
