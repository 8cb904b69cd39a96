// Instantiations of the block-descent kernel for reduced blocks (contact heads only; full width, width of the sweeps): 64/32.
#include "ops_solver_kernel.h"
namespace nkh {
namespace solver {
template __global__ void BlockDescentTileKernel<64, true, 32>(ModelView, DataView, BlockDescentSolveParams, uint32_t, uint32_t, uint32_t, uint32_t);
}  // namespace solver
}  // namespace nkh
