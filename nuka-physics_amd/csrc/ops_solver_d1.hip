// Dense instantiations of the block-descent kernel (three waves a SIMD) for reduced blocks whose sweeps are at most 20
// wide (full width, width of the sweeps): 24/12, 28/16, 32/16, 36/20, 40/20.
#define NKH_SOLVER_DENSE
#include "ops_solver_kernel.h"
namespace nkh {
namespace solver {
namespace dense {
template __global__ void BlockDescentTileKernel<24, true, 12>(ModelView, DataView, BlockDescentSolveParams, uint32_t, uint32_t, uint32_t, uint32_t);
template __global__ void BlockDescentTileKernel<28, true, 16>(ModelView, DataView, BlockDescentSolveParams, uint32_t, uint32_t, uint32_t, uint32_t);
template __global__ void BlockDescentTileKernel<32, true, 16>(ModelView, DataView, BlockDescentSolveParams, uint32_t, uint32_t, uint32_t, uint32_t);
template __global__ void BlockDescentTileKernel<36, true, 20>(ModelView, DataView, BlockDescentSolveParams, uint32_t, uint32_t, uint32_t, uint32_t);
template __global__ void BlockDescentTileKernel<40, true, 20>(ModelView, DataView, BlockDescentSolveParams, uint32_t, uint32_t, uint32_t, uint32_t);
}  // namespace dense
}  // namespace solver
}  // namespace nkh
