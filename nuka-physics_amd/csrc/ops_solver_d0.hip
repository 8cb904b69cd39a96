// Dense instantiations of the block-descent kernel (three waves a SIMD, contact heads only) for padded widths 4 ... 20.
#define NKH_SOLVER_DENSE
#include "ops_solver_kernel.h"
namespace nkh {
namespace solver {
namespace dense {
template __global__ void BlockDescentTileKernel<4, true>(ModelView, DataView, BlockDescentSolveParams, uint32_t, uint32_t, uint32_t, uint32_t);
template __global__ void BlockDescentTileKernel<8, true>(ModelView, DataView, BlockDescentSolveParams, uint32_t, uint32_t, uint32_t, uint32_t);
template __global__ void BlockDescentTileKernel<12, true>(ModelView, DataView, BlockDescentSolveParams, uint32_t, uint32_t, uint32_t, uint32_t);
template __global__ void BlockDescentTileKernel<16, true>(ModelView, DataView, BlockDescentSolveParams, uint32_t, uint32_t, uint32_t, uint32_t);
template __global__ void BlockDescentTileKernel<20, true>(ModelView, DataView, BlockDescentSolveParams, uint32_t, uint32_t, uint32_t, uint32_t);
}  // namespace dense
}  // namespace solver
}  // namespace nkh
