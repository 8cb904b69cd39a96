// Launch side of the block-descent solve: head capacity, LDS sizing and the table of kernels, one per padded width.
// The kernel template lives in ops_solver_kernel.h; its instantiations are spread over ops_solver_w*.hip so that
// they compile in parallel.
#include "ops_solver_kernel.h"

namespace nkh {
namespace solver {
#define NKH_DECLARE_WIDTH(N) \
    extern template __global__ void BlockDescentTileKernel<N>(ModelView, DataView, BlockDescentSolveParams, uint32_t);
NKH_DECLARE_WIDTH(4) NKH_DECLARE_WIDTH(8) NKH_DECLARE_WIDTH(12) NKH_DECLARE_WIDTH(16) NKH_DECLARE_WIDTH(20) NKH_DECLARE_WIDTH(24)
NKH_DECLARE_WIDTH(28) NKH_DECLARE_WIDTH(32) NKH_DECLARE_WIDTH(36) NKH_DECLARE_WIDTH(40) NKH_DECLARE_WIDTH(44) NKH_DECLARE_WIDTH(48)
NKH_DECLARE_WIDTH(52) NKH_DECLARE_WIDTH(56) NKH_DECLARE_WIDTH(60) NKH_DECLARE_WIDTH(64)
#undef NKH_DECLARE_WIDTH
}  // namespace solver


uint32_t SolverHeadCapacity(const ModelView& m, uint32_t slots, size_t lds_budget_bytes) {
    const uint32_t want = slots * (m.max_points_per_slot == 0u ? kPointsPerSlot : m.max_points_per_slot);
    for (uint32_t cap = want; cap >= 1u; --cap)
        if (size_t{solver::SolverLdsFloats(m.dof, cap)} * sizeof(float) <= lds_budget_bytes) return cap;
    return 0u;
}

namespace {
using namespace solver;
using SolverKernel = void (*)(ModelView, DataView, BlockDescentSolveParams, uint32_t);
// One instantiation per padded width.
const SolverKernel kSolverKernels[16] = {
    BlockDescentTileKernel<4>, BlockDescentTileKernel<8>, BlockDescentTileKernel<12>, BlockDescentTileKernel<16>,
    BlockDescentTileKernel<20>, BlockDescentTileKernel<24>, BlockDescentTileKernel<28>, BlockDescentTileKernel<32>,
    BlockDescentTileKernel<36>, BlockDescentTileKernel<40>, BlockDescentTileKernel<44>, BlockDescentTileKernel<48>,
    BlockDescentTileKernel<52>, BlockDescentTileKernel<56>, BlockDescentTileKernel<60>, BlockDescentTileKernel<64>};
}  // namespace

void InitSolverKernels() {
    for (SolverKernel kernel : kSolverKernels) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        (void)hipGetLastError();
    }
}

Status OpBlockDescentSolve(const ModelView& m, const DataView& d, const void* params, hipStream_t stream) {
    const auto* p = static_cast<const BlockDescentSolveParams*>(params);
    if (p == nullptr) return Status::Failed;
    if (p->env_count == 0u || p->rows_per_env == 0u || p->articulation_count == 0u) return Status::Ok;
    if (p->articulation_count != p->env_count || m.dof == 0u || m.dof > kMaxDof || p->max_dof != m.max_dof ||
        p->iterations == 0u) return Status::InvalidArgument;
    const size_t budget = 150u * 1024u;
    const uint32_t cap = SolverHeadCapacity(m, p->contact_slots_per_env == 0u ? 1u : p->contact_slots_per_env, budget);
    if (cap == 0u) return Status::InvalidArgument;
    const size_t lds = size_t{solver::SolverLdsFloats(m.dof, cap)} * sizeof(float);
    hipLaunchKernelGGL(kSolverKernels[solver::PaddedWidth(m.dof) / 4u - 1u], dim3(p->env_count), dim3(solver::kWave), lds, stream, m, d, *p, cap);
    return hipGetLastError() == hipSuccess ? Status::Ok : Status::Failed;
}

}  // namespace nkh
