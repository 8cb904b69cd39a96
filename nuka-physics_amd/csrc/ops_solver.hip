// Launch side of the block-descent solve: head capacity, LDS sizing and the table of kernels, one per padded width.
// The kernel template lives in ops_solver_kernel.h; its instantiations are spread over ops_solver_w*.hip (general)
// and ops_solver_s*.hip (contact heads only) so that they compile in parallel.
#include "ops_solver_kernel.h"

namespace nkh {
namespace solver {
#define NKH_DECLARE_WIDTH(N) \
    extern template __global__ void BlockDescentTileKernel<N, false>(ModelView, DataView, BlockDescentSolveParams, uint32_t, uint32_t, uint32_t, uint32_t); \
    extern template __global__ void BlockDescentTileKernel<N, true>(ModelView, DataView, BlockDescentSolveParams, uint32_t, uint32_t, uint32_t, uint32_t);
NKH_DECLARE_WIDTH(4) NKH_DECLARE_WIDTH(8) NKH_DECLARE_WIDTH(12) NKH_DECLARE_WIDTH(16) NKH_DECLARE_WIDTH(20) NKH_DECLARE_WIDTH(24)
NKH_DECLARE_WIDTH(28) NKH_DECLARE_WIDTH(32) NKH_DECLARE_WIDTH(36) NKH_DECLARE_WIDTH(40) NKH_DECLARE_WIDTH(44) NKH_DECLARE_WIDTH(48)
NKH_DECLARE_WIDTH(52) NKH_DECLARE_WIDTH(56) NKH_DECLARE_WIDTH(60) NKH_DECLARE_WIDTH(64)
#undef NKH_DECLARE_WIDTH
// reduced blocks (contact heads only): width N with the sweeps K wide
#define NKH_DECLARE_REDUCED(N, K) \
    extern template __global__ void BlockDescentTileKernel<N, true, K>(ModelView, DataView, BlockDescentSolveParams, uint32_t, uint32_t, uint32_t, uint32_t);
NKH_DECLARE_REDUCED(24, 12) NKH_DECLARE_REDUCED(28, 16) NKH_DECLARE_REDUCED(32, 16) NKH_DECLARE_REDUCED(36, 20) NKH_DECLARE_REDUCED(40, 20)
NKH_DECLARE_REDUCED(44, 24) NKH_DECLARE_REDUCED(48, 24) NKH_DECLARE_REDUCED(52, 28) NKH_DECLARE_REDUCED(56, 28) NKH_DECLARE_REDUCED(60, 32)
NKH_DECLARE_REDUCED(64, 32)
#undef NKH_DECLARE_REDUCED
// The dense build of the same template (ops_solver_kernel.h compiled with NKH_SOLVER_DENSE: three waves a SIMD), for the
// widths it is instantiated at in ops_solver_d*.hip.
namespace dense {
template <int N, bool kContactsOnly, int K = N>
__global__ void BlockDescentTileKernel(ModelView, DataView, BlockDescentSolveParams, uint32_t, uint32_t, uint32_t, uint32_t);
#define NKH_DECLARE_DENSE(N, K) \
    extern template __global__ void BlockDescentTileKernel<N, true, K>(ModelView, DataView, BlockDescentSolveParams, uint32_t, uint32_t, uint32_t, uint32_t);
NKH_DECLARE_DENSE(4, 4) NKH_DECLARE_DENSE(8, 8) NKH_DECLARE_DENSE(12, 12) NKH_DECLARE_DENSE(16, 16) NKH_DECLARE_DENSE(20, 20)
NKH_DECLARE_DENSE(24, 12) NKH_DECLARE_DENSE(28, 16) NKH_DECLARE_DENSE(32, 16) NKH_DECLARE_DENSE(36, 20) NKH_DECLARE_DENSE(40, 20)
#undef NKH_DECLARE_DENSE
}  // namespace dense
}  // namespace solver


// Heads the solver's LDS holds: the contact heads (each stages three Jacobian rows) plus one unit head per joint row
// slot.  Returns the contact-head capacity that fits `lds_budget_bytes`, 0 when not even one does.
uint32_t SolverHeadCapacity(const ModelView& m, uint32_t slots, size_t lds_budget_bytes) {
    // a contact point is one head, or four under the pyramidal cone of the MuJoCo law (one scalar head an edge)
    const uint32_t heads_per_point = m.any_mujoco != 0u && m.contact_cone == 0u ? kRowsPerPoint : 1u;
    const uint32_t want = slots * (m.max_points_per_slot == 0u ? kPointsPerSlot : m.max_points_per_slot) * heads_per_point;
    const uint32_t joint_heads = m.joint_limit_rows + m.joint_friction_rows + m.joint_drive_rows;
    for (uint32_t staged = want; staged >= 1u; --staged)
        if (size_t{solver::SolverLdsFloats(m.dof, staged + joint_heads, staged)} * sizeof(float) <= lds_budget_bytes) return staged;
    return 0u;
}

namespace {
using namespace solver;

// OrderTilesKernel (block_descent_tile.cuh:3097-3121 orders tiles for its persistent kernel; here the order feeds the
// grid): environments sorted by the work their previous solve took, costliest first, so that the few long solves
// start at once instead of trailing the launch.  One workgroup, counting sort on a 256-level key; the order inside a
// level is arbitrary, which changes when an environment runs and nothing it computes.
__global__ void __launch_bounds__(1024) OrderTilesKernel(DataView d, uint32_t env_count) {
    __shared__ uint32_t bins[256];
    __shared__ uint32_t top;
    const uint32_t t = threadIdx.x;
    if (t < 256u) bins[t] = 0u;
    if (t == 0u) top = 0u;
    __syncthreads();
    uint32_t largest = 0u;
    for (uint32_t e = t; e < env_count; e += 1024u) largest = max(largest, d.solver_cost[e]);
    atomicMax(&top, largest);
    __syncthreads();
    const uint32_t scale = top / 256u + 1u;
    for (uint32_t e = t; e < env_count; e += 1024u) atomicAdd(&bins[255u - min(d.solver_cost[e] / scale, 255u)], 1u);
    __syncthreads();
    // exclusive prefix of the 256 counts: a scan inside each of the first four wavefronts, then their totals
    __shared__ uint32_t wave_total[4];
    uint32_t count = 0u, through = 0u;
    if (t < 256u) {
        count = bins[t];
        through = count;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const uint32_t other = __shfl_up(through, o, 64);
            if (int(t & 63u) >= o) through += other;
        }
        if ((t & 63u) == 63u) wave_total[t >> 6u] = through;
    }
    __syncthreads();
    if (t < 256u) {
        uint32_t before = 0u;
        for (uint32_t w = 0u; w < (t >> 6u); ++w) before += wave_total[w];
        bins[t] = before + through - count;
    }
    __syncthreads();
    for (uint32_t e = t; e < env_count; e += 1024u) d.tile_order[atomicAdd(&bins[255u - min(d.solver_cost[e] / scale, 255u)], 1u)] = e;
}


using SolverKernel = void (*)(ModelView, DataView, BlockDescentSolveParams, uint32_t, uint32_t, uint32_t, uint32_t);
// Two instantiations per padded width: the general one, and the one for worlds whose heads are contact heads only,
// at most one a lane.
#define NKH_WIDTHS(V) \
    BlockDescentTileKernel<4, V>, BlockDescentTileKernel<8, V>, BlockDescentTileKernel<12, V>, BlockDescentTileKernel<16, V>, \
    BlockDescentTileKernel<20, V>, BlockDescentTileKernel<24, V>, BlockDescentTileKernel<28, V>, BlockDescentTileKernel<32, V>, \
    BlockDescentTileKernel<36, V>, BlockDescentTileKernel<40, V>, BlockDescentTileKernel<44, V>, BlockDescentTileKernel<48, V>, \
    BlockDescentTileKernel<52, V>, BlockDescentTileKernel<56, V>, BlockDescentTileKernel<60, V>, BlockDescentTileKernel<64, V>
const SolverKernel kSolverKernels[2][16] = {{NKH_WIDTHS(false)}, {NKH_WIDTHS(true)}};
#undef NKH_WIDTHS
// One reduced instantiation per padded width from 24 on: the sweeps run at about half the width.  A world takes it
// when no contact can reach a coordinate from that width on (ModelView::contact_dof_end).
struct ReducedKernel { uint32_t width, reduced; SolverKernel kernel; };
const ReducedKernel kReducedKernels[] = {
    {24u, 12u, BlockDescentTileKernel<24, true, 12>}, {28u, 16u, BlockDescentTileKernel<28, true, 16>}, {32u, 16u, BlockDescentTileKernel<32, true, 16>},
    {36u, 20u, BlockDescentTileKernel<36, true, 20>}, {40u, 20u, BlockDescentTileKernel<40, true, 20>}, {44u, 24u, BlockDescentTileKernel<44, true, 24>},
    {48u, 24u, BlockDescentTileKernel<48, true, 24>}, {52u, 28u, BlockDescentTileKernel<52, true, 28>}, {56u, 28u, BlockDescentTileKernel<56, true, 28>},
    {60u, 32u, BlockDescentTileKernel<60, true, 32>}, {64u, 32u, BlockDescentTileKernel<64, true, 32>}};
// The dense kernels: (padded width of the block, width of the sweeps), contact heads only.
const ReducedKernel kDenseKernels[] = {
    {4u, 4u, dense::BlockDescentTileKernel<4, true, 4>}, {8u, 8u, dense::BlockDescentTileKernel<8, true, 8>},
    {12u, 12u, dense::BlockDescentTileKernel<12, true, 12>}, {16u, 16u, dense::BlockDescentTileKernel<16, true, 16>},
    {20u, 20u, dense::BlockDescentTileKernel<20, true, 20>}, {24u, 12u, dense::BlockDescentTileKernel<24, true, 12>},
    {28u, 16u, dense::BlockDescentTileKernel<28, true, 16>}, {32u, 16u, dense::BlockDescentTileKernel<32, true, 16>},
    {36u, 20u, dense::BlockDescentTileKernel<36, true, 20>}, {40u, 20u, dense::BlockDescentTileKernel<40, true, 20>}};
// Batches from this many environments on take a dense kernel where there is one: twice the 3072 wave slots three waves
// a SIMD make of 256 compute units.  A dense wave runs slower than a two-wave one (fewer registers, some spilled), so
// below that the launch is over sooner with the two-wave kernel: its length is then the longest environment's, not the
// machine's throughput.  Measured on the 36-coordinate humanoid: 4096 environments +9 % with the dense kernel, 5120
// +1 %, 6144 -8 %, 8192 -8 %, 65536 -9 %; the 18-coordinate quadruped -9 % at 6144 and -14 % at 65536.
#ifndef NKH_DENSE_BATCH
#define NKH_DENSE_BATCH 6144
#endif
constexpr uint32_t kDenseBatch = NKH_DENSE_BATCH;
}  // namespace

void InitSolverKernels() {
    for (const auto& variant : kSolverKernels) {
        for (SolverKernel kernel : variant) {
            (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            (void)hipGetLastError();
        }
    }
    for (const ReducedKernel& reduced : kReducedKernels) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(reduced.kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        (void)hipGetLastError();
    }
    for (const ReducedKernel& dense : kDenseKernels) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(dense.kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        (void)hipGetLastError();
    }
}

// The width the sweeps of a world's solve run at: its coordinates, or the K of a reduced block where no contact of the
// world reaches the coordinates from K on and a kernel is compiled for that.
static uint32_t SolverWorkingWidth(const ModelView& m, bool contacts_only) {
    if (contacts_only)
        for (const ReducedKernel& reduced : kReducedKernels)
            if (reduced.width == solver::PaddedWidth(m.dof) && m.contact_dof_end != 0u && m.contact_dof_end <= reduced.reduced &&
                reduced.reduced <= m.dof) return reduced.reduced;   // (0: a host that did not say; the full width is always right)
    return m.dof;
}
// worlds whose heads are contact heads only, at most one a lane (the elliptic cone of the MuJoCo law is answered by the
// general kernel only)
static bool ContactHeadsOnly(const ModelView& m, uint32_t staged) {
    const uint32_t joint_heads = m.joint_limit_rows + m.joint_friction_rows + m.joint_drive_rows;
    return joint_heads == 0u && staged <= uint32_t(solver::kWave) && !(m.any_mujoco != 0u && m.contact_cone == 1u);
}
// `dense_out`: whether the kernel is a dense one (three waves a SIMD)
static SolverKernel KernelOfWidth(const ModelView& m, bool contacts_only, uint32_t width, uint32_t env_count, bool* dense_out = nullptr) {
    if (dense_out != nullptr) *dense_out = false;
    if (contacts_only && env_count >= kDenseBatch)
        for (const ReducedKernel& dense : kDenseKernels)
            if (dense.width == solver::PaddedWidth(m.dof) && dense.reduced == solver::PaddedWidth(width) && (width == m.dof || dense.reduced == width)) {
                if (dense_out != nullptr) *dense_out = true;
                return dense.kernel;
            }
    if (width != m.dof)
        for (const ReducedKernel& reduced : kReducedKernels)
            if (reduced.width == solver::PaddedWidth(m.dof) && reduced.reduced == width) return reduced.kernel;
    return kSolverKernels[contacts_only ? 1 : 0][solver::PaddedWidth(m.dof) / 4u - 1u];
}
// Blocks (one wavefront, one environment each) of a world's full-capacity solve launch that a compute unit holds at
// once, as the runtime's occupancy query answers for the kernel and the LDS the launch asks for; 0 without a solve.
uint32_t SolverBlocksPerUnit(const ModelView& m, uint32_t env_count) {
    if (m.rows_per_env == 0u || m.dof == 0u) return 0u;
    const uint32_t staged = SolverHeadCapacity(m, std::max(m.contact_slots, 1u), 150u * 1024u);
    if (staged == 0u) return 0u;
    const uint32_t joint_heads = m.joint_limit_rows + m.joint_friction_rows + m.joint_drive_rows;
    const bool contacts_only = ContactHeadsOnly(m, staged);
    const uint32_t width = SolverWorkingWidth(m, contacts_only);
    const size_t lds = size_t{solver::ReducedSolverLdsFloats(m.dof, width, staged + joint_heads, staged,
                                                             solver::RowsFromLinks(width, contacts_only, m.rows_from_links))} * sizeof(float);
    int blocks = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&blocks, reinterpret_cast<const void*>(KernelOfWidth(m, contacts_only, width, env_count)),
                                                     solver::kWave, lds) != hipSuccess) {
        (void)hipGetLastError();
        return 0u;
    }
    return uint32_t(std::max(blocks, 0));
}
uint32_t SolverMassFactorFloats(const ModelView& m) {
    if (m.rows_per_env == 0u || m.dof == 0u) return 0u;
    const uint32_t width = SolverSweepWidth(m);
    return solver::MassFactorInMemory(width) ? solver::FactorFloats(solver::PaddedWidth(width)) : 0u;
}
uint32_t SolverSweepWidth(const ModelView& m) {
    if (m.rows_per_env == 0u || m.dof == 0u) return m.dof;
    const uint32_t staged = SolverHeadCapacity(m, std::max(m.contact_slots, 1u), 150u * 1024u);
    return SolverWorkingWidth(m, staged != 0u && ContactHeadsOnly(m, staged));
}

Status OpBlockDescentSolve(const ModelView& m, const DataView& d, const void* params, hipStream_t stream) {
    const auto* p = static_cast<const BlockDescentSolveParams*>(params);
    if (p == nullptr) return Status::Failed;
    if (p->env_count == 0u || p->rows_per_env == 0u || p->articulation_count == 0u) return Status::Ok;
    if (p->articulation_count != p->env_count || m.dof == 0u || m.dof > kMaxDof || p->max_dof != m.max_dof ||
        p->iterations == 0u) return Status::InvalidArgument;
    const size_t budget = 150u * 1024u;
    const uint32_t staged = SolverHeadCapacity(m, p->contact_slots_per_env == 0u ? 1u : p->contact_slots_per_env, budget);
    if (staged == 0u) return Status::InvalidArgument;
    const uint32_t joint_heads = m.joint_limit_rows + m.joint_friction_rows + m.joint_drive_rows;
    const bool contacts_only = ContactHeadsOnly(m, staged);
    const uint32_t width = SolverWorkingWidth(m, contacts_only);
    const auto lds_bytes = [&](uint32_t contact_heads) {
        return size_t{solver::ReducedSolverLdsFloats(m.dof, width, contact_heads + joint_heads, contact_heads,
                                                     solver::RowsFromLinks(width, contacts_only, m.rows_from_links))} * sizeof(float);
    };
    bool dense = false;
    const SolverKernel kernel = KernelOfWidth(m, contacts_only, width, p->env_count, &dense);
    // widths past kTwoWaveWidth run one wave a SIMD: four blocks a compute unit at most, whatever their LDS; the dense
    // kernels run three, twelve blocks
    const size_t most_blocks = dense ? 12u : solver::PaddedWidth(width) > uint32_t(solver::kTwoWaveWidth) ? 4u : 8u;
    const auto blocks_per_unit = [&](uint32_t contact_heads) { return std::min<size_t>(most_blocks, (160u * 1024u) / lds_bytes(contact_heads)); };
    // The LDS a block needs grows with the contact heads it can stage, and a scene's slots (every pair that may ever
    // touch, at its largest manifold) outnumber the contacts an environment usually has.  Where a smaller capacity
    // lets more blocks share a compute unit, environments with few contact points go to a launch of that capacity:
    // up to three such launches, for eight, four and two blocks a unit, before the full one.  Each launch takes the
    // environments whose contact points fall in its range; an environment's results do not depend on its launch.
    hipLaunchKernelGGL(OrderTilesKernel, dim3(1), dim3(1024), 0, stream, d, p->env_count);
    uint32_t first_points = 0u;
    // (a launch takes its environments by their contact points, one head a point: not under the pyramidal cone, whose
    // worlds go to the one full launch)
    const bool one_head_a_point = !(m.any_mujoco != 0u && m.contact_cone == 0u);
    if (p->contact_slots_per_env != 0u && one_head_a_point) {
        for (const size_t blocks : {size_t{12u}, size_t{8u}, size_t{4u}, size_t{2u}}) {
            if (blocks > most_blocks) continue;                            // more blocks than the waves allow
            if (blocks_per_unit(staged) >= blocks) break;                  // the full capacity does as well
            uint32_t few = staged;
            while (few > 8u && blocks_per_unit(few) < blocks) --few;
            if (blocks_per_unit(few) < blocks || few < first_points) continue;   // not even eight heads fit that often
            hipLaunchKernelGGL(kernel, dim3(p->env_count), dim3(solver::kWave), lds_bytes(few), stream, m, d, *p, few + joint_heads, few,
                               first_points, few);
            first_points = few + 1u;
        }
    }
    hipLaunchKernelGGL(kernel, dim3(p->env_count), dim3(solver::kWave), lds_bytes(staged), stream, m, d, *p, staged + joint_heads, staged,
                       first_points, kInvalid);
    return hipGetLastError() == hipSuccess ? Status::Ok : Status::Failed;
}

}  // namespace nkh
