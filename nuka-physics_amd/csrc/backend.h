// Internal interface between the PHI-shaped backend (backend.hip) and the host world (world.hip).
#pragma once

#include <hip/hip_runtime.h>

#include "../../include/nuka_phi.h"
#include "nk_types.h"

namespace nkh {

// A backend on `device`; `borrowed_stream` non-null is used as is, else an owned stream at default priority.
void* CreateBackend(int device, void* borrowed_stream);
hipStream_t BackendStream(void* backend);
nuka_phi_buffer_type* BackendDeviceBufferType(void* backend);
nuka_phi_buffer_type* BackendHostBufferType(void* backend);
bool BackendSupportsOp(NkOp op);
// Raises the dynamic-LDS limit of the wide kernels once, outside any stream capture.
void InitArticulationKernels();
void InitSolverKernels();
void InitContactKernels();
uint32_t SolverHeadCapacity(const ModelView& m, uint32_t slots, size_t lds_budget_bytes);
// the width the sweeps of the world's block-descent solve run at: its coordinates, or fewer for a reduced block
uint32_t SolverSweepWidth(const ModelView& m);
// blocks of the world's full-capacity solve launch that one compute unit holds at once (runtime occupancy query for
// the kernel a batch of `env_count` environments takes)
uint32_t SolverBlocksPerUnit(const ModelView& m, uint32_t env_count);
// words per environment of DataView::solver_mass_factor: the solve's factor of the mass matrix where its block is too
// wide to keep it in LDS, else none
uint32_t SolverMassFactorFloats(const ModelView& m);

}  // namespace nkh
