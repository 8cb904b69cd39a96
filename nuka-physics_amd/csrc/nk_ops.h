// Op entry points of the HIP backend.  Each has the reference's OpFn shape
// (src/phi/backend_cuda/ops/registry.cuh:27): Status(const ModelView&, const DataView&, const void* params, stream).
#pragma once

#include <hip/hip_runtime.h>

#include "nk_types.h"

namespace nkh {

using OpFn = Status (*)(const ModelView&, const DataView&, const void*, hipStream_t);

Status OpFkWorldPoses(const ModelView&, const DataView&, const void*, hipStream_t);
Status OpArticulationDynamics(const ModelView&, const DataView&, const void*, hipStream_t);
Status OpIntegratePosition(const ModelView&, const DataView&, const void*, hipStream_t);
Status OpFkLinkVelocities(const ModelView&, const DataView&, const void*, hipStream_t);
Status OpApplyDrives(const ModelView&, const DataView&, const void*, hipStream_t);
Status OpIntegrateVelocity(const ModelView&, const DataView&, const void*, hipStream_t);
Status OpSyncLinkBodyPose(const ModelView&, const DataView&, const void*, hipStream_t);
Status OpBuildAabbs(const ModelView&, const DataView&, const void*, hipStream_t);
Status OpLbvhBuild(const ModelView&, const DataView&, const void*, hipStream_t);
Status OpLbvhQueryPairs(const ModelView&, const DataView&, const void*, hipStream_t);
Status OpNarrowphasePrimitives(const ModelView&, const DataView&, const void*, hipStream_t);
Status OpNarrowphaseHeightfield(const ModelView&, const DataView&, const void*, hipStream_t);
Status OpAssembleRows(const ModelView&, const DataView&, const void*, hipStream_t);
Status OpContactWarmStart(const ModelView&, const DataView&, const void*, hipStream_t);
Status OpBlockDescentSolve(const ModelView&, const DataView&, const void*, hipStream_t);
Status OpReadoutDrives(const ModelView&, const DataView&, const void*, hipStream_t);
Status OpReadoutContactWrench(const ModelView&, const DataView&, const void*, hipStream_t);
Status OpAccumulateStep(const ModelView&, const DataView&, const void*, hipStream_t);
Status OpArticulationDamping(const ModelView&, const DataView&, const void*, hipStream_t);
Status OpReferenceWeights(const ModelView&, const DataView&, const void*, hipStream_t);
Status OpSnapshotStepVelocity(const ModelView&, const DataView&, const void*, hipStream_t);

// A free body's part of IntegrateVelocity and IntegratePosition (ModelView::free_body; ops_rigid.hip)
Status BodyIntegrateVelocity(const ModelView&, const DataView&, const IntegrateVelocityParams&, hipStream_t);
Status BodyIntegratePosition(const ModelView&, const DataView&, const IntegratePositionParams&, hipStream_t);

// IntegratePosition, FkWorldPoses, FkLinkVelocities and (when `bodies` is not null) SyncLinkBodyPose as one launch, for
// a plan whose op list holds them in a row; Unsupported when they must run one by one.
Status OpStepTail(const ModelView&, const DataView&, const IntegratePositionParams*, const FkWorldPosesParams*,
                  const FkLinkVelocitiesParams*, const SyncLinkBodyPoseParams*, hipStream_t);
// SyncLinkBodyPose, BuildAabbs, LbvhBuild, LbvhQueryPairs and NarrowphasePrimitives as one launch, likewise.
Status OpCollisionHead(const ModelView&, const DataView&, const SyncLinkBodyPoseParams*, const BuildAabbsParams*,
                       const LbvhQueryPairsParams*, const NarrowphasePrimitivesParams*, hipStream_t);

}  // namespace nkh
