// Shared POD types of the HIP backend: status codes, the op ids and parameter PODs the PHI seam carries
// (same names and field meaning as src/phi/op_schema.hpp), and the flat device-pointer views the ops read.
#pragma once

#include <cstddef>
#include <cstdint>

namespace nkh {

// src/phi/status.hpp
enum class Status : uint8_t { Ok, Unsupported, Failed, OutOfMemory, InvalidArgument };

// Subset of src/phi/op_catalog.inc in catalog order; ids are this backend's own.
enum class NkOp : uint16_t {
    ApplyDrives, ArticulationDynamics, IntegrateVelocity, FkWorldPoses, IntegratePosition, BuildAabbs, LbvhBuild,
    LbvhQueryPairs, NarrowphasePrimitives, AssembleRows, SyncLinkBodyPose, NarrowphaseHeightfield, ContactWarmStart,
    SnapshotStepVelocity, FkLinkVelocities, BlockDescentSolve, ResetEnvs, SnapshotState, RestoreState,
    ReadoutDrives, ReadoutContactWrench, AccumulateStep,
    Count
};

const char* OpName(NkOp op);

constexpr uint32_t kInvalid = 0xFFFFFFFFu;
constexpr uint32_t kMaxDof = 64u;          // src/phi/articulation_contract.hpp:25
constexpr uint32_t kShapeStride = 13u;     // src/phi/op_schema.hpp:26
constexpr uint32_t kRowWords = 26u;        // src/nk/solve/nk_row.hpp:99-100
constexpr uint32_t kPointsPerSlot = 4u;    // src/nk/solve/nk_row.hpp:59
constexpr uint32_t kRowsPerPoint = 4u;     // src/nk/solve/nk_row.hpp:61

// src/phi/articulation_contract.hpp:8-16
enum : uint8_t { kRevolute = 0, kPrismatic = 1, kFixed = 2, kFloatingBase = 3, kSpherical = 4 };
// src/collision/shape_kind.hpp:9-18
enum : uint32_t { kShapeSphere = 0, kShapeCapsule = 1, kShapeBox = 2, kShapePlane = 3, kShapeCylinder = 7 };
// src/nk/solve/nk_row.hpp:14-19
enum : uint32_t { kSideRigid = 0, kSideArtic = 1, kSideStatic = 3 };
// src/nk/solve/nk_row.hpp:41-57
enum : uint32_t {
    kRowActive = 1u << 0, kRowFriction = 1u << 1, kRowBlockNormal = 1u << 2, kRowBlockTangent = 1u << 3,
    kRowJointLimitLower = 1u << 4, kRowJointLimitUpper = 1u << 5,
    kRowContactNormal = 1u << 6, kRowVelocityOnly = 1u << 7, kRowSpeculative = 1u << 8, kRowMuJoCo = 1u << 11
};
// src/phi/op_schema.hpp:36-52
enum : uint32_t {
    kEnvStatusPairOverflow = 1u << 0, kEnvStatusDofOverflow = 1u << 2, kEnvStatusInvalidEndpoint = 1u << 6,
    kEnvStatusControlFailure = 1u << 10, kEnvStatusSolverFailure = 1u << 13
};
// src/phi/articulation_contract.hpp:16-23
enum : uint32_t { kDrivePdPosition = 0, kDriveTorque = 1, kDriveVelocity = 2, kDriveComputedTorque = 3, kDriveOsc = 4, kDriveActuator = 5 };
constexpr uint32_t kContactLawSpeculative = 2u;   // src/nk/solve/nk_row.hpp:37

// Template tables, stored once and shared by every environment (the reference replicates them per env,
// src/nk/model/model.hpp:154-157).  Counts are per environment.
struct ModelView {
    uint32_t links_per_env, bodies_per_env, dof, max_dof, max_depth, contact_slots, rows_per_env, contact_rows_per_env;
    uint32_t profile_count, floating_root;
    uint32_t max_points_per_slot;   // most points a manifold of the template's admitted pairs can hold (sizes the solver's staged rows)
    uint32_t excluded_pair_count;
    // joint row slots after the contact rows: 2 per link, 1 per link, 1 per link, or 0 (scene/cook/cook_to_model.cpp:706-719)
    uint32_t joint_limit_rows, joint_friction_rows, joint_drive_rows, drive_mode;
    const uint8_t* joint_type;
    const uint32_t* parent_link;
    const float* joint_axis;
    const float* parent_offset;
    const float* link_local_pose;
    const float* link_inertial_frame;
    const float* link_inertia;
    const float* joint_damping;
    const float* joint_armature;
    const float* joint_stiffness;
    const float* joint_spring_reference;
    const float* joint_limit_lower;
    const float* joint_limit_upper;
    const float* joint_frictionloss;
    const uint8_t* joint_limit_flags;   // bit 0: lower bound authored, bit 1: upper
    const uint32_t* link_body;
    const uint32_t* link_tree_depth;
    const uint32_t* link_child_range;
    const uint32_t* link_children;
    const uint32_t* link_dof;
    const uint32_t* dof_link;
    const uint32_t* dof_component;
    const uint64_t* link_dof_mask;   // DoFs on the path from each link to the root
    const uint32_t* link_geom_kind;
    const float* link_geom_local;
    const float* shape_table;
    const uint32_t* body_to_link;
    const uint32_t* body_to_articulation;
    const uint32_t* body_collidable_link;
    const uint32_t* body_collidable_body;
    const float* body_collidable_local;
    const float* profile_mu;
    const uint64_t* excluded_pairs;   // sorted (a << 32 | b) keys of collidable rows that never pair, a < b
};

// Mutable per-environment fields, env-major with the element layout of the reference's public fields
// (src/nk/model/fields.yaml), so buffer views are zero-copy.
struct DataView {
    float *q, *qdot, *qddot, *tau, *base_pose, *link_pose, *link_velocity, *link_acceleration, *link_wrench;
    float *articulation_bias, *articulation_qdd, *m, *m_factor, *qdot_flat, *qdot_pseudo, *link_velocity_pseudo;
    float *body_pose, *body_aabb_lo, *body_aabb_hi;
    uint32_t *candidate_pairs, *pair_count;
    uint32_t *ucontact_count, *ucontact_a, *ucontact_b, *ucontact_law, *ucontact_row_range;
    float *ucontact_point, *ucontact_normal, *ucontact_depth;
    uint64_t *ucontact_id_pair, *ucontact_id_feature;
    float *urows, *lambda, *row_penetration, *row_cj_point, *row_cj_point_b, *chain_jacobian, *chain_jacobian_b;
    uint32_t *row_cj_link, *row_cj_link_b, *row_count, *contact_count, *contact_row_extent;
    uint32_t *env_status, *vbd_velocity_sweep_count;
    float *solver_residual, *solver_penalty;
    float *solver_velocity, *solver_free;   // block velocities kept between solves (carried constraint velocity)
    // contact cache carried between steps (fields.yaml:524-539, 155, 791, 844)
    uint64_t *contact_material, *contact_cache_pair, *contact_cache_feature, *contact_cache_material;
    float *contact_cache_lambda, *contact_cache_normal;
    uint32_t *contact_cache_age, *contact_cache_current_owner, *contact_cache_old_keep, *contact_cache_extent;
    uint32_t *contact_warm_start_counts, *contact_cache_match;
    // drives (fields.yaml:49-53, 328, 658-668, 548-551, 906)
    float *drive_target, *drive_stiffness, *drive_damping, *drive_force_limit, *drive_joint_force_limit;
    float *velocity_target, *actuator_noload_speed, *joint_f, *joint_gravity_force;
    float *drive_command, *drive_dissipation, *drive_lower, *drive_upper;
    float *joint_limit_impulse, *actuator_effort_requested, *actuator_effort, *actuator_saturated;
    // contact readout (fields.yaml contact_point .. link_contact_wrench), written by ReadoutContactWrench on demand
    float *contact_point, *contact_normal, *contact_force, *ucontact_impulse, *link_contact_wrench;
    uint32_t *contact_side_a_kind, *contact_side_b_kind, *contact_side_a_index, *contact_side_b_index, *contact_link;
    uint32_t *reset_env_ids;                // staging of nuka_world_reset_envs
    uint32_t *solver_cost, *tile_order;     // decaying maximum of the solves' work per environment; launch order of the next solve (costliest first)
    uint32_t *row_unit;                     // per row: the one coordinate a single-coordinate row acts on, ~0u otherwise
    float *row_unit_value;                  // its Jacobian entry there
    float *snapshot;                        // SnapshotState / RestoreState storage
    // sums over the substeps of one step (fields.yaml:627-632), written by AccumulateStep
    uint32_t *step_env_status;
    float *step_link_impulse, *step_link_moment, *step_joint_limit_impulse;
};

// --- parameter PODs (field names follow src/phi/op_schema.hpp) -------------------------------------------
struct FkWorldPosesParams { uint32_t articulation_count, total_link_count; };
struct FkLinkVelocitiesParams { uint32_t articulation_count, total_link_count; };
struct ApplyDrivesParams {   // op_schema.hpp:79-88
    float dt;
    uint32_t total_link_count, defer_velocity_damping, mode, links_per_env, bodies_per_env, articulation_count;
    float gravity[3];
    uint32_t affine;   // this backend's own: 0 leaves `tau` as the applied generalized force (no drive rows cooked)
};
struct ReadoutDrivesParams { float dt; uint32_t total_link_count, links_per_env, rows_per_env, first_drive_row; };   // op_schema.hpp:100-106
struct ArticulationDynamicsParams {   // op_schema.hpp:108-121
    float dt;
    uint32_t max_dof;
    uint32_t integrate_velocity = 1u;
    uint32_t fold_drive_damping = 0u;
    uint32_t reuse_mass = 0u;
    float gravity[3];
    uint32_t articulation_count;
    uint32_t total_link_count;
    uint32_t apply_link_wrench = 0u;
    uint32_t max_links = 0u;
    uint32_t links_per_env = 0u;
    uint32_t bodies_per_env = 0u;
};
struct IntegrateVelocityParams { float dt; float gravity[3]; uint32_t total_body_count, clear_body_forces; };
struct IntegratePositionParams { float dt; uint32_t total_link_count, articulation_count, total_body_count, env_count, pos_pass, mimic_couplings; };
struct SyncLinkBodyPoseParams { uint32_t env_count, links_per_env, bodies_per_env, family, selected_env_count; };
struct BuildAabbsParams { uint32_t env_count, bodies_per_env, family; float margin, dt, query_reach; };
struct LbvhBuildParams { uint32_t env_count, bodies_per_env, family; };
struct LbvhQueryPairsParams { uint32_t env_count, bodies_per_env, family, max_contacts_per_env, rigid_slot_cap, max_pairs, excluded_count; };
struct NarrowphasePrimitivesParams { uint32_t env_count, bodies_per_env, union_slot_count, rigid_slot_cap; float contact_margin, dt, query_reach; };
struct AssembleRowsParams {
    uint32_t env_count, articulation_count, total_link_count, max_dof, union_slot_count, rows_per_env, contact_rows_per_env;
    uint32_t full_row_slot_count, bodies_per_env, base_link_count, position_pass, family;
    float dt, overlap_recovery_velocity, contact_margin;
    uint32_t joint_limit_rows_per_env, joint_friction_rows_per_env, joint_drive_rows_per_env;
    float baumgarte_max_velocity;
};
struct ContactWarmStartParams { uint32_t phase, env_count, slot_count, rows_per_env, full_row_slot_count, decay_steps; };
struct BlockDescentSolveParams {   // op_schema.hpp:549-636 (the tile-route subset)
    float dt;
    uint32_t env_count, rows_per_env, total_body_count, articulation_count, max_dof, max_independent_dof;
    uint32_t base_link_count, contact_rows_per_env, contact_slots_per_env;
    uint32_t iterations = 10u;
    uint32_t position_iterations;
    float position_beta, position_slop, position_max_velocity;
    float velocity_tolerance;
    uint32_t joint_limit_rows_per_env;
};
struct ReadoutContactWrenchParams {   // op_schema.hpp:746-755
    float dt;
    uint32_t env_count, base_link_count, max_contacts_per_env, rows_per_env, full_row_slot_count, contact_rows_per_env;
};
struct SnapshotParams { uint32_t env_count, selected_env_count; };
// op_schema.hpp:170-180; the flags this path uses (the particle and free-body ones have no counterpart here)
constexpr uint32_t kAccumulateOutputs = 1u, kAccumulateLinkWrench = 2u, kAccumulateJointLimit = 4u, kFinalizeLinkWrench = 8u;
struct AccumulateStepParams { uint32_t env_count, links_per_env, flags, first, last; float substep_dt, inv_outer_dt; };

}  // namespace nkh
