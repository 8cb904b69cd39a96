// Shared POD types of the HIP backend: status codes, the op ids and parameter PODs the PHI seam carries
// (same names and field meaning as src/phi/op_schema.hpp), and the flat device-pointer views the ops read.
#pragma once

#include <cstddef>
#include <cstdint>

namespace nkh {

// src/phi/status.hpp
enum class Status : uint8_t { Ok, Unsupported, Failed, OutOfMemory, InvalidArgument };

// The closed op set of src/phi/op_catalog.inc, in the catalog's order, so that an op id here is the reference's
// NkOp value (src/phi/op_schema.hpp:60-65).  This backend serves the ops of the articulation step; the others have a
// null slot in its table: supports_op answers 0 and a dispatch answers Unsupported.
#define NKH_OP_CATALOG(X) \
    X(ApplyDrives) X(ApplyDynamicsDrives) X(ArticulationDynamics) X(IntegrateVelocity) X(FkWorldPoses) X(IntegratePosition) \
    X(BuildAabbs) X(LbvhBuild) X(LbvhQueryPairs) X(NarrowphasePrimitives) X(NarrowphaseSdf) X(AssembleRows) X(ParticleAeroDrag) \
    X(ParticlePredict) X(ParticleFinalize) X(MpmPredict) X(MpmExchange) X(MpmCommit) X(ReadoutContactWrench) X(ExportObs) \
    X(ResetEnvs) X(SnapshotState) X(RestoreState) X(RandomizeMaterialBuckets) X(RandomizeBodyParams) X(SyncLinkBodyPose) \
    X(NarrowphaseBodyParticle) X(NarrowphaseHeightfield) X(ContactWarmStart) X(SnapshotStepVelocity) \
    X(ParticleProjectionVelocity) X(ParticleContactDelta) X(AccumulateStep) X(FkLinkVelocities) X(ReadoutDrives) \
    X(RefitParticleSurfaces) X(SampleObservation) X(ResetObservation) X(ReadoutMotion) X(SampleStateSensor) X(AdvanceSensorTime) \
    X(ReadoutSensorWrenches) X(ReadoutContactRegion) X(ClothPredict) X(ClothContactRestart) X(ClothFinalize) X(OgcDetect) \
    X(ReadoutEnergyLedger) X(ReadoutContactAudit) X(MimicReduce) X(BlockDescentSolve) X(RecordTelemetry) X(ReferenceWeights) \
    X(ArticulationDamping) X(ReadoutIntervalState) X(ContactRefresh)
enum class NkOp : uint16_t {
#define X(name) name,
    NKH_OP_CATALOG(X)
#undef X
    Count
};

const char* OpName(NkOp op);

constexpr uint32_t kInvalid = 0xFFFFFFFFu;
constexpr uint32_t kSweepLinks = 10u;      // links a pass of the dynamics' tree sweeps: six lanes a link
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
    kRowContactNormal = 1u << 6, kRowVelocityOnly = 1u << 7, kRowSpeculative = 1u << 8, kRowMuJoCo = 1u << 11,
    kRowPyramidal = 1u << 12
};
// src/phi/op_schema.hpp:36-52
enum : uint32_t {
    kEnvStatusPairOverflow = 1u << 0, kEnvStatusDofOverflow = 1u << 2, kEnvStatusGyroFailure = 1u << 5, kEnvStatusInvalidEndpoint = 1u << 6,
    kEnvStatusControlFailure = 1u << 10, kEnvStatusSolverFailure = 1u << 13
};
// src/phi/articulation_contract.hpp:16-23
enum : uint32_t { kDrivePdPosition = 0, kDriveTorque = 1, kDriveVelocity = 2, kDriveComputedTorque = 3, kDriveOsc = 4, kDriveActuator = 5 };
constexpr uint32_t kContactLawCompliant = 0u, kContactLawVelocity = 1u, kContactLawSpeculative = 2u;   // src/nk/solve/nk_row.hpp:35-37

// Template tables, stored once and shared by every environment (the reference replicates them per env,
// src/nk/model/model.hpp:154-157).  Counts are per environment.
struct ModelView {
    uint32_t links_per_env, bodies_per_env, dof, max_dof, max_depth, contact_slots, rows_per_env, contact_rows_per_env;
    uint32_t profile_count, floating_root;
    uint32_t max_points_per_slot;   // most points a manifold of the template's admitted pairs can hold (sizes the solver's staged rows)
    uint32_t excluded_pair_count;
    uint32_t sweep_passes;     // passes of the dynamics' tree sweeps (sweep_links)
    uint32_t pairable_count;   // collidable rows that can pass the shape filter with some partner (pairable_rows, ascending)
    uint32_t contact_dof_end;  // one past the last coordinate on the path to the root of any link that carries a shape: no contact row reaches a later one (0: not known)
    // 1: every contact row acts on the articulation through one link (no admitted pair joins two of its links' shapes) and
    // every coordinate is a hinge, a slider or one of a floating root's six: a contact row's entries then follow from the
    // row's wrench and the coordinates' motion axes, and the solve of a wide block need not keep the rows themselves
    uint32_t rows_from_links;
    // joint row slots after the contact rows: 2 per link, 1 per link, 1 per link, or 0 (scene/cook/cook_to_model.cpp:706-719)
    uint32_t joint_limit_rows, joint_friction_rows, joint_drive_rows, drive_mode;
    // the MuJoCo contact law: some profile is MuJoCo-sourced; the cone of its contacts (0 pyramidal, 1 elliptic) and impratio
    uint32_t any_mujoco, contact_cone;
    float contact_impratio;
    uint32_t integrator;   // 0 native; 1, 2: ArticulationDamping follows the solve (2: with the servos' velocity gains)
    // 1: the template's one link is a free rigid body, stepped by the rigid-body ops (ops_rigid.hip): its six coordinates
    // are its linear velocity and its angular velocity about the centre of mass, in world axes
    uint32_t free_body;
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
    const uint8_t* joint_law;           // 1: MuJoCo-sourced joint rows
    const float* joint_limit_margin;
    const float* joint_limit_reference;     // [link][7] solref, solimp
    const float* joint_friction_reference;  // [link][7]
    const uint32_t* link_body;
    const uint32_t* link_tree_depth;
    const uint32_t* link_child_range;
    const uint32_t* link_children;
    const uint32_t* sweep_links;       // [sweep_passes][kSweepLinks]: the links a depth at a time, ten a pass, kInvalid where a pass ends early
    const uint32_t* link_push_order;   // children in the order the composite-inertia pass adds them to their parents, then kInvalid
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
    const uint32_t* pairable_rows;
    const float* profile_mu;
    const uint32_t* profile_law;      // [profile] 1: MuJoCo-sourced (constraint/law_source.hpp)
    const float* profile_solref;      // [profile][2]
    const float* profile_solimp;      // [profile][5]
    const float* profile_margin;      // [profile][2] margin, gap
    const float* profile_mix;         // [profile][3] priority, solmix, condim
    const uint64_t* excluded_pairs;   // sorted (a << 32 | b) keys of collidable rows that never pair, a < b
};

// Mutable per-environment fields, env-major with the element layout of the reference's public fields
// (src/nk/model/fields.yaml), so buffer views are zero-copy.
struct DataView {
    float *q, *qdot, *qddot, *tau, *base_pose, *link_pose, *link_velocity, *link_acceleration, *link_wrench;
    float *articulation_bias, *articulation_qdd, *m, *m_factor, *qdot_flat, *qdot_pseudo, *link_velocity_pseudo;
    float *body_pose, *body_aabb_lo, *body_aabb_hi;
    // the free body of a free_body world, one an environment (fields.yaml:102-103, 569; articulation.cu:1068-1070)
    float *body_linear_velocity, *body_angular_velocity, *body_world_inv_inertia, *body_gyro_residual;
    float *body_inv_mass, *body_inv_inertia, *body_inertial_frame;   // fields.yaml:17, 108, 568: 1 / mass, 1 / principal moments, the inertial frame in the body's
    uint32_t *body_gyro_iterations, *body_gyro_status;
    uint32_t *candidate_pairs, *pair_count;
    uint32_t *ucontact_count, *ucontact_a, *ucontact_b, *ucontact_law, *ucontact_row_range;
    float *ucontact_point, *ucontact_normal, *ucontact_depth;
    uint64_t *ucontact_id_pair, *ucontact_id_feature;
    float *urows, *lambda, *row_penetration, *row_cj_point, *row_cj_point_b, *chain_jacobian, *chain_jacobian_b;
    uint32_t *row_cj_link, *row_cj_link_b, *row_count, *contact_count, *contact_row_extent;
    uint32_t *env_status, *vbd_velocity_sweep_count;
    float *solver_residual, *solver_penalty;
    float *solver_velocity, *solver_free;   // block velocities kept between solves (carried constraint velocity)
    // the MuJoCo contact law (fields.yaml body_invweight0, dof_invweight0, row_invweight, row_reference_velocity_gain,
    // step_qdot_flat): reference weights at the creation pose, per row the weight and the gain on the start velocity
    float *body_invweight0, *dof_invweight0, *row_invweight, *row_reference_velocity_gain, *step_qdot_flat;
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
    float* solver_mass_factor;              // [env][FactorFloats]: the solve's own factor of the mass matrix, for blocks too wide to keep it in LDS
    uint32_t *solver_cost, *tile_order;     // decaying maximum of the solves' work per environment; launch order of the next solve (costliest first)
    uint32_t *row_unit;                     // per row: the one coordinate a single-coordinate row acts on, ~0u otherwise
    float *row_unit_value;                  // its Jacobian entry there
    float *snapshot;                        // SnapshotState / RestoreState storage
    // sums over the substeps of one step (fields.yaml:627-632), written by AccumulateStep
    uint32_t *step_env_status;
    float *step_link_impulse, *step_link_moment, *step_joint_limit_impulse;
};

// --- parameter PODs ----------------------------------------------------------------------------------------
// Layout-identical to src/phi/op_schema.hpp for every op this backend serves: same members, order and types, so an
// OpCall filled by the reference's Pipeline (src/nk/pipeline/pipeline.cpp:187-1020) reads correctly here.  Members
// that describe what this path does not build (particles, grids, hulls, heightfields, cloth, telemetry) are carried and
// must be zero where a nonzero value would ask for that work; an op answers Unsupported otherwise.  What the kernels
// need beyond these members they derive from the ModelView.
struct ApplyDrivesParams {   // op_schema.hpp:79-88
    float dt;
    uint32_t total_link_count;
    uint32_t defer_velocity_damping;
    uint32_t mode;
    uint32_t links_per_env;
    uint32_t bodies_per_env = 0u;
    uint32_t articulation_count = 0u;
    float gravity[3] = {};
};
struct ReadoutDrivesParams {   // op_schema.hpp:100-106
    float dt;
    uint32_t total_link_count;
    uint32_t links_per_env;
    uint32_t rows_per_env;
    uint32_t first_drive_row;
};
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
struct ReferenceWeightsParams {   // op_schema.hpp:123-130
    uint32_t max_dof;
    uint32_t articulation_count;
    uint32_t total_link_count;
    uint32_t articulations_per_env;
    uint32_t bodies_per_env;
    uint32_t total_body_count;
};
struct ArticulationDampingParams {   // op_schema.hpp:132-141
    float dt;
    uint32_t max_dof;
    uint32_t articulation_count;
    uint32_t total_link_count;
    uint32_t actuator_derivative;
    uint32_t mode;
    uint32_t readout_drives = 0u;
};
struct IntegrateVelocityParams {   // op_schema.hpp:143-150
    float dt;
    float gravity[3];
    uint32_t total_link_count;
    uint32_t articulation_count;
    uint32_t total_body_count;
    uint32_t clear_body_forces = 1u;
};
struct SnapshotStepVelocityParams {   // op_schema.hpp:153-160
    uint32_t env_count;
    uint32_t articulation_count;
    uint32_t max_dof;
    uint32_t base_link_count;
    uint32_t total_body_count;
    uint32_t total_particle_count;
};
// op_schema.hpp:162-168; the flags this path uses (the particle and free-body ones have no counterpart here)
constexpr uint32_t kAccumulateOutputs = 1u, kAccumulateLinkWrench = 2u, kAccumulateJointLimit = 4u, kFinalizeLinkWrench = 8u;
struct AccumulateStepParams {   // op_schema.hpp:170-180
    uint32_t env_count = 0u;
    uint32_t bodies_per_env = 0u;
    uint32_t links_per_env = 0u;
    uint32_t artics_per_env = 0u;
    uint32_t flags = 0u;
    uint32_t first = 0u;
    uint32_t last = 0u;
    float substep_dt = 0.0f;
    float inv_outer_dt = 0.0f;
};
struct FkWorldPosesParams {   // op_schema.hpp:182-187
    uint32_t articulation_count;
    uint32_t total_link_count;
    uint32_t articulations_per_env;
    uint32_t selected_env_count;
};
struct FkLinkVelocitiesParams {   // op_schema.hpp:189-192
    uint32_t articulation_count;
    uint32_t total_link_count;
};
struct IntegratePositionParams {   // op_schema.hpp:194-202
    float dt;
    uint32_t total_link_count;
    uint32_t articulation_count;
    uint32_t total_body_count;
    uint32_t pos_pass;
    uint32_t env_count = 1u;
    uint32_t mimic_couplings = 0u;
};
struct BuildAabbsParams {   // op_schema.hpp:221-228
    float dt = 0.0f;
    float query_reach = 0.02f;   // collision/contact_query.hpp:16
    float margin;
    uint32_t family;
    uint32_t env_count;
    uint32_t bodies_per_env;
};
struct LbvhBuildParams {   // op_schema.hpp:230-236
    uint32_t family;
    uint32_t env_count;
    uint32_t bodies_per_env;
    uint64_t workspace_bytes = 0u;
    uint32_t tree_queries = 0u;
};
struct LbvhQueryPairsParams {   // op_schema.hpp:238-249
    uint32_t max_pairs;
    uint32_t family;
    uint32_t env_count;
    uint32_t bodies_per_env;
    uint32_t max_contacts_per_env;
    uint32_t filter_cross_env;
    uint32_t excluded_count;
    uint32_t contact_pair_count = 0u;
    uint32_t rigid_slot_cap;
    uint64_t workspace_bytes;
};
struct NarrowphasePrimitivesParams {   // op_schema.hpp:392-413
    float contact_margin;
    uint32_t num_material_buckets;
    uint32_t contact_pairs = 0u;
    float dt = 0.0f;
    float query_reach = 0.02f;
    uint8_t max_contacts_per_pair;
    float ground_height;
    uint32_t foot_count;
    uint32_t env_count;
    uint32_t base_link_count;
    uint32_t family;
    uint32_t union_slot_count;
    uint32_t rigid_slot_cap;
    uint32_t bodies_per_env;
    uint32_t hull_vert_count;
    uint32_t particles_per_env;
    uint32_t articulations_per_env;
    uint32_t max_foot_contacts;
    uint32_t max_body_samples;
    uint32_t convex_pairs;
};
struct SyncLinkBodyPoseParams {   // op_schema.hpp:434-440
    uint32_t family;
    uint32_t env_count;
    uint32_t links_per_env;
    uint32_t bodies_per_env;
    uint32_t selected_env_count;
};
struct NarrowphaseHeightfieldParams {   // op_schema.hpp:442-457
    uint32_t family;
    uint32_t env_count;
    uint32_t slot_stride;
    uint32_t rigid_slot_cap;
    uint32_t bodies_per_env;
    uint32_t hull_vert_count;
    float contact_margin;
    uint32_t has_heightfield;
    float origin_x, origin_y, origin_z;
    float cell_size;
    uint32_t nrow, ncol;
    float min_z, max_z;
    uint32_t data_offset;
    uint32_t hf_body_row;
};
struct VertexBlockLayout {   // op_schema.hpp:535-547; all zero on this path
    uint32_t begin = 0u;
    uint32_t vertices = 0u;
    uint32_t dynamic_vertices = 0u;
    uint32_t colors = 0u;
    uint32_t particles_per_env = 0u;
    uint32_t env_count = 0u;
    uint32_t elements = 0u;
    uint32_t coarse_levels = 0u;
    uint32_t coarse_nodes = 0u;
    uint32_t coarse_dense_nodes = 0u;
};
struct AssembleRowsParams {   // op_schema.hpp:549-594
    uint32_t grid_nodes_per_env = 0u;
    float dt;
    uint32_t slot_count;
    uint32_t max_dof;
    uint32_t env_count;
    uint32_t articulation_count;
    uint32_t total_link_count;
    uint32_t family;
    uint32_t union_slot_count;
    uint32_t rows_per_env;
    uint32_t contact_rows_per_env;
    uint32_t joint_limit_rows_per_env;
    uint32_t joint_friction_rows_per_env;
    uint32_t joint_drive_rows_per_env;
    uint32_t mimic_couplings_per_env;
    uint32_t full_row_slot_count;
    uint32_t ogc_slot_count = 0u;
    uint32_t bodies_per_env;
    uint32_t base_link_count;
    float solref[2];
    float solimp[5];
    float impratio;
    bool refsafe;
    uint32_t cone;
    uint32_t particles_per_env;
    uint32_t num_material_buckets;
    uint32_t contact_pairs = 0u;
    float baumgarte_max_velocity;
    float contact_margin;
    uint32_t position_pass = 0u;
    float overlap_recovery_velocity = 0.0f;
    uint32_t point_endpoints_per_env = 0u;
    uint32_t point_endpoint_terms_per_env = 0u;
    VertexBlockLayout vertex_blocks{};
    uint32_t measure_contact_response = 0u;
};
struct BlockDescentSolveParams {   // op_schema.hpp:596-640
    float dt;
    uint32_t iterations = 10u;
    uint32_t env_count = 0u;
    uint32_t rows_per_env = 0u;
    uint32_t total_particle_count = 0u;
    uint32_t total_body_count = 0u;
    uint32_t total_grid_count = 0u;
    uint32_t articulation_count = 0u;
    uint32_t max_dof = 0u;
    uint32_t base_link_count = 0u;
    uint32_t contact_rows_per_env = 0u;
    uint32_t contact_slots_per_env = 0u;
    uint32_t distinct_owner_rows_per_env = 0u;
    uint32_t joint_limit_rows_per_env = 0u;
    uint64_t incidence_per_env = 0u;
    uint32_t measure_contact_residual = 0u;
    uint64_t workspace_words = 0u;
    VertexBlockLayout vertex_blocks{};
    uint32_t measure_vertex_audit = 0u;
    uint32_t mimic_couplings = 0u;
    uint32_t max_independent_dof = kMaxDof;
    uint32_t material_cells_per_env = 0u;
    uint32_t grid_particles_per_env = 0u;
    uint32_t grid_dims[3] = {};
    uint32_t clear_failure_diagnostics = 1u;
    uint32_t substep_index = 0u;
    uint32_t position_iterations = 0u;
    float position_beta = 0.0f;
    float position_slop = 0.0f;
    float position_max_velocity = 0.0f;
    float velocity_tolerance = 0.0f;
    uint32_t trace_sweeps = 0u;
    uint32_t telemetry = 0u;
    uint32_t contact_anchors = 0u;
};
struct ReadoutContactWrenchParams {   // op_schema.hpp:746-755
    float dt;
    uint32_t env_count;
    uint32_t base_link_count;
    uint32_t max_contacts_per_env;
    uint32_t rows_per_env;
    uint32_t full_row_slot_count;
    uint32_t contact_rows_per_env;
    uint64_t workspace_bytes;
};
struct ContactWarmStartParams {   // op_schema.hpp:951-959
    uint32_t phase;
    uint32_t env_count;
    uint32_t slot_count;
    uint32_t rows_per_env;
    uint32_t full_row_slot_count;
    uint32_t decay_steps;
    uint64_t workspace_bytes = 0u;
};

}  // namespace nkh
