/*
 * CPU oracle for the batched articulation step: TEST INFRASTRUCTURE ONLY.
 *
 * A plain-C, one-environment-at-a-time fp32 restatement of the reference's CUDA kernels for
 * forward kinematics, RNEA bias + CRBA + LDL^T forward dynamics, the contact pipeline of analytic
 * primitive pairs (pairs, manifolds, rows, chain Jacobians) and the UABD tile block-descent solve with its
 * split-impulse position pass.  Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline
 * leg may load it, and only as the checker.  Nothing shipped links or calls it.
 *
 * Every function in nko_*.c cites the reference file:line it follows.  Compile without fast-math and
 * with -ffp-contract=off: fused multiply-adds appear only where the reference writes fmaf itself.
 *
 * Parity status per function group (what pins it beyond "it restates the reference"; tests/ holds each check):
 *   cook / spatial inertia  : pinned (parallel-axis closed form)
 *   forward kinematics      : pinned (float64 rotation-matrix kinematics on all four configurations)
 *   dynamics (bias, M, LDL) : pinned (pendulum closed form with damping, spring, armature; M as the kinetic-energy
 *                             form and the bias as the Euler-Lagrange bias of an independent float64 model built
 *                             from finite differences of poses; first-order energy drift and momentum laws of
 *                             free motion, fixed and floating base; LDL^T reconstruction and dense solves)
 *   link velocities, integration : pinned (pose rates of the float64 model; the conservation runs above)
 *   pairs / slots / rows    : pinned (brute-force O(B^2) overlap enumeration in canonical order; integer exact)
 *   manifolds, compose, contact id, query band, filter, projection roundoff :
 *                             pinned bit-exact against oracle/_ref (the reference's own host headers) and the
 *                             committed vectors tests/golden/rowmath_vectors.npz; the prim-frame bake is device-only
 *                             code and is pinned by the rotation-matrix closed form instead.  Every pair kind of
 *                             PrimitivePair is covered (sphere, capsule, box, plane, cylinder; box x box included)
 *   row math (AL impulses)  : pinned bit-exact against oracle/_ref (augmented_row.hpp), the committed vectors, and
 *                             the known answers in tests/math/test_contact_tangent.cpp; the compliant-row terms and
 *                             the elliptic cone likewise, with the hand-evaluated table of
 *                             tests/constraint/test_solref_solimp.cpp
 *   MuJoCo contact law      : pinned (merged profile terms bit-exact against the reference's MergeContactParams in
 *                             oracle/_ref; reference weights against the closed forms of a free body and a pendulum
 *                             and a dense float64 J M^-1 J^T of a chain; the compliant normal, tangent and pyramid
 *                             edge rows against the pinned row math and the geometry of the pyramid; a resting
 *                             sphere's depth against the closed form of the spring-damper reference, both cones)
 *   chain Jacobian          : pinned (J qdot == contact point velocity of the float64 model)
 *   contact cache           : pinned by behaviour (seeding of a persisting contact, one-step retention and decay,
 *                             layout invariants); the merged profile terms of the material key against the
 *                             reference's MergeContactParams.  The key's hash routine is device-only code:
 *                             PARITY UNPINNED for its constants.
 *   drives, joint rows      : pinned (gravity-free pendulum: implicit-Euler PD step, force-limit clamp, limit stop and
 *                             push-out, dry friction hold / slip; torque-mode drive rows against the direct-torque path)
 *   contact readout         : pinned (weight of a resting ball, Coulomb friction and its moment, link wrenches adding up
 *                             to the generalized impulse the solve applied)
 *   substeps                : pinned (n substeps of dt are n steps of dt / n bit for bit; the step's status, joint limit
 *                             impulses and link contact wrenches are the or, the sum and the time average of those steps')
 *   free rigid body         : pinned (free flight: the parabola of the centre of mass, angular momentum and kinetic
 *                             energy of a tumbling body over thousands of steps, the precession rate of a symmetric top
 *                             against its closed form, the free-rotation solve against the midpoint rule's own
 *                             equation; the row entries J [v; w] against the velocity of the contact point; a box at rest
 *                             on a plane carries its weight; a sliding box stops by Coulomb's law)
 *   UABD fixed point        : pinned (closed-form resting, falling, sticking and sliding ball; Coulomb / KKT
 *                             conditions and momentum balance of converged solves)
 *   UABD iterate path       : PARITY UNPINNED - penalty heuristic, first-sweep segment search, FISTA
 *                             restart timing, secant relaxation and the 8-epsilon waivers decide the
 *                             multipliers held after a fixed sweep budget; only a running reference
 *                             could pin them and none can run here.
 */
#ifndef NUKA_ORACLE_H_
#define NUKA_ORACLE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Layout-identical to nuka_template_desc_t / nuka_world_desc_t of include/nuka_hip.h so that one
 * host-side description drives both the product library and this checker. */
typedef struct nko_template_desc {
    uint32_t struct_size;
    uint32_t link_count;
    uint32_t body_count;
    uint32_t profile_count;
    uint32_t max_contacts_per_env;
    uint32_t reserved0;
    const uint8_t* joint_type;
    const uint32_t* parent_link;
    const float* joint_axis;
    const float* parent_offset;
    const float* link_local_pose;
    const float* link_inertial_frame;
    const float* link_mass;
    const float* link_diag_inertia;
    const float* joint_damping;
    const float* joint_armature;
    const float* joint_stiffness;
    const float* joint_spring_reference;
    const uint32_t* body_role;
    const uint32_t* body_link;
    const float* body_local;
    const uint32_t* shape_kind;
    const float* shape_params;
    const uint32_t* shape_contype;
    const uint32_t* shape_conaffinity;
    const uint32_t* shape_group;
    const uint32_t* shape_profile;
    const float* profile_mu;
    /* joint rows and drives; read only when struct_size covers them */
    const float* joint_limit_lower;
    const float* joint_limit_upper;
    const uint8_t* joint_limit_flags;
    const float* joint_frictionloss;
    uint32_t drive_mode;
    uint32_t drive_rows;
    /* collidable rows that never pair; read only when struct_size covers them */
    const uint32_t* excluded_pairs;
    uint32_t excluded_pair_count;
    uint32_t reserved1;
    /* MuJoCo-law contact profiles; read only when struct_size covers them */
    const uint32_t* profile_law;
    const float* profile_solref;
    const float* profile_solimp;
    const float* profile_margin;
    uint32_t contact_cone;
    float contact_impratio;
    const int32_t* profile_priority;
    const float* profile_solmix;
    const uint32_t* profile_condim;
    /* MuJoCo-sourced joints and integrator; read only when struct_size covers them */
    const uint8_t* joint_law;
    const float* joint_limit_margin;
    const float* joint_limit_reference;
    const float* joint_friction_reference;
    uint32_t integrator;
    uint32_t free_body;   /* 1: the template's one link (floating root) is a free rigid body, stepped by the rigid-body ops */
} nko_template_desc;

typedef struct nko_world_desc {
    uint32_t struct_size;
    uint32_t env_count;
    float fixed_dt;
    float gravity[3];
    uint32_t solver_vel_iters;
    uint32_t solver_pos_iters;
    float solver_contact_margin;
    float solver_pos_beta;
    float solver_pos_slop;
    float solver_velocity_tolerance;
    float solver_baumgarte_max_velocity;
    float solver_overlap_recovery_velocity;
    uint32_t solver_fold_drive_damping;   /* read only when struct_size covers it */
    uint32_t solver_substeps;             /* 0 => 1; read, like the next member, only when struct_size covers it */
    uint32_t contact_detection_substeps;  /* 0 or 1 */
} nko_world_desc;

typedef struct nko_world nko_world;

nko_world* nko_world_create(const nko_template_desc* tmpl, const nko_world_desc* desc);
void nko_world_destroy(nko_world* w);
/* Host pointer and byte size of a named env-major field (or template table); 0 on success. */
int nko_world_field(nko_world* w, const char* name, void** ptr, size_t* bytes);
/* Comma-separated list of the field names nko_world_field serves. */
const char* nko_world_field_names(void);
void nko_world_set_threads(nko_world* w, int threads);
/* The line search's stopping rule.  0 (the default): the reference's (SearchTileLine, block_descent_tile.cuh:2089-2125),
 * whose rounding magnitude counts the heads' responses.  1: the magnitude also counts the rounding of the heads'
 * residuals, curvature x (|residual| + |move|) x |step| a head axis - the rule the HIP kernels apply - so that a test
 * can tell the kernels' arithmetic from that one deliberate difference. */
void nko_world_set_line_rule(nko_world* w, int rule);
uint32_t nko_real_bytes(void);
uint32_t nko_world_dof(const nko_world* w);
uint32_t nko_world_rows_per_env(const nko_world* w);

/* One call per reference op (src/nk/pipeline/pipeline.cpp op order). */
void nko_fk_world_poses(nko_world* w);
void nko_apply_drives(nko_world* w);
void nko_articulation_dynamics(nko_world* w, uint32_t integrate_velocity);
void nko_sync_link_body_pose(nko_world* w);
void nko_build_aabbs(nko_world* w);
void nko_query_pairs(nko_world* w);
void nko_narrowphase(nko_world* w);
void nko_assemble_rows(nko_world* w);
void nko_contact_warm_start(nko_world* w, uint32_t phase);
void nko_block_descent_solve(nko_world* w);
void nko_readout_drives(nko_world* w);
void nko_readout_contact_wrench(nko_world* w);   /* on demand: not part of nko_world_step until it has been called once,
                                                    then every interval ends with it (nk/pipeline/world.cpp:905-975) */
void nko_integrate_position(nko_world* w);
/* a free_body world's ops (articulation.cu:1019-1049 BodyIntegrateVelocityKernel with the tile's rigid block,
 * :1058-1117 BodyIntegratePositionKernel) and the free-rotation solve alone (rigid_types.cuh:38-121) */
void nko_body_integrate_velocity(nko_world* w);
void nko_body_integrate_position(nko_world* w);
uint32_t nko_solve_free_rotation(const float w0[3], const float inv_i[3], float dt, float midpoint[3], float* residual, uint32_t* iterations);
void nko_fk_link_velocities(nko_world* w);
/* The whole op list of one step, in the reference's order. */
void nko_world_step(nko_world* w);
/* ReferenceWeights (articulation.cu:425-500): body_invweight0 and dof_invweight0 at the current poses; creation runs it
 * once at the template's rest pose. */
void nko_reference_weights(nko_world* w);
void nko_snapshot_step_velocity(nko_world* w);
/* ArticulationDamping (articulation.cu:950-1000): the step's velocity change through (M + dt D)^-1 M */
void nko_articulation_damping(nko_world* w);
/* scene/contact_filter.hpp:100-137 MergeContactParams.  A side is mu1, mu2, solref[2], solimp[5], margin, gap, priority,
 * solmix, condim; out = mu1, mu2, solref[2], solimp[5], margin, gap, condim */
void nko_merge_contact_params(const float a[14], const float b[14], float out[12]);
uint64_t nko_contact_material_merged(const float merged[12], uint32_t law, uint32_t cone);

/* Stand-alone pieces exposed for unit pins. */
void nko_make_spatial_inertia(float mass, const float diag[3], const float inertial_frame[7], float out[36]);
void nko_factor_mass(const float* mass, float* factor, uint32_t n, uint32_t stride);
void nko_solve_mass(const float* factor, float* value, uint32_t n, uint32_t stride);
float nko_mass_coupling(const float* factor, uint32_t n, const float* v, const float* extra);
void nko_scalar_impulse(float dual, float rho, float residual, float compliance, float lower, float upper,
                        float out[2]);
void nko_tangent_impulse(const float dual[3], float rho, const float residual[3], float normal_impulse,
                         float mu_first, float mu_second, float impulse[3], float curvature[6]);
void nko_relax_contact_impulse(const float dual[3], const float next[3], float last_step[3], float* last_weight,
                               float last_point[3], float out[3]);
float nko_cone_argument(float dual, float rho, float mu, float residual);
/* FactorTileBlock + SolveTileBlock (block_descent_tile.cuh:1622-1666) up to 32 coordinates, FactorTileColumns +
 * SolveWideTileBlock (:209-252, 1866-1895) past them; see nko_solver.c */
int nko_tile_cholesky_solve(const float* h, uint32_t n, const float* g, float* factor, float* d);
/* The compliant (MuJoCo-law) row terms and the elliptic cone of the reference's row math (constraint/solref_solimp.hpp,
 * nk/solve/augmented_row.hpp:48-108), as the contact rows of a MuJoCo-sourced profile and the block descent use them. */
void nko_compliant_row_terms(const float solref[2], const float solimp[5], float pos_imp, float pos_aref, float vel, float invweight,
                             float dt, int refsafe, float out[6]);
void nko_discretize_compliant_row(float R, float aref_bias, float damping, float dt, float out[3]);
void nko_elliptic_impulse(const float dual[3], float cap, const float residual[3], const float compliance[3], float mu_first, float out[9]);
void nko_elliptic_multiplier_step(const float dual[3], const float next[3], float cap, const float compliance[3], float out[3]);
double nko_momentum_restart(const float point[3], const float next[3], const float base[3], const float scale[3]);
double nko_contact_projection_roundoff(const float start[3], const float end[3], const float axis[3]);
float nko_contact_query_reach(float thickness, float margin);
float nko_contact_motion_radius(float base, float dt, float sa, float sb, float relax);
int nko_shape_filter_admits(uint32_t ta, uint32_t aa, uint32_t ga, uint32_t tb, uint32_t ab, uint32_t gb);
int nko_pair_excluded(const nko_world* w, uint32_t a, uint32_t b);
int nko_pair_has_manifold(uint32_t kind_a, uint32_t kind_b);   /* the analytic pairs of PrimitivePair */
void nko_compose_transform(const float parent[7], const float child[7], float out[7]);
void nko_make_contact_id(uint32_t a, uint32_t b, const float local_a[3], const float local_b[3], uint32_t feature,
                         uint32_t manifold_slot, uint64_t out[2]);
/* analytical_manifold.hpp:931-966 PrimitivePair on two baked frames (cx, cy, cz, t) */
uint32_t nko_primitive_pair_frames(uint32_t kind_a, const float frame_a[12], const float params_a[4], uint32_t kind_b,
                                   const float frame_b[12], const float params_b[4], float query, float points[12],
                                   float normals[12], float penetration[4], uint64_t keys[4]);
/* cx, cy, cz, t of the baked prim frame (narrowphase_prims.cu:34-46 MakePrim) */
void nko_prim_frame(const float pose[7], float frame[12]);
uint32_t nko_sphere_plane(const float sphere_pose[7], float radius, const float plane_pose[7], float query,
                          float point[3], float normal[3], float* penetration);
uint32_t nko_box_plane(const float box_pose[7], const float half[3], const float plane_pose[7], float query,
                       float points[12], float normal[3], float penetration[4], uint32_t feature[4]);
void nko_contact_tangent_basis(const float normal[3], float t1[3], float t2[3]);

#ifdef __cplusplus
}
#endif
#endif
