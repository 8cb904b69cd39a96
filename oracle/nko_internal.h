/* Internal declarations of the CPU oracle (test infrastructure; see nuka_oracle.h). */
#ifndef NKO_INTERNAL_H_
#define NKO_INTERNAL_H_

#include <float.h>
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include "nuka_oracle.h"

#define NKO_INVALID 0xFFFFFFFFu
#define NKO_MAX_DOF 64u

/* phi/articulation_contract.hpp:8-16 */
enum { NKO_REVOLUTE = 0, NKO_PRISMATIC = 1, NKO_FIXED = 2, NKO_FLOATING = 3, NKO_SPHERICAL = 4 };
/* collision/shape_kind.hpp:9-18 */
enum { NKO_SPHERE = 0, NKO_CAPSULE = 1, NKO_BOX = 2, NKO_PLANE = 3, NKO_CYLINDER = 7 };
/* nk/solve/nk_row.hpp:14-19 */
enum { NKO_SIDE_RIGID = 0, NKO_SIDE_ARTIC = 1, NKO_SIDE_STATIC = 3 };
/* nk/solve/nk_row.hpp:41-57 */
enum {
    NKO_ROW_ACTIVE = 1u << 0, NKO_ROW_BLOCK_NORMAL = 1u << 2, NKO_ROW_BLOCK_TANGENT = 1u << 3,
    NKO_ROW_JOINT_LIMIT_LOWER = 1u << 4, NKO_ROW_JOINT_LIMIT_UPPER = 1u << 5,
    NKO_ROW_CONTACT_NORMAL = 1u << 6, NKO_ROW_VELOCITY_ONLY = 1u << 7, NKO_ROW_SPECULATIVE = 1u << 8,
    NKO_ROW_MUJOCO = 1u << 11, NKO_ROW_PYRAMIDAL = 1u << 12, NKO_ROW_FRICTION = 1u << 1
};
/* phi/op_schema.hpp:36-52 */
enum { NKO_STATUS_PAIR_OVERFLOW = 1u << 0, NKO_STATUS_DOF_OVERFLOW = 1u << 2, NKO_STATUS_GYRO_FAILURE = 1u << 5, NKO_STATUS_INVALID_ENDPOINT = 1u << 6,
       NKO_STATUS_CONTROL_FAILURE = 1u << 10, NKO_STATUS_SOLVER_FAILURE = 1u << 13 };
/* phi/articulation_contract.hpp:16-23 */
enum { NKO_DRIVE_PD_POSITION = 0, NKO_DRIVE_TORQUE = 1, NKO_DRIVE_VELOCITY = 2, NKO_DRIVE_COMPUTED_TORQUE = 3,
       NKO_DRIVE_OSC = 4, NKO_DRIVE_ACTUATOR = 5 };

typedef struct { float x, y, z; } v3;
typedef struct { float w, x, y, z; } quat;
typedef struct { v3 p; quat r; } xform;

/* nk/solve/nk_row.hpp:75-101: 26 words. */
typedef struct {
    uint32_t kind, index;
    v3 jlin, jang;
} nko_row_side;
typedef struct {
    uint32_t flags, group_first, group_normal_count, env;
    float rhs, compliance_alpha, lower, upper, mu, friction_secondary;
    nko_row_side a, b;
} nko_row;

/* Cooked template shared by every environment. */
typedef struct {
    uint32_t nl, nb, nv, max_dof, slots, rows_per_env, contact_rows_per_env, n_profiles, max_depth;
    /* joint row slots after the contact rows: 2 per link, 1 per link, 1 per link, or 0 (cook_to_model.cpp:706-719) */
    uint32_t joint_limit_rows, joint_friction_rows, joint_drive_rows, drive_mode;
    int floating;
    uint8_t* joint_type;
    uint32_t* parent_link;
    float* joint_axis;          /* nl*3 */
    float* parent_offset;       /* nl*3 */
    float* link_local_pose;     /* nl*7 */
    float* link_inertial_frame; /* nl*7 */
    float* link_inertia;        /* nl*36 */
    float* joint_damping, *joint_armature, *joint_stiffness, *joint_spring_reference;
    float* joint_limit_lower, *joint_limit_upper, *joint_frictionloss;   /* nl */
    uint8_t* joint_limit_flags;                                          /* nl: bit 0 lower, bit 1 upper */
    uint32_t* link_body;        /* nl */
    uint32_t* link_tree_depth;  /* nl */
    uint32_t* link_child_range; /* nl*2 */
    uint32_t* link_children;    /* nl */
    uint32_t* link_dof;         /* nl: first dof of the link */
    uint32_t* dof_link;         /* max_dof */
    uint32_t* dof_component;    /* max_dof, ~0 for scalar joints */
    float* link_geom_local;     /* nl*7 */
    uint32_t* link_geom_kind;   /* nl */
    float* shape_table;         /* nb*13 words */
    uint64_t* excluded_pairs;   /* sorted (a << 32 | b) keys of collidable rows that never pair, a < b */
    uint32_t excluded_count;
    uint32_t* body_to_link, *body_to_articulation, *body_collidable_link, *body_collidable_body;
    float* body_collidable_local; /* nb*7 */
    float* body_init_pose;        /* nb*7 */
    float* profile_mu;            /* n_profiles*2 */
    /* MuJoCo-law profiles (scene_ir.hpp:116; contact_filter.hpp:20-37): law source, solref, solimp, margin and gap */
    uint32_t* profile_law;        /* n_profiles */
    float* profile_mix;           /* n_profiles*3: priority, solmix, condim */
    uint8_t* joint_law;           /* nl: 1 MuJoCo-sourced joint rows */
    float *joint_limit_margin, *joint_limit_reference, *joint_friction_reference;   /* nl, nl*7 (solref, solimp), nl*7 */
    uint32_t integrator;          /* 0 native; 1 MuJoCo Euler (implicit joint damping after the solve); 2 with actuator derivatives */
    float* profile_solref;        /* n_profiles*2 */
    float* profile_solimp;        /* n_profiles*5 */
    float* profile_margin;        /* n_profiles*2 */
    uint32_t cone;                /* constraint::FrictionCone: 0 pyramidal, 1 elliptic */
    float impratio;
    int any_mujoco;
    /* the template's one link is a free rigid body, stepped by the reference's rigid-body ops (nko_rigid.c) */
    int free_body;
    float body_mass, body_diag_inertia[3];
} nko_template;

struct nko_world {
    nko_template t;
    nko_world_desc cfg;
    uint32_t env_count;
    int threads;
    int line_rule;   /* nko_world_set_line_rule */
    uint64_t step_index;
    /* env-major state */
    float *q, *qdot, *qddot, *tau, *base_pose, *link_pose, *link_velocity, *link_acceleration, *link_wrench;
    float *articulation_bias, *articulation_qdd, *m, *m_factor, *qdot_flat;
    float *qdot_pseudo, *link_velocity_pseudo;
    float *body_pose, *body_aabb_lo, *body_aabb_hi;
    /* the free body of a free_body world, one an environment (fields.yaml:102-103, 569; articulation.cu:1068-1070) */
    float *body_linear_velocity, *body_angular_velocity, *body_world_inv_inertia, *body_gyro_residual;
    uint32_t *body_gyro_iterations, *body_gyro_status;
    uint32_t *candidate_pairs, *pair_count;
    uint32_t *ucontact_count, *ucontact_a, *ucontact_b, *ucontact_law, *ucontact_row_range;
    float *ucontact_point, *ucontact_normal, *ucontact_depth;
    uint64_t *ucontact_id_pair, *ucontact_id_feature;
    float *urows, *lambda, *row_penetration, *row_cj_point, *row_cj_point_b, *chain_jacobian, *chain_jacobian_b;
    uint32_t *row_cj_link, *row_cj_link_b, *row_count, *contact_count, *contact_row_extent;
    uint32_t *env_status, *vbd_velocity_sweep_count;
    float *solver_residual;
    /* solver state kept between steps (block_descent.cu BlockScratch articulation_velocity/free) */
    float *solver_velocity, *solver_free, *solver_penalty;
    /* MuJoCo-law reference weights and per-row records (fields.yaml:863, 168-169) */
    float *body_invweight0, *dof_invweight0, *row_invweight, *row_reference_velocity_gain, *step_qdot_flat;
    /* contact cache carried between steps (fields.yaml:524-539, 155, 791, 844) */
    uint64_t *contact_material, *contact_cache_pair, *contact_cache_feature, *contact_cache_material;
    float *contact_cache_lambda, *contact_cache_normal;
    uint32_t *contact_cache_age, *contact_cache_current_owner, *contact_cache_old_keep, *contact_cache_extent;
    uint32_t *contact_warm_start_counts, *contact_cache_match;
    /* drives (fields.yaml:49-53, 328, 658-668, 548-551, 906) */
    float *drive_target, *drive_stiffness, *drive_damping, *drive_force_limit, *drive_joint_force_limit;
    float *velocity_target, *actuator_noload_speed, *joint_f, *joint_gravity_force;
    float *drive_command, *drive_dissipation, *drive_lower, *drive_upper;
    float *joint_limit_impulse, *actuator_effort_requested, *actuator_effort, *actuator_saturated;
    /* contact readout (ops/readout.cu ReadoutContactWrench) */
    float *contact_point, *contact_normal, *contact_force, *ucontact_impulse, *link_contact_wrench;
    uint32_t *contact_side_a_kind, *contact_side_b_kind, *contact_side_a_index, *contact_side_b_index, *contact_link;
    int fold_drive_damping;
    /* a step of several substeps (nk/pipeline/pipeline.cpp:56-180; ops/readout.cu AccumulateStepKernel) */
    uint32_t substeps;
    float outer_dt;
    int readout_in_step;
    uint32_t* step_env_status;
    float *step_link_impulse, *step_link_moment, *step_joint_limit_impulse;
};

/* ---- math (nko_math.c) ------------------------------------------------- */
static inline v3 v3_make(float x, float y, float z) { v3 r = {x, y, z}; return r; }
static inline v3 v3_add(v3 a, v3 b) { return v3_make(a.x + b.x, a.y + b.y, a.z + b.z); }
static inline v3 v3_sub(v3 a, v3 b) { return v3_make(a.x - b.x, a.y - b.y, a.z - b.z); }
static inline v3 v3_scale(v3 a, float s) { return v3_make(a.x * s, a.y * s, a.z * s); }
static inline float v3_dot(v3 a, v3 b) { return a.x * b.x + a.y * b.y + a.z * b.z; }
static inline v3 v3_cross(v3 a, v3 b) {
    return v3_make(a.y * b.z - a.z * b.y, a.z * b.x - a.x * b.z, a.x * b.y - a.y * b.x);
}
static inline float nko_rsqrt(float x) { return 1.0f / sqrtf(x); }
static inline quat quat_make(float w, float x, float y, float z) { quat q = {w, x, y, z}; return q; }
static inline xform xform_load(const float* p) {
    xform t; t.p = v3_make(p[0], p[1], p[2]); t.r = quat_make(p[3], p[4], p[5], p[6]); return t;
}
static inline void xform_store(float* p, xform t) {
    p[0] = t.p.x; p[1] = t.p.y; p[2] = t.p.z; p[3] = t.r.w; p[4] = t.r.x; p[5] = t.r.y; p[6] = t.r.z;
}
/* 32-bit patterns kept in scalar words.  In the double-precision build (nko_double.h) the word is a double that holds
 * the single-precision value of the pattern exactly, NaN payloads and subnormals included. */
#ifndef NKO_DOUBLE
typedef float nko_f32;
#endif
static inline uint32_t f2u(float f) { const nko_f32 g = (nko_f32)f; uint32_t u; memcpy(&u, &g, 4); return u; }
static inline float u2f(uint32_t u) { nko_f32 g; memcpy(&g, &u, 4); return g; }

quat nko_quat_mul(quat a, quat b);
quat nko_quat_normalize_rsqrt(quat q, float eps);
v3 nko_rotate_normalized(quat q, v3 v);
v3 nko_rotate_inverse(quat q, v3 v);
v3 nko_rotate_forward(quat q, v3 v);
v3 nko_prim_rotate(quat q, v3 v);
xform nko_compose_frame(xform parent, xform local);
xform nko_compose_hd(xform parent, xform child);
uint32_t nko_joint_dof(uint8_t type);

void nko_env_fk(const nko_world* w, uint32_t env);
void nko_env_apply_drives(nko_world* w, uint32_t env);
void nko_env_readout_drives(nko_world* w, uint32_t env);
void nko_env_joint_rows(nko_world* w, uint32_t env);
void nko_env_readout_contact_wrench(nko_world* w, uint32_t env);
void nko_env_dynamics(nko_world* w, uint32_t env, uint32_t integrate_velocity);
void nko_env_integrate_position(nko_world* w, uint32_t env);
void nko_env_body_integrate_velocity(nko_world* w, uint32_t env);
void nko_env_body_integrate_position(nko_world* w, uint32_t env);
void nko_body_center_of_mass(const nko_world* w, uint32_t env, float out[3]);
void nko_factor_mass(const float* mass, float* factor, uint32_t n, uint32_t stride);
void nko_env_link_velocities(nko_world* w, uint32_t env);
void nko_env_articulation_damping(nko_world* w, uint32_t env);
void nko_env_reference_weights(nko_world* w, uint32_t env);
/* the generalized force of a force f and a moment tau applied at `point`, added into one link's coordinates */
void nko_accumulate_chain(const nko_world* w, uint32_t env, uint32_t link_local, uint32_t dof_index, v3 point, v3 f, v3 tau, float* out);
void nko_env_sync_body_pose(nko_world* w, uint32_t env);
void nko_env_aabbs(nko_world* w, uint32_t env);
void nko_env_pairs(nko_world* w, uint32_t env);
int nko_template_pair_excluded(const nko_template* t, uint32_t a, uint32_t b);   /* a < b */
void nko_env_narrowphase(nko_world* w, uint32_t env);
void nko_env_assemble_rows(nko_world* w, uint32_t env);
void nko_env_warm_start_prepare(nko_world* w, uint32_t env);
void nko_env_warm_start_commit(nko_world* w, uint32_t env);
uint64_t nko_contact_material(float mu1, float mu2, uint32_t law);
void nko_env_solve(nko_world* w, uint32_t env);
void nko_joint_transform(const nko_world* w, uint32_t env, uint32_t link, float X[36]);
void nko_motion_subspace(uint8_t type, v3 axis, float s[6]);

#endif
