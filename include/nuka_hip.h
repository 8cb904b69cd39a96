/*
 * C ABI of the MI355X articulation-step library (libnuka_hip.so).  Plain pointers and sizes only.
 *
 * Two groups of declarations:
 *   - what the reference's stable C surface (src/include/nuka/nuka.h) declares for the batched articulation step, under
 *     the reference's own names and with its layouts, signatures and numeric values: result codes, device and world
 *     descriptors, nuka_world_create_from_scene, step / reset / checkpoint / parameter / execution-mode calls, the
 *     NUKA_FIELD_* ids of the fields this library serves, buffer views and byte transfers.  A caller compiled against
 *     nuka.h that uses only these links against this library unchanged; every such entry cites the lines it matches.
 *   - the library's own additions, which no reference name is reused for: the cooked-template creator
 *     (nuka_hip_world_desc_t, nuka_world_create_from_template), scene handles (nuka_scene_*,
 *     nuka_hip_world_create_from_scene_handle), per-op dispatch, the extended field ids (every internal field by
 *     name, from NUKA_HIP_FIELD_BASE up) and the timing helpers the benchmark uses.
 */
#ifndef NUKA_HIP_H_
#define NUKA_HIP_H_

#include <stddef.h>
#include <stdint.h>

#include "nuka_phi.h"

#ifdef __cplusplus
extern "C" {
#endif

/* nuka.h:22-32.  Code 3 is the reference's device-runtime error; NUKA_RESULT_DEVICE_ERROR names the same value. */
typedef enum nuka_result_t {
    NUKA_RESULT_OK = 0,
    NUKA_RESULT_INVALID_ARG = 1,
    NUKA_RESULT_NULL_HANDLE = 2,
    NUKA_RESULT_CUDA_ERROR = 3,
    NUKA_RESULT_DEVICE_ERROR = 3,
    NUKA_RESULT_FILE_NOT_FOUND = 4,
    NUKA_RESULT_PARSE_ERROR = 5,
    NUKA_RESULT_OUT_OF_MEMORY = 6,
    NUKA_RESULT_NOT_SUPPORTED = 7,
    NUKA_RESULT_INTERNAL = 100
} nuka_result_t;

typedef struct nuka_device_t* nuka_device_handle;
typedef struct nuka_world_t* nuka_world_handle;

/* nuka.h:40-44 */
const char* nuka_result_message(nuka_result_t result);
const char* nuka_last_error_message(void);

/* nuka.h:46-51, member for member.  `cuda_stream` (the reference's name for the member) non-null is a borrowed
 * hipStream_t; null creates an owned stream at default priority. */
typedef struct nuka_device_desc_t {
    uint32_t gpu_index;
    void* cuda_stream;
    uint8_t backend_selection_layer_enabled;
} nuka_device_desc_t;
nuka_result_t nuka_device_create(const nuka_device_desc_t* desc, nuka_device_handle* out);
void nuka_device_destroy(nuka_device_handle device);
/* The PHI backend a device owns (src/c_abi/internal.hpp:57-69 DeviceRecord). */
nuka_phi_backend* nuka_device_backend(nuka_device_handle device);

/* Cook inputs of one environment (src/runtime/articulation/articulation_state.cpp:345-435 BuildArticulationHostState,
 * src/scene/cook/cook_to_model.cpp collidable rows).  Arrays are per link / per collidable row. */
typedef struct nuka_template_desc_t {
    uint32_t struct_size;
    uint32_t link_count;
    uint32_t body_count;
    uint32_t profile_count;
    uint32_t max_contacts_per_env;   /* contact slots per env; 0 => admitted collidable pairs of the template */
    uint32_t reserved0;
    const uint8_t* joint_type;       /* phi/articulation_contract.hpp:8-16; link 0 is the root */
    const uint32_t* parent_link;     /* ~0u for the root */
    const float* joint_axis;         /* [link][3], in the child joint frame */
    const float* parent_offset;      /* [link][3], nullable */
    const float* link_local_pose;    /* [link][7] px py pz qw qx qy qz, parent to child at q = 0 */
    const float* link_inertial_frame;/* [link][7] */
    const float* link_mass;          /* [link] */
    const float* link_diag_inertia;  /* [link][3] */
    const float* joint_damping;      /* [link], nullable */
    const float* joint_armature;     /* [link], nullable */
    const float* joint_stiffness;    /* [link], nullable */
    const float* joint_spring_reference; /* [link], nullable */
    const uint32_t* body_role;       /* 0 static, 1 the link's own body row, 2 extra collidable of a link */
    const uint32_t* body_link;       /* owning link for roles 1 and 2 */
    const float* body_local;         /* [row][7]: world pose (static) or pose in the owning link's frame */
    const uint32_t* shape_kind;      /* collision/shape_kind.hpp:9-18: sphere 0, capsule 1, box 2, plane 3, cylinder 7;
                                        ~0u for no shape */
    const float* shape_params;       /* [row][4]: radius | radius, half length along local z | half extents */
    const uint32_t* shape_contype;
    const uint32_t* shape_conaffinity;
    const uint32_t* shape_group;
    const uint32_t* shape_profile;   /* friction profile row, ~0u for the default (mu 1) */
    const float* profile_mu;         /* [profile][2] */
    /* Joint rows and drives (src/scene/cook/cook_to_model.cpp:696-719); read only when struct_size covers them. */
    const float* joint_limit_lower;  /* [link], nullable */
    const float* joint_limit_upper;  /* [link], nullable */
    const uint8_t* joint_limit_flags;/* [link] bit 0: lower bound authored, bit 1: upper; nullable.  Any bit set gives
                                        every link its two limit row slots */
    const float* joint_frictionloss; /* [link], nullable; any positive entry gives every link a friction row slot */
    uint32_t drive_mode;             /* phi/articulation_contract.hpp:16-23: 0 PD position, 1 torque, 2 velocity, 5 actuator */
    uint32_t drive_rows;             /* 0: the field `tau` is the applied generalized force and no drive rows exist;
                                        1: the reference's actuation - ApplyDrives turns the drive_* fields into one
                                        bounded-effort row per link, overwrites `tau` with `joint_f` and ReadoutDrives
                                        reports the applied effort (src/nk/pipeline/world.cpp:61) */
    /* Collidable rows that never pair (src/scene/cooker.cpp:470-538 excluded_body_pairs, carried to collidable rows
     * at src/scene/cook/cook_to_model.cpp:1468-1490); read only when struct_size covers them.  Two rows of one link
     * are excluded by the cook itself. */
    const uint32_t* excluded_pairs;  /* [pair][2] collidable rows, either order; nullable */
    uint32_t excluded_pair_count;
    uint32_t reserved1;
    /* The MuJoCo contact law (src/constraint/law_source.hpp; src/scene/contact_filter.hpp:20-37 ContactParamsIn), read
     * only when struct_size covers it.  A pair with a MuJoCo-sourced profile on either side builds compliant rows from
     * the merged solref/solimp of both sides (src/phi/backend_cuda/ops/assemble_rows.cu:540-800) in place of the
     * native velocity rows. */
    const uint32_t* profile_law;     /* [profile] 0 native, 1 MuJoCo-sourced; nullable */
    const float* profile_solref;     /* [profile][2] timeconst, dampratio (or -stiffness, -damping); nullable => 0.02, 1 */
    const float* profile_solimp;     /* [profile][5] dmin dmax width midpoint power; nullable => 0.9 0.95 0.001 0.5 2 */
    const float* profile_margin;     /* [profile][2] margin, gap; nullable => 0, 0 */
    uint32_t contact_cone;           /* <option cone>: 0 pyramidal (four edge rows a point), 1 elliptic */
    float contact_impratio;          /* <option impratio>; 0 => 1 */
    /* How two sides' profiles merge (src/scene/contact_filter.hpp:89-137), read only when struct_size covers them */
    const int32_t* profile_priority; /* [profile] the higher priority gives friction and condim and all of the mixing
                                        weight; nullable => 0 */
    const float* profile_solmix;     /* [profile] mixing weight at equal priority; nullable => 1 */
    const uint32_t* profile_condim;  /* [profile] 3: a normal and two friction rows a point; 1: the normal alone;
                                        nullable => 3 */
    /* MuJoCo-sourced joints and integrator (src/scene/cook/cook_to_model.cpp:662-693; src/nk/pipeline/pipeline.cpp:264-265,
     * 939-951), read only when struct_size covers them.  Such a joint's limit and dry-friction rows are compliant rows
     * of its own solref / solimp (src/phi/backend_cuda/ops/assemble_rows.cu:860-877, 921-931). */
    const uint8_t* joint_law;              /* [link] 0 native, 1 MuJoCo-sourced; nullable */
    const float* joint_limit_margin;       /* [link]; nullable => 0 */
    const float* joint_limit_reference;    /* [link][7] solref[2], solimp[5] of the limit rows; nullable => 0.02 1, 0.9 0.95 0.001 0.5 2 */
    const float* joint_friction_reference; /* [link][7] of the dry-friction row; nullable => the same */
    uint32_t integrator;                   /* 0 native (damping of drives folded into the solve); 1 MuJoCo's Euler: joint
                                              damping applied implicitly after the solve, the step's velocity change
                                              through (M + dt D)^-1 M; 2 implicit / implicitfast: the servos' velocity
                                              gains join D */
    uint32_t free_body;                    /* 1: the template's one link (link_count 1, a floating root) is a free rigid body.
                                              The reference's rigid-body ops step it (BodyIntegrateVelocityKernel,
                                              src/phi/backend_cuda/ops/articulation.cu:1019-1049; the six by six block of the
                                              tile, ops/block_descent_rigid.cuh:4-48, ops/block_descent_tile.cuh:541-603;
                                              BodyIntegratePositionKernel with the free-rotation solve, articulation.cu:1058-1117,
                                              ops/rigid_types.cuh:38-121): base_pose is the body's pose, link_mass,
                                              link_diag_inertia and link_inertial_frame its inertial parameters,
                                              BODY_LINEAR_VELOCITY / BODY_ANGULAR_VELOCITY its state (world axes, about the
                                              centre of mass), link_wrench the force and torque applied at the centre of
                                              mass.  One free body an environment; statics beside it */
} nuka_template_desc_t;

/* The world options of the cooked-template creator (the library's own descriptor; the reference's nuka_world_desc_t
 * follows below).  Zero keeps the default of the reference field of the same name (nuka.h:160-173). */
typedef struct nuka_hip_world_desc_t {
    uint32_t struct_size;
    uint32_t env_count;
    float fixed_dt;                  /* 0 => 1/240 */
    float gravity[3];
    uint32_t solver_vel_iters;       /* 0 => 10 (op_schema.hpp:598) */
    uint32_t solver_pos_iters;       /* 0 => 4; ~0u => no position pass */
    float solver_contact_margin;
    float solver_pos_beta;           /* 0 => 0.3 */
    float solver_pos_slop;           /* 0 => 1e-3 */
    float solver_velocity_tolerance; /* 0 => 1e-5 (op_schema.hpp:663) */
    float solver_baumgarte_max_velocity;   /* 0 => 3e38 */
    float solver_overlap_recovery_velocity;
    uint32_t solver_fold_drive_damping;    /* 0 => on (pipeline.hpp:48-49): a drive's velocity feedback is solved
                                              implicitly through the mass matrix; ~0u => off.  Read only when
                                              struct_size covers it */
    uint32_t solver_substeps;              /* nuka.h:171: substeps of dt / substeps each step runs; 0 => 1.  Status words
                                              are or-ed over the substeps, joint limit impulses summed, the links'
                                              contact wrenches averaged over the step (src/nk/pipeline/pipeline.cpp:118-180).
                                              Read, like the next member, only when struct_size covers it */
    uint32_t contact_detection_substeps;   /* nuka.h:172: 0 or 1; substeps that share a detection are NOT_SUPPORTED */
} nuka_hip_world_desc_t;

/* nuka.h:57-173, member for member: same names, types, order and therefore offsets.  nuka_world_create_from_scene reads
 * scene_path, env_count, fixed_dt, determinism, control_mode, gravity_*, solver_vel_iters, solver_pos_iters,
 * solver_contact_margin, solver_baumgarte_max_velocity, solver_overlap_recovery_velocity, solver_substeps and
 * contact_detection_substeps.  The members that ask for what this library does not build must be zero (null), else the
 * creation is refused with NUKA_RESULT_NOT_SUPPORTED: terrain_*, instance_count above 1, contact_family,
 * heightfield_*, curric_*, terrain_feature_cell, cloth_integrator, ogc_contact_capacity, control modes 3 and 4.
 * solver_max_pairs is accepted and has no effect (every admitted pair of an environment has its own slot here). */
typedef struct nuka_world_desc_t {
    const char* scene_path;
    uint32_t env_count;
    float fixed_dt;
    uint8_t determinism;             /* 0 or 1; both run the same deterministic kernels */
    uint8_t control_mode;            /* 0 PD position, 1 torque, 2 velocity, 3 computed torque, 4 OSC, 5 actuator */
    uint32_t osc_task_link;
    float terrain_step_height;
    float terrain_step_width;
    float terrain_platform_width;
    float terrain_grid_width;
    float terrain_grid_height_max;
    uint32_t instance_count;
    float instance_spacing;
    uint32_t contact_family;
    uint32_t heightfield_terrain_type;
    uint32_t heightfield_nrow;
    uint32_t heightfield_ncol;
    float heightfield_cell;
    const char* heightfield_image_path;
    float heightfield_radius_x;
    float heightfield_radius_y;
    float heightfield_elevation_z;
    float heightfield_base_z;
    float gravity_x;                 /* all three zero => {0, 0, -9.81} */
    float gravity_y;
    float gravity_z;
    uint32_t curric_levels;
    uint32_t curric_types;
    float terrain_feature_cell;
    uint32_t solver_vel_iters;       /* 0 => 10 */
    uint32_t solver_pos_iters;       /* 0 => 4 */
    float solver_contact_margin;
    uint32_t solver_max_pairs;
    float solver_baumgarte_max_velocity;
    uint32_t cloth_integrator;
    uint32_t ogc_contact_capacity;
    float solver_overlap_recovery_velocity;
    uint32_t solver_substeps;
    uint32_t contact_detection_substeps;
} nuka_world_desc_t;

/* Scene files (src/import/mjcf_importer.cpp LoadMjcf and src/import/urdf_importer.cpp LoadUrdf, then the articulation
 * part of the cook): a robot description read into the cook inputs of one environment.  One articulation per file.
 * MJCF: bodies, default classes, hinge / slide / free joints (several per body), inertial elements or geom-derived
 * mass, sphere / capsule / box / cylinder / plane collision geoms, joint ranges, damping, armature, frictionloss,
 * springs, <contact><exclude>, and position / velocity / motor actuators.  URDF: links with inertial and collision
 * elements (box, sphere, cylinder, capsule), revolute / continuous / prismatic / fixed joints with origin, axis, limits,
 * dynamics and effort (a bounded torque motor), nuka:exclude.  A body never pairs with its parent body or with a body
 * welded to it (src/scene/cooker.cpp:470-538).  Joint and contact rows use this library's native laws (no solref /
 * solimp compliance). */
typedef struct nuka_scene_t* nuka_scene_handle;
/* Keep the shapes this library has manifolds for and drop (and count) the other colliding geoms; the robot's geoms
 * share one negative collision group, so that they meet static shapes and not each other. */
#define NUKA_SCENE_PLANE_CONTACTS_ONLY 1u
/* URDF only: the root link is welded to the world (the importer's fix_base option, src/import/urdf_importer.cpp:655-661);
 * without it the root link floats. */
#define NUKA_SCENE_FIXED_BASE 2u
/* A static ground plane z = 0 joins the file's collidables (a URDF describes the robot only). */
#define NUKA_SCENE_GROUND_PLANE 4u
/* MJCF only: the geoms keep the native contact law (speculative velocity rows).  Without it every geom is
 * MuJoCo-sourced, as in the reference's importer (src/import/mjcf_importer.cpp:790): its friction, solref, solimp,
 * margin and gap make a contact profile of the MuJoCo law, with the cone and impratio of <option>. */
#define NUKA_SCENE_NATIVE_CONTACT_LAW 8u
/* MJCF only: the joints keep the native limit and dry-friction rows and the native integrator.  Without it every joint is
 * MuJoCo-sourced (src/import/mjcf_importer.cpp:1193, 1720): its limit rows are compliant rows of margin / solreflimit /
 * solimplimit, its dry friction of solreffriction / solimpfriction, and joint damping is applied implicitly after the
 * solve as <option integrator> says (Euler by default; implicit and implicitfast add the servos' velocity gains). */
#define NUKA_SCENE_NATIVE_JOINT_LAW 16u
nuka_result_t nuka_scene_load_mjcf(const char* path, uint32_t flags, nuka_scene_handle* out);
nuka_result_t nuka_scene_load_urdf(const char* path, uint32_t flags, nuka_scene_handle* out);
void nuka_scene_destroy(nuka_scene_handle scene);
/* The cook inputs; the arrays live as long as the scene. */
const nuka_template_desc_t* nuka_scene_template(nuka_scene_handle scene);
typedef struct nuka_scene_info_t {
    uint32_t link_count, body_count, actuator_count, dropped_geom_count, floating_root, drive_mode;
    float timestep;
    float gravity[3];
} nuka_scene_info_t;
nuka_result_t nuka_scene_get_info(nuka_scene_handle scene, nuka_scene_info_t* out);
/* The MJCF body behind a link ("<body>_anchor" for the static anchor of a jointed root, "<body>/<joint>" for the
 * massless links between several joints of one body) and the joint that moves it ("" for a welded body). */
const char* nuka_scene_link_name(nuka_scene_handle scene, uint32_t link);
const char* nuka_scene_joint_name(nuka_scene_handle scene, uint32_t link);
/* What the file authors beyond the template, per link: initial coordinate, drive stiffness / damping / force limit from
 * its actuators and the joint's actuator force range; base_pose[7] of a floating root.  Null outputs are skipped. */
nuka_result_t nuka_scene_initial_state(nuka_scene_handle scene, float* q, float* base_pose, float* drive_stiffness,
                                       float* drive_damping, float* drive_force_limit, float* drive_joint_force_limit);
/* A loaded scene's template in every environment, its initial state and drive parameters uploaded (PD targets hold
 * the initial pose), and that state kept as what nuka_world_reset returns to.  `desc->fixed_dt` of 0 takes the file's
 * timestep; gravity of all zeros takes the file's. */
nuka_result_t nuka_hip_world_create_from_scene_handle(nuka_device_handle device, nuka_scene_handle scene,
                                                      const nuka_hip_world_desc_t* desc, nuka_world_handle* out);

/* nuka.h:175-177, src/c_abi/world.cpp:590-635: the file at desc->scene_path read by its extension (.xml or .mjcf as
 * MJCF, .urdf as URDF; .nks and OpenUSD files are NUKA_RESULT_NOT_SUPPORTED, as is any other extension) and stepped in
 * desc->env_count environments.  As in the reference a null desc, a null scene_path, fixed_dt <= 0, env_count 0,
 * determinism above 1 or an unknown control mode is NUKA_RESULT_INVALID_ARG and a null device NUKA_RESULT_NULL_HANDLE;
 * a file that cannot be opened is NUKA_RESULT_FILE_NOT_FOUND and one that cannot be read as its format, or holds what
 * this library has no path for (meshes, several articulations), NUKA_RESULT_PARSE_ERROR or NUKA_RESULT_NOT_SUPPORTED
 * with the reason in nuka_last_error_message.  The control mode is the descriptor's, the drive gains the file's. */
nuka_result_t nuka_world_create_from_scene(nuka_device_handle device, const nuka_world_desc_t* desc, nuka_world_handle* out);

/* The cooked-template creator: what SceneIR -> CookToModel produces for one environment, passed directly. */
nuka_result_t nuka_world_create_from_template(nuka_device_handle device, const nuka_template_desc_t* tmpl,
                                              const nuka_hip_world_desc_t* desc, nuka_world_handle* out);
void nuka_world_destroy(nuka_world_handle world);            /* nuka.h:253 */
nuka_result_t nuka_world_step(nuka_world_handle world);      /* nuka.h:254, src/c_abi/world.cpp:696-698 */
nuka_result_t nuka_world_step_n(nuka_world_handle world, uint32_t step_count);   /* nuka.h:255, world.cpp:700-731 */

/* nuka.h:257-279 */
typedef enum nuka_execution_mode_t { NUKA_EXECUTION_EAGER = 0, NUKA_EXECUTION_GRAPH = 1 } nuka_execution_mode_t;
nuka_result_t nuka_world_set_execution_mode(nuka_world_handle world, nuka_execution_mode_t mode);
/* nuka.h:261-275, 342: how the world executes - mode, whether a captured graph stands, captures and graph replays so
 * far, and the last failure of a dispatch, capture or replay (status mapped to a result, the op, the HIP error code). */
enum { NUKA_EXECUTION_INFO_VERSION = 1 };
typedef struct nuka_world_execution_info_t {
    uint32_t struct_size;
    uint32_t schema_version;
    nuka_execution_mode_t mode;
    uint32_t graph_ready;
    uint64_t capture_attempts;
    uint64_t graph_replays;
    nuka_result_t last_result;
    uint32_t failed_op;
    int32_t native_error;
    char message[256];
} nuka_world_execution_info_t;
nuka_result_t nuka_world_get_execution_info(nuka_world_handle world, nuka_world_execution_info_t* out);
nuka_result_t nuka_world_set_velocity_iterations(nuka_world_handle world, uint32_t iterations);   /* nuka.h:289 */
nuka_result_t nuka_world_get_velocity_iterations(nuka_world_handle world, uint32_t* out_iterations);
nuka_result_t nuka_world_synchronize(nuka_world_handle world);   /* nuka.h:376 */
nuka_result_t nuka_world_reset(nuka_world_handle world);         /* nuka.h:380 */
/* nuka.h:381-385: duplicates are ignored, count 0 is a no-op, an id out of range returns INVALID_ARG and changes nothing */
nuka_result_t nuka_world_reset_envs(nuka_world_handle world, const uint32_t* env_ids, uint32_t count);
/* No counterpart in the reference.  nuka_world_reset_envs for callers that cannot allocate (tight serving loops,
 * harnesses that forbid hipMalloc): the same kernel and the same result, with the ids staged in a device array of
 * static storage, NUKA_RESET_ENVS_STATIC_MAX words that each GPU the library has opened holds until the process ends,
 * instead of in memory the library allocates.  Takes no device memory and no host heap memory.  More ids than the
 * maximum are refused with NUKA_RESULT_INVALID_ARG (nuka_last_error_message says so).  The call blocks the host on the
 * world's stream (it waits for the stream before it stages the ids and again before it returns), so it does not belong
 * inside a stream capture.  Every call on one GPU shares that GPU's array; the library serialises such calls on a
 * process-wide lock held until the call's reset has finished, so they do not overlap. */
#define NUKA_RESET_ENVS_STATIC_MAX 16384u
nuka_result_t nuka_world_reset_envs_static(nuka_world_handle world, const uint32_t* env_ids, uint32_t count);

/* nuka.h:386-398: a checkpoint holds the persistent physics of every environment, in device memory here.  Restore
 * is enqueued on the world's stream (no host wait) and refuses a checkpoint of another world. */
typedef struct nuka_checkpoint_t* nuka_checkpoint_handle;
nuka_result_t nuka_world_checkpoint_capture(nuka_world_handle world, nuka_checkpoint_handle* out);
nuka_result_t nuka_world_checkpoint_restore(nuka_world_handle world, nuka_checkpoint_handle checkpoint);
void nuka_checkpoint_destroy(nuka_checkpoint_handle checkpoint);
nuka_result_t nuka_checkpoint_byte_size(nuka_checkpoint_handle checkpoint, uint64_t* out_bytes);
/* nuka.h:394-398: a checkpoint as a file - a header with the layout hash of the world it was taken of (environment
 * count, names and sizes of the persistent fields) and the persistent bytes.  Reading makes a checkpoint of `world`
 * from the file; a file of another layout, a truncated one or one that is no checkpoint is INVALID_ARG.  The format is
 * this library's own, not the reference's. */
nuka_result_t nuka_checkpoint_write(nuka_checkpoint_handle checkpoint, const char* path);
nuka_result_t nuka_world_checkpoint_read(nuka_world_handle world, const char* path, nuka_checkpoint_handle* out);
/* nuka.h:401-402: 1 when both checkpoints were taken of worlds of one layout and hold the same persistent bytes, else 0 */
nuka_result_t nuka_checkpoint_equal(nuka_checkpoint_handle a, nuka_checkpoint_handle b, uint32_t* out_equal);
/* nuka.h:403-404, src/c_abi/checkpoint.cpp:601-636: 64-bit FNV-1a over a domain string, the byte count and the
 * persistent physics bytes in field order.  Waits for the device.  Two runs of one build from the same inputs hash
 * alike; the value is not comparable with the reference's, whose persistent arena holds other fields. */
nuka_result_t nuka_world_state_hash(nuka_world_handle world, uint64_t* out_hash);

/* nuka.h:433-434, nk::World::RefreshPoses (src/nk/pipeline/world.cpp:778-793): link and body poses from the joint
 * coordinates and base poses, without advancing time. */
nuka_result_t nuka_world_forward_kinematics(nuka_world_handle world);

/* The tunable parameters of a world (nuka.h:281-285, 304-341; src/c_abi/params.cpp): world options and values of one
 * template link that hold in every environment.  Indices, keys, units and ranges are the reference's:
 *   0 gravity_z            1 velocity_iterations   2 link_mass        3 joint_damping
 *   4 joint_armature       5 joint_frictionloss    6 drive_stiffness  7 drive_force_limit
 * Parameters 0 and 1 have one element, the others one per template link.  A LIVE value applies at the next step and
 * survives nuka_world_reset.  link_mass keeps the link's centre of mass and its rotational inertia about it;
 * drive_stiffness also sets the drive's damping to 2 sqrt(stiffness), as the cook derives it.  joint_frictionloss is
 * REBUILD (set returns NOT_SUPPORTED) in a world cooked without joint friction rows.  NOT_SUPPORTED also for a joint
 * parameter of a link whose joint has no scalar coordinate (the root, a fixed joint) and for a drive parameter in a
 * world without drive rows. */
typedef enum nuka_param_type_t { NUKA_PARAM_F32 = 0, NUKA_PARAM_U32 = 1 } nuka_param_type_t;
typedef enum nuka_param_tier_t { NUKA_PARAM_LIVE = 0, NUKA_PARAM_REBUILD = 1 } nuka_param_tier_t;
enum { NUKA_PARAM_INFO_VERSION = 1 };
typedef struct nuka_param_info_t {
    uint32_t struct_size;
    uint32_t schema_version;
    char key[48];
    char unit[16];
    char scene_field[48];
    nuka_param_type_t type;
    nuka_param_tier_t tier;
    uint32_t count;
    double min_value;
    double max_value;
} nuka_param_info_t;
nuka_result_t nuka_world_param_count(nuka_world_handle world, uint32_t* out_count);
/* every entry carries struct_size and schema_version on entry; capacity covers the count */
nuka_result_t nuka_world_get_param_infos(nuka_world_handle world, nuka_param_info_t* infos, uint32_t capacity);
nuka_result_t nuka_world_get_param(nuka_world_handle world, uint32_t param, uint32_t element, double* out_value);
nuka_result_t nuka_world_set_param(nuka_world_handle world, uint32_t param, uint32_t element, double value);
nuka_result_t nuka_world_set_link_mass(nuka_world_handle world, uint32_t link_index, float mass);   /* nuka.h:282 */
nuka_result_t nuka_world_set_gravity_z(nuka_world_handle world, float gravity_z);                   /* nuka.h:285 */

/* nk::World::DispatchOp (src/nk/pipeline/world.hpp): one op of the pipeline with the pipeline's own parameters.
 * `variant` 1 on ArticulationDynamics dispatches it with integrate_velocity = 0, the probe
 * tests/oracle/featherstone_oracle_harness.cpp:174-182 uses. */
nuka_result_t nuka_world_dispatch_op(nuka_world_handle world, uint16_t op, uint32_t variant);

/* nuka.h:496-958: the public field ids, with the reference's numeric values, for the fields this library serves
 * (any other value below NUKA_HIP_FIELD_BASE is NUKA_RESULT_NOT_SUPPORTED, as the reference answers for a field a world
 * does not hold).  A view of one of these has the reference's element stride (src/c_abi/dlpack_table.hpp:101-330): 28
 * bytes for a pose, 24 for a spatial vector, 12 for a vector, the field's element size otherwise. */
typedef enum nuka_state_field_t {
    NUKA_FIELD_RIGID_BODY_TRANSFORM = 0,        /* body_pose */
    NUKA_FIELD_ARTICULATION_LINK_POSE = 1,      /* link_pose */
    NUKA_FIELD_JOINT_POSITION = 2,              /* q */
    NUKA_FIELD_JOINT_VELOCITY = 3,              /* qdot */
    NUKA_FIELD_CONTACT_POINTS = 5,              /* contact_point */
    NUKA_FIELD_DRIVE_TARGET = 6,
    NUKA_FIELD_LINK_VELOCITY = 7,
    NUKA_FIELD_DRIVE_STIFFNESS = 8,
    NUKA_FIELD_DRIVE_DAMPING = 9,
    NUKA_FIELD_DRIVE_FORCE_LIMIT = 10,
    NUKA_FIELD_BASE_POSE = 11,
    NUKA_FIELD_TORQUE_INPUT = 12,               /* the storage of DRIVE_TARGET, as in the reference */
    NUKA_FIELD_VELOCITY_TARGET = 13,
    NUKA_FIELD_ACTUATOR_NOLOAD_SPEED = 14,
    NUKA_FIELD_LINK_CONTACT_WRENCH = 16,
    NUKA_FIELD_CONTACT_NORMAL = 17,
    NUKA_FIELD_CONTACT_FORCE = 18,
    NUKA_FIELD_CONTACT_LINK = 19,
    NUKA_FIELD_JOINT_FEEDFORWARD = 22,          /* joint_f */
    NUKA_FIELD_BODY_LINEAR_VELOCITY = 25,       /* per body row; a free body's values in its own row */
    NUKA_FIELD_BODY_ANGULAR_VELOCITY = 26,
    NUKA_FIELD_JOINT_LIMIT_IMPULSE = 27,
    NUKA_FIELD_ACTUATOR_EFFORT_REQUESTED = 28,
    NUKA_FIELD_ACTUATOR_EFFORT = 29,
    NUKA_FIELD_ACTUATOR_SATURATED = 30,
    NUKA_FIELD_CONTACT_SIDE_A_KIND = 33,
    NUKA_FIELD_CONTACT_SIDE_B_KIND = 34,
    NUKA_FIELD_CONTACT_SIDE_A_INDEX = 35,
    NUKA_FIELD_CONTACT_SIDE_B_INDEX = 36,
    NUKA_FIELD_ENV_STATUS = 39,
    NUKA_FIELD_CONTACT_WARM_START_COUNTS = 70,
    NUKA_FIELD_VBD_VELOCITY_SWEEP_COUNT = 79,
    NUKA_FIELD_UCONTACT_ROW_RANGE = 103,
    NUKA_FIELD_LINK_WRENCH = 105,
    NUKA_FIELD_UCONTACT_COUNT = 107,
    NUKA_FIELD_UCONTACT_POINT = 108,
    NUKA_FIELD_SOLVER_RESIDUAL = 109,
    NUKA_FIELD_UCONTACT_NORMAL = 128,
    NUKA_FIELD_UCONTACT_DEPTH = 129,
    NUKA_FIELD_UCONTACT_LAW = 132,
    NUKA_FIELD_UCONTACT_SIDE_A = 134,
    NUKA_FIELD_UCONTACT_SIDE_B = 135,
    NUKA_FIELD_UCONTACT_IMPULSE = 138,
    NUKA_FIELD_JOINT_GRAVITY_FORCE = 157,
    NUKA_FIELD_ROW_PENETRATION = 161,
    NUKA_FIELD_ROW_LAMBDA = 162,
    /* The library's own ids: every field of the world by its name in src/nk/model/fields.yaml (m, m_factor, urows,
     * chain_jacobian, ...), NUKA_HIP_FIELD_BASE + its place in nuka_field_names().  Views of these count 4- or 8-byte
     * scalars. */
    NUKA_HIP_FIELD_BASE = 0x10000,
    NUKA_HIP_FIELD_NONE = 0x7FFFFFFF
} nuka_state_field_t;
/* NUKA_HIP_FIELD_NONE when the library serves no field of that name. */
nuka_state_field_t nuka_field_from_name(const char* name);
const char* nuka_field_names(void);   /* comma separated */

/* nuka.h:1158-1168 */
typedef struct nuka_buffer_view_t {
    void* device_ptr;
    size_t element_count;
    uint32_t element_stride_bytes;
    uint8_t dtype;   /* 0 float32, 1 uint32, 2 uint64, 3 uint8 */
} nuka_buffer_view_t;
nuka_result_t nuka_world_get_buffer_view(nuka_world_handle world, nuka_state_field_t field, nuka_buffer_view_t* out);
/* nuka.h:1181-1188: byte transfers relative to the field's base; out-of-range is INVALID_ARG, never a clamp. */
nuka_result_t nuka_world_upload_field(nuka_world_handle world, nuka_state_field_t field, const void* bytes, size_t nbytes,
                                      size_t byte_offset);
nuka_result_t nuka_world_download_field(nuka_world_handle world, nuka_state_field_t field, void* bytes, size_t nbytes,
                                        size_t byte_offset);

/* What a caller binds names, columns and its own stream to (nuka.h:34-40, 292-299, 478-494, 1222-1281, 1283-1301;
 * src/c_abi/error.cpp:69-72, cuda_interop.cpp:20-58, world.cpp:759-768, 1170-1294, 1345-1413), under the reference's
 * names, layouts and error behaviour. */
typedef struct nuka_version_t {
    uint16_t major;
    uint16_t minor;
    uint16_t patch;
} nuka_version_t;
nuka_version_t nuka_get_version(void);   /* the version of the C ABI this header follows: 0.1.0 */
enum { NUKA_RUNTIME_INFO_VERSION = 1 };
typedef struct nuka_runtime_info_t {
    uint32_t struct_size;
    uint32_t schema_version;
    int32_t cuda_runtime_version;   /* here: hipRuntimeGetVersion */
    int32_t cuda_driver_version;    /* here: hipDriverGetVersion */
} nuka_runtime_info_t;
/* struct_size and schema_version are set by the caller, else INVALID_ARG */
nuka_result_t nuka_get_runtime_info(nuka_runtime_info_t* out);
/* The stream the world executes on (a hipStream_t), and a caller's hipEvent_t recorded on it after all submitted work */
nuka_result_t nuka_world_get_stream(nuka_world_handle world, void** out_stream);
nuka_result_t nuka_world_record_event(nuka_world_handle world, void* cuda_event);
typedef struct nuka_solver_options_t {
    uint32_t cone;         /* constraint/solver_contract.hpp:8: 0 pyramidal, 1 elliptic */
    uint32_t integrator;   /* :9: 0 Euler, 3 implicitfast (what the template's integrator 2 runs) */
    float impratio;
    uint32_t refsafe;
} nuka_solver_options_t;
nuka_result_t nuka_world_get_solver_options(nuka_world_handle world, nuka_solver_options_t* out);
/* The name of the joint whose child is link `link_index` (any environment's copy: env-concatenated link order), else
 * the link's own name.  `out` null is a size query; a `cap` too small for name + NUL is INVALID_ARG with *out_len still
 * set; NOT_SUPPORTED for a world that was not created from a scene file. */
nuka_result_t nuka_world_get_dof_name(nuka_world_handle world, uint32_t link_index, char* out, size_t cap, size_t* out_len);
typedef enum nuka_kinematic_joint_t {
    NUKA_KINEMATIC_ROOT = 0,
    NUKA_KINEMATIC_FIXED = 1,
    NUKA_KINEMATIC_REVOLUTE = 2,
    NUKA_KINEMATIC_PRISMATIC = 3,
    NUKA_KINEMATIC_SPHERICAL = 4    /* never reported: this path builds no ball joints */
} nuka_kinematic_joint_t;
typedef struct nuka_kinematic_link_t {
    uint32_t parent_index;          /* UINT32_MAX for a root */
    uint32_t articulation_index;
    nuka_kinematic_joint_t joint_type;
    float local_pose[7];            /* parent to child at coordinate zero (xyz, wxyz); identity for a root */
    float axis[3];                  /* in the child frame */
} nuka_kinematic_link_t;
nuka_result_t nuka_world_get_kinematic_link(nuka_world_handle world, uint32_t link_index, nuka_kinematic_link_t* out);
typedef struct nuka_link_binding_t {
    uint32_t body_index;            /* the link's own collidable row, UINT32_MAX without one */
    uint32_t articulation_index;
    uint32_t is_root;
    uint32_t is_floating;
} nuka_link_binding_t;
nuka_result_t nuka_world_get_link_binding(nuka_world_handle world, uint32_t link_index, nuka_link_binding_t* out);
/* One collision shape of the template with its pose in an environment now (xyz, wxyz): a link's shape follows the
 * link's pose of the last forward kinematics, any other row its own body pose. */
typedef struct nuka_collider_t {
    uint32_t kind;
    uint32_t is_static;
    float params[4];
    float pose[7];
} nuka_collider_t;
/* `out` null: *out_count = rows only; a capacity below the rows or an environment out of range is INVALID_ARG */
nuka_result_t nuka_world_get_colliders(nuka_world_handle world, uint32_t env_index, nuka_collider_t* out, uint32_t capacity,
                                       uint32_t* out_count);

/* Memory and execution figures (nuka.h:343-374; src/c_abi/device.cpp:101-108, world.cpp:910-990), through the backend's
 * own resource_info and plan_metrics entries.  A null handle or out pointer is refused here (NULL_HANDLE, INVALID_ARG). */
typedef struct nuka_device_resource_info_t {
    uint64_t free_bytes, total_bytes, thread_stack_limit_bytes;
    uint64_t graph_used_bytes, graph_reserved_bytes;
    uint32_t compute_units, threads_per_unit;
} nuka_device_resource_info_t;
typedef struct nuka_world_resource_info_t {
    uint64_t model_bytes, persistent_bytes, scratch_bytes;   /* the template's tables; what a checkpoint keeps; the rest of the arena */
    uint32_t env_count, contacts_per_env, rows_per_env, dofs_per_articulation;
    uint32_t bodies_per_env, particles_per_env;              /* particles: always 0 on this path */
} nuka_world_resource_info_t;
typedef struct nuka_resource_field_t {
    char name[64];           /* the reference's field name where it has one, else this library's */
    uint64_t offset, bytes;  /* place in the world's one arena */
    uint32_t owner, arena;   /* owner 0: the template (model), 1: per-environment data; arena 0 persistent, 1 scratch */
} nuka_resource_field_t;
typedef struct nuka_execution_window_t {
    double gpu_ms;           /* device time between begin and end on the world's stream */
    uint64_t graph_replays, nodes, kernels, clears, copies;   /* replays inside the window; the captured graph's make-up */
} nuka_execution_window_t;
nuka_result_t nuka_device_get_resource_info(nuka_device_handle device, nuka_device_resource_info_t* out);
nuka_result_t nuka_world_get_resource_info(nuka_world_handle world, nuka_world_resource_info_t* out);
uint32_t nuka_world_resource_field_count(nuka_world_handle world);
/* the caller allocates nuka_world_resource_field_count entries */
nuka_result_t nuka_world_get_resource_fields(nuka_world_handle world, nuka_resource_field_t* out);
nuka_result_t nuka_world_begin_execution_window(nuka_world_handle world, void** window);
/* ends and frees the window; waits for the work inside it */
nuka_result_t nuka_world_end_execution_window(nuka_world_handle world, void* window, nuka_execution_window_t* out);

/* Counts of the cooked world. */
typedef struct nuka_world_info_t {
    uint32_t env_count, links_per_env, bodies_per_env, dof, max_dof, contact_slots_per_env, rows_per_env, op_count;
    /* coordinates the sweeps of the contact solve work on: dof, or fewer where no contact of the world can reach the
     * later coordinates and the solve eliminates those once per step */
    uint32_t solver_width;
    /* one-wavefront blocks of the contact solve's full-capacity launch that a compute unit (four SIMDs) holds at once,
     * by the runtime's occupancy query for that kernel and its LDS (a world of 6144 environments or more takes the
     * kernels built for three waves a SIMD where there is one for its width: 12 instead of 8); 0 for a world without
     * a contact solve */
    uint32_t solver_blocks_per_cu;
} nuka_world_info_t;
nuka_result_t nuka_world_get_info(nuka_world_handle world, nuka_world_info_t* out);

/* Timing on the world's own stream with device events, as tests/perf/test_go2_4096env_step_time.cpp:118-137
 * (back-to-back steps, one wait at the end) and, per op, as the eager profiler behind NUKA_STEP_TIMING
 * (src/phi/backend_cuda/cuda_backend.cu:78-120, 188-221). */
/* `from` non-null: every step is preceded by a restore of that checkpoint (inside the timed region), so that each
 * timed step runs on the same state; null: the steps follow one another. */
nuka_result_t nuka_world_time_steps(nuka_world_handle world, nuka_checkpoint_handle from, uint32_t step_count,
                                    float* out_total_ms);
/* out_ms has one slot per pipeline op (nuka_world_info_t::op_count); out_ops receives their op ids. */
nuka_result_t nuka_world_profile_ops(nuka_world_handle world, nuka_checkpoint_handle from, uint32_t step_count,
                                     float* out_ms, uint16_t* out_ops);
/* Device-to-device copy of `bytes` bytes repeated `repeats` times on the world's stream; the streaming-copy ceiling. */
nuka_result_t nuka_device_copy_bandwidth(nuka_device_handle device, size_t bytes, uint32_t repeats, float* out_gb_per_s);

#ifdef __cplusplus
}
#endif
#endif
