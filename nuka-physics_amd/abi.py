"""ctypes mirror of include/nuka_hip.h: descriptor structs, result codes and the host-side template container.

The structs are plain C layouts (pointers and sizes), the same ones the reference's ctypes caller style uses
(examples/sim_val/nuka_cabi.py); nothing here touches torch.
"""
import ctypes as C

import numpy as np

INVALID = 0xFFFFFFFF

# phi/articulation_contract.hpp:8-16
JOINT_REVOLUTE, JOINT_PRISMATIC, JOINT_FIXED, JOINT_FLOATING = 0, 1, 2, 3
# collision/shape_kind.hpp:9-18
SHAPE_SPHERE, SHAPE_CAPSULE, SHAPE_BOX, SHAPE_PLANE, SHAPE_CYLINDER, SHAPE_NONE = 0, 1, 2, 3, 7, INVALID
# collidable row roles of the template description
ROLE_STATIC, ROLE_LINK_BODY, ROLE_PROXY = 0, 1, 2

# constraint/law_source.hpp: where a shape's contact law comes from; nk/solve/row_types.hpp cone of the MuJoCo law
LAW_NATIVE, LAW_MUJOCO = 0, 1
CONE_PYRAMIDAL, CONE_ELLIPTIC = 0, 1
# the integrator of the step: native, MuJoCo's Euler (joint damping implicit after the solve), implicit / implicitfast
INTEGRATOR_NATIVE, INTEGRATOR_MUJOCO_EULER, INTEGRATOR_MUJOCO_IMPLICIT = 0, 1, 2
SOLVER_REFERENCE = (0.02, 1.0, 0.9, 0.95, 0.001, 0.5, 2.0)   # solref, solimp of constraint::SolverReference

# phi/articulation_contract.hpp:16-23
DRIVE_PD_POSITION, DRIVE_TORQUE, DRIVE_VELOCITY, DRIVE_COMPUTED_TORQUE, DRIVE_OSC, DRIVE_ACTUATOR = 0, 1, 2, 3, 4, 5

# nuka.h:22-32
RESULT_OK, RESULT_INVALID_ARG, RESULT_NULL_HANDLE, RESULT_DEVICE_ERROR = 0, 1, 2, 3
RESULT_OUT_OF_MEMORY, RESULT_NOT_SUPPORTED, RESULT_INTERNAL = 6, 7, 100

_PF = C.POINTER(C.c_float)
_PU = C.POINTER(C.c_uint32)
_PB = C.POINTER(C.c_uint8)


class TemplateDescC(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32), ("link_count", C.c_uint32), ("body_count", C.c_uint32),
        ("profile_count", C.c_uint32), ("max_contacts_per_env", C.c_uint32), ("reserved0", C.c_uint32),
        ("joint_type", _PB), ("parent_link", _PU), ("joint_axis", _PF), ("parent_offset", _PF),
        ("link_local_pose", _PF), ("link_inertial_frame", _PF), ("link_mass", _PF), ("link_diag_inertia", _PF),
        ("joint_damping", _PF), ("joint_armature", _PF), ("joint_stiffness", _PF), ("joint_spring_reference", _PF),
        ("body_role", _PU), ("body_link", _PU), ("body_local", _PF), ("shape_kind", _PU), ("shape_params", _PF),
        ("shape_contype", _PU), ("shape_conaffinity", _PU), ("shape_group", _PU), ("shape_profile", _PU),
        ("profile_mu", _PF),
        ("joint_limit_lower", _PF), ("joint_limit_upper", _PF), ("joint_limit_flags", _PB), ("joint_frictionloss", _PF),
        ("drive_mode", C.c_uint32), ("drive_rows", C.c_uint32),
        ("excluded_pairs", _PU), ("excluded_pair_count", C.c_uint32), ("reserved1", C.c_uint32),
        ("profile_law", _PU), ("profile_solref", _PF), ("profile_solimp", _PF), ("profile_margin", _PF),
        ("contact_cone", C.c_uint32), ("contact_impratio", C.c_float),
        ("profile_priority", C.POINTER(C.c_int32)), ("profile_solmix", _PF), ("profile_condim", _PU),
        ("joint_law", _PB), ("joint_limit_margin", _PF), ("joint_limit_reference", _PF), ("joint_friction_reference", _PF),
        ("integrator", C.c_uint32), ("free_body", C.c_uint32),
    ]


class WorldDescC(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32), ("env_count", C.c_uint32), ("fixed_dt", C.c_float), ("gravity", C.c_float * 3),
        ("solver_vel_iters", C.c_uint32), ("solver_pos_iters", C.c_uint32), ("solver_contact_margin", C.c_float),
        ("solver_pos_beta", C.c_float), ("solver_pos_slop", C.c_float), ("solver_velocity_tolerance", C.c_float),
        ("solver_baumgarte_max_velocity", C.c_float), ("solver_overlap_recovery_velocity", C.c_float),
        ("solver_fold_drive_damping", C.c_uint32), ("solver_substeps", C.c_uint32), ("contact_detection_substeps", C.c_uint32),
    ]


class SceneWorldDescC(C.Structure):
    """nuka_world_desc_t of nuka.h:57-173, member for member (the descriptor nuka_world_create_from_scene takes)."""
    _fields_ = [
        ("scene_path", C.c_char_p), ("env_count", C.c_uint32), ("fixed_dt", C.c_float), ("determinism", C.c_uint8),
        ("control_mode", C.c_uint8), ("osc_task_link", C.c_uint32), ("terrain_step_height", C.c_float),
        ("terrain_step_width", C.c_float), ("terrain_platform_width", C.c_float), ("terrain_grid_width", C.c_float),
        ("terrain_grid_height_max", C.c_float), ("instance_count", C.c_uint32), ("instance_spacing", C.c_float),
        ("contact_family", C.c_uint32), ("heightfield_terrain_type", C.c_uint32), ("heightfield_nrow", C.c_uint32),
        ("heightfield_ncol", C.c_uint32), ("heightfield_cell", C.c_float), ("heightfield_image_path", C.c_char_p),
        ("heightfield_radius_x", C.c_float), ("heightfield_radius_y", C.c_float), ("heightfield_elevation_z", C.c_float),
        ("heightfield_base_z", C.c_float), ("gravity_x", C.c_float), ("gravity_y", C.c_float), ("gravity_z", C.c_float),
        ("curric_levels", C.c_uint32), ("curric_types", C.c_uint32), ("terrain_feature_cell", C.c_float),
        ("solver_vel_iters", C.c_uint32), ("solver_pos_iters", C.c_uint32), ("solver_contact_margin", C.c_float),
        ("solver_max_pairs", C.c_uint32), ("solver_baumgarte_max_velocity", C.c_float), ("cloth_integrator", C.c_uint32),
        ("ogc_contact_capacity", C.c_uint32), ("solver_overlap_recovery_velocity", C.c_float), ("solver_substeps", C.c_uint32),
        ("contact_detection_substeps", C.c_uint32),
    ]


# nuka.h:496-958: the public field ids this library serves, by the name of the world field behind each
PUBLIC_FIELDS = {
    "RIGID_BODY_TRANSFORM": (0, "body_pose", 28), "ARTICULATION_LINK_POSE": (1, "link_pose", 28), "JOINT_POSITION": (2, "q", 4),
    "JOINT_VELOCITY": (3, "qdot", 4), "CONTACT_POINTS": (5, "contact_point", 12), "DRIVE_TARGET": (6, "drive_target", 4),
    "LINK_VELOCITY": (7, "link_velocity", 24), "DRIVE_STIFFNESS": (8, "drive_stiffness", 4), "DRIVE_DAMPING": (9, "drive_damping", 4),
    "DRIVE_FORCE_LIMIT": (10, "drive_force_limit", 4), "BASE_POSE": (11, "base_pose", 28), "TORQUE_INPUT": (12, "drive_target", 4),
    "VELOCITY_TARGET": (13, "velocity_target", 4), "ACTUATOR_NOLOAD_SPEED": (14, "actuator_noload_speed", 4),
    "LINK_CONTACT_WRENCH": (16, "link_contact_wrench", 24), "CONTACT_NORMAL": (17, "contact_normal", 12),
    "CONTACT_FORCE": (18, "contact_force", 12), "CONTACT_LINK": (19, "contact_link", 4), "JOINT_FEEDFORWARD": (22, "joint_f", 4),
    "BODY_LINEAR_VELOCITY": (25, "body_linear_velocity", 12), "BODY_ANGULAR_VELOCITY": (26, "body_angular_velocity", 12),
    "JOINT_LIMIT_IMPULSE": (27, "joint_limit_impulse", 8), "ACTUATOR_EFFORT_REQUESTED": (28, "actuator_effort_requested", 4),
    "ACTUATOR_EFFORT": (29, "actuator_effort", 4), "ACTUATOR_SATURATED": (30, "actuator_saturated", 4),
    "CONTACT_SIDE_A_KIND": (33, "contact_side_a_kind", 4), "CONTACT_SIDE_B_KIND": (34, "contact_side_b_kind", 4),
    "CONTACT_SIDE_A_INDEX": (35, "contact_side_a_index", 4), "CONTACT_SIDE_B_INDEX": (36, "contact_side_b_index", 4),
    "ENV_STATUS": (39, "env_status", 4), "CONTACT_WARM_START_COUNTS": (70, "contact_warm_start_counts", 8),
    "VBD_VELOCITY_SWEEP_COUNT": (79, "vbd_velocity_sweep_count", 4), "UCONTACT_ROW_RANGE": (103, "ucontact_row_range", 8),
    "LINK_WRENCH": (105, "link_wrench", 24), "UCONTACT_COUNT": (107, "ucontact_count", 4), "UCONTACT_POINT": (108, "ucontact_point", 48),
    "SOLVER_RESIDUAL": (109, "solver_residual", 16), "UCONTACT_NORMAL": (128, "ucontact_normal", 48),
    "UCONTACT_DEPTH": (129, "ucontact_depth", 16), "UCONTACT_LAW": (132, "ucontact_law", 4), "UCONTACT_SIDE_A": (134, "ucontact_a", 16),
    "UCONTACT_SIDE_B": (135, "ucontact_b", 16), "UCONTACT_IMPULSE": (138, "ucontact_impulse", 48),
    "JOINT_GRAVITY_FORCE": (157, "joint_gravity_force", 4), "ROW_PENETRATION": (161, "row_penetration", 4), "ROW_LAMBDA": (162, "lambda", 4),
}


class BufferViewC(C.Structure):   # nuka.h:1158-1164
    _fields_ = [("device_ptr", C.c_void_p), ("element_count", C.c_size_t), ("element_stride_bytes", C.c_uint32),
                ("dtype", C.c_uint8)]


IDENTITY7 = np.array([0, 0, 0, 1, 0, 0, 0], dtype=np.float32)


class Template:
    """Host-side authoring description of one environment: an articulation tree plus its collidable rows."""

    def __init__(self):
        self.links = []
        self.bodies = []
        self.profiles = []
        self.max_contacts_per_env = 0
        self.drive_mode = DRIVE_TORQUE
        self.drive_rows = False   # True: affine drives through joint drive rows; False: `tau` is the applied force
        self.excluded = []        # pairs of collidable rows that never pair (rows of one link are excluded by the cook)
        self.contact_cone = CONE_PYRAMIDAL   # friction cone of MuJoCo-law contacts (<option cone>)
        self.contact_impratio = 1.0          # <option impratio>
        self.integrator = INTEGRATOR_NATIVE  # <option integrator> of a MuJoCo-sourced scene
        self.free_body = False    # True: the template's one link (floating root) is a free rigid body (rigid-body ops)

    def add_link(self, joint_type, parent, axis=(0, 0, 1), local_pos=(0, 0, 0), local_rot=(1, 0, 0, 0), mass=1.0,
                 diag_inertia=(0.01, 0.01, 0.01), com=(0, 0, 0), damping=0.0, armature=0.0, stiffness=0.0,
                 spring_ref=0.0, parent_offset=(0, 0, 0), lower=None, upper=None, frictionloss=0.0, law=LAW_NATIVE,
                 limit_margin=0.0, limit_reference=SOLVER_REFERENCE, friction_reference=SOLVER_REFERENCE):
        self.links.append(dict(joint_type=joint_type, parent=INVALID if parent is None else parent, axis=axis,
                               local=list(local_pos) + list(local_rot), mass=mass, diag=diag_inertia,
                               inertial=list(com) + [1, 0, 0, 0], damping=damping, armature=armature,
                               stiffness=stiffness, spring_ref=spring_ref, parent_offset=parent_offset,
                               lower=lower, upper=upper, frictionloss=frictionloss, law=law, limit_margin=limit_margin,
                               limit_reference=tuple(limit_reference), friction_reference=tuple(friction_reference)))
        return len(self.links) - 1

    def add_profile(self, mu1, mu2=None, law=LAW_NATIVE, solref=(0.02, 1.0), solimp=(0.9, 0.95, 0.001, 0.5, 2.0), margin=0.0,
                    gap=0.0, priority=0, solmix=1.0, condim=3):
        """A contact profile; `law`, `solref`, `solimp`, `margin` and `gap` matter to MuJoCo-law contacts only
        (scene/contact_filter.hpp:20-37 holds the defaults)."""
        self.profiles.append(dict(mu=(mu1, mu1 if mu2 is None else mu2), law=law, solref=tuple(solref), solimp=tuple(solimp),
                                  margin=(margin, gap), priority=priority, solmix=solmix, condim=condim))
        return len(self.profiles) - 1

    def add_body(self, role, link=None, kind=SHAPE_NONE, params=(0, 0, 0, 0), local_pos=(0, 0, 0),
                 local_rot=(1, 0, 0, 0), contype=1, conaffinity=1, group=0, profile=INVALID):
        self.bodies.append(dict(role=role, link=INVALID if link is None else link, kind=kind, params=params,
                                local=list(local_pos) + list(local_rot), contype=contype, conaffinity=conaffinity,
                                group=group, profile=profile))
        return len(self.bodies) - 1

    def exclude(self, row_a, row_b):
        self.excluded.append((row_a, row_b))

    @property
    def link_count(self):
        return len(self.links)

    @property
    def dof(self):
        width = {JOINT_REVOLUTE: 1, JOINT_PRISMATIC: 1, JOINT_FIXED: 0, JOINT_FLOATING: 6}
        return sum(width[l["joint_type"]] for l in self.links)

    def arrays(self):
        f32, u32 = np.float32, np.uint32
        L, B = self.links, self.bodies
        return dict(
            joint_type=np.array([l["joint_type"] for l in L], dtype=np.uint8),
            parent_link=np.array([l["parent"] for l in L], dtype=u32),
            joint_axis=np.array([l["axis"] for l in L], dtype=f32).reshape(-1),
            parent_offset=np.array([l["parent_offset"] for l in L], dtype=f32).reshape(-1),
            link_local_pose=np.array([l["local"] for l in L], dtype=f32).reshape(-1),
            link_inertial_frame=np.array([l["inertial"] for l in L], dtype=f32).reshape(-1),
            link_mass=np.array([l["mass"] for l in L], dtype=f32),
            link_diag_inertia=np.array([l["diag"] for l in L], dtype=f32).reshape(-1),
            joint_damping=np.array([l["damping"] for l in L], dtype=f32),
            joint_armature=np.array([l["armature"] for l in L], dtype=f32),
            joint_stiffness=np.array([l["stiffness"] for l in L], dtype=f32),
            joint_spring_reference=np.array([l["spring_ref"] for l in L], dtype=f32),
            joint_limit_lower=np.array([0.0 if l["lower"] is None else l["lower"] for l in L], dtype=f32),
            joint_limit_upper=np.array([0.0 if l["upper"] is None else l["upper"] for l in L], dtype=f32),
            joint_limit_flags=np.array([(l["lower"] is not None) + 2 * (l["upper"] is not None) for l in L], dtype=np.uint8),
            joint_frictionloss=np.array([l["frictionloss"] for l in L], dtype=f32),
            joint_law=np.array([l["law"] for l in L], dtype=np.uint8),
            joint_limit_margin=np.array([l["limit_margin"] for l in L], dtype=f32),
            joint_limit_reference=np.array([l["limit_reference"] for l in L], dtype=f32).reshape(-1),
            joint_friction_reference=np.array([l["friction_reference"] for l in L], dtype=f32).reshape(-1),
            body_role=np.array([b["role"] for b in B], dtype=u32),
            body_link=np.array([b["link"] for b in B], dtype=u32),
            body_local=np.array([b["local"] for b in B], dtype=f32).reshape(-1),
            shape_kind=np.array([b["kind"] for b in B], dtype=u32),
            shape_params=np.array([b["params"] for b in B], dtype=f32).reshape(-1),
            shape_contype=np.array([b["contype"] for b in B], dtype=u32),
            shape_conaffinity=np.array([b["conaffinity"] for b in B], dtype=u32),
            shape_group=np.array([b["group"] for b in B], dtype=u32),
            shape_profile=np.array([b["profile"] for b in B], dtype=u32),
            profile_mu=np.array([p["mu"] for p in self.profiles], dtype=f32).reshape(-1),
            profile_law=np.array([p["law"] for p in self.profiles], dtype=u32),
            profile_solref=np.array([p["solref"] for p in self.profiles], dtype=f32).reshape(-1),
            profile_solimp=np.array([p["solimp"] for p in self.profiles], dtype=f32).reshape(-1),
            profile_margin=np.array([p["margin"] for p in self.profiles], dtype=f32).reshape(-1),
            profile_priority=np.array([p["priority"] for p in self.profiles], dtype=np.int32),
            profile_solmix=np.array([p["solmix"] for p in self.profiles], dtype=f32),
            profile_condim=np.array([p["condim"] for p in self.profiles], dtype=u32),
            excluded_pairs=np.array(self.excluded, dtype=u32).reshape(-1),
        )

    def to_c(self):
        """Returns (TemplateDescC, keepalive) - the arrays must outlive the call that consumes the struct."""
        a = self.arrays()
        d = TemplateDescC()
        d.struct_size = C.sizeof(TemplateDescC)
        d.link_count, d.body_count, d.profile_count = len(self.links), len(self.bodies), len(self.profiles)
        d.max_contacts_per_env = self.max_contacts_per_env
        d.drive_mode, d.drive_rows = self.drive_mode, 1 if self.drive_rows else 0
        d.excluded_pair_count = len(self.excluded)
        d.contact_cone, d.contact_impratio = self.contact_cone, self.contact_impratio
        d.integrator = self.integrator
        d.free_body = 1 if self.free_body else 0
        ctype = {np.dtype(np.float32): C.c_float, np.dtype(np.uint32): C.c_uint32, np.dtype(np.uint8): C.c_uint8, np.dtype(np.int32): C.c_int32}
        for name, arr in a.items():
            arr = np.ascontiguousarray(arr)
            a[name] = arr
            if arr.size:
                setattr(d, name, arr.ctypes.data_as(C.POINTER(ctype[arr.dtype])))
        return d, a


def world_desc(env_count, dt, gravity=(0.0, 0.0, -9.81), vel_iters=0, pos_iters=0, contact_margin=0.0,
               velocity_tolerance=0.0, fold_drive_damping=True, substeps=0):
    d = WorldDescC()
    d.struct_size = C.sizeof(WorldDescC)
    d.env_count, d.fixed_dt = env_count, dt
    d.gravity[0], d.gravity[1], d.gravity[2] = gravity
    d.solver_vel_iters, d.solver_pos_iters = vel_iters, pos_iters
    d.solver_contact_margin = contact_margin
    d.solver_velocity_tolerance = velocity_tolerance
    d.solver_fold_drive_damping = 0 if fold_drive_damping else INVALID
    d.solver_substeps = substeps
    return d
