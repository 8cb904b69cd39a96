"""MI355X-native batched articulation step for Nuka-Physics: Python host layer over the C ABI of libnuka_hip.so.

The package directory name carries a hyphen, so load it by path (see __graft_entry__.load_package) or put its parent
on sys.path under the module name ``nuka_physics_amd``.  Everything computes in the HIP library; there is no CPU
fallback, and a missing library or GPU raises.
"""
import ctypes as C
import os
import subprocess

import numpy as np

from . import abi, synthetic  # noqa: F401
from .abi import BufferViewC, TemplateDescC, WorldDescC

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libnuka_hip.so")

_DTYPES = {0: np.float32, 1: np.uint32, 2: np.uint64, 3: np.uint8}


class NukaError(RuntimeError):
    def __init__(self, code, message):
        super().__init__(f"nuka result {code}: {message}")
        self.code = code


class WorldInfoC(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in ("env_count", "links_per_env", "bodies_per_env", "dof", "max_dof",
                                          "contact_slots_per_env", "rows_per_env", "op_count", "solver_width", "solver_blocks_per_cu")]


class SceneInfoC(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in ("link_count", "body_count", "actuator_count", "dropped_geom_count", "floating_root",
                                          "drive_mode")] + [("timestep", C.c_float), ("gravity", C.c_float * 3)]


SCENE_PLANE_CONTACTS_ONLY = 1
SCENE_FIXED_BASE = 2
SCENE_GROUND_PLANE = 4
SCENE_NATIVE_CONTACT_LAW = 8
SCENE_NATIVE_JOINT_LAW = 16


class ParamInfoC(C.Structure):
    """nuka_param_info_t"""
    _fields_ = [("struct_size", C.c_uint32), ("schema_version", C.c_uint32), ("key", C.c_char * 48), ("unit", C.c_char * 16),
                ("scene_field", C.c_char * 48), ("type", C.c_int), ("tier", C.c_int), ("count", C.c_uint32),
                ("min_value", C.c_double), ("max_value", C.c_double)]


class ExecutionInfoC(C.Structure):
    """nuka_world_execution_info_t"""
    _fields_ = [("struct_size", C.c_uint32), ("schema_version", C.c_uint32), ("mode", C.c_int), ("graph_ready", C.c_uint32),
                ("capture_attempts", C.c_uint64), ("graph_replays", C.c_uint64), ("last_result", C.c_int), ("failed_op", C.c_uint32),
                ("native_error", C.c_int32), ("message", C.c_char * 256)]


class VersionC(C.Structure):
    """nuka_version_t"""
    _fields_ = [("major", C.c_uint16), ("minor", C.c_uint16), ("patch", C.c_uint16)]


class RuntimeInfoC(C.Structure):
    """nuka_runtime_info_t"""
    _fields_ = [("struct_size", C.c_uint32), ("schema_version", C.c_uint32), ("cuda_runtime_version", C.c_int32),
                ("cuda_driver_version", C.c_int32)]


class SolverOptionsC(C.Structure):
    """nuka_solver_options_t"""
    _fields_ = [("cone", C.c_uint32), ("integrator", C.c_uint32), ("impratio", C.c_float), ("refsafe", C.c_uint32)]


class KinematicLinkC(C.Structure):
    """nuka_kinematic_link_t"""
    _fields_ = [("parent_index", C.c_uint32), ("articulation_index", C.c_uint32), ("joint_type", C.c_int), ("local_pose", C.c_float * 7),
                ("axis", C.c_float * 3)]


class LinkBindingC(C.Structure):
    """nuka_link_binding_t"""
    _fields_ = [(n, C.c_uint32) for n in ("body_index", "articulation_index", "is_root", "is_floating")]


class ColliderC(C.Structure):
    """nuka_collider_t"""
    _fields_ = [("kind", C.c_uint32), ("is_static", C.c_uint32), ("params", C.c_float * 4), ("pose", C.c_float * 7)]


class DeviceResourceInfoC(C.Structure):
    """nuka_device_resource_info_t"""
    _fields_ = [(n, C.c_uint64) for n in ("free_bytes", "total_bytes", "thread_stack_limit_bytes", "graph_used_bytes",
                                          "graph_reserved_bytes")] + [("compute_units", C.c_uint32), ("threads_per_unit", C.c_uint32)]


class WorldResourceInfoC(C.Structure):
    """nuka_world_resource_info_t"""
    _fields_ = [(n, C.c_uint64) for n in ("model_bytes", "persistent_bytes", "scratch_bytes")] + \
               [(n, C.c_uint32) for n in ("env_count", "contacts_per_env", "rows_per_env", "dofs_per_articulation", "bodies_per_env",
                                          "particles_per_env")]


class ResourceFieldC(C.Structure):
    """nuka_resource_field_t"""
    _fields_ = [("name", C.c_char * 64), ("offset", C.c_uint64), ("bytes", C.c_uint64), ("owner", C.c_uint32), ("arena", C.c_uint32)]


class ExecutionWindowC(C.Structure):
    """nuka_execution_window_t"""
    _fields_ = [("gpu_ms", C.c_double)] + [(n, C.c_uint64) for n in ("graph_replays", "nodes", "kernels", "clears", "copies")]


KINEMATIC_ROOT, KINEMATIC_FIXED, KINEMATIC_REVOLUTE, KINEMATIC_PRISMATIC = 0, 1, 2, 3
PARAM_INFO_VERSION = 1
PARAM_LIVE, PARAM_REBUILD = 0, 1
PARAMS = ("gravity_z", "velocity_iterations", "link_mass", "joint_damping", "joint_armature", "joint_frictionloss", "drive_stiffness",
          "drive_force_limit")


class DeviceDescC(C.Structure):   # nuka.h:46-51
    _fields_ = [("gpu_index", C.c_uint32), ("cuda_stream", C.c_void_p), ("backend_selection_layer_enabled", C.c_uint8)]


FIELD_BASE, FIELD_NONE = 0x10000, 0x7FFFFFFF   # NUKA_HIP_FIELD_BASE, NUKA_HIP_FIELD_NONE
RESET_ENVS_STATIC_MAX = 16384   # NUKA_RESET_ENVS_STATIC_MAX of include/nuka_hip.h

EXPORTS = [
    "nuka_result_message", "nuka_last_error_message", "nuka_device_create", "nuka_device_destroy", "nuka_device_backend",
    "nuka_world_create_from_template", "nuka_world_destroy", "nuka_world_step", "nuka_world_step_n",
    "nuka_world_set_execution_mode", "nuka_world_set_velocity_iterations", "nuka_world_get_velocity_iterations",
    "nuka_world_synchronize", "nuka_world_reset", "nuka_world_reset_envs", "nuka_world_reset_envs_static", "nuka_world_checkpoint_capture", "nuka_world_checkpoint_restore",
    "nuka_checkpoint_destroy", "nuka_checkpoint_byte_size", "nuka_world_dispatch_op", "nuka_field_from_name", "nuka_field_names",
    "nuka_world_get_buffer_view", "nuka_world_upload_field", "nuka_world_download_field", "nuka_world_get_info",
    "nuka_world_time_steps", "nuka_world_profile_ops", "nuka_device_copy_bandwidth", "nuka_hip_register_backend_entry",
    "nuka_hip_op_count", "nuka_hip_op_name", "nuka_hip_op_from_name",
    "nuka_scene_load_mjcf", "nuka_scene_load_urdf", "nuka_scene_destroy", "nuka_scene_template", "nuka_scene_get_info", "nuka_scene_link_name",
    "nuka_scene_joint_name", "nuka_scene_initial_state", "nuka_world_create_from_scene", "nuka_hip_world_create_from_scene_handle",
    "nuka_checkpoint_equal", "nuka_world_state_hash", "nuka_world_forward_kinematics", "nuka_world_param_count", "nuka_world_get_param_infos",
    "nuka_world_get_param", "nuka_world_set_param", "nuka_world_set_link_mass", "nuka_world_set_gravity_z",
    "nuka_checkpoint_write", "nuka_world_checkpoint_read", "nuka_world_get_execution_info",
    "nuka_get_version", "nuka_get_runtime_info", "nuka_world_get_stream", "nuka_world_record_event", "nuka_world_get_solver_options",
    "nuka_world_get_dof_name", "nuka_world_get_kinematic_link", "nuka_world_get_link_binding", "nuka_world_get_colliders",
    "nuka_device_get_resource_info", "nuka_world_get_resource_info", "nuka_world_resource_field_count", "nuka_world_get_resource_fields",
    "nuka_world_begin_execution_window", "nuka_world_end_execution_window",
]


def build(force=False):
    """Compiles csrc/*.hip for gfx950 into lib/libnuka_hip.so (hipcc cross-compiles without a GPU)."""
    cmd = ["make", "-C", os.path.join(HERE, "csrc"), "-j8"] + (["-B"] if force else [])
    subprocess.run(cmd, check=True, stdout=subprocess.DEVNULL, stderr=subprocess.PIPE)


_lib = None


def lib():
    """The loaded C-ABI library; raises when it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise FileNotFoundError(f"{LIB_PATH} is missing: run __graft_entry__.build() first")
        L = C.CDLL(LIB_PATH)
        L.nuka_result_message.restype = C.c_char_p
        L.nuka_last_error_message.restype = C.c_char_p
        L.nuka_field_names.restype = C.c_char_p
        L.nuka_hip_op_name.restype = C.c_char_p
        L.nuka_hip_op_name.argtypes = [C.c_uint16]
        L.nuka_hip_op_from_name.argtypes = [C.c_char_p]
        L.nuka_hip_register_backend_entry.restype = C.c_void_p
        L.nuka_device_backend.restype = C.c_void_p
        L.nuka_device_backend.argtypes = [C.c_void_p]
        L.nuka_device_create.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
        L.nuka_device_destroy.argtypes = [C.c_void_p]
        L.nuka_world_create_from_template.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.POINTER(C.c_void_p)]
        L.nuka_world_destroy.argtypes = [C.c_void_p]
        L.nuka_world_step.argtypes = [C.c_void_p]
        L.nuka_world_step_n.argtypes = [C.c_void_p, C.c_uint32]
        L.nuka_world_set_execution_mode.argtypes = [C.c_void_p, C.c_int]
        L.nuka_world_set_velocity_iterations.argtypes = [C.c_void_p, C.c_uint32]
        L.nuka_world_get_velocity_iterations.argtypes = [C.c_void_p, C.POINTER(C.c_uint32)]
        L.nuka_world_synchronize.argtypes = [C.c_void_p]
        L.nuka_world_reset.argtypes = [C.c_void_p]
        L.nuka_world_reset_envs.argtypes = [C.c_void_p, C.c_void_p, C.c_uint32]
        L.nuka_world_dispatch_op.argtypes = [C.c_void_p, C.c_uint16, C.c_uint32]
        L.nuka_field_from_name.argtypes = [C.c_char_p]
        L.nuka_field_from_name.restype = C.c_uint32
        L.nuka_world_get_buffer_view.argtypes = [C.c_void_p, C.c_uint32, C.POINTER(BufferViewC)]
        L.nuka_world_upload_field.argtypes = [C.c_void_p, C.c_uint32, C.c_void_p, C.c_size_t, C.c_size_t]
        L.nuka_world_download_field.argtypes = [C.c_void_p, C.c_uint32, C.c_void_p, C.c_size_t, C.c_size_t]
        L.nuka_world_get_info.argtypes = [C.c_void_p, C.POINTER(WorldInfoC)]
        L.nuka_world_time_steps.argtypes = [C.c_void_p, C.c_void_p, C.c_uint32, C.POINTER(C.c_float)]
        L.nuka_world_profile_ops.argtypes = [C.c_void_p, C.c_void_p, C.c_uint32, C.POINTER(C.c_float), C.POINTER(C.c_uint16)]
        L.nuka_world_checkpoint_capture.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
        L.nuka_world_checkpoint_restore.argtypes = [C.c_void_p, C.c_void_p]
        L.nuka_checkpoint_destroy.argtypes = [C.c_void_p]
        L.nuka_checkpoint_byte_size.argtypes = [C.c_void_p, C.POINTER(C.c_uint64)]
        L.nuka_device_copy_bandwidth.argtypes = [C.c_void_p, C.c_size_t, C.c_uint32, C.POINTER(C.c_float)]
        L.nuka_scene_load_mjcf.argtypes = [C.c_char_p, C.c_uint32, C.POINTER(C.c_void_p)]
        L.nuka_scene_load_urdf.argtypes = [C.c_char_p, C.c_uint32, C.POINTER(C.c_void_p)]
        L.nuka_scene_destroy.argtypes = [C.c_void_p]
        L.nuka_scene_template.argtypes = [C.c_void_p]
        L.nuka_scene_template.restype = C.POINTER(TemplateDescC)
        L.nuka_scene_get_info.argtypes = [C.c_void_p, C.POINTER(SceneInfoC)]
        L.nuka_scene_link_name.argtypes = [C.c_void_p, C.c_uint32]
        L.nuka_scene_link_name.restype = C.c_char_p
        L.nuka_scene_joint_name.argtypes = [C.c_void_p, C.c_uint32]
        L.nuka_scene_joint_name.restype = C.c_char_p
        L.nuka_scene_initial_state.argtypes = [C.c_void_p] + [C.c_void_p] * 6
        L.nuka_hip_world_create_from_scene_handle.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.POINTER(C.c_void_p)]
        L.nuka_world_create_from_scene.argtypes = [C.c_void_p, C.c_void_p, C.POINTER(C.c_void_p)]
        L.nuka_checkpoint_equal.argtypes = [C.c_void_p, C.c_void_p, C.POINTER(C.c_uint32)]
        L.nuka_world_state_hash.argtypes = [C.c_void_p, C.POINTER(C.c_uint64)]
        L.nuka_world_forward_kinematics.argtypes = [C.c_void_p]
        L.nuka_world_param_count.argtypes = [C.c_void_p, C.POINTER(C.c_uint32)]
        L.nuka_world_get_param_infos.argtypes = [C.c_void_p, C.POINTER(ParamInfoC), C.c_uint32]
        L.nuka_world_get_param.argtypes = [C.c_void_p, C.c_uint32, C.c_uint32, C.POINTER(C.c_double)]
        L.nuka_world_set_param.argtypes = [C.c_void_p, C.c_uint32, C.c_uint32, C.c_double]
        L.nuka_world_set_link_mass.argtypes = [C.c_void_p, C.c_uint32, C.c_float]
        L.nuka_world_set_gravity_z.argtypes = [C.c_void_p, C.c_float]
        L.nuka_checkpoint_write.argtypes = [C.c_void_p, C.c_char_p]
        L.nuka_world_checkpoint_read.argtypes = [C.c_void_p, C.c_char_p, C.POINTER(C.c_void_p)]
        L.nuka_world_get_execution_info.argtypes = [C.c_void_p, C.POINTER(ExecutionInfoC)]
        L.nuka_get_version.restype = VersionC
        L.nuka_get_runtime_info.argtypes = [C.POINTER(RuntimeInfoC)]
        L.nuka_world_get_stream.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
        L.nuka_world_record_event.argtypes = [C.c_void_p, C.c_void_p]
        L.nuka_world_get_solver_options.argtypes = [C.c_void_p, C.POINTER(SolverOptionsC)]
        L.nuka_world_get_dof_name.argtypes = [C.c_void_p, C.c_uint32, C.c_char_p, C.c_size_t, C.POINTER(C.c_size_t)]
        L.nuka_world_get_kinematic_link.argtypes = [C.c_void_p, C.c_uint32, C.POINTER(KinematicLinkC)]
        L.nuka_world_get_link_binding.argtypes = [C.c_void_p, C.c_uint32, C.POINTER(LinkBindingC)]
        L.nuka_world_get_colliders.argtypes = [C.c_void_p, C.c_uint32, C.POINTER(ColliderC), C.c_uint32, C.POINTER(C.c_uint32)]
        L.nuka_device_get_resource_info.argtypes = [C.c_void_p, C.POINTER(DeviceResourceInfoC)]
        L.nuka_world_get_resource_info.argtypes = [C.c_void_p, C.POINTER(WorldResourceInfoC)]
        L.nuka_world_resource_field_count.argtypes = [C.c_void_p]
        L.nuka_world_resource_field_count.restype = C.c_uint32
        L.nuka_world_get_resource_fields.argtypes = [C.c_void_p, C.POINTER(ResourceFieldC)]
        L.nuka_world_begin_execution_window.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
        L.nuka_world_end_execution_window.argtypes = [C.c_void_p, C.c_void_p, C.POINTER(ExecutionWindowC)]
        _lib = L
    return _lib


def _check(code):
    if code != 0:
        raise NukaError(code, lib().nuka_last_error_message().decode() or lib().nuka_result_message(code).decode())


def version():
    """nuka_get_version as (major, minor, patch)."""
    v = lib().nuka_get_version()
    return v.major, v.minor, v.patch


def runtime_info():
    """nuka_get_runtime_info: the HIP runtime and driver versions in the reference's record."""
    info = RuntimeInfoC(C.sizeof(RuntimeInfoC), 1, 0, 0)
    _check(lib().nuka_get_runtime_info(C.byref(info)))
    return info


class Device:
    """nuka_device_create / nuka_device_destroy."""

    def __init__(self, gpu_index=0):
        self._h = C.c_void_p()
        desc = DeviceDescC(gpu_index, None, 0)
        _check(lib().nuka_device_create(C.byref(desc), C.byref(self._h)))

    def close(self):
        if self._h:
            lib().nuka_device_destroy(self._h)
            self._h = C.c_void_p()

    def resource_info(self):
        """nuka_device_get_resource_info: free and total device memory, compute units and threads a unit."""
        out = DeviceResourceInfoC()
        _check(lib().nuka_device_get_resource_info(self._h, C.byref(out)))
        return out

    def copy_bandwidth(self, nbytes=1 << 30, repeats=10):
        out = C.c_float()
        _check(lib().nuka_device_copy_bandwidth(self._h, nbytes, repeats, C.byref(out)))
        return out.value


class Scene:
    """A robot description file (MJCF, or URDF by its extension) read into the cook inputs of one environment
    (nuka_scene_*; host code, no GPU)."""

    def __init__(self, path, flags=0):
        self._h = C.c_void_p()
        load = lib().nuka_scene_load_urdf if str(path).lower().endswith(".urdf") else lib().nuka_scene_load_mjcf
        _check(load(os.fsencode(path), flags, C.byref(self._h)))
        info = SceneInfoC()
        _check(lib().nuka_scene_get_info(self._h, C.byref(info)))
        self.info = info
        self.link_count = info.link_count
        self.link_names = [lib().nuka_scene_link_name(self._h, l).decode() for l in range(info.link_count)]
        self.joint_names = [lib().nuka_scene_joint_name(self._h, l).decode() for l in range(info.link_count)]

    def close(self):
        if self._h:
            lib().nuka_scene_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        self.close()

    def to_c(self):
        """(TemplateDescC, keepalive), as abi.Template.to_c(): the arrays belong to the scene."""
        return lib().nuka_scene_template(self._h).contents, self

    def template_arrays(self):
        """The template description as numpy copies, keyed like abi.Template.arrays()."""
        d = lib().nuka_scene_template(self._h).contents
        nl, nb, npf = d.link_count, d.body_count, d.profile_count
        shapes = dict(joint_type=nl, parent_link=nl, joint_axis=3 * nl, link_local_pose=7 * nl, link_inertial_frame=7 * nl, link_mass=nl,
                      link_diag_inertia=3 * nl, joint_damping=nl, joint_armature=nl, joint_stiffness=nl, joint_spring_reference=nl,
                      body_role=nb, body_link=nb, body_local=7 * nb, shape_kind=nb, shape_params=4 * nb, shape_contype=nb,
                      shape_conaffinity=nb, shape_group=nb, shape_profile=nb, profile_mu=2 * npf, joint_limit_lower=nl,
                      profile_law=npf if d.profile_law else 0, profile_solref=2 * npf if d.profile_solref else 0,
                      profile_solimp=5 * npf if d.profile_solimp else 0, profile_margin=2 * npf if d.profile_margin else 0,
                      profile_priority=npf if d.profile_priority else 0, profile_solmix=npf if d.profile_solmix else 0,
                      profile_condim=npf if d.profile_condim else 0, joint_law=nl if d.joint_law else 0,
                      joint_limit_margin=nl if d.joint_limit_margin else 0, joint_limit_reference=7 * nl if d.joint_limit_reference else 0,
                      joint_friction_reference=7 * nl if d.joint_friction_reference else 0,
                      joint_limit_upper=nl, joint_limit_flags=nl, joint_frictionloss=nl, excluded_pairs=2 * d.excluded_pair_count)
        out = {name: np.ctypeslib.as_array(getattr(d, name), shape=(count,)).copy() if count else np.zeros(0, np.float32)
               for name, count in shapes.items()}
        out.update(drive_mode=d.drive_mode, drive_rows=d.drive_rows, contact_cone=d.contact_cone, contact_impratio=d.contact_impratio, integrator=d.integrator)
        return out

    def initial_state(self):
        nl = self.link_count
        names = ("q", "base_pose", "drive_stiffness", "drive_damping", "drive_force_limit", "drive_joint_force_limit")
        out = {n: np.zeros(7 if n == "base_pose" else nl, np.float32) for n in names}
        _check(lib().nuka_scene_initial_state(self._h, *[out[n].ctypes.data for n in names]))
        return out


class World:
    """One cooked template stepped over `env_count` environments on the GPU (nuka_world_*)."""

    def __init__(self, device, template, desc):
        self.device = device
        self._h = C.c_void_p()
        if isinstance(desc, abi.SceneWorldDescC):      # the reference's entry point: the descriptor names the scene file
            _check(lib().nuka_world_create_from_scene(device._h, C.byref(desc), C.byref(self._h)))
        elif isinstance(template, Scene):
            _check(lib().nuka_hip_world_create_from_scene_handle(device._h, template._h, C.byref(desc), C.byref(self._h)))
        else:
            tdesc, keep = template.to_c()
            _check(lib().nuka_world_create_from_template(device._h, C.byref(tdesc), C.byref(desc), C.byref(self._h)))
            del keep
        info = WorldInfoC()
        _check(lib().nuka_world_get_info(self._h, C.byref(info)))
        self.info = info
        self.env_count, self.link_count, self.dof = info.env_count, info.links_per_env, info.dof
        self.rows_per_env, self.op_count = info.rows_per_env, info.op_count

    def close(self):
        if self._h:
            lib().nuka_world_destroy(self._h)
            self._h = C.c_void_p()

    def _field(self, name):
        fid = lib().nuka_field_from_name(name.encode())
        if fid == FIELD_NONE:
            raise KeyError(name)
        view = BufferViewC()
        _check(lib().nuka_world_get_buffer_view(self._h, fid, C.byref(view)))
        return fid, view

    def public_view(self, public_name):
        """The buffer view of a NUKA_FIELD_* id (its numeric value from nuka.h) and the bytes behind it."""
        fid = abi.PUBLIC_FIELDS[public_name][0]
        view = BufferViewC()
        _check(lib().nuka_world_get_buffer_view(self._h, fid, C.byref(view)))
        raw = np.empty(view.element_count * view.element_stride_bytes, np.uint8)
        _check(lib().nuka_world_download_field(self._h, fid, raw.ctypes.data, raw.nbytes, 0))
        return view, raw

    def download(self, name):
        fid, view = self._field(name)
        out = np.empty(view.element_count, dtype=_DTYPES[view.dtype])
        _check(lib().nuka_world_download_field(self._h, fid, out.ctypes.data, out.nbytes, 0))
        return out

    def upload(self, name, values):
        fid, view = self._field(name)
        arr = np.ascontiguousarray(np.asarray(values, dtype=_DTYPES[view.dtype]).reshape(-1))
        if arr.size != view.element_count:
            raise ValueError(f"{name}: expected {view.element_count} elements, got {arr.size}")
        _check(lib().nuka_world_upload_field(self._h, fid, arr.ctypes.data, arr.nbytes, 0))

    def set_state(self, state):
        E, nl = self.env_count, self.link_count
        self.upload("q", state["q"])
        self.upload("qdot", state["qdot"])
        self.upload("tau", state["tau"])
        self.upload("base_pose", state["base_pose"])
        lv = np.zeros((E, nl, 6), np.float32)
        lv[:, 0, :] = state["root_twist"]
        self.upload("link_velocity", lv)
        for name in ("body_linear_velocity", "body_angular_velocity"):   # a free body's state, per body row
            if name in state:
                self.upload(name, state[name])

    def op(self, name, variant=0):
        op = lib().nuka_hip_op_from_name(name.encode())
        if op < 0:
            raise KeyError(name)
        _check(lib().nuka_world_dispatch_op(self._h, op, variant))

    def step(self, n=1):
        _check(lib().nuka_world_step_n(self._h, n))

    def synchronize(self):
        _check(lib().nuka_world_synchronize(self._h))

    def checkpoint(self):
        """nuka_world_checkpoint_capture: the persistent physics of every environment, kept in device memory."""
        handle = C.c_void_p()
        _check(lib().nuka_world_checkpoint_capture(self._h, C.byref(handle)))
        return handle

    def restore(self, checkpoint):
        """nuka_world_checkpoint_restore, enqueued on the world's stream."""
        _check(lib().nuka_world_checkpoint_restore(self._h, checkpoint))

    def step_from(self, checkpoint, n=1):
        """n times: restore the checkpoint, then one step - every step runs on the checkpointed state."""
        L, h = lib(), self._h
        for _ in range(n):
            _check(L.nuka_world_checkpoint_restore(h, checkpoint))
            _check(L.nuka_world_step(h))

    def reset(self):
        _check(lib().nuka_world_reset(self._h))

    def reset_envs(self, env_ids, static=False):
        """Masked reset; `static` takes the entry point that stages the ids in the library's static device array."""
        ids = np.ascontiguousarray(np.asarray(env_ids, dtype=np.uint32))
        call = lib().nuka_world_reset_envs_static if static else lib().nuka_world_reset_envs
        _check(call(self._h, C.c_void_p(ids.ctypes.data), C.c_uint32(ids.size)))

    def set_execution_mode(self, graph):
        _check(lib().nuka_world_set_execution_mode(self._h, 1 if graph else 0))

    def set_velocity_iterations(self, n):
        _check(lib().nuka_world_set_velocity_iterations(self._h, n))

    def forward_kinematics(self):
        """nuka_world_forward_kinematics: link and body poses from the joint coordinates, no time advanced."""
        _check(lib().nuka_world_forward_kinematics(self._h))

    def state_hash(self):
        out = C.c_uint64()
        _check(lib().nuka_world_state_hash(self._h, C.byref(out)))
        return out.value

    def checkpoints_equal(self, a, b):
        out = C.c_uint32()
        _check(lib().nuka_checkpoint_equal(a, b, C.byref(out)))
        return bool(out.value)

    def write_checkpoint(self, checkpoint, path):
        _check(lib().nuka_checkpoint_write(checkpoint, str(path).encode()))

    def read_checkpoint(self, path):
        """nuka_world_checkpoint_read: a checkpoint of this world from a file a world of the same layout wrote."""
        handle = C.c_void_p()
        _check(lib().nuka_world_checkpoint_read(self._h, str(path).encode(), C.byref(handle)))
        return handle

    def execution_info(self):
        info = ExecutionInfoC()
        info.struct_size, info.schema_version = C.sizeof(ExecutionInfoC), 1
        _check(lib().nuka_world_get_execution_info(self._h, C.byref(info)))
        return info

    def resource_info(self):
        out = WorldResourceInfoC()
        _check(lib().nuka_world_get_resource_info(self._h, C.byref(out)))
        return out

    def resource_fields(self):
        """nuka_world_get_resource_fields: every field's place in the world's arena."""
        records = (ResourceFieldC * max(lib().nuka_world_resource_field_count(self._h), 1))()
        _check(lib().nuka_world_get_resource_fields(self._h, records))
        return list(records)[:lib().nuka_world_resource_field_count(self._h)]

    def begin_execution_window(self):
        window = C.c_void_p()
        _check(lib().nuka_world_begin_execution_window(self._h, C.byref(window)))
        return window

    def end_execution_window(self, window):
        out = ExecutionWindowC()
        _check(lib().nuka_world_end_execution_window(self._h, window, C.byref(out)))
        return out

    def stream(self):
        """nuka_world_get_stream: the hipStream_t the world executes on, as an integer address."""
        out = C.c_void_p()
        _check(lib().nuka_world_get_stream(self._h, C.byref(out)))
        return out.value

    def record_event(self, event):
        """nuka_world_record_event: records the caller's hipEvent_t (an address) after the work submitted so far."""
        _check(lib().nuka_world_record_event(self._h, C.c_void_p(event)))

    def solver_options(self):
        out = SolverOptionsC()
        _check(lib().nuka_world_get_solver_options(self._h, C.byref(out)))
        return out

    def dof_name(self, link_index):
        """nuka_world_get_dof_name by its two calls: the size query, then the name."""
        length = C.c_size_t()
        _check(lib().nuka_world_get_dof_name(self._h, link_index, None, 0, C.byref(length)))
        buffer = C.create_string_buffer(length.value + 1)
        _check(lib().nuka_world_get_dof_name(self._h, link_index, buffer, length.value + 1, C.byref(length)))
        return buffer.value.decode()

    def kinematic_link(self, link_index):
        out = KinematicLinkC()
        _check(lib().nuka_world_get_kinematic_link(self._h, link_index, C.byref(out)))
        return out

    def link_binding(self, link_index):
        out = LinkBindingC()
        _check(lib().nuka_world_get_link_binding(self._h, link_index, C.byref(out)))
        return out

    def colliders(self, env_index):
        """nuka_world_get_colliders: the count query, then the records of one environment."""
        count = C.c_uint32()
        _check(lib().nuka_world_get_colliders(self._h, env_index, None, 0, C.byref(count)))
        records = (ColliderC * max(count.value, 1))()
        _check(lib().nuka_world_get_colliders(self._h, env_index, records, count.value, C.byref(count)))
        return list(records)[:count.value]

    def param_infos(self):
        """nuka_world_get_param_infos as a list of dicts, in parameter order."""
        count = C.c_uint32()
        _check(lib().nuka_world_param_count(self._h, C.byref(count)))
        infos = (ParamInfoC * count.value)()
        for info in infos:
            info.struct_size, info.schema_version = C.sizeof(ParamInfoC), PARAM_INFO_VERSION
        _check(lib().nuka_world_get_param_infos(self._h, infos, count.value))
        return [{"key": i.key.decode(), "unit": i.unit.decode(), "scene_field": i.scene_field.decode(), "type": i.type, "tier": i.tier,
                 "count": i.count, "min": i.min_value, "max": i.max_value} for i in infos]

    def get_param(self, key, element=0):
        out = C.c_double()
        _check(lib().nuka_world_get_param(self._h, PARAMS.index(key), element, C.byref(out)))
        return out.value

    def set_param(self, key, element, value):
        """nuka_world_set_param: a world option or one template link's value, in every environment, from the next step on."""
        _check(lib().nuka_world_set_param(self._h, PARAMS.index(key), element, float(value)))

    def set_link_mass(self, link, mass):
        _check(lib().nuka_world_set_link_mass(self._h, link, mass))

    def set_gravity_z(self, gravity_z):
        _check(lib().nuka_world_set_gravity_z(self._h, gravity_z))

    def time_steps(self, n, checkpoint=None):
        """Milliseconds of n steps by device events on the world's stream; with a checkpoint every step starts from it."""
        out = C.c_float()
        _check(lib().nuka_world_time_steps(self._h, checkpoint, n, C.byref(out)))
        return out.value

    def profile_ops(self, steps, checkpoint=None):
        info = WorldInfoC()
        _check(lib().nuka_world_get_info(self._h, C.byref(info)))
        self.op_count = info.op_count   # a demanded readout joins the pipeline
        ms = (C.c_float * self.op_count)()
        ops = (C.c_uint16 * self.op_count)()
        _check(lib().nuka_world_profile_ops(self._h, checkpoint, steps, ms, ops))
        return [(lib().nuka_hip_op_name(ops[i]).decode(), ms[i] / steps) for i in range(self.op_count)]
