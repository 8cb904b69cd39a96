"""ctypes driver of the CPU oracle (test infrastructure: tests/, smoke() and bench.py's cpu_baseline leg only)."""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "_build", "libnuka_oracle.so")
LIB64_PATH = os.path.join(HERE, "_build", "libnuka_oracle_f64.so")   # the same sources with every scalar a double
REF_PATH = os.path.join(HERE, "_ref", "libnuka_ref.so")

U32_FIELDS = {"candidate_pairs", "pair_count", "ucontact_count", "ucontact_a", "ucontact_b", "ucontact_law",
              "ucontact_row_range", "row_cj_link", "row_cj_link_b", "row_count", "contact_count",
              "contact_row_extent", "env_status", "vbd_velocity_sweep_count", "link_tree_depth",
              "link_child_range", "link_children", "link_dof", "dof_link", "dof_component", "link_body",
              "body_to_link", "body_collidable_link", "body_collidable_body", "contact_cache_age",
              "contact_cache_current_owner", "contact_cache_old_keep", "contact_cache_extent", "contact_warm_start_counts",
              "contact_side_a_kind", "contact_side_b_kind", "contact_side_a_index", "contact_side_b_index", "contact_link",
              "body_gyro_iterations", "body_gyro_status"}
U64_FIELDS = {"ucontact_id_pair", "ucontact_id_feature", "contact_material", "contact_cache_pair", "contact_cache_feature",
              "contact_cache_material"}


def build(force=False):
    """Compiles the oracle (and, where the reference tree is mounted, the reference-header shim)."""
    # make compares the sources' and headers' times with the library's: an up-to-date library costs nothing
    subprocess.run(["make", "-C", HERE, "_build/libnuka_oracle.so", "_build/libnuka_oracle_f64.so"] + (["-B"] if force else []), check=True,
                   stdout=subprocess.DEVNULL)
    if os.path.isdir("/root/reference/src") and (force or not os.path.exists(REF_PATH)):
        subprocess.run(["make", "-C", HERE, "ref"], check=True, stdout=subprocess.DEVNULL)


_lib = None
_lib64 = None


def lib64():
    """The double-precision build: the world entry points only (what steps a world and reads its fields)."""
    global _lib64
    if _lib64 is None:
        build()
        L = C.CDLL(LIB64_PATH)
        _declare_world_entry_points(L)
        assert L.nko_real_bytes() == 8
        _lib64 = L
    return _lib64


def _declare_world_entry_points(L):
    L.nko_world_create.restype = C.c_void_p
    L.nko_world_create.argtypes = [C.c_void_p, C.c_void_p]
    L.nko_world_destroy.argtypes = [C.c_void_p]
    L.nko_world_field.argtypes = [C.c_void_p, C.c_char_p, C.POINTER(C.c_void_p), C.POINTER(C.c_size_t)]
    L.nko_world_field_names.restype = C.c_char_p
    L.nko_world_set_threads.argtypes = [C.c_void_p, C.c_int]
    L.nko_world_set_line_rule.argtypes = [C.c_void_p, C.c_int]
    L.nko_world_dof.argtypes = [C.c_void_p]
    L.nko_world_dof.restype = C.c_uint32
    L.nko_world_rows_per_env.argtypes = [C.c_void_p]
    L.nko_world_rows_per_env.restype = C.c_uint32
    L.nko_real_bytes.restype = C.c_uint32
    for name in ("fk_world_poses", "sync_link_body_pose", "build_aabbs", "query_pairs", "narrowphase",
                 "assemble_rows", "block_descent_solve", "integrate_position", "fk_link_velocities", "apply_drives",
                 "readout_drives", "readout_contact_wrench", "reference_weights", "snapshot_step_velocity",
                 "articulation_damping", "body_integrate_velocity", "body_integrate_position"):
        getattr(L, "nko_" + name).argtypes = [C.c_void_p]
    L.nko_articulation_dynamics.argtypes = [C.c_void_p, C.c_uint32]
    L.nko_contact_warm_start.argtypes = [C.c_void_p, C.c_uint32]
    L.nko_world_step.argtypes = [C.c_void_p]


def widened(struct, arrays=None):
    """A descriptor struct for the double-precision build: the same members in the same order with every float a
    double, arrays of floats converted (`arrays`: the float32 arrays behind the struct's pointers, by member name).
    Returns the struct and what must stay alive with it."""
    fields, keep = [], []
    for name, ctype in struct._fields_:
        if ctype is C.c_float:
            ctype = C.c_double
        elif isinstance(ctype, type) and issubclass(ctype, C.Array) and ctype._type_ is C.c_float:
            ctype = C.c_double * ctype._length_
        elif ctype == C.POINTER(C.c_float):
            ctype = C.POINTER(C.c_double)
        fields.append((name, ctype))
    wide = type(type(struct).__name__ + "F64", (C.Structure,), {"_fields_": fields})()
    for (name, old), (_, new) in zip(struct._fields_, fields):
        value = getattr(struct, name)
        if new == C.POINTER(C.c_double):
            source = None if arrays is None else arrays.get(name)
            if source is not None and source.size:
                converted = np.ascontiguousarray(source, dtype=np.float64)
                keep.append(converted)
                setattr(wide, name, converted.ctypes.data_as(new))
        elif isinstance(new, type) and issubclass(new, C.Array):
            for i in range(new._length_):
                getattr(wide, name)[i] = value[i]
        else:
            setattr(wide, name, value)
    if hasattr(wide, "struct_size"):
        wide.struct_size = C.sizeof(wide)
    return wide, keep


def lib():
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(LIB_PATH)
        L.nko_world_create.restype = C.c_void_p
        L.nko_world_create.argtypes = [C.c_void_p, C.c_void_p]
        L.nko_world_destroy.argtypes = [C.c_void_p]
        L.nko_world_field.argtypes = [C.c_void_p, C.c_char_p, C.POINTER(C.c_void_p), C.POINTER(C.c_size_t)]
        L.nko_world_field_names.restype = C.c_char_p
        L.nko_world_set_threads.argtypes = [C.c_void_p, C.c_int]
        L.nko_world_set_line_rule.argtypes = [C.c_void_p, C.c_int]
        L.nko_world_dof.argtypes = [C.c_void_p]
        L.nko_world_dof.restype = C.c_uint32
        L.nko_world_rows_per_env.argtypes = [C.c_void_p]
        L.nko_world_rows_per_env.restype = C.c_uint32
        for name in ("fk_world_poses", "sync_link_body_pose", "build_aabbs", "query_pairs", "narrowphase",
                     "assemble_rows", "block_descent_solve", "integrate_position", "fk_link_velocities", "apply_drives",
                     "readout_drives", "readout_contact_wrench", "reference_weights", "snapshot_step_velocity",
                     "articulation_damping", "body_integrate_velocity", "body_integrate_position"):
            getattr(L, "nko_" + name).argtypes = [C.c_void_p]
        L.nko_articulation_dynamics.argtypes = [C.c_void_p, C.c_uint32]
        L.nko_contact_warm_start.argtypes = [C.c_void_p, C.c_uint32]
        L.nko_world_step.argtypes = [C.c_void_p]
        L.nko_mass_coupling.restype = C.c_float
        _lib = L
    return _lib


class OracleWorld:
    def __init__(self, template, desc, threads=1, double=False):
        """`double`: the double-precision build of the same sources - every field then reads and writes as float64."""
        self._double = double
        L = self._lib = lib64() if double else lib()
        tdesc, self._keep = template.to_c()
        if double:
            tdesc, kept = widened(tdesc, self._keep)
            desc, _ = widened(desc)
            self._keep = (self._keep, kept)
        self._h = L.nko_world_create(C.byref(tdesc), C.byref(desc))
        if not self._h:
            raise RuntimeError("oracle: template rejected")
        L.nko_world_set_threads(self._h, threads)
        self.env_count = desc.env_count
        self.link_count = template.link_count
        self.dof = L.nko_world_dof(self._h)
        self.rows_per_env = L.nko_world_rows_per_env(self._h)

    def set_line_rule(self, rule):
        """1: the line search stops by the rule of the HIP kernels instead of the reference's (nuka_oracle.h)."""
        self._lib.nko_world_set_line_rule(self._h, int(rule))

    def close(self):
        if self._h:
            self._lib.nko_world_destroy(self._h)
            self._h = None

    def __del__(self):
        self.close()

    def field(self, name):
        ptr, nbytes = C.c_void_p(), C.c_size_t()
        if self._lib.nko_world_field(self._h, name.encode(), C.byref(ptr), C.byref(nbytes)) != 0:
            raise KeyError(name)
        dtype = np.uint32 if name in U32_FIELDS else np.uint64 if name in U64_FIELDS else np.float64 if self._double else np.float32
        count = nbytes.value // np.dtype(dtype).itemsize
        if count == 0:
            return np.zeros(0, dtype)
        return np.ctypeslib.as_array(C.cast(ptr, C.POINTER(np.ctypeslib.as_ctypes_type(dtype))), shape=(count,))

    def download(self, name):
        return self.field(name).copy()

    def upload(self, name, values):
        f = self.field(name)
        f[:] = np.asarray(values, dtype=f.dtype).reshape(-1)

    def set_state(self, state):
        E, nl = self.env_count, self.link_count
        self.upload("q", state["q"])
        self.upload("qdot", state["qdot"])
        self.upload("tau", state["tau"])
        self.upload("base_pose", state["base_pose"])
        lv = self.field("link_velocity").reshape(E, nl, 6)
        lv[:] = 0.0
        lv[:, 0, :] = state["root_twist"]
        for name in ("body_linear_velocity", "body_angular_velocity"):   # a free body's state, per body row
            if name in state:
                self.upload(name, state[name])

    def op(self, name, *args):
        getattr(self._lib, "nko_" + name)(self._h, *args)

    def step(self, n=1):
        for _ in range(n):
            self._lib.nko_world_step(self._h)
