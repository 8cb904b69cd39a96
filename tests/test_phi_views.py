"""The two views at the PHI seam, field by field, against the reference's field table.

ModelView and DataView (src/nk/model/generated/views.hpp) are generated from src/nk/model/fields.yaml: one device
pointer per field.  This backend's views hold the fields its ops touch; tests/golden/fields_layout.json is that table
read off the reference (tests/golden/make_fields_layout.py).  Every member that stands for a field of the table must
carry its name (or the name recorded as its counterpart), its scalar type, the entity it is counted by and the scalars
per entity; what remains must be declared as the backend's own.  The by-name binding a host uses to fill the views is
exercised on plain host memory (no device call)."""
import ctypes as C
import json
import os

import pytest

from conftest import ROOT, nk

SCALARS = {"f32": (0, 1), "u32": (1, 1), "u64": (2, 1), "u8": (3, 1), "vec3": (0, 3), "quat": (0, 4), "transform": (0, 7), "spatial6": (0, 6),
           "mat36": (0, 36), "symmat3": (0, 6)}
# NUKA_HIP_PER_*; one articulation an environment on this path: per articulation is per environment
PER = {"env": 0, "articulation": 0, "link": 1, "body": 2, "dof": 3, "articulation_dof": 3, "articulation_dof2": 4, "contact_slot": 5, "row_slot": 6,
       "row_dof": 7, "scalar": 8}


class ViewField(C.Structure):
    _fields_ = [("name", C.c_char_p), ("reference_name", C.c_char_p), ("owner", C.c_uint8), ("dtype", C.c_uint8), ("per", C.c_uint8),
                ("scalars_per_entity", C.c_uint32)]


def view_fields():
    L = nk.lib()
    L.nuka_hip_view_field_count.restype = C.c_uint32
    out = []
    for i in range(L.nuka_hip_view_field_count()):
        f = ViewField()
        assert L.nuka_hip_view_field(i, C.byref(f)) == 0
        out.append(f)
    assert L.nuka_hip_view_field(len(out), C.byref(ViewField())) == -1
    return out


def test_every_served_field_is_the_reference_field_of_that_name():
    table = json.load(open(os.path.join(ROOT, "tests", "golden", "fields_layout.json")))["fields"]
    fields = view_fields()
    own = [f.name.decode() for f in fields if f.reference_name is None]
    assert len(fields) - len(own) >= 120 and len(own) <= 24
    for f in fields:
        name = f.name.decode()
        if f.reference_name is None:
            assert name not in table, f"{name} is a field of the reference and must be bound to it"
            continue
        ref = table[f.reference_name.decode()]
        dtype, width = SCALARS[ref["dtype"]]
        assert f.dtype == dtype, (name, ref)
        assert f.owner == (0 if ref["owner"] == "model" else 1) or name in ("body_invweight0", "dof_invweight0"), (name, ref)
        if ref["per"] == "scalar":
            assert f.per == PER["scalar"] and ref["count"], (name, ref)      # sized by its own count on both sides
            continue
        assert f.per == PER[ref["per"]], (name, f.per, ref)
        assert f.scalars_per_entity == width * ref["elem"], (name, f.scalars_per_entity, ref)


def test_views_bind_by_reference_name():
    """A host hands (name, pointer) pairs under the reference's names; members without a pair are reported."""
    L = nk.lib()
    L.nuka_hip_model_view_bytes.restype = C.c_size_t
    L.nuka_hip_data_view_bytes.restype = C.c_size_t
    model = (C.c_char * L.nuka_hip_model_view_bytes())()
    data = (C.c_char * L.nuka_hip_data_view_bytes())()
    fields = view_fields()
    names = [(f.reference_name or f.name) for f in fields if f.name not in (b"lambda", b"solver_cost")]
    pointers = [0x1000 + 0x100 * i for i in range(len(names))]
    c_names = (C.c_char_p * len(names))(*names)
    c_pointers = (C.c_void_p * len(names))(*pointers)
    missing = C.create_string_buffer(256)
    unset = L.nuka_hip_bind_views(c_names, c_pointers, len(names), model, data, missing, 256)
    assert unset == 2 and sorted(missing.value.decode().split(",")) == ["lambda", "solver_cost"]
    # a second call adds to what is bound
    rest = (C.c_char_p * 2)(b"lambda", b"solver_cost")
    rest_pointers = (C.c_void_p * 2)(0xAAA000, 0xBBB000)
    assert L.nuka_hip_bind_views(rest, rest_pointers, 2, model, data, missing, 256) == 0 and missing.value == b""
    # the reference's name and the member's own both reach dof_link
    alias = (C.c_char_p * 1)(b"dof_to_link")
    alias_pointer = (C.c_void_p * 1)(0xCCC000)
    assert L.nuka_hip_bind_views(alias, alias_pointer, 1, model, data, None, 0) == 0
    for name, value in (("links_per_env", 31), ("dof", 36), ("contact_dof_end", 18)):
        assert L.nuka_hip_model_view_set_count(model, name.encode(), value) == 0
    assert L.nuka_hip_model_view_set_count(model, b"no_such_count", 1) == -1
    words = (C.c_uint32 * 4).from_buffer(model)
    assert words[0] == 31 and words[2] == 36                     # links_per_env, bodies_per_env, dof head the model view


def test_the_adapter_is_reached_through_get_proc_address():
    L = nk.lib()
    L.nuka_hip_register_backend_entry.restype = C.c_void_p
    entry = L.nuka_hip_register_backend_entry()
    table = C.cast(C.cast(entry, C.POINTER(C.c_void_p))[0], C.POINTER(C.c_void_p))       # RegistryEntryI: 4 function pointers
    get_proc_address = C.CFUNCTYPE(C.c_void_p, C.c_void_p, C.c_char_p)(table[3])
    for name in ("nuka_hip_view_field_count", "nuka_hip_view_field", "nuka_hip_model_view_bytes", "nuka_hip_data_view_bytes",
                 "nuka_hip_bind_views", "nuka_hip_model_view_set_count"):
        address = get_proc_address(entry, name.encode())
        assert address == C.cast(getattr(L, name), C.c_void_p).value, name
    assert get_proc_address(entry, b"no_such_entry") is None
