"""The C-ABI library loads and exports every symbol include/*.h declares (no compute calls: runs without a GPU)."""
import ctypes as C
import os
import re

from conftest import ROOT, nk


def declared_functions():
    names = []
    for header in ("nuka_hip.h", "nuka_phi.h"):
        text = open(os.path.join(ROOT, "include", header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        text = re.sub(r"typedef struct\s+\w+\s*\{.*?\}\s*\w+;", "", text, flags=re.S)
        names += re.findall(r"\b(nuka_\w+)\s*\(", text)
    return sorted(set(names))


def test_library_exports_every_declared_symbol():
    lib = C.CDLL(nk.LIB_PATH)
    names = declared_functions()
    assert len(names) >= 28
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, f"declared but not exported: {missing}"
    assert set(nk.EXPORTS) <= set(names)


def test_struct_layouts_match_the_header():
    # 6 u32 + 22 pointers, then 4 pointers + 2 u32 of joint rows, then a pointer + 2 u32 of excluded pairs; 15 4-byte words
    assert C.sizeof(nk.abi.TemplateDescC) == 6 * 4 + 22 * 8 + 4 * 8 + 2 * 4 + 8 + 2 * 4 + 4 * 8 + 2 * 4 + 3 * 8 + 4 * 8 + 2 * 4
    assert C.sizeof(nk.abi.WorldDescC) == 17 * 4


def test_headers_compile_as_c_and_agree_with_the_ctypes_mirror(tmp_path):
    """include/*.h are plain C: a C99 program that includes them reports the size of each descriptor and the offset of
    every member the ctypes mirror declares, and the two layouts agree."""
    import subprocess
    members = {"nuka_template_desc_t": nk.abi.TemplateDescC, "nuka_hip_world_desc_t": nk.abi.WorldDescC, "nuka_world_desc_t": nk.abi.SceneWorldDescC, "nuka_device_desc_t": nk.DeviceDescC, "nuka_scene_info_t": nk.SceneInfoC,
               "nuka_param_info_t": nk.ParamInfoC, "nuka_world_execution_info_t": nk.ExecutionInfoC, "nuka_world_info_t": nk.WorldInfoC,
               "nuka_buffer_view_t": nk.abi.BufferViewC}
    lines = ['#include <stddef.h>', '#include <stdio.h>', '#include "nuka_phi.h"', '#include "nuka_hip.h"', 'int main(void) {']
    for name, mirror in members.items():
        lines.append(f'    printf("{name} %zu\\n", sizeof({name}));')
        for field, _ in mirror._fields_:
            lines.append(f'    printf("{name}.{field} %zu\\n", offsetof({name}, {field}));')
    lines += ['    return 0;', '}']
    source = tmp_path / "layout.c"
    source.write_text("\n".join(lines) + "\n")
    binary = tmp_path / "layout"
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-pedantic", "-I", os.path.join(ROOT, "include"), str(source), "-o", str(binary)], check=True)
    reported = dict(line.split() for line in subprocess.run([str(binary)], check=True, capture_output=True, text=True).stdout.splitlines())
    for name, mirror in members.items():
        assert int(reported[name]) == C.sizeof(mirror), name
        for field, _ in mirror._fields_:
            assert int(reported[f"{name}.{field}"]) == getattr(mirror, field).offset, f"{name}.{field}"


def test_op_catalog_names_round_trip():
    lib = nk.lib()
    count = lib.nuka_hip_op_count()
    names = [lib.nuka_hip_op_name(i).decode() for i in range(count)]
    for expected in ("FkWorldPoses", "ArticulationDynamics", "SyncLinkBodyPose", "BuildAabbs", "LbvhQueryPairs",
                     "NarrowphasePrimitives", "AssembleRows", "ContactWarmStart", "BlockDescentSolve", "IntegratePosition",
                     "FkLinkVelocities", "ApplyDrives", "ReadoutDrives", "ReadoutContactWrench", "AccumulateStep"):
        assert expected in names
        assert lib.nuka_hip_op_from_name(expected.encode()) == names.index(expected)
    assert lib.nuka_hip_op_from_name(b"NoSuchOp") == -1


def test_field_names_cover_the_seam_fields():
    lib = nk.lib()
    fields = lib.nuka_field_names().decode().strip(",").split(",")
    for name in ("q", "qdot", "qddot", "tau", "base_pose", "link_pose", "link_velocity", "link_acceleration", "m",
                 "m_factor", "articulation_bias", "candidate_pairs", "pair_count", "ucontact_count", "ucontact_point",
                 "ucontact_normal", "ucontact_depth", "ucontact_row_range", "urows", "lambda", "chain_jacobian",
                 "chain_jacobian_b", "env_status", "solver_residual", "vbd_velocity_sweep_count", "link_inertia",
                 "shape_table", "drive_target", "drive_stiffness", "drive_damping", "drive_force_limit", "velocity_target",
                 "joint_f", "drive_command", "actuator_effort", "joint_limit_impulse"):
        assert name in fields
        assert lib.nuka_field_from_name(name.encode()) == nk.FIELD_BASE + fields.index(name)     # the library's own ids
    assert lib.nuka_field_from_name(b"no_such_field") == nk.FIELD_NONE
    # every public id the header declares names a field of the world, and no library id collides with a public one
    header = open(os.path.join(ROOT, "include", "nuka_hip.h")).read()
    declared = {m.group(1): int(m.group(2)) for m in re.finditer(r"NUKA_FIELD_(\w+) = (\d+)", header)}
    assert declared == {k: v[0] for k, v in nk.abi.PUBLIC_FIELDS.items()}
    assert all(v[1] in fields for v in nk.abi.PUBLIC_FIELDS.values()) and max(declared.values()) < nk.FIELD_BASE


def test_result_messages():
    lib = nk.lib()
    assert lib.nuka_result_message(0) == b"ok"
    assert lib.nuka_result_message(7) == b"not supported"
