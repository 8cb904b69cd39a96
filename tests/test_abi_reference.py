"""include/nuka_hip.h against the reference's own src/include/nuka/nuka.h, where the reference tree is mounted: every
struct, enum constant and function that both headers declare must agree - sizes, member offsets, numeric values and
full signatures.  Two C++ programs, one per header, print the same report; the reports are compared line by line.
(The headers cannot share a translation unit: they declare the same names.)"""
import os
import re
import subprocess

import pytest

from conftest import ROOT

REFERENCE = "/root/reference/src/include/nuka/nuka.h"
MINE = os.path.join(ROOT, "include", "nuka_hip.h")
pytestmark = pytest.mark.skipif(not os.path.exists(REFERENCE), reason="the reference tree is not mounted")


def strip_comments(text):
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return re.sub(r"//[^\n]*", "", text)


def declarations(path):
    """(structs {name: [members]}, enum constants, functions) a header declares."""
    text = strip_comments(open(path).read())
    structs = {}
    for body, name in re.findall(r"typedef struct\s+\w+\s*\{(.*?)\}\s*(\w+)\s*;", text, flags=re.S):
        members = []
        for line in body.split(";"):
            line = line.strip()
            if not line or "(" in line:          # function pointers are compared through the whole struct's size
                continue
            for part in line.split(","):
                found = re.search(r"(\w+)\s*(\[[^\]]*\]\s*)*$", part.strip())
                if found:
                    members.append(found.group(1))
        structs[name] = members
    constants = set()
    for body in re.findall(r"enum\s*\w*\s*\{(.*?)\}", text, flags=re.S):
        constants.update(re.findall(r"\b(NUKA_\w+)\b\s*(?:=|,|$)", body, flags=re.M))
    functions = set(re.findall(r"\b(nuka_\w+)\s*\(", re.sub(r"typedef struct\s+\w+\s*\{.*?\}\s*\w+\s*;", "", text, flags=re.S)))
    functions = {f for f in functions if not f.endswith("_t")}
    return structs, constants, functions


def report(header, include_dir, structs, constants, functions, tmp_path, tag):
    lines = ["#include <cstddef>", "#include <cstdio>", "#include <typeinfo>", f'#include "{header}"', "int main() {"]
    for name, members in sorted(structs.items()):
        lines.append(f'    std::printf("sizeof {name} %zu\\n", sizeof({name}));')
        for m in members:
            lines.append(f'    std::printf("offsetof {name}.{m} %zu\\n", offsetof({name}, {m}));')
    for c in sorted(constants):
        lines.append(f'    std::printf("value {c} %lld\\n", (long long)({c}));')
    for f in sorted(functions):
        lines.append(f'    std::printf("signature {f} %s\\n", typeid(decltype(&{f})).name());')
    lines += ["    return 0;", "}"]
    source = tmp_path / f"{tag}.cpp"
    source.write_text("\n".join(lines) + "\n")
    binary = tmp_path / tag
    subprocess.run(["g++", "-std=c++17", "-I", include_dir, str(source), "-o", str(binary)], check=True)
    return subprocess.run([str(binary)], check=True, capture_output=True, text=True).stdout.splitlines()


def test_everything_both_headers_declare_agrees(tmp_path):
    ref_structs, ref_constants, ref_functions = declarations(REFERENCE)
    my_structs, my_constants, my_functions = declarations(MINE)
    structs = {}
    for name in sorted(set(ref_structs) & set(my_structs)):
        assert ref_structs[name] == my_structs[name], f"{name}: members differ from nuka.h: {my_structs[name]} vs {ref_structs[name]}"
        structs[name] = my_structs[name]
    constants = ref_constants & my_constants
    functions = ref_functions & my_functions
    # what the path needs from the reference's surface must be among the shared names
    for name in ("nuka_world_desc_t", "nuka_device_desc_t", "nuka_buffer_view_t", "nuka_param_info_t", "nuka_world_execution_info_t"):
        assert name in structs, name
    for name in ("nuka_world_create_from_scene", "nuka_device_create", "nuka_world_step", "nuka_world_step_n", "nuka_world_reset_envs",
                 "nuka_world_get_buffer_view", "nuka_world_upload_field", "nuka_world_download_field", "nuka_world_checkpoint_capture",
                 "nuka_world_set_param", "nuka_world_set_execution_mode", "nuka_world_state_hash"):
        assert name in functions, name
    assert {"NUKA_FIELD_JOINT_POSITION", "NUKA_FIELD_ARTICULATION_LINK_POSE", "NUKA_FIELD_ROW_LAMBDA", "NUKA_RESULT_CUDA_ERROR",
            "NUKA_RESULT_NOT_SUPPORTED", "NUKA_EXECUTION_GRAPH", "NUKA_PARAM_REBUILD"} <= constants
    # a library-only name must not be a name of the reference
    assert not any(n.startswith("NUKA_HIP_") for n in ref_constants)
    theirs = report("nuka/nuka.h", os.path.dirname(os.path.dirname(REFERENCE)), structs, constants, functions, tmp_path, "reference")
    ours = report("nuka_hip.h", os.path.join(ROOT, "include"), structs, constants, functions, tmp_path, "library")
    assert len(ours) == len(theirs) and len(ours) > 150
    differing = [(a, b) for a, b in zip(ours, theirs) if a != b]
    assert not differing, differing[:10]
    print(f"{len(structs)} structs, {len(constants)} constants and {len(functions)} functions agree with nuka.h")
