"""The PHI op contract of the backend against the reference's: every NkOp value (src/phi/op_catalog.inc order) and the
size and every member offset of the parameter struct of every op served (src/phi/op_schema.hpp), as recorded in
tests/golden/op_schema_layout.json with the line of each struct.  The library's side is measured, not restated: a C++
program including csrc/nk_types.h prints sizeof and offsetof.  Where the reference tree is mounted the recorded layout is
also rebuilt from the reference's header and must not have drifted."""
import json
import os
import subprocess

from conftest import ROOT

GOLDEN = os.path.join(ROOT, "tests", "golden", "op_schema_layout.json")
CSRC = os.path.join(ROOT, "nuka-physics_amd", "csrc")


def test_op_ids_and_parameter_structs_have_the_reference_layout(tmp_path):
    expected = json.load(open(GOLDEN))
    lines = ["#include <cstddef>", "#include <cstdio>", '#include "nk_types.h"', "using namespace nkh;", "int main() {"]
    for op in expected["ops"]:
        lines.append(f'    std::printf("op {op} %u\\n", unsigned(NkOp::{op}));')
    lines.append('    std::printf("op Count %u\\n", unsigned(NkOp::Count));')
    for struct, layout in expected["structs"].items():
        lines.append(f'    std::printf("sizeof {struct} %zu\\n", sizeof({struct}));')
        for member in layout["members"]:
            lines.append(f'    std::printf("offsetof {struct}.{member} %zu\\n", offsetof({struct}, {member}));')
    lines += ["    return 0;", "}"]
    source, binary = tmp_path / "layout.cpp", tmp_path / "layout"
    source.write_text("\n".join(lines) + "\n")
    subprocess.run(["g++", "-std=c++17", "-Wno-invalid-offsetof", "-I", CSRC, str(source), "-o", str(binary)], check=True)
    out = subprocess.run([str(binary)], check=True, capture_output=True, text=True).stdout
    measured = {" ".join(line.split()[:2]): int(line.split()[2]) for line in out.splitlines()}
    for op, value in expected["ops"].items():
        assert measured[f"op {op}"] == value, f"NkOp::{op} (op_catalog.inc entry {value})"
    assert measured["op Count"] == expected["op_count"]
    for struct, layout in expected["structs"].items():
        where = f"op_schema.hpp:{layout['line']}"
        assert measured[f"sizeof {struct}"] == layout["size"], f"{struct} ({where})"
        for member, offset in layout["members"].items():
            assert measured[f"offsetof {struct}.{member}"] == offset, f"{struct}.{member} ({where})"
    # the library's struct has no member the reference's lacks: it ends where the reference's does (sizes agree above)
    # and every member counted by the compiler is one of the recorded ones
    assert expected["ops"]["BlockDescentSolve"] == 50 and expected["ops"]["ArticulationDynamics"] == 2


def test_recorded_layout_is_what_the_reference_header_says():
    import importlib.util
    import pytest
    if not os.path.isdir("/root/reference/src/phi"):
        pytest.skip("the reference tree is not mounted")
    spec = importlib.util.spec_from_file_location("make_op_schema_layout", os.path.join(ROOT, "tests", "golden", "make_op_schema_layout.py"))
    module = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(module)
    assert module.reference_layout() == json.load(open(GOLDEN))


def test_layout_rules_of_the_generator_match_the_compiler(tmp_path):
    """The generator computes offsets from declarations; the same declarations compiled by g++ must give the same
    numbers (checked on the library's own copy of the structs, which the first test ties to the recorded layout)."""
    import importlib.util
    spec = importlib.util.spec_from_file_location("make_op_schema_layout", os.path.join(ROOT, "tests", "golden", "make_op_schema_layout.py"))
    module = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(module)
    text = open(os.path.join(CSRC, "nk_types.h")).read().replace("kMaxDof", "64")
    known = {}
    computed = {s: module.layout_of(text, s, known) for s in module.STRUCTS}
    recorded = json.load(open(GOLDEN))["structs"]
    for struct in module.STRUCTS:
        assert computed[struct]["size"] == recorded[struct]["size"] and computed[struct]["members"] == recorded[struct]["members"], struct
