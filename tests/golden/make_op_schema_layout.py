"""Writes tests/golden/op_schema_layout.json: the value of every NkOp and the size and member offsets of the parameter
structs of the ops this library serves, read off the reference's src/phi/op_catalog.inc and src/phi/op_schema.hpp.
The header itself does not compile outside the reference's build (it pulls in generated code), so the offsets are
computed from the member declarations as written there - scalar types of 1, 4 and 8 bytes, arrays and one nested
struct, laid out by the x86-64 rules (natural alignment, size rounded up to the largest alignment) - and each struct
carries the line of op_schema.hpp it was read from.  Data only: names and numbers.  Run where /root/reference is mounted."""
import json
import os
import re
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
REFERENCE = "/root/reference/src"
STRUCTS = ["VertexBlockLayout", "ApplyDrivesParams", "ReadoutDrivesParams", "ArticulationDynamicsParams", "IntegrateVelocityParams",
           "SnapshotStepVelocityParams", "AccumulateStepParams", "FkWorldPosesParams", "FkLinkVelocitiesParams",
           "IntegratePositionParams", "BuildAabbsParams", "LbvhBuildParams", "LbvhQueryPairsParams", "NarrowphasePrimitivesParams",
           "SyncLinkBodyPoseParams", "NarrowphaseHeightfieldParams", "AssembleRowsParams", "BlockDescentSolveParams",
           "ReadoutContactWrenchParams", "ContactWarmStartParams"]
SCALARS = {"float": 4, "uint32_t": 4, "int32_t": 4, "uint64_t": 8, "uint8_t": 1, "bool": 1, "uint16_t": 2}


def members_of(text, struct):
    """[(type, name, element count)] of a struct as declared, and the line it starts on."""
    found = re.search(r"struct " + struct + r"\s*\{(.*?)\n\};", text, flags=re.S)
    line = text[:found.start()].count("\n") + 1
    body = re.sub(r"//[^\n]*", "", found.group(1))
    members = []
    for statement in body.split(";"):
        statement = statement.strip()
        if not statement:
            continue
        kind, rest = statement.split(None, 1)
        for part in rest.split(","):
            part = re.sub(r"=.*$", "", part.strip(), flags=re.S)        # default initialiser
            part = re.sub(r"\{\s*\}", "", part).strip()
            name, dims = re.match(r"(\w+)\s*((?:\[\s*\w+\s*\]\s*)*)$", part).groups()
            count = 1
            for d in re.findall(r"\[\s*(\w+)\s*\]", dims):
                count *= int(d)
            members.append((kind, name, count))
    return members, line


def layout_of(text, struct, known):
    members, line = members_of(text, struct)
    offset, largest, offsets = 0, 1, {}
    for kind, name, count in members:
        size, align = (SCALARS[kind], SCALARS[kind]) if kind in SCALARS else known[kind]
        offset = (offset + align - 1) // align * align
        offsets[name] = offset
        offset += size * count
        largest = max(largest, align)
    size = (offset + largest - 1) // largest * largest
    known[struct] = (size, largest)
    return {"line": line, "size": size, "members": offsets}


def reference_layout():
    schema = open(os.path.join(REFERENCE, "phi", "op_schema.hpp")).read()
    ops = re.findall(r"NUKA_OP\((\w+),", open(os.path.join(REFERENCE, "phi", "op_catalog.inc")).read())
    known = {}
    return {"ops": {name: index for index, name in enumerate(ops)}, "op_count": len(ops),
            "structs": {s: layout_of(schema, s, known) for s in STRUCTS}}


if __name__ == "__main__":
    if not os.path.isdir(REFERENCE):
        sys.exit("the reference tree is not mounted")
    layout = reference_layout()
    with open(os.path.join(ROOT, "tests", "golden", "op_schema_layout.json"), "w") as out:
        json.dump(layout, out, indent=1, sort_keys=True)
    print(len(layout["ops"]), "ops,", len(layout["structs"]), "structs")
