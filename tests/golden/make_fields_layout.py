"""Writes tests/golden/fields_layout.json: every field of the reference's field table (src/nk/model/fields.yaml) with
its element type, the entity it has one element group for, the elements a group (`elem`, 1 where not given), its owner
and, for fields sized by a count of their own, that count as written.  Data only: names and numbers, with the line of
fields.yaml each was read from.  Run where /root/reference is mounted."""
import json
import os

import yaml

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
SOURCE = "/root/reference/src/nk/model/fields.yaml"


def main():
    text = open(SOURCE).read()
    lines = text.splitlines()
    table = yaml.safe_load(text)
    fields = {}
    for f in table["fields"]:
        line = next(i + 1 for i, l in enumerate(lines) if f"name: {f['name']}," in l or f"name: {f['name']} " in l or l.rstrip().endswith(f"name: {f['name']}}}"))
        fields[f["name"]] = {"dtype": f["dtype"], "per": f["per"], "elem": int(f.get("elem", 1)), "owner": f["owner"],
                             "count": f.get("count"), "line": line}
    out = {"source": "src/nk/model/fields.yaml", "schema": table["schema"], "fields": fields}
    with open(os.path.join(ROOT, "tests", "golden", "fields_layout.json"), "w") as fh:
        json.dump(out, fh, indent=0, sort_keys=True)
    print(len(fields), "fields")


if __name__ == "__main__":
    main()
