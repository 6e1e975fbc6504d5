"""Writes tests/golden/struct_fields.json: for every argument struct this library mirrors, the ordered list of
(type, field name) as the reference's headers declare it.  Run in a container that has /root/reference; the
test that reads the JSON (tests/test_abi.py) needs only the JSON.

The reference headers are read as text (no import, nothing executed)."""
import json
import os
import re
import sys

REF = os.environ.get("PTL_REFERENCE", "/root/reference")
HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))


def struct_fields(text):
    """{struct name: [[type, field], ...]} of every `struct X { ... };` definition in a C header."""
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    out = {}
    for m in re.finditer(r"struct\s+(\w+)\s*\{([^{}]*)\}\s*;", text):
        fields = []
        for decl in m.group(2).split(";"):
            decl = " ".join(decl.replace("__restrict__", " ").split())
            if not decl:
                continue
            mm = re.match(r"^(.*?)([A-Za-z_]\w*)\s*(\[\w*\])?$", decl)
            typ, name = mm.group(1), mm.group(2)
            typ = re.sub(r"\s*\*\s*", " *", typ).strip() + (mm.group(3) or "")
            fields.append([typ, name])
        out[m.group(1)] = fields
    return out


def main():
    mine = struct_fields(open(os.path.join(ROOT, "include", "ptl_structs.h")).read())
    ref = {}
    inc = os.path.join(REF, "lib", "include")
    for f in sorted(os.listdir(inc)):
        if f.endswith(".h"):
            for name, fields in struct_fields(open(os.path.join(inc, f)).read()).items():
                ref.setdefault(name, {"header": "lib/include/" + f, "fields": fields})
    missing = [n for n in mine if n not in ref]
    # structs this library adds (no counterpart in the reference) are listed, not silently dropped
    data = {"reference_structs": {n: ref[n] for n in mine if n in ref}, "extensions": sorted(missing)}
    with open(os.path.join(HERE, "struct_fields.json"), "w") as f:
        json.dump(data, f, indent=1, sort_keys=True)
    print("%d structs written, extensions: %s" % (len(data["reference_structs"]), data["extensions"]))


if __name__ == "__main__":
    sys.exit(main())
