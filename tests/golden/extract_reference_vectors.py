#!/usr/bin/env python3
"""Extract the known-answer vectors held by the reference's own tests into JSON fixtures.

Reads the `static const TensorData NAME = {{dims}, {values}};` tables of
/root/reference/test/test_ops.cpp (:24-470 and :663-666) and
/root/reference/test/test_resnode.cpp (:35-134) and writes them, as data only, to
tests/golden/test_ops.json and tests/golden/test_resnode.json.  Only numeric tables are
taken; no code of the reference is copied.  Run once in a container that has
/root/reference mounted:

    python tests/golden/extract_reference_vectors.py
"""
import json
import os
import re
import sys

REF = os.environ.get("SAGA_REFERENCE", "/root/reference")
HERE = os.path.dirname(os.path.abspath(__file__))

TABLE = re.compile(
    r"static\s+const\s+TensorData\s+(\w+)\s*=\s*\{\s*\{([^}]*)\}\s*,\s*\{(.*?)\}\s*\}\s*;",
    re.S,
)


def parse(path):
    text = open(path).read()
    text = re.sub(r"//[^\n]*", "", text)
    out = {}
    for name, dims, vals in TABLE.findall(text):
        d = [int(t) for t in dims.replace("\n", " ").split(",") if t.strip()]
        v = [float(t) for t in vals.replace("\n", " ").split(",") if t.strip()]
        out[name] = {"dims": d, "data": v}
    return out


def main():
    for src, dst in (("test/test_ops.cpp", "test_ops.json"),
                     ("test/test_resnode.cpp", "test_resnode.json")):
        tables = parse(os.path.join(REF, src))
        if not tables:
            sys.exit("no tables found in " + src)
        with open(os.path.join(HERE, dst), "w") as f:
            json.dump({"source": src, "tensors": tables}, f, indent=0)
        print(dst, {k: (v["dims"], len(v["data"])) for k, v in tables.items()})


if __name__ == "__main__":
    main()
