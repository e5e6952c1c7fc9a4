"""Writes tests/golden/zk_tables.json from the data the reference holds as text.

The reference keeps no test vectors for its GPU kernels.  What it does hold is
two 256-entry exp2 tables (and the log2(e) constants) inside its proving
circuits, which re-derive every kernel result and would fail to prove if the
kernels used different tables:
    zk/src/index.ts:2645-2681   q19Table   (softmax Q19,   2^(-i/256) * 2^19)
    zk/src/index.ts:3382-3418   q23Table   (SiLU/sigmoid,  2^(+i/256) * 2^23)
    zk/src/index.ts:2618, 3377  LOG2E_Q19, LOG2E_Q23
This script reads those literals AS TEXT (nothing from the reference is
imported or executed) and stores the numbers.  It only runs where
/root/reference is mounted; the JSON it writes is the committed fixture.
"""
import json
import os
import re

REF = os.environ.get("ZK_REFERENCE", "/root/reference")
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "zk_tables.json")


def table(text, name):
    m = re.search(r"const %s = \[(.*?)\];" % name, text, re.S)
    vals = [int(v) for v in re.findall(r"UInt64\.from\((\d+)n\)", m.group(1))]
    assert len(vals) == 256, (name, len(vals))
    return vals


def const(text, name):
    m = re.search(r"const %s = (?:UInt64\.from\()?(\d+)n" % name, text)
    return int(m.group(1))


def main():
    with open(os.path.join(REF, "zk/src/index.ts"), encoding="utf-8") as f:
        text = f.read()
    data = {
        "source": "zk/src/index.ts (q19Table, q23Table, LOG2E_Q19, LOG2E_Q23), parsed as text",
        "LOG2E_Q19": const(text, "LOG2E_Q19"),
        "LOG2E_Q23": const(text, "LOG2E_Q23"),
        "q19Table": table(text, "q19Table"),
        "q23Table": table(text, "q23Table"),
    }
    with open(OUT, "w") as f:
        json.dump(data, f, indent=0)
    print("wrote", OUT, data["LOG2E_Q19"], data["LOG2E_Q23"], data["q19Table"][:3], data["q23Table"][-3:])


if __name__ == "__main__":
    main()
