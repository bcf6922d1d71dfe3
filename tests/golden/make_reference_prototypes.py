#!/usr/bin/env python3
"""Writes tests/golden/reference_prototypes.json: the C prototypes that the cgo preamble of the
reference's cgo_bridge/bridge.go declares (return type and parameter types, names dropped) for
every function include/gometal_hip.h also declares.  Data for tests/test_abi_symbols.py, which
checks that a Go build of cgo_bridge would bind to this library's header unchanged.

Run in the build container (it reads /root/reference):  python tests/golden/make_reference_prototypes.py
"""
import json
import os
import re
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))


def prototypes(text):
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    out = {}
    for m in re.finditer(r"([A-Za-z_][A-Za-z0-9_ \*]*?)\s*\b([a-z_][a-z0-9_]*)\s*\(([^;{()]*)\)\s*;", text, re.S):
        ret, name, params = " ".join(m.group(1).split()), m.group(2), m.group(3)

        def kind(p):
            p = " ".join(p.split())
            if p in ("void", ""):
                return None
            mm = re.match(r"^(.*?)([A-Za-z_][A-Za-z0-9_]*)$", p)
            t = mm.group(1).strip() if mm and mm.group(1).strip() else p
            t = t.replace(" *", "*").replace("* ", "*").replace("const ", "")
            return "bool" if t == "_Bool" else t

        out[name] = {"ret": ret.replace("extern ", ""), "params": [k for k in map(kind, params.split(",")) if k]}
    return out


def header_prototypes():
    with open(os.path.join(ROOT, "include", "gometal_hip.h")) as f:
        return prototypes(f.read())


def main():
    with open("/root/reference/cgo_bridge/bridge.go") as f:
        src = f.read()
    preamble = src[src.index("/*") + 2:src.index('*/\nimport "C"')]
    ref = prototypes(preamble)
    mine = header_prototypes()
    shared = {name: ref[name] for name in sorted(mine) if name in ref}
    path = os.path.join(HERE, "reference_prototypes.json")
    with open(path, "w") as f:
        json.dump({"source": "cgo_bridge/bridge.go, cgo preamble", "prototypes": shared}, f, indent=1)
    print("wrote", path, len(shared), "prototypes;", len(mine) - len(shared), "functions of the header are additions")


if __name__ == "__main__":
    sys.exit(main())
