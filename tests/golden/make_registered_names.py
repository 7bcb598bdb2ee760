"""Writes tests/golden/registered_names.json: the operator names and, per class, the method names
that the reference registers in its TORCH_LIBRARY(recis) block (csrc/bind.cc:46-211), read from the
text of that file. Run in the container that holds /root/reference:

    python tests/golden/make_registered_names.py
"""
import json
import os
import re

SRC = "/root/reference/csrc/bind.cc"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "registered_names.json")


def main():
    text = open(SRC).read()
    text = text[text.index("TORCH_LIBRARY(recis"):]
    ops, classes, attributes = [], {}, {}
    current = None
    for stmt in text.split(";"):
        m = re.search(r'm\.class_<[^>]*>\(\s*"([^"]+)"\s*\)', stmt)
        if m:
            current = m.group(1)
            classes[current] = re.findall(r'\.def(?:_static)?\(\s*"([^"]+)"', stmt)
            for attr in re.findall(r'\.def_readonly\(\s*"([^"]+)"', stmt):
                attributes.setdefault(current, []).append(attr)
            continue
        m = re.search(r'm\.def\(\s*"([^"]+)"', stmt)
        if m:
            ops.append(m.group(1))
    with open(OUT, "w") as f:
        json.dump({"source": "csrc/bind.cc", "ops": sorted(ops), "classes": {k: sorted(v) for k, v in sorted(classes.items())},
                   "readonly_attributes": attributes},
                  f, indent=1)
    print("wrote %s: %d ops, %d classes" % (OUT, len(ops), len(classes)))


if __name__ == "__main__":
    main()
