"""Writes reference_api_signatures.json: side, return type, name and parameter types of every
function that the reference's public header (library/include/roc_shmem.hpp) declares.  The header
is read as text; nothing of the reference is compiled or run.
Usage: python tests/golden/make_api_signatures.py [reference root]"""
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
from api_names import declarations_of  # noqa: E402

root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
decls = declarations_of([os.path.join(root, "library", "include", "roc_shmem.hpp")])
with open(os.path.join(HERE, "reference_api_signatures.json"), "w") as f:
    f.write('{"source": "library/include/roc_shmem.hpp", "declarations": [\n')
    f.write(",\n".join(json.dumps([side, ret, name, list(params)]) for side, ret, name, params in decls))
    f.write("\n]}\n")
print("%d declarations" % len(decls))
