"""Writes reference_api_names.json: the names of the functions that the reference's public header
(library/include/roc_shmem.hpp) declares, per side.  The header is read as text; nothing of the
reference is compiled or run.  Usage: python tests/golden/make_api_names.py [reference root]"""
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
from api_names import names_of  # noqa: E402

root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
host, device = names_of([os.path.join(root, "library", "include", "roc_shmem.hpp")])
with open(os.path.join(HERE, "reference_api_names.json"), "w") as f:
    json.dump({"source": "library/include/roc_shmem.hpp", "host": host, "device": device}, f, indent=0)
    f.write("\n")
print("host %d, device %d" % (len(host), len(device)))
