"""Writes tests/golden/ref_config_entries.json: a handful of entries of the two tuning tables the reference
ships (configs/moe_jit_257_256_7168.json, configs/moe_jit_512_256_2048.json) plus lookups worked out by hand
from the nearest-key rule of alpha_moe_python/utils.py:19-29.  Data only; run once in the build container:
    python tests/golden/make_config_fixture.py /root/reference
"""
import json
import os
import sys

ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
keep = ["1", "7", "8", "16", "64", "512", "2048", "4096", "8192"]
out = {}
for name in ("moe_jit_257_256_7168.json", "moe_jit_512_256_2048.json"):
    with open(os.path.join(ref, "configs", name)) as fh:
        table = json.load(fh)
    out[name] = {"n_keys": len(table), "first_keys": list(table)[:12], "entries": {k: table[k] for k in keep}}
with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "ref_config_entries.json"), "w") as fh:
    json.dump(out, fh, indent=1)
