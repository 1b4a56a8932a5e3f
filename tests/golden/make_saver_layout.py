#!/usr/bin/env python3
"""Writes tests/golden/saver_layout.json: what the reference's own MmapSaver (trak/savers.py) leaves
on disk, and reports on reopening, after the call sequence of saver_scenario.py, in float32 and in
float16.  Run once, in the container that has the reference checked out at /root/reference:
    python tests/golden/make_saver_layout.py
Only the snapshot is committed; the reference itself never travels."""
import json
import os
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
sys.path.insert(0, os.environ.get("TRAK_REFERENCE", "/root/reference"))

import saver_scenario  # noqa: E402
from trak.savers import MmapSaver  # noqa: E402

result = {}
for half in (False, True):
    with tempfile.TemporaryDirectory() as d:
        reopened = saver_scenario.run(MmapSaver, d, use_half_precision=half)
        result["float16" if half else "float32"] = {"files": saver_scenario.snapshot(d), "reopened": reopened}
path = os.path.join(HERE, "saver_layout.json")
with open(path, "w") as f:
    json.dump(result, f, indent=1, sort_keys=True)
print("wrote", path, os.path.getsize(path), "bytes")
