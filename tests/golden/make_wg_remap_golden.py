"""Writes tests/golden/wg_remap_460x64_wgm8.npy from the reference's golden file.

The reference keeps exactly one CPU-checkable fixture for this path: src/gemm/ref/res, the captured
output of src/gemm/ref/map.cpp (WorkGroupMapping = 8 on a 460 x 64 grid): 29,440 lines
"(wg0,wg1)--->(new0, new1) in original map".  This script parses that text into an int16 array of
rows (wg0, wg1, new0, new1).  It reads the file as data; it runs nothing from the reference.

    python tests/golden/make_wg_remap_golden.py [/root/reference]
"""
import os
import re
import sys

import numpy as np

ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
src = os.path.join(ref, "src", "gemm", "ref", "res")
pat = re.compile(r"\((\d+),\s*(\d+)\)--->\s*\((\d+),\s*(\d+)\) in original map")
rows = []
with open(src) as f:
    for line in f:
        m = pat.match(line.strip())
        if m:
            rows.append([int(x) for x in m.groups()])
a = np.array(rows, dtype=np.int16)
assert a.shape == (460 * 64, 4), a.shape
out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "wg_remap_460x64_wgm8.npy")
np.save(out, a)
print("wrote", out, a.shape)
