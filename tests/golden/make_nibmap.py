"""Writes tests/golden/nibmap_4bit.json from the reference's NIBMAP data table.

The table (engine-rs/src/nibmap.rs:3-20) is a golden data vector the reference holds for the 4-bit tile
layout: for tile cell (row, col) the four nibble positions (little-endian slot order) of its 16-bit
trellis state.  Only the numbers are read; the file is parsed as text, nothing is imported or executed.
Run here (the reference checkout is not present on the GPU box): python tests/golden/make_nibmap.py
"""
import json, re, sys
from pathlib import Path

src = Path(sys.argv[1] if len(sys.argv) > 1 else "/root/reference/engine-rs/src/nibmap.rs").read_text()
body = src[src.index("= [") + 2:]
nums = [int(t) for t in re.findall(r"\d+", body)]
assert len(nums) == 16 * 16 * 4, len(nums)
table = [[[nums[(r * 16 + c) * 4 + s] for s in range(4)] for c in range(16)] for r in range(16)]
out = Path(__file__).with_name("nibmap_4bit.json")
out.write_text(json.dumps({"source": "engine-rs/src/nibmap.rs:3-20", "shape": [16, 16, 4], "nibmap": table}))
print("wrote", out)
