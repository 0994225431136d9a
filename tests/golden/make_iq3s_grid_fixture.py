"""Writes tests/golden/iq3s_grid_check.json: checksums of the IQ3_S codebook grid as the
reference states it (the IQ3S_GRID table of src/quant/iq3_s.rs, ggml's iq3s_grid), read from
the reference's source text.  The product and the oracle each hold the grid in their own
packed form; the tests expand both and compare against these figures.

Run in the build container (the reference tree is not present elsewhere):
    python tests/golden/make_iq3s_grid_fixture.py [/root/reference]
"""
import json
import os
import re
import sys
import zlib

import numpy as np


def read_grid(ref_root):
    text = open(os.path.join(ref_root, "src", "quant", "iq3_s.rs")).read()
    body = text[text.index("pub const IQ3S_GRID"):]
    body = body[body.index("= [") + 3:body.index("];")]
    vals = [int(v, 16) for v in re.findall(r"0x([0-9a-fA-F]{8})", body)]
    return np.array(vals, dtype="<u4")


if __name__ == "__main__":
    grid = read_grid(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
    by = grid.view(np.uint8)
    out = {
        "source": "src/quant/iq3_s.rs IQ3S_GRID (512 little-endian u32, four bytes in 1..15 each)",
        "count": int(grid.size),
        "crc32_le_bytes": zlib.crc32(grid.tobytes()),
        "sum": int(grid.astype(np.uint64).sum()),
        "xor": int(np.bitwise_xor.reduce(grid)),
        "byte_histogram": {str(v): int((by == v).sum()) for v in range(1, 16, 2)},
        "strictly_increasing": bool(np.all(np.diff(grid.astype(np.int64)) > 0)),
        "entries_at": {str(i): int(grid[i]) for i in (0, 1, 255, 256, 511)},
    }
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "iq3s_grid_check.json")
    with open(dst, "w") as f:
        json.dump(out, f, indent=1)
        f.write("\n")
    print(out)
