"""Writes tests/golden/reference_arch_tiles.json: the (types, M0, N0, K0) entries
of the reference's tables of architecture-specific mmt4d tile functions
(arch/x86_64/mmt4d_x86_64_tiles.inl, arch/arm_64/mmt4d_arm_64_tiles.inl), i.e.
the tile shapes a compiler targeting those CPUs hands to the microkernel.
Run in a container that has the reference tree: python tests/golden/make_tile_list.py
"""
import json
import os
import re

HERE = os.path.dirname(os.path.abspath(__file__))
UK = "/root/reference/runtime/src/iree/builtins/ukernel"
FILES = ["arch/x86_64/mmt4d_x86_64_tiles.inl", "arch/arm_64/mmt4d_arm_64_tiles.inl"]

entries = set()
for rel in FILES:
    for line in open(os.path.join(UK, rel)):
        m = re.match(r"\s*IREE_UK_MMT4D_TILE\(\s*(\w+)\s*,\s*(\w+)\s*,\s*(\w+)\s*,\s*(\w+)\s*,\s*(\d+)\s*,\s*(\d+)\s*,\s*(\d+)\s*,", line)
        if m:
            arch, lhs, rhs, out, m0, n0, k0 = m.groups()
            entries.add((arch, lhs + rhs + out, int(m0), int(n0), int(k0)))
rows = [{"arch": a, "type": t, "M0": m0, "N0": n0, "K0": k0} for (a, t, m0, n0, k0) in sorted(entries)]
with open(os.path.join(HERE, "reference_arch_tiles.json"), "w") as f:
    json.dump({"source": FILES, "tiles": rows}, f, indent=0)
print(len(rows), "tile shapes")
