"""Writes tests/golden/had_digests.json: sha256 of every order-K Hadamard table of the reference
(lib/utils/matmul_had.py:129-95715), as row-major int8 bytes (+1 -> 0x01, -1 -> 0xFF).

The reference file is parsed as TEXT with `ast` (nothing is imported or executed): every
`get_had{N}` function's torch.FloatTensor([...]) literal is evaluated as a nested list.  This is
a different reader from the one that produced qtip_amd/utils/hadamard_tables.npz
(make_hadamard_tables.py scans for sign characters), so a slip in either shows as a digest
mismatch in tests/test_oracle.py.

  python tests/golden/make_had_digests.py [/root/reference]
"""
import ast
import hashlib
import json
import os
import re
import sys

import numpy as np

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
HERE = os.path.dirname(os.path.abspath(__file__))


def main():
    tree = ast.parse(open(os.path.join(REF, "lib", "utils", "matmul_had.py")).read())
    out = {}
    for node in tree.body:
        if not isinstance(node, ast.FunctionDef):
            continue
        m = re.fullmatch(r"get_had(\d+)", node.name)
        if not m:
            continue
        order = int(m.group(1))
        lists = [c.args[0] for c in ast.walk(node)
                 if isinstance(c, ast.Call) and c.args and isinstance(c.args[0], ast.List)]
        assert len(lists) == 1, (node.name, len(lists))
        h = np.array(ast.literal_eval(lists[0]), dtype=np.float64)
        assert h.shape == (order, order) and np.all(np.abs(h) == 1.0), node.name
        out[f"had{order}"] = {
            "order": order,
            "sha256": hashlib.sha256(h.astype(np.int8).tobytes()).hexdigest(),
            "row0": h[0].astype(int).tolist(),
            "col0_sum": int(h[:, 0].sum()),
            "symmetric": bool(np.array_equal(h, h.T)),
        }
    with open(os.path.join(HERE, "had_digests.json"), "w") as f:
        json.dump(out, f, indent=1, sort_keys=True)
    print({k: v["sha256"][:12] for k, v in out.items()})


if __name__ == "__main__":
    main()
