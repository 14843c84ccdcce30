"""Build step: write hadamard_tables.npz (packed sign bits of the order-K tables).

The layer transform is (H_K (x) H_{n/K}) with H_K one of twelve fixed
Hadamard matrices (orders 12 ... 172, from N. Sloane's public library) that
the reference keeps as number literals in lib/utils/matmul_had.py:129-95715.
A quantised checkpoint only decodes correctly with exactly those matrices, so
they are data of the format.  This script reads that file as TEXT (it is not
imported or executed), extracts the +1/-1 literals of every `get_hadN`
function and stores them as packed bits (bit set = -1), 15 KB in total.

Run once in a container that has the reference checkout:
    python tests/golden/make_hadamard_tables.py [/root/reference]
The .npz it writes (qtip_amd/utils/hadamard_tables.npz) is committed; nothing reads the reference
at run time.  tests/golden/had_digests.json (make_had_digests.py, an independent parse of the same
literals) pins its contents.
"""
import os
import re
import sys

import numpy as np

ORDERS = (12, 20, 28, 36, 52, 60, 108, 116, 124, 140, 156, 172)


def parse(text):
    tables = {}
    starts = [(m.start(), int(m.group(1))) for m in re.finditer(r"^def get_had(\d+)\(\):", text, re.M)]
    starts.sort()
    for idx, (pos, order) in enumerate(starts):
        end = starts[idx + 1][0] if idx + 1 < len(starts) else len(text)
        body = text[pos:end]
        body = body[body.index("FloatTensor"):]
        vals = re.findall(r"[+-]\s*1\b", body)
        arr = np.array([1 if v[0] == "+" else -1 for v in vals], dtype=np.int64)
        if arr.size != order * order:
            raise SystemExit(f"had{order}: found {arr.size} entries, want {order * order}")
        h = arr.reshape(order, order)
        if not np.array_equal(h @ h.T, order * np.eye(order, dtype=np.int64)):
            raise SystemExit(f"had{order}: H H^T != K I")
        tables[order] = h
    return tables


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    with open(os.path.join(ref, "lib", "utils", "matmul_had.py")) as f:
        tables = parse(f.read())
    missing = [o for o in ORDERS if o not in tables]
    if missing:
        raise SystemExit(f"missing orders {missing}")
    out = {f"had{o}": np.packbits((tables[o] < 0).astype(np.uint8).reshape(-1)) for o in ORDERS}
    root = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    dst = os.path.join(root, "qtip_amd", "utils", "hadamard_tables.npz")
    np.savez(dst, **out)
    print("wrote", dst, {k: v.size for k, v in out.items()})


if __name__ == "__main__":
    main()
