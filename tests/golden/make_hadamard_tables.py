"""Writes tests/golden/hadamard_tables.npz: the 12- and 40-point sign matrices the reference's
12N / 40N transforms are generated from (the `+`/`-` string literals ``had_12_paley`` and ``had_40_tpal``
of csrc/hadamard/code_gen.py, which its generator turns into hadamard_mult_thread_12 / _40).

The reference file is read as TEXT: the literals are cut out with a regular expression and turned into
+1 / -1 arrays; nothing from the reference is imported or executed.  Run in the build container only
(the reference tree does not travel): python tests/golden/make_hadamard_tables.py [reference root]
"""
import os
import re
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def table(text, name):
    m = re.search(r'^' + re.escape(name) + r'\s*=\s*"""(.*?)"""', text, re.S | re.M)
    if m is None:
        raise SystemExit(f"{name}: literal not found")
    rows = [r for r in m.group(1).split() if r]
    n = len(rows)
    if any(len(r) != n or set(r) - set("+-") for r in rows):
        raise SystemExit(f"{name}: not a square +/- table")
    return np.array([[1 if c == "+" else -1 for c in r] for r in rows], np.int8)


def main():
    root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    with open(os.path.join(root, "csrc", "hadamard", "code_gen.py"), encoding="utf-8") as f:
        text = f.read()
    h12, h40 = table(text, "had_12_paley"), table(text, "had_40_tpal")
    assert h12.shape == (12, 12) and h40.shape == (40, 40)
    np.savez_compressed(os.path.join(HERE, "hadamard_tables.npz"), had_12_paley=h12, had_40_tpal=h40)
    print("wrote hadamard_tables.npz", h12.shape, h40.shape)


if __name__ == "__main__":
    main()
