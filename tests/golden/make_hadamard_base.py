"""Writes tests/golden/hadamard_base.json: the rows of this library's 12 x 12, 20 x 20, 28 x 28 and
40 x 40 Hadamard base matrices as strings of '+' and '-' (row r, column c), as the oracle's
textbook constructions give them.

    python tests/golden/make_hadamard_base.py

The file freezes the matrices: weights that were rotated offline with this library stay loadable
only as long as the online rotation uses the very same matrices, so tests/test_hadamard_base_frozen.py
holds both the oracle (oracle/uniql_oracle.py::hadamard_base_matrix) and the kernels' tables
(uniql_amd/csrc/hadamard_base.hpp) to it.  Run this script again only to ADD a base; a diff in an
existing entry is a format break.
"""
import json
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import uniql_oracle as O  # noqa: E402


def main():
    out = {}
    for base in (12, 20, 28, 40):
        h = O.hadamard_base_matrix(base)
        out[str(base)] = ["".join("+" if v > 0 else "-" for v in row) for row in h]
    path = os.path.join(ROOT, "tests", "golden", "hadamard_base.json")
    with open(path, "w") as f:
        json.dump(out, f, indent=1)
    print("wrote", path)


if __name__ == "__main__":
    main()
