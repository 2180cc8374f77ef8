"""The base matrices of the 12N / 20N / 28N / 40N transforms are frozen by a fixture: the oracle's
constructions and the bit masks the kernels read must both equal tests/golden/hadamard_base.json
(written by tests/golden/make_hadamard_base.py).  Their equality with the reference's tables is
NOT claimed (those are not in the reference's tree: parity unpinned); what is pinned is that this
library's own matrices never change under a model that was rotated with them."""
import json
import os
import re
import warnings

import numpy as np
import pytest

from oracle import uniql_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def frozen():
    with open(os.path.join(ROOT, "tests", "golden", "hadamard_base.json")) as f:
        raw = json.load(f)
    return {int(k): np.array([[1 if ch == "+" else -1 for ch in row] for row in rows], dtype=np.int64)
            for k, rows in raw.items()}


def kernel_tables():
    """base -> list of 64-bit masks from csrc/hadamard_base.hpp: word c has bit r set where H[r][c] is -1."""
    text = open(os.path.join(ROOT, "uniql_amd", "csrc", "hadamard_base.hpp")).read()
    tables = {}
    for base, body in re.findall(r"kHadamard(\d+)\[\d+\]\s*=\s*\{([^}]*)\}", text):
        tables[int(base)] = [int(v, 16) for v in re.findall(r"0x([0-9a-fA-F]+)ull", body)]
    return tables


@pytest.mark.parametrize("base", [12, 20, 28, 40])
def test_fixture_is_a_hadamard_matrix(frozen, base):
    h = frozen[base]
    assert h.shape == (base, base)
    assert np.array_equal(h @ h.T, base * np.eye(base, dtype=np.int64))


@pytest.mark.parametrize("base", [12, 20, 28, 40])
def test_oracle_matrix_is_frozen(frozen, base):
    assert np.array_equal(O.hadamard_base_matrix(base), frozen[base])


@pytest.mark.parametrize("base", [12, 20, 28, 40])
def test_kernel_table_is_frozen(frozen, base):
    masks = kernel_tables()[base]
    assert len(masks) == base
    h = np.array([[-1 if (masks[c] >> r) & 1 else 1 for c in range(base)] for r in range(base)], dtype=np.int64)
    assert np.array_equal(h, frozen[base])


def test_first_use_warns_and_can_be_refused(monkeypatch):
    """The composite variants announce that their matrices are this library's own: once per base,
    silenced or turned into a refusal by UNIQL_AMD_COMPOSITE_HADAMARD (no GPU: only the notice runs)."""
    from uniql_amd import ops
    monkeypatch.setattr(ops, "_composite_warned", set())
    monkeypatch.delenv("UNIQL_AMD_COMPOSITE_HADAMARD", raising=False)
    with pytest.warns(ops.UnpinnedHadamardWarning, match="28 x 28"):
        ops._composite_notice(28)
    with warnings.catch_warnings():
        warnings.simplefilter("error")
        ops._composite_notice(28)          # second use of the same base: silent
        monkeypatch.setenv("UNIQL_AMD_COMPOSITE_HADAMARD", "quiet")
        ops._composite_notice(12)          # silenced
    monkeypatch.setenv("UNIQL_AMD_COMPOSITE_HADAMARD", "error")
    with pytest.raises(NotImplementedError):
        ops._composite_notice(20)
