"""Holds oracle.hcsim to tests/golden/sim_golden.json: what the reference's own
simulator (python/hckernel/kernel_api.py:106-211,297-376) returned for the
bodies of tests/golden/sim_cases.py, written by tests/golden/make_sim_golden.py.

These are the behaviours that follow from numpy.ma internals and that no test
or document of the reference fixes: in-place operators on partially active
tiles, loads from tiles that are already masked, domain masking of / // % **,
NumPy functions and reductions applied to tiles, compressed() and repr, Python
and NumPy scalars next to a tile, every installed operator on int32, float32
and bool tiles, stores of numpy.ma results, and reductions (sum, max, min,
mean, var, std) over elements that a zero divisor deactivated, together with
arithmetic on the deactivated row and column scalars that come out of them.

Rule: wherever the reference returned a value, the oracle returns the same
bytes (dtype, shape, content).  Where the reference raised there is no result
to agree with; the oracle may define one, and the names where it does are
listed here, so a new divergence cannot slip in as an "extension".
"""

import os
import sys

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))

import sim_cases                                    # noqa: E402

import oracle.hcsim as hcsim                        # noqa: E402

GOLDEN = os.path.join(HERE, "golden", "sim_golden.json")

# The reference raises, the oracle returns a value:
#  * an operand that is not a tile on the left of an operator: the reference
#    installs no reflected methods (kernel_api.py:185-195), so `2 * tile`
#    is a TypeError there, and so is `numpy.float32(2) / tile` (every arithmetic
#    operator of a NumPy scalar; its comparisons are reflected by Python and
#    work); the oracle gives the commuted result.
#  * `int_tile ** 2`: numpy.ma returns its scalar "no mask", which the
#    reference's mask property cannot invert (kernel_api.py:93-103); the oracle
#    treats it as all active.
#  * len(tile): no __len__ on the reference's wrapper type.
ORACLE_DEFINES = ("_left_", "domain_masking/int_pow", "compressed_repr/len")


def _text(a):
    return bytes(a).decode(errors="replace")


@pytest.fixture(scope="module")
def golden():
    return sim_cases.load(GOLDEN)


def test_fixture_is_for_this_numpy(golden):
    # the recorded behaviours are numpy.ma's; a different NumPy means the
    # fixture has to be written again from the reference
    made_with = _text(golden["numpy_version"])
    assert made_with.split(".")[:2] == np.__version__.split(".")[:2], (made_with, np.__version__)


@pytest.mark.parametrize("case", sorted(sim_cases.CASES))
def test_oracle_equals_reference_simulator(golden, case):
    want = {k: v for k, v in golden.items() if k.startswith(case + "/")}
    got = {f"{case}/{k}": np.asarray(v) for k, v in sim_cases.CASES[case](hcsim).items()}
    assert want, "case missing from the fixture: run tests/golden/make_sim_golden.py"
    raised = [k[:-len(".raises")] for k in want if k.endswith(".raises")]
    for k, w in want.items():
        if k.endswith(".raises"):
            stem = k[:-len(".raises")]
            if k in got:
                # same exception family; the mask assertion is the reference's own
                assert _text(got[k]).split(":")[0] == _text(w).split(":")[0], k
            else:
                assert any(tag in k for tag in ORACLE_DEFINES), \
                    f"{stem}: the reference raises {_text(w)}, the oracle returns a value"
            continue
        assert k in got, f"{k}: the reference returns a value, the oracle does not"
        g = got[k]
        assert g.dtype == w.dtype and g.shape == w.shape, (k, g.dtype, w.dtype, g.shape, w.shape)
        assert g.tobytes() == w.tobytes(), (k, g.tolist(), w.tolist())
    for k in got:
        if k not in want:
            assert any(k.startswith(r) for r in raised) and any(t in k for t in ORACLE_DEFINES), \
                f"{k}: recorded by the oracle only"


def test_headline_behaviours(golden):
    """The pinned facts, spelled out (they read off the fixture, so a fixture
    that changes under a new NumPy shows here by name)."""
    g = golden
    # (i) an in-place operator never widens activity and only updates elements
    #     active on both sides
    assert g["inplace_partial/narrow_plus_wider.active"].tolist() == [1, 1, 1, 0, 0, 0, 0, 0]
    assert g["inplace_partial/partial_plus_narrower.value"].tolist() == [3, 2, 7, 4, 5, 0, 0, 0]
    # (ii) a load from a masked tile inherits its activity
    assert g["load_from_masked/vload_window.active"].sum() == 4
    # (iii) x / 0 is deactivated and the store leaves the destination alone
    assert g["domain_masking/dst"][0, 1] == sim_cases.POISON
    # (iv) np.dot sees inactive elements as zeros and returns a plain array
    assert _text(g["numpy_functions/np_dot.kind"]) == "ndarray"
    # (vi) a Python scalar promotes a float32 tile to float64 (numpy.ma wraps it
    #      in a 0-d float64 array), a NumPy scalar of the tile's type does not
    assert _text(g["scalar_promotion/f32.mul_pyfloat.dtype"]) == "float64"
    assert _text(g["scalar_promotion/f32.mul_npf32.dtype"]) == "float32"


def test_headline_behaviours_of_reductions_over_deactivated_elements(golden):
    """What numpy.ma does where elements or whole rows are deactivated (rows of the
    case: 1 has zero divisors only, 2 a negative divisor sum, 4 divisors that add
    up to zero, 5 an inf in the dividend)."""
    g = golden
    rows = g["masked_reductions/dst_rows"]
    names = ["mean", "sum", "max", "min", "var", "std1", "plain_mean", "plain_var", "plain_std", "sqrt_sum",
             "sum_ratio", "one_plus_ratio", "python_one_plus_ratio"]
    r = {n: rows[i] for i, n in enumerate(names)}
    # a per-row result is stored in full; a fold without active elements holds 0
    # (sum, and the mean and variance made of it) or numpy.ma's fill value 1e20
    assert r["sum"][1] == 0 and r["mean"][1] == 0 and r["var"][1] == 0
    assert r["max"][1] == np.float32(1e20) and r["min"][1] == np.float32(1e20)
    # the mean divides by the number of active elements: one of row 0's five divisors is zero
    assert r["mean"][0] * 4 == r["sum"][0]
    # a mean that is not finite is deactivated, the variance of that row is an active 0
    assert np.isinf(r["plain_mean"][5]) and r["plain_var"][5] == 0 and r["plain_std"][5] == 0
    # numpy.sqrt of a negative sum: deactivated, fill value 0
    assert r["sqrt_sum"][2] == 0
    # a deactivated quotient holds the dividend; a NumPy scalar's + computes on it
    # (1 + dividend), a Python scalar's leaves its own first operand (1)
    assert r["sum_ratio"][4] == -1.5 and r["one_plus_ratio"][4] == -0.5 and r["python_one_plus_ratio"][4] == 1.0
    # tiles computed from a deactivated row scalar are not stored
    tiles = g["masked_reductions/dst_tiles"]
    assert (tiles[0][[0, 1, 4, 5]] == sim_cases.POISON).all() and (tiles[0][[2, 3]] != sim_cases.POISON).all()
    # down columns: a column without an active quotient
    cols = g["masked_reductions/dst_cols"]
    assert cols[0][3] == 0 and cols[1][3] == np.float32(1e20)
