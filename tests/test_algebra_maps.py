"""The rearrangement that carries the other algebras onto the quaternion kernels (phx_algebra_map of the library,
the table its rearrangement kernels use), checked on the CPU against the reference's sign tables (through the
oracle, which restates src/algebras.cc:5-145 and is pinned entry by entry against the reference's own object
code): multiplying two multivectors blade by blade with the algebra's table must equal mapping both to their
quaternion-like halves, multiplying those with the quaternion table in the block form [[A, B], [-B, A]] (input half
x output half), and mapping back.  Host-only: the library is loaded, no GPU call is made."""
import numpy as np
import pytest

import oracle
from phoenix_core_amd import algebras, ops


def blade_terms(algebra):
    """The table's entries (left, right, positive) per output blade."""
    dims, entries, layout, _ = oracle.sign_table(algebra)
    assert dims == algebras.DIMS[algebra]
    return [entries[layout[k]:layout[k + 1]] for k in range(dims)]


def table_product(algebra, a, b):
    """Left-times-right product of two multivectors by the reference's table."""
    out = np.zeros(algebras.DIMS[algebra])
    for k, terms in enumerate(blade_terms(algebra)):
        for left, right, positive in terms:
            out[k] += (1.0 if positive else -1.0) * a[left] * b[right]
    return out


def halves_of(m, algebra):
    """Multivector [D] -> its quaternion-like halves [halves, 4] by the library's map."""
    dims, halves, blade, sign = algebras.blade_map(algebra)
    assert dims == algebras.DIMS[algebra] == len(m)
    return np.array([[sign[4 * h + p] * m[blade[4 * h + p]] if blade[4 * h + p] >= 0 else 0.0 for p in range(4)]
                     for h in range(halves)])


def from_halves(q, algebra):
    dims, halves, blade, sign = algebras.blade_map(algebra)
    out = np.full(dims, np.nan)
    for h in range(halves):
        for p in range(4):
            if blade[4 * h + p] >= 0:
                out[blade[4 * h + p]] = sign[4 * h + p] * q[h, p]
    assert not np.isnan(out).any()  # every blade has a seat
    return out


@pytest.mark.parametrize("algebra", [ops.REAL, ops.COMPLEX, ops.GA_300])
def test_composition_equals_the_algebra(algebra):
    r = np.random.default_rng(algebra)
    d = algebras.DIMS[algebra]
    for _ in range(20):
        a, b = r.standard_normal(d), r.standard_normal(d)
        want = table_product(algebra, a, b)
        xa, wb = halves_of(a, algebra), halves_of(b, algebra)
        halves = len(xa)
        # filter blocks, input half x output half: [[A, B], [-B, A]]
        block = (lambda i, o: wb[0]) if halves == 1 else (lambda i, o: wb[0] if i == o else (wb[1] if i == 0 else -wb[1]))
        y = np.zeros((halves, 4))
        for o in range(halves):
            for i in range(halves):
                y[o] += table_product(ops.QUATERNION, xa[i], block(i, o))
        np.testing.assert_allclose(from_halves(y, algebra), want, rtol=1e-12, atol=1e-12)
        # the embedded algebras stay inside their sub-algebra: components that are zero on the way in stay zero
        _, _, blade, _ = algebras.blade_map(algebra)
        for h in range(halves):
            for p in range(4):
                if blade[4 * h + p] < 0:
                    assert abs(y[h, p]) < 1e-12


def test_quaternion_map_is_the_identity():
    assert algebras.blade_map(ops.QUATERNION) == (4, 1, [0, 1, 2, 3, -1, -1, -1, -1], [1, 1, 1, 1, 0, 0, 0, 0])
