"""Pins the oracle's lowering / lifting / remap against evidence that does not come from the
oracle itself: the hand-checked matrices of the reference's lowering note, a brute-force
restatement of the definition, and the adjoint identity between lowering and lifting."""
import importlib.util
import os

import numpy as np
import pytest

from conftest import ROOT

_spec = importlib.util.spec_from_file_location(
    "lowering_tex_examples", os.path.join(ROOT, "tests", "golden", "lowering_tex_examples.py"))
_tex = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(_tex)


def brute_lower(x, k, s, p):
    """Definition: row (bi,r,c) is vec over (dd,kr,kc) of the padded window (tex eq. 4)."""
    b, d, n, _ = x.shape
    m = (n + 2 * p - k) // s + 1
    xp = np.zeros((b, d, n + 2 * p, n + 2 * p), x.dtype)
    xp[:, :, p:p + n, p:p + n] = x
    out = np.zeros((b * m * m, d * k * k), x.dtype)
    for bi in range(b):
        for r in range(m):
            for c in range(m):
                out[(bi * m + r) * m + c] = xp[bi, :, r * s:r * s + k, c * s:c * s + k].reshape(-1)
    return out


def brute_lift(y, b, d, n, k, s, p):
    """Definition of the adjoint: scatter-add every lowered entry back to its source pixel.
    y is [k*k*d][b*m*m]."""
    m = (n + 2 * p - k) // s + 1
    y = y.reshape(d, k, k, b, m, m).astype(np.float64)
    out = np.zeros((b, d, n + 2 * p + k, n + 2 * p + k), np.float64)
    for kr in range(k):
        for kc in range(k):
            for r in range(m):
                for c in range(m):
                    out[:, :, r * s + kr, c * s + kc] += y[:, kr, kc, :, r, c].T
    return out[:, :, p:p + n, p:p + n]


@pytest.mark.parametrize("idx", range(len(_tex.EXAMPLES)))
def test_tex_known_answers(oracle, idx):
    n, k, p, s, D, expect = _tex.EXAMPLES[idx]
    got = oracle.lower_cube(D.reshape(1, 1, n, n), k, s, p)
    np.testing.assert_array_equal(got, expect)


SHAPES = [  # b d n k s p
    (2, 3, 7, 3, 1, 0), (2, 3, 7, 3, 2, 1), (1, 8, 9, 5, 1, 2), (3, 16, 6, 3, 1, 1),
    (2, 9, 11, 5, 4, 2), (1, 1, 28, 5, 1, 0), (2, 3, 23, 11, 4, 0), (1, 10, 8, 3, 3, 2),
    (1, 2, 5, 5, 1, 0), (2, 1, 4, 1, 1, 0),
]


@pytest.mark.parametrize("shape", SHAPES)
def test_lower_matches_definition(oracle, shape):
    b, d, n, k, s, p = shape
    rng = np.random.default_rng(hash(shape) % 2**31)
    x = rng.standard_normal((b, d, n, n)).astype(np.float32)
    np.testing.assert_array_equal(oracle.lower_cube(x, k, s, p), brute_lower(x, k, s, p))


@pytest.mark.parametrize("shape", SHAPES)
def test_lift_matches_definition_and_adjoint(oracle, shape):
    b, d, n, k, s, p = shape
    m = (n + 2 * p - k) // s + 1
    rng = np.random.default_rng(hash(shape) % 2**31 + 1)
    # small integers: every fp32 sum is exact, so equality is bit-level
    y = rng.integers(-4, 5, size=(k * k * d, b * m * m)).astype(np.float32)
    got = oracle.inverse_lower_cube(y, b, d, n, k, s, p)
    np.testing.assert_array_equal(got, brute_lift(y, b, d, n, k, s, p).astype(np.float32))
    # <lower(x), y^T> == <x, lift(y)> with integer tensors (exact)
    x = rng.integers(-3, 4, size=(b, d, n, n)).astype(np.float32)
    lhs = np.sum(oracle.lower_cube(x, k, s, p).astype(np.float64) * y.T)
    rhs = np.sum(x.astype(np.float64) * got)
    assert lhs == rhs


def test_lift_accumulation_order(oracle):
    """The addends of one pixel arrive in (kr ascending, kc ascending) order; with values whose
    fp32 sum depends on the order, any other order gives a different bit pattern."""
    b, d, n, k, s, p = 1, 1, 3, 3, 1, 1
    m = 3
    y = np.zeros((k * k, m * m), np.float32)
    # centre pixel (1,1) receives entry (kr,kc) from output position (r,c) = (2-kr, 2-kc)
    vals = np.array([1e8, 1.0, -1e8, 3.0, 1e-3, 7.0, 2.5e7, -2.5e7, 0.125], np.float32)
    for kr in range(k):
        for kc in range(k):
            y[kr * k + kc, (2 - kr) * m + (2 - kc)] = vals[kr * k + kc]
    got = oracle.inverse_lower_cube(y, b, d, n, k, s, p)[0, 0, 1, 1]
    acc = np.float32(0)
    for v in vals:
        acc = np.float32(acc + v)
    assert got == acc
    rev = np.float32(0)
    for v in vals[::-1]:
        rev = np.float32(rev + v)
    assert rev != acc  # the probe really is order sensitive


def test_remap_closed_form(oracle):
    rng = np.random.default_rng(5)
    for (R, Cc, depth, batch) in [(3, 3, 4, 2), (5, 5, 10, 4), (1, 1, 7, 3), (2, 3, 1, 5)]:
        x = rng.standard_normal((depth * batch, R, Cc)).astype(np.float32)
        got = oracle.remap(x, R, Cc, depth, batch)
        # forward use: source is [depth][batch] slices -> destination [batch][depth]
        expect = x.reshape(depth, batch, R, Cc).transpose(1, 0, 2, 3).reshape(depth * batch, R, Cc)
        np.testing.assert_array_equal(got, expect)
        # applying it with the roles swapped is the inverse permutation
        back = oracle.remap(got, R, Cc, batch, depth)
        np.testing.assert_array_equal(back, x)
