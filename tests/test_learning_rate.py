"""The learning-rate schedule (Util::get_learning_rate, src/util.h:76-93), both copies of it: the
oracle's C restatement and the C++ one the device updaters use (`cct_solver_learning_rate`, host
arithmetic, no GPU).  Each is pinned by evidence that is not the other:

  * float64 closed forms at parameters where a wrong exponent sign, swapped gamma/power, a float
    instead of an integer step count, or iter/max_iter inverted changes the value well beyond the
    tolerance;
  * identities of each schedule (ratio at a step boundary, geometric ratio, half height at the
    sigmoid's centre and its point symmetry, end points of poly, inv at power 1);
  * the learning rates Caffe prints while training LeNet with its stock solver
    (base_lr 0.01, lr_policy "inv", gamma 0.0001, power 0.75): the reference states that its
    schedule is Caffe's (src/util.h:72-75).
"""
import math

import numpy as np
import pytest

from caffecontroll_amd import nets
from caffecontroll_amd.bridges import solver_param

REL = 2e-6  # float32 rounding of a handful of operations


def _oracle(oracle):
    return lambda policy, base, gamma, it, step, power, max_iter: oracle.learning_rate(policy, base, gamma, it, step, power, max_iter)


def _host(_):
    def f(policy, base, gamma, it, step, power, max_iter):
        sp = solver_param(base_lr=base, lr_policy=policy, gamma=gamma, stepsize=int(step), power=power, max_iter=int(max_iter))
        return nets.solver_learning_rate(sp, int(it))
    return f


IMPLS = {"oracle": _oracle, "host": _host}


@pytest.fixture(params=sorted(IMPLS))
def lr(request, oracle):
    return IMPLS[request.param](oracle)


def closed_form(policy, base, gamma, it, step, power, max_iter):
    base, gamma, power = float(np.float32(base)), float(np.float32(gamma)), float(np.float32(power))
    if policy == "fixed":
        return base
    if policy == "step":
        return base * gamma ** (it // step)
    if policy == "exp":
        return base * gamma ** it
    if policy == "inv":
        return base / (1.0 + gamma * it) ** power
    if policy == "poly":
        return base * (1.0 - it / max_iter) ** power
    if policy == "sigmoid":
        return base / (1.0 + math.exp(-gamma * (it - step)))
    raise AssertionError(policy)


# (policy, base_lr, gamma, stepsize, power, max_iter): gamma != power, gamma != 1/gamma, step > 1
CASES = [
    ("fixed", 0.05, 0.3, 7, 2.0, 50),
    ("step", 0.01, 0.1, 100, 0.75, 1000),
    ("step", 0.2, 0.5, 7, 3.0, 50),
    ("exp", 0.01, 0.999, 100, 0.75, 1000),
    ("exp", 0.5, 0.9, 7, 3.0, 50),
    ("inv", 0.01, 0.0001, 100, 0.75, 1000),
    ("inv", 0.3, 0.05, 7, 2.0, 50),
    ("poly", 0.01, 0.1, 100, 0.5, 1000),
    ("poly", 0.3, 0.05, 7, 2.0, 450),
    ("sigmoid", 0.01, -0.05, 100, 0.75, 1000),
    ("sigmoid", 0.3, 0.25, 7, 2.0, 50),
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "%s-%g-%g" % (c[0], c[1], c[2]))
def test_closed_forms(lr, case):
    policy, base, gamma, step, power, max_iter = case
    its = sorted({0, 1, 2, step - 1, step, step + 1, 2 * step - 1, 2 * step, 2 * step + 1, 3 * step + 2, 40, 399})
    for it in its:
        if policy == "poly" and it > max_iter:
            continue
        got = lr(policy, base, gamma, it, step, power, max_iter)
        want = closed_form(policy, base, gamma, it, step, power, max_iter)
        assert got == pytest.approx(want, rel=REL, abs=1e-12), (policy, it, got, want)


def test_step_is_piecewise_constant_with_ratio_gamma(lr):
    base, gamma, step = 0.01, 0.1, 100
    f = lambda it: lr("step", base, gamma, it, step, 0.0, 0)
    assert f(0) == f(1) == f(step - 1) == np.float32(base)           # integer division, not a real quotient
    assert f(step) == f(step + 1) == f(2 * step - 1)
    assert f(step) == pytest.approx(base * gamma, rel=REL)
    assert f(2 * step + 1) == pytest.approx(base * gamma * gamma, rel=REL)
    assert f(step) < f(step - 1) and f(2 * step) < f(step)            # decays for gamma < 1


def test_exp_is_geometric(lr):
    f = lambda it: lr("exp", 0.5, 0.9, it, 7, 3.0, 50)
    assert f(0) == np.float32(0.5)
    for it in (0, 1, 5, 20):
        assert f(it + 1) / f(it) == pytest.approx(0.9, rel=REL)


def test_inv_known_values_and_limits(lr):
    # Caffe's LeNet solver: base_lr 0.01, gamma 0.0001, power 0.75.  The tutorial's training log
    # prints "Iteration 100, lr = 0.00992565", "Iteration 200, lr = 0.00985258", ... (6 digits).
    f = lambda it: lr("inv", 0.01, 0.0001, it, 0, 0.75, 0)
    for it, printed in ((100, 0.00992565), (200, 0.00985258), (300, 0.00978075), (400, 0.00971013),
                        (500, 0.00964069), (5000, 0.00737788), (9900, 0.00596843)):
        assert "%.6g" % f(it) == "%.6g" % printed, (it, f(it), printed)
    assert f(0) == np.float32(0.01)
    # power 1, gamma 1: base / (1 + iter) exactly representable cases
    g = lambda it: lr("inv", 1.0, 1.0, it, 0, 1.0, 0)
    assert g(1) == 0.5 and g(3) == 0.25 and g(7) == 0.125
    # swapping gamma and power would give (1 + 0.75 it)^-0.0001: far from this
    assert f(1000) < 0.0094


def test_poly_end_points_and_linear_case(lr):
    f = lambda it, power=2.0: lr("poly", 0.3, 0.05, it, 7, power, 400)
    assert f(0) == np.float32(0.3)
    assert f(400) == 0.0
    assert f(100, 1.0) == pytest.approx(0.3 * 0.75, rel=REL)          # power 1: a straight line
    assert f(100) == pytest.approx(0.3 * 0.75 ** 2, rel=REL)
    assert f(300) < f(100)


def test_sigmoid_centre_and_symmetry(lr):
    base, gamma, step = 0.3, 0.25, 40
    f = lambda it: lr("sigmoid", base, gamma, it, step, 0.0, 0)
    assert f(step) == pytest.approx(base / 2, rel=REL)
    for d in (1, 3, 10):
        assert f(step + d) + f(step - d) == pytest.approx(base, rel=2 * REL)
    assert f(step + 10) > f(step) > f(step - 10)                      # positive gamma rises with iter
    h = lambda it: lr("sigmoid", base, -gamma, it, step, 0.0, 0)
    assert h(step + 10) < h(step) < h(step - 10)                      # the usual decaying use


def test_rejected_policies(oracle):
    assert math.isnan(oracle.learning_rate("multistep", 0.01, 0.1, 1, 10, 0, 0))
    for policy in ("multistep", "nope"):
        sp = solver_param(lr_policy=policy)
        assert math.isnan(nets.solver_learning_rate(sp, 3))


def test_oracle_and_host_agree_bit_for_bit(oracle):
    """Same float/double steps in both copies: identical float results, so the stepped-SGD parity
    test on the device can demand equality."""
    for policy, base, gamma, step, power, max_iter in CASES:
        sp = solver_param(base_lr=base, lr_policy=policy, gamma=gamma, stepsize=step, power=power, max_iter=max_iter)
        for it in range(0, 3 * step + 3):
            if policy == "poly" and it > max_iter:
                break
            a = oracle.learning_rate(policy, base, gamma, it, step, power, max_iter)
            b = nets.solver_learning_rate(sp, it)
            assert np.float32(a).tobytes() == np.float32(b).tobytes(), (policy, it, a, b)
