"""Pins the oracle's iRPROP- (Neural_Network__iRPROP_minus.cpp:21-67; Igel & Huesken 2000, the variant without weight
backtracking) by what the published rule fixes: a slope that keeps its sign grows the step geometrically up to the cap and
moves the weight against the slope by that step; a sign change shrinks the step down to the floor, takes no step and
forgets the slope, so the update after it moves by the shrunk step without growing it; a zero slope moves nothing.
A five-update trace is counted by hand."""
import ctypes as C

import numpy as np

from myea_amd import binding as mb
from tests.common import oracle_hyper
from tests.oracle_lib import load_oracle


def _update(h, w, g, steps, slopes):
    lib = load_oracle()
    arrays = [np.ascontiguousarray(a, dtype=np.float32) for a in (w, g, steps, slopes)]
    lib.myea_oracle_irprop_minus(C.byref(h), len(arrays[0]), *(C.c_void_p(a.ctypes.data) for a in arrays))
    return arrays


def test_constant_sign_grows_the_step_geometrically_up_to_the_cap():
    h = oracle_hyper(rprop_increase_factor=1.5, rprop_delta_max=2.0)
    w, steps, slopes = np.zeros(2, np.float32), np.full(2, 0.1, np.float32), np.zeros(2, np.float32)
    moved = []
    for k in range(10):
        before = w.copy()
        w, g, steps, slopes = _update(h, w, np.array([0.3, -7.0], np.float32), steps, slopes)
        assert not g.any()                                   # the gradient is consumed
        moved.append(w - before)
        want = min(0.1 * 1.5 ** k, 2.0)                      # the first update has no earlier slope: the step as it is
        np.testing.assert_allclose(steps, [want, want], rtol=1e-6)
        np.testing.assert_allclose(moved[-1], [-want, want], rtol=1e-6)   # against the slope, whatever its size


def test_hand_trace_with_a_sign_change():
    h = oracle_hyper(rprop_increase_factor=1.2, rprop_decrease_factor=0.5, rprop_delta_min=1e-6, rprop_delta_max=50.0)
    w, steps, slopes = np.array([1.0], np.float32), np.array([0.1], np.float32), np.array([0.0], np.float32)
    trace = []
    for grad in (2.0, 3.0, -1.0, -1.0, -4.0):
        w, _, steps, slopes = _update(h, w, np.array([grad], np.float32), steps, slopes)
        trace.append((float(w[0]), float(steps[0]), float(slopes[0])))
    want = [(0.9, 0.1, 2.0),        # no earlier slope: step 0.1 against the slope
            (0.78, 0.12, 3.0),      # same sign: 0.1 * 1.2
            (0.78, 0.06, 0.0),      # sign change: step halved, no move, slope forgotten
            (0.84, 0.06, -1.0),     # forgotten slope: the halved step as it is, upwards
            (0.912, 0.072, -4.0)]   # same sign again: 0.06 * 1.2
    np.testing.assert_allclose(np.array(trace), np.array(want), rtol=2e-6, atol=1e-7)


def test_floor_and_zero_slope():
    h = oracle_hyper(rprop_decrease_factor=0.5, rprop_delta_min=0.04)
    w, _, steps, slopes = _update(h, np.array([0.5, 0.5], np.float32), np.array([-1.0, 0.0], np.float32), np.array([0.05, 0.05], np.float32), np.array([1.0, 1.0], np.float32))
    np.testing.assert_allclose(steps, [0.04, 0.05], rtol=1e-6)     # 0.025 floored at 0.04; a zero slope leaves the step
    np.testing.assert_allclose(w, [0.5, 0.5])                       # neither moves: forgotten slope, zero slope
    np.testing.assert_allclose(slopes, [0.0, 0.0])
