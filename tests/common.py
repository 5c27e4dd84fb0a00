"""Shared builders for the parity tests: seeded synthetic nets and data in the reference's layouts."""
import ctypes as C
import os
from contextlib import contextmanager

import numpy as np

from myea_amd import binding as mb
from myea_amd.synthetic import glorot_parameters, one_hot   # noqa: F401 (re-exported for the tests)
from tests.oracle_lib import load_oracle


@contextmanager
def environment(**kw):
    """environment variables for the library's switches, restored afterwards"""
    old = {k: os.environ.get(k) for k in kw}
    os.environ.update({k: str(v) for k, v in kw.items()})
    try:
        yield
    finally:
        for k, v in old.items():
            if v is None:
                del os.environ[k]
            else:
                os.environ[k] = v


def oracle_desc(layers, batch_size, recurrent_depth=1):
    """make_desc through the oracle build of the layout code (no HIP library needed on CPU)."""
    return mb.make_desc(layers, batch_size, recurrent_depth, lib=load_oracle())


def oracle_hyper(**kw):
    return mb.default_hyper(lib=load_oracle(), **kw)


def run_step(net, B, X, Y, training_size=None, update=True):
    """the 4-call loop of Dataset::Train_Batch_BP (Neural_Network/Dataset.cpp:645-658) + Update_Parameter"""
    net.Forward_Pass(B, X)
    net.Compute__Error(B, Y)
    net.Backward_Pass(B)
    net.Update_Derivative_Weight(B, 1, net.desc.n_layers)
    if update:
        net.Update_Parameter(B, training_size or B)


def assert_close(a, b, rel=1e-4, abs_=1e-5, what=""):
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    assert a.shape == b.shape, (what, a.shape, b.shape)
    err = np.abs(a - b)
    tol = abs_ + rel * np.abs(b)
    bad = err > tol
    if bad.any():
        i = int(np.argmax(err - tol))
        raise AssertionError("%s: %d / %d out of tolerance; worst at %d: got %.9g want %.9g (err %.3g, tol %.3g)"
                             % (what, int(bad.sum()), a.size, i, a.flat[i], b.flat[i], err.flat[i], tol.flat[i]))


def assert_close_or_nearer_truth(got, oracle, truth, rel=1e-4, abs_=1e-5, what="", require_nearer=True):
    """Elementwise: `got` is within tolerance of the fp32 oracle, or - where the oracle's own fp32 rounding is the
    larger error - at least as near to the float64 `truth` as the oracle is.  At most 0.1 % of the entries (3 for
    small vectors) may need the second clause, and none may be farther than the tolerance from the truth.
    require_nearer=False keeps only "within tolerance of the truth" for those entries: for tiny-batch normalisation,
    where both fp32 results scatter around the truth by about the tolerance."""
    got, oracle, truth = (np.asarray(x, dtype=np.float64) for x in (got, oracle, truth))
    tol = abs_ + rel * np.abs(oracle)
    off = np.abs(got - oracle) > tol
    if not off.any():
        return
    assert off.sum() <= max(3, 1e-3 * got.size), "%s: %d / %d entries differ from the oracle" % (what, int(off.sum()), got.size)
    nearer = np.abs(got - truth) <= np.abs(oracle - truth)
    inside = np.abs(got - truth) <= abs_ + rel * np.abs(truth)
    bad = off & ~(inside & (nearer | (not require_nearer)))
    if bad.any():
        i = int(np.argmax(bad))
        raise AssertionError("%s: entry %d got %.9g oracle %.9g float64 %.9g" % (what, i, got.flat[i], oracle.flat[i], truth.flat[i]))
