"""The float64 checker of the full-size parity tests, held against the oracle at small sizes on the CPU: the products it
lists for every entry of the flat gradient (dense layers, LSTM layers of one and two directions with their peepholes and
the bias slots neighbouring layers share) must add up to the gradient the oracle computed."""
import numpy as np
import pytest

from myea_amd import binding as mb
from tests.common import glorot_parameters, oracle_desc, oracle_hyper, run_step
from tests.full_size_support import GradientTerms, assert_sums_match
from tests.oracle_lib import OracleNetwork

CASES = [
    ("dense", [dict(units=7), dict(units=9, activation="TANH"), dict(units=5, activation="SIGMOID")], 1, 6, 6),
    ("lstm-x2-head", [dict(units=5), dict(type="lstm", units=6), dict(type="lstm", units=4), dict(units=6, activation="LINEAR")], 5, 4, 5),
    ("two-directions", [dict(units=4), dict(type="lstm", units=6, bidirectional=True), dict(units=7, activation="TANH")], 4, 3, 3),
]


@pytest.mark.parametrize("name,specs,T,B,Bmax", CASES, ids=[c[0] for c in CASES])
def test_listed_products_add_up_to_the_oracles_gradient(name, specs, T, B, Bmax):
    desc = oracle_desc(specs, Bmax, T)
    net = OracleNetwork(desc, oracle_hyper(type_loss_function=mb.LOSS["MSE"]))
    net.set_state_propagation(mb.STATE_TRAINING)
    net.upload_parameters(glorot_parameters(desc, 5, bias_range=0.3))
    net.Clear_Training_Arrays()
    rng = np.random.default_rng(5)
    X = rng.normal(0, 1, (B, T * specs[0]["units"])).astype(np.float32)
    Y = rng.normal(0, 1, (B, T * specs[-1]["units"])).astype(np.float32)
    run_step(net, B, X, Y, update=False)
    g = net.download_gradient()
    sums, mags = GradientTerms(desc, net, X, B).exact(np.arange(desc.total_parameters))
    assert np.abs(sums - g).max() <= 1e-5 * max(1.0, float(np.abs(g).max()))
    assert (mags >= np.abs(sums) - 1e-12).all() and np.count_nonzero(g) > 0.8 * g.size


def test_the_three_clauses():
    oracle = np.array([1.0, 2.0, 3.0, 4.0, 5.0])
    exact = lambda idx: (np.array([1.0, 2.5, 3.0, 4.0, 5.0])[idx], np.array([1.0, 1.0, 1e6, 1.0, 1.0])[idx])
    got = np.array([1.00005, 2.4, 3.05, 4.0, 5.0])       # inside the oracle's tolerance; nearer to the exact sum; within four ulps of 1e6
    counts = assert_sums_match(got, oracle, exact, "clauses")
    assert counts["outside_oracle_tolerance"] == 2 and counts["nearer_than_oracle"] == 1 and counts["within_ulp_of_magnitudes"] == 1
    with pytest.raises(AssertionError):
        assert_sums_match(np.array([1.0, 2.0, 3.0, 4.1, 5.0]), oracle, exact, "a wrong entry")
