"""The committed regression vectors (tests/golden/*.npz, written by tests/golden/make_golden.py with the CPU oracle): the
oracle must still reproduce them (CPU), and the HIP path must meet them through the C ABI within the parity tolerance
(rel 1e-4 / abs 1e-5).  They are the oracle's own record, not outputs of the reference, which ships none."""
import numpy as np
import pytest

from myea_amd import binding as mb
from tests.common import assert_close
from tests.golden.make_golden import CASES, fixture_path, run_case


def _load(name):
    with np.load(fixture_path(name), allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


@pytest.mark.parametrize("name", sorted(CASES))
def test_oracle_reproduces_the_committed_vectors(name):
    from tests.oracle_lib import OracleNetwork, load_oracle
    want = _load(name)
    got = run_case(name, lambda desc, h: OracleNetwork(desc, h), lib=load_oracle())
    assert sorted(got) == sorted(want)
    for k in want:
        # the same C code on the same inputs: equal up to what another compiler's contraction choices could move
        assert_close(got[k], want[k], 1e-6, 1e-7 * max(1.0, float(np.abs(want[k]).max())), what="%s %s" % (name, k))


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(CASES))
def test_hip_path_meets_the_committed_vectors(name):
    want = _load(name)
    got = run_case(name, lambda desc, h: mb.HipNetwork(desc, h))
    for k in ("outputs", "gradient", "parameters"):
        assert_close(got[k], want[k], 1e-4, 1e-5 * max(1.0, float(np.abs(want[k]).max())), what="%s %s" % (name, k))
    assert got["loss"][1] == want["loss"][1]
    assert_close(got["loss"][:1], want["loss"][:1], 1e-4, 1e-6, what="%s accumulated loss" % name)
