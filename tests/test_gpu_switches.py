"""The environment switches that exist for A/B timing must not move a result: with MYEA_SIDE_STREAM=0 (no second stream
for a bidirectional layer's second direction or for the bias reductions) and MYEA_GEMM_PAIR=0 (dX and dW launched apart)
a child process computes the same cases as this one and every array must come out bit for bit equal."""
import os
import subprocess
import sys

import numpy as np
import pytest

from myea_amd import binding as mb
from tests.golden.make_golden import run_case

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLDEN_CASES = ["bilstm_softmax_clip_adabound", "mlp_bn_relu_dropout_nesterov", "lstm_x2_linear_amsgrad"]


def wide_stack():
    """a dense stack wide enough at a batch of 1024 for the paired launch and the side-stream reductions to happen"""
    from tests.common import glorot_parameters, one_hot
    specs = [dict(units=1024), dict(units=2048, activation="RELU"), dict(units=2048, activation="TANH"), dict(units=2048, activation="RELU"), dict(units=1000, activation="SOFTMAX")]
    B = 1024
    desc = mb.make_desc(specs, B)
    net = mb.HipNetwork(desc, mb.default_hyper(type_optimizer_function=mb.OPTIMIZER["ADAM"], type_loss_function=mb.LOSS["CROSS_ENTROPY"]))
    rng = np.random.default_rng(5)
    net.set_state_propagation(mb.STATE_TRAINING)
    net.upload_parameters(glorot_parameters(desc, 5, bias_range=0.2))
    net.Clear_Training_Arrays()
    X = rng.normal(0, 1, (B, 1024)).astype(np.float32)
    Y = one_hot(rng.integers(0, 1000, B), 1000)
    for _ in range(2):
        net.Forward_Pass(B, X)
        net.Compute__Error(B, Y)
        net.Backward_Pass__Update_Derivative_Weight(B)
        g = net.download_gradient()
        net.Update_Parameter(B, B)
    return dict(gradient=g, parameters=net.download_parameters())


def compute_all():
    out = {}
    for name in GOLDEN_CASES:
        for k, v in run_case(name, lambda desc, h: mb.HipNetwork(desc, h)).items():
            out["%s.%s" % (name, k)] = v
    for k, v in wide_stack().items():
        out["wide.%s" % k] = v
    return out


def test_switched_off_paths_give_the_same_bits(tmp_path):
    here = compute_all()
    target = str(tmp_path / "switched_off.npz")
    env = dict(os.environ, MYEA_SIDE_STREAM="0", MYEA_GEMM_PAIR="0")
    code = "import sys, numpy as np; sys.path.insert(0, %r); from tests.test_gpu_switches import compute_all; np.savez(%r, **compute_all())" % (ROOT, target)
    done = subprocess.run([sys.executable, "-c", code], env=env, cwd=ROOT, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
    assert done.returncode == 0, done.stdout[-2000:]
    with np.load(target, allow_pickle=False) as there:
        assert sorted(there.files) == sorted(here)
        for k in here:
            assert np.array_equal(here[k], there[k]), k
