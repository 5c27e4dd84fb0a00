"""Regression vectors for the training step: small seeded networks walked for a few steps, with the parameters, the
gradient of the last step and the accumulated loss written to tests/golden/*.npz.

The reference ships no vectors, fixtures or tests of its own, so these are NOT its outputs: they are what the CPU oracle
(oracle/myea_oracle.c, pinned against mathematics by tests/test_oracle_*.py) produced when this file was last run, kept so
that a later change to the oracle or to the HIP path that moves a result shows up against a fixed record.
Regenerate (after an intended change of behaviour only):  python -m tests.golden.make_golden
"""
import os

import numpy as np

from myea_amd import binding as mb

HERE = os.path.dirname(os.path.abspath(__file__))

CASES = {
    # BASELINE config 1's shape shrunk: tanh hidden layer, sigmoid head, SGD with momentum, MSE
    "mlp_tanh_sigmoid_momentum": dict(
        layers=[dict(units=12), dict(units=16, activation="TANH"), dict(units=5, activation="SIGMOID")], batch=8, depth=1, steps=3, head="uniform",
        hyper=dict(type_optimizer_function="GD", learning_rate=0.05, learning_momentum=0.9, type_loss_function="MSE")),
    # config 2's shape shrunk: ReLU stack, softmax + cross-entropy, Adam
    "mlp_relu_softmax_adam": dict(
        layers=[dict(units=10), dict(units=24, activation="RELU"), dict(units=24, activation="RELU"), dict(units=6, activation="SOFTMAX")], batch=16, depth=1, steps=3,
        head="one_hot", hyper=dict(type_optimizer_function="ADAM", type_loss_function="CROSS_ENTROPY")),
    # config 3's shape shrunk: two LSTM layers with peepholes, linear head, AMSGrad
    "lstm_x2_linear_amsgrad": dict(
        layers=[dict(units=6), dict(type="lstm", units=8), dict(type="lstm", units=8), dict(units=8, activation="LINEAR")], batch=5, depth=6, steps=2, head="normal",
        hyper=dict(type_optimizer_function="AMSGRAD", type_loss_function="MSE")),
    # config 4's shape shrunk: BatchNorm before ReLU, inverted dropout, Nesterov
    "mlp_bn_relu_dropout_nesterov": dict(
        layers=[dict(units=16)] + [dict(units=32, activation="RELU", normalization="BATCH_NORMALIZATION", norm_before=True, dropout="BERNOULLI_INVERTED", keep=0.5)] * 2
               + [dict(units=7, activation="SOFTMAX")], batch=24, depth=1, steps=2, head="one_hot",
        hyper=dict(type_optimizer_function="GD", use_Nesterov=1, learning_rate=0.01, learning_momentum=0.9, type_loss_function="CROSS_ENTROPY")),
    # config 5's shape shrunk: bidirectional LSTM, per-step softmax, clip by global norm, AdaBound
    "bilstm_softmax_clip_adabound": dict(
        layers=[dict(units=5), dict(type="lstm", units=8, bidirectional=True), dict(units=3, activation="SOFTMAX")], batch=4, depth=7, steps=2, head="one_hot",
        hyper=dict(type_optimizer_function="ADABOUND", type_loss_function="CROSS_ENTROPY", use_clip_gradient=1, clip_gradient=1.0)),
}


def _hyper(spec, lib=None):
    kw = dict(spec)
    kw["type_optimizer_function"] = mb.OPTIMIZER[kw["type_optimizer_function"]]
    kw["type_loss_function"] = mb.LOSS[kw["type_loss_function"]]
    return mb.default_hyper(lib=lib, **kw)


def case_inputs(name):
    """descriptor-independent data of a case: everything comes from one seeded generator, in a fixed order"""
    c = CASES[name]
    rng = np.random.default_rng(abs(hash_name(name)))
    n_in, n_out, B, T = c["layers"][0]["units"], c["layers"][-1]["units"], c["batch"], c["depth"]
    X = rng.normal(0, 1, (B, T * n_in)).astype(np.float32)
    if c["head"] == "one_hot":
        Y = np.zeros((B * T, n_out), dtype=np.float32)
        Y[np.arange(B * T), rng.integers(0, n_out, B * T)] = 1.0
        Y = Y.reshape(B, T * n_out)
    elif c["head"] == "uniform":
        Y = rng.uniform(0, 1, (B, T * n_out)).astype(np.float32)
    else:
        Y = rng.normal(0, 1, (B, T * n_out)).astype(np.float32)
    return rng, X, Y


def hash_name(name):
    h = 2166136261
    for ch in name.encode():
        h = ((h ^ ch) * 16777619) & 0xffffffff
    return h


def run_case(name, make_network, lib=None):
    """walks the case on a network built by make_network(desc, hyper); returns the arrays a fixture holds"""
    from tests.common import glorot_parameters
    c = CASES[name]
    desc = mb.make_desc(c["layers"], c["batch"], c["depth"], lib=lib)
    net = make_network(desc, _hyper(c["hyper"], lib))
    rng, X, Y = case_inputs(name)
    net.set_state_propagation(mb.STATE_TRAINING)
    net.upload_parameters(glorot_parameters(desc, hash_name(name) & 0xffff, bias_range=0.2))
    net.Clear_Training_Arrays()
    B = c["batch"]
    gradient = None
    for step in range(c["steps"]):
        if desc.total_mask_units:
            net.upload_masks((rng.uniform(0, 1, desc.total_mask_units) < 0.5).astype(np.uint8))
        net.Forward_Pass(B, X)
        net.Compute__Error(B, Y)
        net.Backward_Pass(B)
        net.Update_Derivative_Weight(B, 1, desc.n_layers)
        gradient = np.asarray(net.download_gradient(), dtype=np.float32).copy()
        net.Update_Parameter(B, B)
    loss = net.get_loss()
    return dict(parameters=np.asarray(net.download_parameters(), dtype=np.float32).copy(), gradient=gradient,
                outputs=np.asarray(net.download_tensor(desc.n_layers - 1, mb.TENSOR["OUTPUTS"]), dtype=np.float32).copy(),
                loss=np.array([loss.loss_values, float(loss.number_loss)], dtype=np.float64))


def fixture_path(name):
    return os.path.join(HERE, name + ".npz")


def main():
    from tests.oracle_lib import OracleNetwork, load_oracle
    for name in CASES:
        out = run_case(name, lambda desc, h: OracleNetwork(desc, h), lib=load_oracle())
        np.savez_compressed(fixture_path(name), **out)
        print(name, {k: v.shape for k, v in out.items()})


if __name__ == "__main__":
    main()
