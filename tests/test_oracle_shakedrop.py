"""Pins the oracle's ShakeDrop on residual blocks against a float64 model with a custom autograd function that multiplies
by one set of draws going forward and by another going back (the published operator, Yamada et al. 2018, applied value by
value as the reference does); cleared masks must reproduce the plain block, the inference pass the 1 - p scaling.
CPU only."""
import numpy as np
import pytest
import torch

from myea_amd import binding as mb
from tests.common import assert_close, glorot_parameters, oracle_desc, oracle_hyper
from tests.oracle_lib import OracleNetwork


class Shake(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, alpha, beta):
        ctx.save_for_backward(beta)
        return x * alpha

    @staticmethod
    def backward(ctx, g):
        return g * ctx.saved_tensors[0], None, None


def _specs(p, norm=False, wide_shortcut=False):
    res = dict(type="residual", block_depth=2, dropout="SHAKEDROP", keep=p)
    if norm:
        res["normalization"] = "BATCH_NORMALIZATION"
    return [dict(units=6), dict(units=12 if wide_shortcut else 10, activation="TANH"), res, dict(units=9, activation="LEAKY_RELU"), dict(units=10, activation="LEAKY_RELU"),
            dict(units=3, activation="LINEAR")]


def _run(specs, B, draws, seed=1, state=mb.STATE_TRAINING):
    desc = oracle_desc(specs, B)
    net = OracleNetwork(desc, oracle_hyper(type_loss_function=mb.LOSS["MSE"]))
    w = glorot_parameters(desc, seed, bias_range=0.3)
    net.set_state_propagation(state)
    net.upload_parameters(w)
    net.Clear_Training_Arrays()
    if draws is not None:
        net.upload_dropout_noise(2, draws)
    rng = np.random.default_rng(seed)
    X, Y = rng.normal(0, 1, (B, 6)).astype(np.float32), rng.normal(0, 1, (B, 3)).astype(np.float32)
    net.Forward_Pass(B, X)
    if state == mb.STATE_TRAINING:
        net.Compute__Error(B, Y); net.Backward_Pass(B); net.Update_Derivative_Weight(B)
    return desc, net, w, X, Y


def _draws(B, W, seed, p=0.5):
    rng = np.random.default_rng(seed)
    mask = (rng.uniform(0, 1, B) < p).astype(np.float32)
    return mask, rng.uniform(-1, 1, (B, W)).astype(np.float32), rng.uniform(0, 1, (B, W)).astype(np.float32)


def _float64(desc, specs, w, X, Y, mask, alpha, beta, norm):
    W = torch.tensor(w.astype(np.float64), requires_grad=True)
    def fc(li, x):
        l = desc.layers[li]
        H = specs[li]["units"]
        In = (l.last_connection_index - l.first_connection_index) // H
        return x @ W[l.first_connection_index:l.last_connection_index].reshape(H, In).T + W[l.first_bias_connection_index:l.first_bias_connection_index + H]
    leaky = lambda s: torch.where(s < 0, 0.01 * s, s)
    x = torch.tensor(X.astype(np.float64))
    h1 = torch.tanh(fc(1, x))
    # members apply on their input side: the first has no activation, the second activates its input
    m1 = fc(3, h1)
    m2 = fc(4, leaky(m1))
    blk = m2
    if norm:
        l = desc.layers[2]
        at = desc.total_weights + desc.total_bias + l.first_normalized_unit_index
        scale, shift = W[at:at + 10], W[at + desc.total_normalized_units:at + desc.total_normalized_units + 10]
        mean = blk.mean(0)
        blk = scale * (blk - mean) / torch.sqrt(((blk - mean) ** 2).mean(0) + 1e-5) + shift
    m = torch.tensor(mask.astype(np.float64))[:, None]
    a = torch.where(m != 0, torch.tensor(alpha.astype(np.float64)), torch.ones_like(blk))
    b = torch.where(m != 0, torch.tensor(beta.astype(np.float64)), torch.ones_like(blk))
    blk = Shake.apply(blk, a, b)
    wide = h1.shape[1]
    if wide > 10:
        pad = ((wide - 10) + 1) // 2
        res = h1 + torch.nn.functional.pad(blk, (pad, wide - 10 - pad))
    else:
        res = h1 + blk
    y = fc(5, res)
    (0.5 * ((y - torch.tensor(Y.astype(np.float64))) ** 2).sum()).backward()
    return y.detach().numpy(), W.grad.numpy()


@pytest.mark.parametrize("norm,wide", [(False, False), (True, False), (False, True)])
def test_shakedrop_against_a_float64_model_with_separate_forward_and_backward_draws(norm, wide):
    B = 8
    specs = _specs(0.5, norm, wide)
    mask, alpha, beta = _draws(B, 10, 3)
    assert mask.any() and not mask.all()
    draws = np.concatenate([mask, alpha.ravel(), beta.ravel()])
    desc, net, w, X, Y = _run(specs, B, draws)
    y, grad = _float64(desc, specs, w, X, Y, mask, alpha, beta, norm)
    assert_close(net.download_tensor(5, mb.TENSOR["OUTPUTS"], B * 3), y.ravel(), rel=1e-5, abs_=2e-6, what="outputs")
    g = net.download_gradient()
    assert_close(g, grad, rel=3e-4, abs_=2e-6 * float(np.abs(grad).max()) + 3e-6, what="gradient")


def test_cleared_masks_reproduce_the_plain_block_and_inference_scales_by_one_minus_p():
    B, p = 7, 0.3
    plain = _specs(p)
    plain[2] = dict(type="residual", block_depth=2)
    d0, a, _, _, _ = _run(plain, B, None)
    d1, b, _, _, _ = _run(_specs(p), B, None)                       # masks all false after create
    assert np.array_equal(a.download_gradient(), b.download_gradient())
    assert np.array_equal(a.download_tensor(5, mb.TENSOR["OUTPUTS"]), b.download_tensor(5, mb.TENSOR["OUTPUTS"]))
    # inference: block output times (1 - p) whatever the draws
    mask, alpha, beta = _draws(B, 10, 5)
    _, c, _, _, _ = _run(_specs(p), B, np.concatenate([mask, alpha.ravel(), beta.ravel()]), state=mb.STATE_INFERENCE)
    _, e, _, _, _ = _run(plain, B, None, state=mb.STATE_INFERENCE)
    h1 = e.download_tensor(1, mb.TENSOR["OUTPUTS"], B * 10)
    blk_plain = e.download_tensor(2, mb.TENSOR["OUTPUTS"], B * 10) - h1
    blk_shake = c.download_tensor(2, mb.TENSOR["OUTPUTS"], B * 10) - h1
    assert_close(blk_shake, blk_plain * np.float32(1 - p), rel=1e-5, abs_=1e-6, what="inference block output")
