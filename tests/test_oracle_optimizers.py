"""Pins the oracle's Update_Parameter (clip-by-global-norm + optimizers) with independent float64 restatements
of the published algorithms, torch.optim where the formulas coincide, and hand traces.  CPU only."""
import numpy as np
import pytest
import torch

from myea_amd import binding as mb
from tests.common import assert_close, oracle_desc, oracle_hyper
from tests.oracle_lib import OracleNetwork

SPECS = [dict(units=5), dict(units=4, activation="TANH"), dict(units=3, activation="SIGMOID")]


def _net(**kw):
    desc = oracle_desc(SPECS, 2)
    net = OracleNetwork(desc, oracle_hyper(**kw))
    return desc, net


def _run(net, w0, grads):
    net.upload_parameters(w0)
    net.Clear_Training_Arrays()
    out = []
    for g in grads:
        net.upload_gradient(g)
        net.Update_Parameter(2, 2)
        assert np.all(net.download_gradient() == 0)   # the update zeroes the gradient (Neural_Network__Adam.cpp:80,94)
        out.append(net.download_parameters().astype(np.float64))
    return out


def _data(P, steps=4, seed=0):
    rng = np.random.default_rng(seed)
    return rng.normal(0, 1, P).astype(np.float32), [rng.normal(0, 0.5, P).astype(np.float32) for _ in range(steps)]


def test_plain_and_momentum_sgd_match_torch():
    desc, net = _net(type_optimizer_function=mb.OPTIMIZER["GD"], learning_rate=0.01, learning_momentum=0.0)
    w0, grads = _data(desc.total_parameters)
    got = _run(net, w0, grads)
    for mu, nesterov in ((0.0, False), (0.9, False)):
        net.set_hyper(oracle_hyper(type_optimizer_function=mb.OPTIMIZER["GD"], learning_rate=0.01, learning_momentum=mu))
        got = _run(net, w0, grads)
        p = torch.tensor(w0.astype(np.float64), requires_grad=True)
        opt = torch.optim.SGD([p], lr=0.01, momentum=mu)
        for k, g in enumerate(grads):
            p.grad = torch.tensor(g.astype(np.float64))
            opt.step()
            assert_close(got[k], p.detach().numpy(), rel=2e-6, abs_=2e-7, what="sgd mu=%g step %d" % (mu, k))
    assert net.get_hyper().optimizer_time_step == len(grads)


def test_nesterov_as_written_in_the_reference():
    """d = lr g + mu d; w -= mu d - lr g  (minus sign on the lr*g term, Neural_Network__Nesterov_Accelerated_Gradient.cpp:48,59).
    Pinned by reading only; the hand trace also shows it is not the textbook form (w -= mu d + lr g)."""
    desc, net = _net(type_optimizer_function=mb.OPTIMIZER["GD"], learning_rate=0.1, learning_momentum=0.5, use_Nesterov=1)
    P = desc.total_parameters
    w0 = np.full(P, 1.0, dtype=np.float32)
    grads = [np.full(P, 2.0, dtype=np.float32), np.full(P, -1.0, dtype=np.float32), np.full(P, 0.5, dtype=np.float32)]
    got = _run(net, w0, grads)
    # step 1: d = .2            w = 1 - (.5*.2 - .2)        = 1.1
    # step 2: d = -.1 + .1 = 0  w = 1.1 - (0 + .1)          = 1.0
    # step 3: d = .05           w = 1.0 - (.025 - .05)      = 1.025
    for k, want in enumerate((1.1, 1.0, 1.025)):
        assert_close(got[k], np.full(P, want), rel=1e-6, abs_=1e-6)
    textbook = 1.0 - (0.5 * 0.2 + 0.2)
    assert abs(got[0][0] - textbook) > 0.3


@pytest.mark.parametrize("amsgrad", [False, True])
def test_adam_and_amsgrad_match_torch_when_epsilon_is_zero(amsgrad):
    """lr_t = lr sqrt(1-b2^t)/(1-b1^t); w -= lr_t m / (sqrt(v) + eps).  With eps = 0 this is exactly torch's Adam
    (which puts eps after the bias correction of v); AMSGrad keeps the running maximum of the raw second moment."""
    kind = "AMSGRAD" if amsgrad else "ADAM"
    desc, net = _net(type_optimizer_function=mb.OPTIMIZER[kind], adam_epsilon=0.0)
    w0, grads = _data(desc.total_parameters, steps=6, seed=3)
    grads[3] = (grads[3] * 0.01).astype(np.float32)  # make v shrink so that the AMSGrad maximum matters
    got = _run(net, w0, grads)
    p = torch.tensor(w0.astype(np.float64), requires_grad=True)
    opt = torch.optim.Adam([p], lr=1e-3, betas=(0.9, 0.999), eps=0.0, amsgrad=amsgrad)
    for k, g in enumerate(grads):
        p.grad = torch.tensor(g.astype(np.float64))
        opt.step()
        assert_close(got[k] - w0, p.detach().numpy() - w0, rel=2e-4, abs_=8e-7, what="%s step %d" % (kind, k))  # fp32 ulp of w ~ 1.2e-7 per step


def _adam_family_f64(kind, w0, grads, lr=1e-3, b1=0.9, b2=0.999, eps=1e-8, final=0.1, gamma=1e-3, wd=0.0, n_weights=0):
    """float64 restatement of Adam (Kingma & Ba, eps outside the sqrt, bias correction folded into the step size),
    AMSGrad (Reddi et al.) and AdaBound (Luo et al., official implementation: step_size / denom clamped to
    [final(1 - 1/(gamma t + 1)), final(1 + 1/(gamma t))])."""
    w = w0.astype(np.float64).copy()
    m = np.zeros_like(w); v = np.zeros_like(w); vh = np.zeros_like(w)
    out = []
    for t, g in enumerate(grads, 1):
        g = g.astype(np.float64)
        m = b1 * m + (1 - b1) * g
        v = b2 * v + (1 - b2) * g * g
        step_size = lr * np.sqrt(1 - b2 ** t) / (1 - b1 ** t)
        if kind == "ADAM":
            upd = step_size * m / (np.sqrt(v) + eps)
        elif kind == "AMSGRAD":
            vh = np.maximum(vh, v)
            upd = step_size * m / (np.sqrt(vh) + eps)
        else:
            lo, hi = final * (1 - 1 / (gamma * t + 1)), final * (1 + 1 / (gamma * t))
            upd = np.clip(step_size / (np.sqrt(v) + eps), lo, hi) * m
        if wd:
            mask = (np.arange(w.size) < n_weights).astype(np.float64)
            upd = upd + mask * wd * w
        w = w - upd
        out.append(w.copy())
    return out


@pytest.mark.parametrize("kind", ["ADAM", "AMSGRAD", "ADABOUND"])
@pytest.mark.parametrize("wd", [0.0, 1e-2])
def test_adam_family_against_float64_restatement(kind, wd):
    desc, net = _net(type_optimizer_function=mb.OPTIMIZER[kind], regularization__weight_decay=wd)
    w0, grads = _data(desc.total_parameters, steps=5, seed=7)
    got = _run(net, w0, grads)
    want = _adam_family_f64(kind, w0, grads, wd=wd, n_weights=desc.total_weights)
    for k in range(len(grads)):
        assert_close(got[k] - w0, want[k] - w0, rel=3e-4, abs_=8e-7, what="%s step %d" % (kind, k))


def test_adabound_bounds_converge_to_final_learning_rate():
    """after many steps both bounds are ~lr_final, so the update is lr_final * m whatever v is"""
    desc, net = _net(type_optimizer_function=mb.OPTIMIZER["ADABOUND"], learning_rate_final=0.05, learning_gamma=1.0)
    P = desc.total_parameters
    h = net.get_hyper(); h.optimizer_time_step = 1e6; net.set_hyper(h)
    w0 = np.zeros(P, dtype=np.float32)
    net.upload_parameters(w0)
    g = np.linspace(-3, 3, P).astype(np.float32)
    net.upload_gradient(g)
    net.Update_Parameter(2, 2)
    assert_close(net.download_parameters(), -0.05 * 0.1 * g.astype(np.float64), rel=1e-4, abs_=1e-9)


def test_clip_gradient_global_norm():
    """one norm over ALL parameters (weights, biases, ...); scale by clip/norm when norm >= clip, including equality."""
    desc, net = _net(type_optimizer_function=mb.OPTIMIZER["GD"], learning_rate=1.0, learning_momentum=0.0, use_clip_gradient=1, clip_gradient=2.0)
    P = desc.total_parameters
    w0 = np.zeros(P, dtype=np.float32)
    g = np.zeros(P, dtype=np.float32); g[0] = 3.0; g[P - 1] = 4.0          # norm 5 spans weights and biases
    got = _run(net, w0, [g])[0]
    assert_close(got, -g.astype(np.float64) * (2.0 / 5.0), rel=1e-6, abs_=1e-7)
    g2 = np.zeros(P, dtype=np.float32); g2[3] = 1.0                         # norm 1 < clip: untouched
    assert_close(_run(net, w0, [g2])[0], -g2.astype(np.float64))
    g3 = np.zeros(P, dtype=np.float32); g3[3] = 2.0                         # norm == clip: scaled by exactly 1
    assert_close(_run(net, w0, [g3])[0], -g3.astype(np.float64))


def test_adam_bias_corrected_rate_is_evaluated_in_float():
    """The reference evaluates lr_t = lr * sqrt(1 - beta2^t) / (1 - beta1^t) with every operand a float
    (NN/Neural_Network__Adam.cpp:58, T_ = float).  With a gradient of constant sign and m = v = 0 at the start, step t moves
    a weight by lr_t * m_t / (sqrt(v_t) + eps): restated here in numpy float32 it must match the oracle bit for bit, and the
    same restatement with lr_t evaluated in double and rounded once must NOT (it differs in the last bits at some t <= 10) -
    the check a double-precision lr_t fails."""
    f = np.float32
    lr, b1, b2, eps = f(1e-3), f(0.9), f(0.999), f(1e-8)
    desc, net = _net(type_optimizer_function=mb.OPTIMIZER["ADAM"], adam_learning_rate=float(lr), adam_beta1=float(b1), adam_beta2=float(b2),
                     adam_epsilon=float(eps), use_adam_bias_correction=1)
    P = desc.total_parameters
    rng = np.random.default_rng(11)
    w0 = rng.normal(0, 1, P).astype(f)
    grads = [rng.normal(0, 0.5, P).astype(f) for _ in range(10)]
    got = [g.astype(f) for g in _run(net, w0, grads)]

    def restate(rate_in_double):
        w, m, v, out = w0.copy(), np.zeros(P, f), np.zeros(P, f), []
        for k, g in enumerate(grads):
            t = f(k + 1)
            m = b1 * m + (f(1) - b1) * g
            v = b2 * v + (f(1) - b2) * g * g
            if rate_in_double:
                lr_t = f(float(lr) * np.sqrt(1.0 - float(b2) ** float(t)) / (1.0 - float(b1) ** float(t)))
            else:
                # powf as the C library gives it: the correctly rounded float power (numpy's float32 power is a different routine)
                p2, p1 = f(float(b2) ** float(t)), f(float(b1) ** float(t))
                lr_t = f(lr * np.sqrt(f(1) - p2, dtype=f)) / (f(1) - p1)
            w = w - lr_t * m / (np.sqrt(v, dtype=f) + eps)
            out.append(w.astype(f))
        return out

    in_float, in_double = restate(False), restate(True)
    assert any(not np.array_equal(a, b) for a, b in zip(in_float, in_double)), "float and double rates coincide on this data: the test pins nothing"
    for k in range(10):
        assert np.array_equal(got[k], in_float[k]), "step %d: the oracle's rate is not the float expression" % (k + 1)


def check_clear_optimizer_touches_the_current_optimizers_state_only(make_net):
    """Clear_Optimizer (NN/Train.cpp:128-263) switches on the optimizer: gradient descent with a momentum clears its previous
    deltas and nothing else; NosAdam its two moments and its running sum; iRPROP+ its losses, derivatives, steps and deltas.
    The step counters restart for all."""
    S = mb.OPT_STATE
    for kind, kw, cleared, kept in (
            ("GD", dict(learning_momentum=0.9), ["PREVIOUS_DELTA"], ["FIRST_MOMENT", "SECOND_MOMENT", "SECOND_MOMENT_HAT", "PREVIOUS_DERIVATIVES"]),
            ("GD", dict(learning_momentum=0.0), [], ["PREVIOUS_DELTA", "FIRST_MOMENT"]),
            ("ADAM", {}, ["FIRST_MOMENT", "SECOND_MOMENT"], ["SECOND_MOMENT_HAT", "PREVIOUS_DELTA"]),
            ("AMSGRAD", {}, ["FIRST_MOMENT", "SECOND_MOMENT", "SECOND_MOMENT_HAT"], ["PREVIOUS_DELTA", "PREVIOUS_DERIVATIVES"]),
            ("NOSADAM", {}, ["FIRST_MOMENT", "SECOND_MOMENT"], ["SECOND_MOMENT_HAT"]),
            ("IRPROP_PLUS", dict(rprop_delta_zero=0.07), ["PREVIOUS_DERIVATIVES", "PREVIOUS_DELTA"], ["FIRST_MOMENT", "SECOND_MOMENT"])):
        desc, net = make_net(type_optimizer_function=mb.OPTIMIZER[kind], **kw)
        P = desc.total_parameters
        for name in S:
            net.upload_optimizer_state(S[name], np.full(P, 2.0, dtype=np.float32))
        h = net.get_hyper()
        h.loss_rprop, h.previous_loss_rprop, h.adam_previous_beta2, h.optimizer_time_step, h.epoch_time_step = 3.0, 4.0, 5.0, 6.0, 7.0
        net.set_hyper(h)
        net.Clear_Training_Arrays()
        for name in cleared:
            assert np.all(net.download_optimizer_state(S[name]) == 0), (kind, name)
        for name in kept:
            assert np.all(net.download_optimizer_state(S[name]) == 2.0), (kind, name)
        steps = net.download_optimizer_state(S["PREVIOUS_STEPS"])
        assert np.all(steps == (np.float32(0.07) if kind == "IRPROP_PLUS" else 2.0)), kind
        h = net.get_hyper()
        assert (h.optimizer_time_step, h.epoch_time_step) == (0.0, 1.0)
        assert (h.loss_rprop, h.previous_loss_rprop) == ((np.finfo(np.float32).max,) * 2 if kind == "IRPROP_PLUS" else (3.0, 4.0)), kind
        assert h.adam_previous_beta2 == (0.0 if kind == "NOSADAM" else 5.0), kind


def test_clear_optimizer_touches_the_current_optimizers_state_only():
    check_clear_optimizer_touches_the_current_optimizers_state_only(_net)
