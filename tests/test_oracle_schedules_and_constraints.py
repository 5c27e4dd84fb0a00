"""Pins the rest of the oracle's Update_Parameter: AMSBound, NosAdam, iRPROP+, the max-norm constraint, normalized
weight decay and cosine warm restarts.  Every check is a closed form, a limiting case that reduces to an optimizer
already pinned elsewhere, an invariant, or a hand trace - none re-types the oracle's loop.  CPU only."""
import math

import numpy as np
import pytest

from myea_amd import binding as mb
from tests.common import assert_close, oracle_desc, oracle_hyper
from tests.oracle_lib import OracleNetwork

SPECS = [dict(units=5), dict(units=4, activation="TANH"), dict(units=3, activation="SIGMOID")]
FLT_MAX = float(np.finfo(np.float32).max)


def _net(specs=SPECS, T=1, **kw):
    desc = oracle_desc(specs, 2, T)
    return desc, OracleNetwork(desc, oracle_hyper(**kw))


def _run(net, w0, grads, B=2, N=2, clear=True):
    net.upload_parameters(w0)
    if clear:
        net.Clear_Training_Arrays()
    out = []
    for g in grads:
        net.upload_gradient(g)
        net.Update_Parameter(B, N)
        assert np.all(net.download_gradient() == 0)
        out.append(net.download_parameters().astype(np.float64))
    return out


def _data(P, steps=4, seed=0):
    rng = np.random.default_rng(seed)
    return rng.normal(0, 1, P).astype(np.float32), [rng.normal(0, 0.5, P).astype(np.float32) for _ in range(steps)]


# ---------------------------------------------------------------------------------------------------------------
# NosAdam (Neural_Network__NosAdam.cpp:43-100)

@pytest.mark.parametrize("gamma", [0.0, 0.1, 0.7])
def test_nosadam_second_moment_is_the_weighted_mean_of_squares(gamma):
    """beta2_t = S_{t-1} / S_t with S_t = sum_{k<=t} k^-gamma telescopes: v_t = sum_k k^-gamma g_k^2 / S_t
    (Huang et al. 2018, eq. 4); gamma = 0 is the plain running mean."""
    desc, net = _net(type_optimizer_function=mb.OPTIMIZER["NOSADAM"], adam_gamma=gamma)
    w0, grads = _data(desc.total_parameters, steps=6, seed=3)
    net.upload_parameters(w0)
    net.Clear_Training_Arrays()
    num = np.zeros(desc.total_parameters); den = 0.0
    for t, g in enumerate(grads, 1):
        net.upload_gradient(g)
        net.Update_Parameter(2, 2)
        wt = float(t) ** -gamma
        num += wt * g.astype(np.float64) ** 2; den += wt
        assert_close(net.download_optimizer_state(mb.OPT_STATE["SECOND_MOMENT"]), num / den, rel=2e-5, abs_=1e-9, what="v at t=%d" % t)
        assert abs(net.get_hyper().adam_previous_beta2 - den) < 1e-5 * den


def test_nosadam_constant_gradient_closed_form():
    """g constant: m_t = (1 - b1^t) g, v_t = g^2, so each step moves the weight by lr sqrt(1 - b2^t) g / (|g| + eps) - the bias
    correction keeps the PLAIN beta2 although the second moment decays with beta2_t (NosAdam.cpp:62 as written)."""
    lr, b2 = 1e-2, 0.999
    desc, net = _net(type_optimizer_function=mb.OPTIMIZER["NOSADAM"], adam_learning_rate=lr, adam_beta2=b2, adam_epsilon=1e-8)
    P = desc.total_parameters
    g = np.linspace(0.5, 2.0, P).astype(np.float32) * np.where(np.arange(P) % 2, 1, -1).astype(np.float32)
    got = _run(net, np.zeros(P, dtype=np.float32), [g] * 5)
    moved = 0.0
    for t in range(1, 6):
        moved += lr * math.sqrt(1 - b2 ** t)
        assert_close(got[t - 1], -np.sign(g) * moved, rel=2e-5, abs_=1e-9, what="t=%d" % t)


# ---------------------------------------------------------------------------------------------------------------
# AMSBound (Neural_Network__AMSBound.cpp:43-110)

def test_amsbound_with_open_bounds_is_amsgrad():
    """gamma -> 0 opens the clip to (0, inf): the step is lr_t m / (sqrt(vhat) + eps), AMSGrad's (pinned against torch.optim)."""
    desc, net = _net(type_optimizer_function=mb.OPTIMIZER["AMSBOUND"], learning_gamma=1e-30, learning_rate_final=0.1)
    w0, grads = _data(desc.total_parameters, steps=5, seed=11)
    grads[2] = grads[2] * 8; grads[3] = grads[3] * 0.05    # vhat must hold its maximum through the small gradients
    got = _run(net, w0, grads)
    net.set_hyper(oracle_hyper(type_optimizer_function=mb.OPTIMIZER["AMSGRAD"]))
    want = _run(net, w0, grads)
    for k in range(len(grads)):
        assert_close(got[k] - w0, want[k] - w0, rel=1e-6, abs_=1e-9, what="step %d" % k)


def test_amsbound_with_closed_bounds_is_final_rate_times_first_moment():
    desc, net = _net(type_optimizer_function=mb.OPTIMIZER["AMSBOUND"], learning_rate_final=0.05, learning_gamma=1.0)
    P = desc.total_parameters
    h = net.get_hyper(); h.optimizer_time_step = 1e6; net.set_hyper(h)
    net.upload_parameters(np.zeros(P, dtype=np.float32))
    g = np.linspace(-3, 3, P).astype(np.float32)
    net.upload_gradient(g)
    net.Update_Parameter(2, 2)
    assert_close(net.download_parameters(), -0.05 * 0.1 * g.astype(np.float64), rel=1e-4, abs_=1e-9)


def test_amsbound_keeps_the_running_maximum_and_clips_by_it():
    """invariants over a run with shrinking gradients: vhat_t = max_k v_k; the per-parameter rate |dw| / |m| lies inside the
    published bounds final (1 - 1/(gamma t + 1)) .. final (1 + 1/(gamma t)) and equals lr_t / (sqrt(vhat) + eps) when that is inside."""
    final, gamma, lr, b1, b2, eps = 0.1, 0.5, 1e-3, 0.9, 0.999, 1e-8
    desc, net = _net(type_optimizer_function=mb.OPTIMIZER["AMSBOUND"], learning_rate_final=final, learning_gamma=gamma, adam_learning_rate=lr)
    P = desc.total_parameters
    w0, grads = _data(P, steps=6, seed=5)
    grads = [g * s for g, s in zip(grads, (4, 2, 1, 0.02, 0.01, 0.01))]
    net.upload_parameters(w0); net.Clear_Training_Arrays()
    vmax = np.zeros(P); prev = w0.astype(np.float64); inside = 0
    for t, g in enumerate(grads, 1):
        net.upload_gradient(g); net.Update_Parameter(2, 2)
        v = net.download_optimizer_state(mb.OPT_STATE["SECOND_MOMENT"]).astype(np.float64)
        vmax = np.maximum(vmax, v)
        hat = net.download_optimizer_state(mb.OPT_STATE["SECOND_MOMENT_HAT"]).astype(np.float64)
        assert_close(hat, vmax, rel=1e-6, abs_=0, what="vhat t=%d" % t)
        m = net.download_optimizer_state(mb.OPT_STATE["FIRST_MOMENT"]).astype(np.float64)
        w = net.download_parameters().astype(np.float64)
        rate = (prev - w) / m
        lo, hi = final * (1 - 1 / (gamma * t + 1)), final * (1 + 1 / (gamma * t))
        assert np.all(rate >= lo * (1 - 1e-3)) and np.all(rate <= hi * (1 + 1e-3))
        free = lr * math.sqrt(1 - b2 ** t) / (1 - b1 ** t) / (np.sqrt(vmax) + eps)
        sel = (free > lo * 1.01) & (free < hi * 0.99) & (np.abs(m) > 1e-3)
        inside += int(sel.sum())
        assert_close(rate[sel], free[sel], rel=2e-3, abs_=0, what="unclipped rate t=%d" % t)
        assert np.all(np.abs(rate[free <= lo * 0.99] / lo - 1) < 2e-3)
        prev = w
    assert inside > 0


# ---------------------------------------------------------------------------------------------------------------
# iRPROP+ (Neural_Network__iRPROP_plus.cpp:28-117; Igel & Huesken 2000)

def test_irprop_plus_constant_sign_grows_the_step_geometrically_up_to_the_cap():
    d0, inc, cap = 0.1, 1.2, 0.2
    desc, net = _net(type_optimizer_function=mb.OPTIMIZER["IRPROP_PLUS"], rprop_delta_zero=d0, rprop_increase_factor=inc, rprop_delta_max=cap)
    P = desc.total_parameters
    sign = np.where(np.arange(P) % 3 == 0, -1.0, 1.0)
    rng = np.random.default_rng(0)
    grads = [(sign * rng.uniform(0.01, 5, P)).astype(np.float32) for _ in range(7)]   # magnitudes must not matter
    got = _run(net, np.zeros(P, dtype=np.float32), grads)
    moved = 0.0
    for k in range(7):
        moved += d0 if k == 0 else min(d0 * inc ** k, cap)    # the first update has no previous slope: plain step
        assert_close(got[k], -sign * moved, rel=2e-6, abs_=1e-7, what="step %d" % k)
    assert net.get_hyper().optimizer_time_step == 0           # iRPROP+ does not count steps
    assert_close(net.download_optimizer_state(mb.OPT_STATE["PREVIOUS_STEPS"]), np.full(P, cap), rel=1e-6)


@pytest.mark.parametrize("worse", [False, True])
def test_irprop_plus_sign_change_hand_trace(worse):
    """one weight, slopes +, +, -, -, + with step0 0.1, x1.2 / x0.5:
       t1 no history    : step 0.1            w = -0.1
       t2 same sign     : step 0.12           w = -0.22, last change -0.12
       t3 sign flips    : step 0.06, the weight goes back by the last change only if the loss got worse; slope forgotten
       t4 slope forgotten -> product 0: moves by the current step 0.06 against the sign (+0.06)
       t5 sign flips against t4's slope: step 0.03, back by t4's change when worse"""
    desc, net = _net(type_optimizer_function=mb.OPTIMIZER["IRPROP_PLUS"], rprop_delta_zero=0.1)
    P = desc.total_parameters
    net.upload_parameters(np.zeros(P, dtype=np.float32)); net.Clear_Training_Arrays()
    h = net.get_hyper()
    assert h.loss_rprop == FLT_MAX and h.previous_loss_rprop == FLT_MAX
    h.loss_rprop, h.previous_loss_rprop = (2.0, 1.0) if worse else (1.0, 2.0)
    net.set_hyper(h)
    want = [-0.1, -0.22, -0.10 if worse else -0.22, None, None]
    want[3] = want[2] + 0.06
    want[4] = want[3] - 0.06 if worse else want[3]
    steps = [0.1, 0.12, 0.06, 0.06, 0.03]
    for t, s in enumerate([3.0, 0.2, -1.0, -7.0, 0.4]):
        net.upload_gradient(np.full(P, s, dtype=np.float32)); net.Update_Parameter(2, 2)
        assert_close(net.download_parameters(), np.full(P, want[t]), rel=1e-6, abs_=1e-7, what="t=%d" % (t + 1))
        assert_close(net.download_optimizer_state(mb.OPT_STATE["PREVIOUS_STEPS"]), np.full(P, steps[t]), rel=1e-6, what="step t=%d" % (t + 1))
    slopes = net.download_optimizer_state(mb.OPT_STATE["PREVIOUS_DERIVATIVES"])
    assert np.all(slopes == 0)                                  # t5 was a flip


def test_irprop_plus_floor_and_zero_gradient():
    desc, net = _net(type_optimizer_function=mb.OPTIMIZER["IRPROP_PLUS"], rprop_delta_zero=0.1, rprop_delta_min=0.04)
    P = desc.total_parameters
    w0 = np.ones(P, dtype=np.float32)
    got = _run(net, w0, [np.zeros(P, dtype=np.float32)])       # sign(0) = 0: nothing moves
    assert np.all(got[0] == 1.0)
    alternating = [np.full(P, s, dtype=np.float32) for s in (1, -1, 1, -1, 1, -1, 1)]
    _run(net, w0, alternating)
    # flips happen on every second update (each flip forgets the slope): 0.1 -> 0.05 -> 0.04 (floor) -> 0.04
    assert_close(net.download_optimizer_state(mb.OPT_STATE["PREVIOUS_STEPS"]), np.full(P, 0.04), rel=1e-6)


# ---------------------------------------------------------------------------------------------------------------
# max-norm constraint (Neural_Network__Regularization__Max_Norm_Constraints.cpp:48-332)

def _rows(desc, w):
    out = []
    for li in range(1, desc.n_layers):
        l = desc.layers[li]
        fan_in = desc.layers[li - 1].n_units
        out.append(w[l.first_connection_index:l.first_connection_index + l.n_units * fan_in].reshape(l.n_units, fan_in))
    return out


def test_max_norm_projects_every_neuron_row_and_leaves_the_rest():
    c = 2.0
    desc, net = _net(type_optimizer_function=mb.OPTIMIZER["GD"], learning_rate=0.05, learning_momentum=0.0)
    w0, grads = _data(desc.total_parameters, steps=1, seed=2)
    free = _run(net, w0, grads)[0]
    net.set_hyper(oracle_hyper(type_optimizer_function=mb.OPTIMIZER["GD"], learning_rate=0.05, learning_momentum=0.0, regularization__max_norm_constraints=c))
    got = _run(net, w0, grads)[0]
    assert np.array_equal(got[desc.total_weights:], free[desc.total_weights:])      # biases are not constrained
    clipped = kept = 0
    for a, b in zip(_rows(desc, got), _rows(desc, free)):
        for ra, rb in zip(a, b):
            nb = np.linalg.norm(rb)
            if nb >= c:
                clipped += 1
                assert abs(np.linalg.norm(ra) - c) < 1e-6
                assert_close(ra, rb * (c / nb), rel=1e-5, abs_=1e-7)              # same direction
            else:
                kept += 1
                assert np.array_equal(ra, rb)
    assert clipped >= 2 and kept >= 2


def test_max_norm_on_an_lstm_block_skips_the_vector_at_index_zero():
    """the LSTM branch tests `first index > start` (:184 ...): the first cell's feed-forward vector, at flat index 0 when the
    LSTM is the first hidden layer, is never projected; every other gate vector is."""
    c = 0.3
    specs = [dict(units=3), dict(type="lstm", units=2, cells_per_block=2), dict(units=4, activation="SIGMOID")]
    desc, net = _net(specs, T=3, type_optimizer_function=mb.OPTIMIZER["GD"], learning_rate=1e-9, learning_momentum=0.0,
                     regularization__max_norm_constraints=c)
    P = desc.total_parameters
    w0 = np.full(P, 0.5, dtype=np.float32)
    got = _run(net, w0, [np.zeros(P, dtype=np.float32)])[0]
    In, K, cpb = 3, 2, 2
    C = K * cpb
    per_block = cpb * (In + C) + 3 * In + 3 * C + 3 * cpb
    l = desc.layers[1]
    assert l.first_connection_index == 0 and l.last_connection_index == K * per_block
    for k in range(K):
        at = k * per_block
        for n in [In, C] * cpb + [In] * 3 + [C] * 3 + [cpb] * 3:
            seg = got[at:at + n]
            if at == 0:
                assert np.all(seg == 0.5)
            else:
                want = min(c, 0.5 * math.sqrt(n))
                assert abs(np.linalg.norm(seg) - want) < 1e-6, (k, at, n)
            at += n
        assert at == (k + 1) * per_block
    out = desc.layers[2]
    rows = got[out.first_connection_index:out.last_connection_index].reshape(4, C)
    assert_close(np.linalg.norm(rows, axis=1), np.full(4, c), rel=1e-5)


# ---------------------------------------------------------------------------------------------------------------
# normalized weight decay (Train.cpp:285-286) and warm restarts (Train.cpp:266-283)

@pytest.mark.parametrize("kind", ["GD", "ADAM"])
def test_normalized_weight_decay_is_decay_times_sqrt_batch_over_set_times_epochs(kind):
    lam = 0.02
    desc, net = _net(type_optimizer_function=mb.OPTIMIZER[kind], learning_momentum=0.0, regularization__weight_decay=lam)
    w0, grads = _data(desc.total_parameters, steps=3, seed=9)
    assert net.get_hyper().use_normalized_weight_decay == 1                         # the reference's default
    h = net.get_hyper(); h.epoch_time_step = 4.0
    net.upload_parameters(w0); net.Clear_Training_Arrays()
    assert net.get_hyper().epoch_time_step == 1.0                                   # Clear_Optimizer resets it
    net.set_hyper(h)
    got = _run(net, w0, grads, B=2, N=32, clear=False)                              # sqrt(2 / (32 * 4)) = 1/8
    plain = oracle_hyper(type_optimizer_function=mb.OPTIMIZER[kind], learning_momentum=0.0, regularization__weight_decay=lam / 8,
                         use_normalized_weight_decay=0)
    net.set_hyper(plain)
    want = _run(net, w0, grads, B=2, N=32)
    for k in range(3):
        assert_close(got[k], want[k], rel=1e-6, abs_=1e-8)
    net.set_hyper(oracle_hyper(type_optimizer_function=mb.OPTIMIZER[kind], learning_momentum=0.0, regularization__weight_decay=0.0))
    none = _run(net, w0, grads, B=2, N=32)
    assert np.abs(none[2][:desc.total_weights] - want[2][:desc.total_weights]).max() > 1e-5   # the decay is visible
    assert_close(none[2][desc.total_weights:], want[2][desc.total_weights:], rel=1e-7, abs_=1e-9)  # ... on weights only


def test_warm_restarts_cosine_schedule_and_restart_side_effects():
    """plain gradient descent on g = 1: w moves by the rate of each step, eta_t = min + (max - min)/2 (1 + cos(pi t / T_i)) with t the
    number of updates since the last restart (Loshchilov & Hutter 2017, eq. 5).  The update that finds t >= T_i still uses the
    minimum, then clears the optimizer, multiplies T_i and decays the maximum."""
    lo, hi, Ti, mult, decay = 1e-3, 0.1, 4.0, 2.0, 0.5
    desc, net = _net(type_optimizer_function=mb.OPTIMIZER["GD"], learning_rate=0.01, learning_momentum=0.9, use_Warm_Restarts=1,
                     warm_restarts_minimum_learning_rate=lo, warm_restarts_maximum_learning_rate=hi, warm_restarts_T_i=Ti,
                     warm_restarts_multiplier=mult, warm_restarts_decay_learning_rate=decay)
    P = desc.total_parameters
    h = net.get_hyper(); h.learning_momentum = 0.0; net.set_hyper(h)
    net.upload_parameters(np.zeros(P, dtype=np.float32)); net.Clear_Training_Arrays()
    moved, t, cyc_T, cyc_hi = 0.0, 0, Ti, hi
    for step in range(16):
        net.upload_gradient(np.ones(P, dtype=np.float32)); net.Update_Parameter(2, 2)
        moved += lo + 0.5 * (cyc_hi - lo) * (1 + math.cos(math.pi * t / cyc_T))
        if t >= cyc_T:
            t, cyc_T, cyc_hi = 0, cyc_T * mult, max(cyc_hi * decay, lo)
        t += 1
        assert_close(net.download_parameters(), np.full(P, -moved), rel=3e-6, abs_=1e-8, what="update %d" % step)
        g = net.get_hyper()
        assert g.optimizer_time_step == t and g.warm_restarts_T_i == cyc_T
        assert abs(g.warm_restarts_maximum_learning_rate - cyc_hi) < 1e-7
    assert cyc_T == Ti * mult * mult                                                # two restarts happened in 16 updates


def test_warm_restart_clears_the_moments_and_scales_the_adam_rate_but_not_its_decay():
    desc, net = _net(type_optimizer_function=mb.OPTIMIZER["ADAM"], adam_learning_rate=1e-3, use_Warm_Restarts=1,
                     warm_restarts_minimum_learning_rate=1e-4, warm_restarts_maximum_learning_rate=1e-2, warm_restarts_T_i=2.0)
    P = desc.total_parameters
    w0, grads = _data(P, steps=4, seed=4)
    net.upload_parameters(w0); net.Clear_Training_Arrays()
    for k in range(3):
        net.upload_gradient(grads[k]); net.Update_Parameter(2, 2)
    # the third update found t = 2 >= T_i: state cleared BEFORE its own moments were written
    m = net.download_optimizer_state(mb.OPT_STATE["FIRST_MOMENT"]).astype(np.float64)
    assert_close(m, 0.1 * grads[2].astype(np.float64), rel=1e-6, abs_=1e-9)
    assert net.get_hyper().optimizer_time_step == 1
    # first update of a run: rate = maximum; Adam's first step is rate * sign(g) (bias-corrected, eps ~ 0)
    net.upload_parameters(w0); net.Clear_Training_Arrays()
    h = net.get_hyper(); h.warm_restarts_T_i = 2.0; h.warm_restarts_maximum_learning_rate = 1e-2; net.set_hyper(h)
    net.upload_gradient(grads[0]); net.Update_Parameter(2, 2)
    assert_close(net.download_parameters().astype(np.float64) - w0, -1e-2 * np.sign(grads[0]), rel=1e-4, abs_=1e-9)
