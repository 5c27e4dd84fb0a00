"""Checkers for the parity tests at the benchmark configurations' full sizes: how a gradient entry that is a sum of tens of
thousands of products is held against the fp32 CPU oracle, and how the step of an Adam-type optimizer is.

A weight-gradient entry is sum over (time step, example) of delta x input.  Two fp32 implementations that add those products
in different orders agree to rel 1e-4 / abs 1e-5 wherever the sum is not much smaller than its terms; where it is, neither
holds more digits than the terms allow, the reference's own path under another number of OpenMP threads included.  So an
entry outside the tolerance of the oracle is taken to float64: the exact sum of the very products (from the oracle's own
delta and input tensors) and the sum of their magnitudes.  It passes when it is within the tolerance of the exact sum, or
at least as near to it as the oracle's entry is, or within four fp32 units in the last place (2^-21) of the sum of
magnitudes - the products themselves are built from fp32 deltas and activations that agree between the two sides to a unit
or two in the last place, so no summation, however exact, can agree more closely than that.  No share of entries is
exempt."""
import numpy as np

from myea_amd import binding as mb

ULPS = 4 * 2.0 ** -23   # of the sum of the terms' magnitudes


def assert_sums_match(got, oracle, exact, what, rel=1e-4, abs_=1e-5, report=None):
    """exact(indices) -> (float64 sums, float64 sums of the terms' magnitudes) for the listed entries of the vector"""
    got, oracle = np.asarray(got, np.float64).ravel(), np.asarray(oracle, np.float64).ravel()
    assert got.shape == oracle.shape, (what, got.shape, oracle.shape)
    off = np.flatnonzero(np.abs(got - oracle) > abs_ + rel * np.abs(oracle))
    counts = dict(entries=got.size, outside_oracle_tolerance=int(off.size), within_exact=0, nearer_than_oracle=0, within_ulp_of_magnitudes=0)
    if off.size:
        truth, mags = exact(off)
        eg, eo = np.abs(got[off] - truth), np.abs(oracle[off] - truth)
        within = eg <= abs_ + rel * np.abs(truth)
        nearer = eg <= eo
        ulp = eg <= ULPS * mags
        counts.update(within_exact=int(within.sum()), nearer_than_oracle=int((~within & nearer).sum()), within_ulp_of_magnitudes=int((~within & ~nearer & ulp).sum()))
        bad = ~(within | nearer | ulp)
        if bad.any():
            i = int(np.argmax(np.where(bad, eg / np.maximum(mags, 1e-300), 0)))
            raise AssertionError("%s: %d of %d entries match neither the oracle nor the exact sum; entry %d: got %.9g oracle %.9g exact %.17g, magnitudes sum to %.6g"
                                 % (what, int(bad.sum()), got.size, int(off[i]), got[off[i]], oracle[off[i]], truth[i], mags[i]))
    if report is not None:
        report[what] = counts
    return counts


class GradientTerms:
    """The products behind every entry of the flat gradient of a stack of fully-connected and one-cell-per-block LSTM
    layers, read from a network's own tensors after Backward_Pass: for a flat index, the list of (u, v) vector pairs whose
    dot products add up to the entry (Update_Derivative_Weight__FC, NN/Neural_Network__Update_Derivative_Weight__OpenMP.cpp:
    178-242; the LSTM layer's, NN/Neural_Network__Recurrent_Update_Derivative_Weight__OpenMP.cpp:168-490: input weights take
    delta[t] x input[t], recurrent weights and the input / forget peepholes delta[next step] x (cell output / cell state)[t],
    the output peephole delta[t] x cell state[t], biases the deltas themselves)."""

    def __init__(self, desc, net, X, B):
        self.desc, self.net, self.B = desc, net, B
        self.T, self.Bmax = desc.number_recurrent_depth, desc.batch_size
        self.cache = {}
        In = desc.layers[0].n_units
        self.cache[("out", 0, 0)] = np.ascontiguousarray(np.asarray(X, np.float32).reshape(B, self.T, In).transpose(1, 0, 2))
        self.ranges = []   # (first, end, kind, layer, direction)
        for li in range(1, desc.n_layers):
            l = desc.layers[li]
            W, Win = self.width(li), self.width(li - 1)
            if l.type_layer == mb.LAYER_FULLY_CONNECTED:
                self.ranges.append((l.first_connection_index, l.first_connection_index + W * Win, "fc_w", li, 0))
                self.ranges.append((l.first_bias_connection_index, l.first_bias_connection_index + W, "fc_b", li, 0))
            elif l.type_layer == mb.LAYER_LSTM:
                assert l.n_cells_per_block == 1
                C = l.n_units
                per_block, G = 4 * (Win + C) + 3, 4 * C
                for direction in range(2 if l.use_bidirectional else 1):
                    first = l.first_connection_index + direction * C * per_block
                    self.ranges.append((first, first + C * per_block, "lstm_w", li, direction))
                    b0 = l.first_bias_connection_index + direction * G
                    self.ranges.append((b0, b0 + G, "lstm_b", li, direction))
            else:
                raise NotImplementedError(l.type_layer)

    def width(self, li):
        l = self.desc.layers[li]
        return l.n_units * (l.n_cells_per_block if l.type_layer == mb.LAYER_LSTM else 1)

    def tensor(self, name, li, direction=0):
        key = (name, li, direction)
        if key not in self.cache:
            kind = mb.TENSOR[{"out": "OUTPUTS", "delta": "ERRORS", "dz": "LSTM_DELTA_CELL_INPUT", "di": "LSTM_DELTA_INPUT_GATE", "df": "LSTM_DELTA_FORGET_GATE",
                              "do": "LSTM_DELTA_OUTPUT_GATE", "c": "LSTM_CELL_STATE", "h": "LSTM_CELL_OUTPUT"}[name]]
            if direction:
                kind |= mb.TENSOR["DIRECTION_BACKWARD"]
            a = np.asarray(self.net.download_tensor(li, kind))
            self.cache[key] = a.reshape(self.T, self.Bmax, -1)[:, :self.B]
        return self.cache[key]

    def pairs(self, index):
        """every (u, v) whose dot product is added into gradient[index] (bias slots of neighbouring layers may overlap)"""
        found = []
        for first, end, kind, li, direction in self.ranges:
            if not first <= index < end:
                continue
            at = index - first
            Win = self.width(li - 1)
            x = self.tensor("out", li - 1)
            if kind == "fc_w":
                found.append((self.tensor("delta", li)[:, :, at // Win], x[:, :, at % Win]))
            elif kind == "fc_b":
                found.append((self.tensor("delta", li)[:, :, at], None))
            elif kind == "lstm_b":
                C = self.width(li)
                found.append((self.tensor(("dz", "di", "df", "do")[at // C], li, direction)[:, :, at % C], None))
            else:
                C = self.width(li)
                k, r = divmod(at, 4 * (Win + C) + 3)
                # delta of the step processed next in the direction's own order against the state of the current one
                nxt = (lambda a: a[:-1]) if direction else (lambda a: a[1:])
                cur = (lambda a: a[1:]) if direction else (lambda a: a[:-1])
                d = lambda name: self.tensor(name, li, direction)[:, :, k]
                if r < Win:
                    found.append((d("dz"), x[:, :, r]))
                elif r < Win + C:
                    found.append((nxt(d("dz")), cur(self.tensor("h", li, direction)[:, :, r - Win])))
                elif r < 4 * Win + C:
                    g, a = divmod(r - Win - C, Win)
                    found.append((d(("di", "df", "do")[g]), x[:, :, a]))
                elif r < 4 * Win + 4 * C:
                    g, a = divmod(r - 4 * Win - C, C)
                    found.append((nxt(d(("di", "df", "do")[g])), cur(self.tensor("h", li, direction)[:, :, a])))
                else:
                    g = r - 4 * Win - 4 * C
                    c = self.tensor("c", li, direction)[:, :, k]
                    found.append((d("do"), c) if g == 2 else (nxt(d(("di", "df")[g])), cur(c)))
        return found   # empty for a bias slot no layer writes (the LSTM bias addressing leaves some)

    def exact(self, indices):
        sums, mags = np.zeros(len(indices)), np.zeros(len(indices))
        for n, index in enumerate(indices):
            for u, v in self.pairs(int(index)):
                u = np.asarray(u, np.float64).ravel()
                v = np.ones_like(u) if v is None else np.asarray(v, np.float64).ravel()
                sums[n] += float(u @ v)
                mags[n] += float(np.abs(u) @ np.abs(v))
        return sums, mags


def _clip_factor(first_moment, gradient, beta1):
    """the factor s a clipped update applied, read back from its first moment m = (1 - beta1) s g on the entries with the
    largest gradients"""
    top = np.argsort(np.abs(gradient))[-4096:]
    return float(np.median(first_moment[top] / ((1.0 - beta1) * gradient[top])))


def assert_first_adam_type_step_matches(gpu, cpu, twin, w, g_gpu, g_cpu, B, h, kinds, what, rel=1e-4, abs_=1e-5):
    """Update_Parameter from cleared optimizer state on three networks that hold the same parameters `w`: the device (its own
    gradient g_gpu), the oracle (its own gradient g_cpu) and a second oracle network `twin` that is handed the device's
    gradient.
    (a) Device against twin - the same gradient on both sides, so the update arithmetic alone: every parameter and every
        entry of the optimizer vectors `kinds`, rel 1e-5.
    (b) Device against oracle, each from its own gradient: parameters within rel / abs and the optimizer vectors within the
        tolerance the gradient's own tolerance turns into (first moment (1 - beta1) s g, second moment (1 - beta2) (s g)^2,
        s the clipping factor), wherever the two gradients agree within rel / abs and the gradient is not below its own
        absolute tolerance.  An Adam-type step has the size lr whatever |g| is, so where |g| < abs_ - rounding noise of
        either side - the step's direction is noise too: those parameters are held to the step's bound, 2.1 lr.
    With clipping by the global norm every step carries one more scalar, s = clip / |g|, and |g| is an fp32 sum over all
    parameters: the reference's serial loop over ten million squares stops taking in addends below half a unit in the last
    place of its running sum (its OpenMP build, which sums per thread, lands elsewhere again), so its s is off in the fourth
    digit.  The factor is therefore held on its own - the device's must be at least as near to clip / (the float64 norm) as
    the oracle's, or within 1e-6 of it - and taken out of the entrywise comparisons of the optimizer vectors; the
    parameters are compared as they are (an Adam-type step barely depends on the gradient's scale) and, in (a), also
    against the float64 closed form of the step from the device's own optimizer vectors."""
    twin.upload_gradient(g_gpu)
    for n in (gpu, cpu, twin):
        n.Update_Parameter(B, B)
    wg, wc, wt = (n.download_parameters().astype(np.float64) for n in (gpu, cpu, twin))
    gg, gc = np.asarray(g_gpu, np.float64), np.asarray(g_cpu, np.float64)
    b1, b2 = float(h.adam_beta1), float(h.adam_beta2)
    states = {kind: tuple(n.download_optimizer_state(mb.OPT_STATE[kind]).astype(np.float64) for n in (gpu, cpu, twin)) for kind in kinds}
    clipped = bool(h.use_clip_gradient)
    s_gpu = s_cpu = s_twin = 1.0
    report = {}
    if clipped:
        m = states["FIRST_MOMENT"]
        s_gpu, s_cpu, s_twin = _clip_factor(m[0], gg, b1), _clip_factor(m[1], gc, b1), _clip_factor(m[2], gg, b1)
        exact = min(1.0, float(h.clip_gradient) / float(np.sqrt((gg * gg).sum())))
        err_gpu, err_twin = abs(s_gpu / exact - 1.0), abs(s_twin / exact - 1.0)
        assert err_gpu <= max(1e-6, err_twin), "%s: clipping factor %.9g, exact %.9g, oracle %.9g" % (what, s_gpu, exact, s_twin)
        report.update(clip_factor_error=err_gpu, oracle_clip_factor_error=err_twin)
    e = np.abs(wg - wt)
    arel, aabs = (rel, abs_) if clipped else (1e-5, 1e-7)
    assert not (e > aabs + arel * np.abs(wt)).any(), "%s: update arithmetic: %d parameters differ, worst %.3g" % (what, int((e > aabs + arel * np.abs(wt)).sum()), float(e.max()))
    agree = np.abs(gg - gc) <= abs_ + rel * np.abs(gc)
    strict = (agree & (np.abs(gc) >= abs_)) | ((gg == 0) & (gc == 0))
    e = np.abs(wg - wc)
    bad = strict & (e > abs_ + rel * np.abs(wc))
    assert not bad.any(), "%s: %d parameters differ from the oracle's, worst %.3g" % (what, int(bad.sum()), float(e[bad].max()))
    lr = float(h.adam_learning_rate)
    assert float(np.abs(wg - w)[~strict].max(initial=0.0)) <= 2.1 * lr, "%s: a parameter with a noise-level gradient moved by more than a step" % what
    for kind in kinds:
        a, b, t = states[kind]
        power = 1 if kind == "FIRST_MOMENT" else 2
        t = t * (s_gpu / s_twin) ** power     # the clipping factors taken out (1 without clipping)
        b = b * (s_gpu / s_cpu) ** power
        e = np.abs(a - t)
        assert not (e > 1e-30 + 1e-5 * np.abs(t)).any(), "%s: update arithmetic: optimizer vector %s: %d entries differ" % (what, kind, int((e > 1e-30 + 1e-5 * np.abs(t)).sum()))
        if kind == "FIRST_MOMENT":
            tol = 1.1 * rel * np.abs(b) + (1.0 - b1) * s_gpu * 1.1 * abs_
        else:
            tol = 2.2 * rel * np.abs(b) + (1.0 - b2) * s_gpu * s_gpu * (2.1 * np.abs(gc) * abs_ + abs_ * abs_)
        bad = agree & (np.abs(a - b) > tol)
        assert not bad.any(), "%s: optimizer vector %s: %d entries differ from the oracle's" % (what, kind, int(bad.sum()))
    if clipped and h.type_optimizer_function == mb.OPTIMIZER["ADABOUND"]:
        # Update_Parameters__AdaBound (NN/Neural_Network__AdaBound.cpp:43-110), first step, from the device's own vectors
        m, v = states["FIRST_MOMENT"][0], states["SECOND_MOMENT"][0]
        lr_t = lr * np.sqrt(1.0 - b2) / (1.0 - b1) if h.use_adam_bias_correction else lr
        lo = float(h.learning_rate_final) * (1.0 - 1.0 / (float(h.learning_gamma) + 1.0))
        hi = float(h.learning_rate_final) * (1.0 + 1.0 / float(h.learning_gamma))
        want = w - np.clip(lr_t / (np.sqrt(v) + float(h.adam_epsilon)), lo, hi) * m
        e = np.abs(wg - want)
        assert not (e > 1e-7 + 1e-5 * np.abs(want)).any(), "%s: parameters against the closed form of the step: %d differ, worst %.3g" % (what, int((e > 1e-7 + 1e-5 * np.abs(want)).sum()), float(e.max()))
    report.update(parameters=int(wg.size), compared_strictly=int(strict.sum()), noise_level_or_disagreeing_gradients=int((~strict).sum()))
    return report
