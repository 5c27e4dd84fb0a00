"""Seeded synthetic parameters and labels in the reference's layouts, for benchmarks, smoke runs and tests."""
import numpy as np

from myea_amd import binding as mb


def glorot_parameters(desc, seed, bias_range=0.1):
    """Glorot-uniform weights per FC layer written into the flat vector; small random biases so that the
    bias path is exercised; scales near 1, shifts near 0 for normalised layers."""
    rng = np.random.default_rng(seed)
    w = np.zeros(desc.total_parameters, dtype=np.float32)
    widths = []
    for i in range(desc.n_layers):
        l = desc.layers[i]
        widths.append(l.n_units * (l.n_cells_per_block if l.type_layer == mb.LAYER_LSTM else 1))
    for i in range(1, desc.n_layers):
        l = desc.layers[i]
        fan_in, fan_out = widths[i - 1], widths[i]
        n = l.last_connection_index - l.first_connection_index
        if n == 0:
            continue  # residual layer: owns no connection
        fan_out = l.n_units * (l.n_cells_per_block if l.type_layer == mb.LAYER_LSTM else 1)
        fan_in = n // fan_out if l.type_layer != mb.LAYER_LSTM else fan_in
        r = np.sqrt(6.0 / (fan_in + fan_out))
        w[l.first_connection_index:l.last_connection_index] = rng.uniform(-r, r, n).astype(np.float32)
    nb = desc.total_bias
    w[desc.total_weights:desc.total_weights + nb] = rng.uniform(-bias_range, bias_range, nb).astype(np.float32)
    tn = desc.total_normalized_units
    if tn:
        base = desc.total_weights + desc.total_bias
        w[base:base + tn] = rng.uniform(0.5, 1.5, tn).astype(np.float32)
        w[base + tn:base + 2 * tn] = rng.uniform(-0.2, 0.2, tn).astype(np.float32)
    return w


def one_hot(labels, n):
    y = np.zeros((len(labels), n), dtype=np.float32)
    y[np.arange(len(labels)), labels] = 1.0
    return y
