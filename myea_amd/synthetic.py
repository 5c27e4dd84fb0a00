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


def simple_debug_layers(inputs=28, outputs=10, units=32, blocks_per_group=3, block_depth=3, widening=-9, normalization="BATCH_NORMALIZATION"):
    """The network the reference's worked example builds (Neural_Network_Launcher_Windows/Source_Files/debug.cpp:81-87, 727-1075):
    an independently recurrent first hidden layer, then three groups of residual blocks whose members are independently recurrent
    layers, a max pooling (kernel 2, stride 2, dilation 0) between the groups, every block `widening / (3 * blocks_per_group)`
    units wider than the one before; ISRLU members, batch normalisation on every hidden and residual layer (before the
    activation), a softmax head.  sMNIST rows: 28 inputs per time step."""
    norm = dict(normalization=normalization, norm_before=True) if normalization != "NONE" else {}
    member = lambda n: dict(type="ind_rnn", units=int(n), activation="ISRLU", **norm)
    layers = [dict(units=inputs), member(units)]
    width, step = float(units), widening / (3.0 * blocks_per_group)
    for group in range(3):
        if group:
            layers.append(dict(type="max_pooling", kernel=2, stride=2, padding=0, dilation=0))
        for _ in range(blocks_per_group):
            width += step
            block = dict(type="residual", block_depth=block_depth)
            if normalization != "NONE":
                block["normalization"] = normalization
            layers.append(block)
            layers += [member(width)] * block_depth
    layers.append(dict(units=outputs, activation="SOFTMAX"))
    return layers
