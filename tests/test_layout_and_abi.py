"""Host-side logic of the C ABI: the index table of myea_net_desc_layout (checked against hand counts that follow
Neural_Network::Compile), defaults, and that the built library exports every declared symbol.  CPU only: no
compute entry point is called."""
import ctypes as C
import os
import re

import numpy as np
import pytest

from myea_amd import binding as mb
from tests.common import oracle_desc, oracle_hyper

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_hyper_defaults_are_the_reference_public_fields():
    h = oracle_hyper()
    assert (h.learning_rate, h.learning_momentum, h.learning_rate_final, h.learning_gamma) == pytest.approx((0.01, 0.9, 0.1, 1e-3))
    assert (h.adam_learning_rate, h.adam_beta1, h.adam_beta2, h.adam_epsilon) == pytest.approx((1e-3, 0.9, 0.999, 1e-8))
    assert (h.clip_gradient, h.accuracy_variance, h.bit_fail_limit) == pytest.approx((1.0, 0.49, 0.35))
    assert (h.normalization_momentum_average, h.normalization_epsilon) == pytest.approx((0.999, 1e-5))
    assert h.batch_renormalization_r_correction_maximum == 1.0 and h.batch_renormalization_d_correction_maximum == 0.0
    assert h.use_adam_bias_correction == 1 and h.use_Nesterov == 0 and h.use_clip_gradient == 0 and h.optimizer_time_step == 0


def test_layout_feedforward_mlp():
    d = oracle_desc([dict(units=784), dict(units=256, activation="TANH"), dict(units=10, activation="SIGMOID")], 128)
    assert d.total_weights == 784 * 256 + 256 * 10 and d.total_bias == 266
    assert d.total_normalized_units == 0 and d.total_parameters == d.total_weights + 266
    assert d.layers[1].first_connection_index == 0 and d.layers[1].last_connection_index == 784 * 256
    assert d.layers[2].first_connection_index == 784 * 256
    assert d.layers[1].first_bias_connection_index == d.total_weights
    assert d.layers[2].first_bias_connection_index == d.total_weights + 256
    assert [d.layers[i].first_mask_index for i in range(3)] == [0, 784, 784 + 256] and d.total_mask_units == 1050


def test_layout_normalised_stack_owns_units_on_every_layer():
    """every layer (input layer included) owns Normalized_unit entries; the scale/shift region appears once any layer
    is normalised; normalised layers keep their (unused) bias slots."""
    d = oracle_desc([dict(units=6), dict(units=8, activation="RELU", normalization="BATCH_NORMALIZATION"),
                     dict(units=5, activation="RELU"), dict(units=3, activation="SOFTMAX")], 4)
    assert d.total_bias == 16 and d.total_normalized_units == 6 + 8 + 5 + 3
    assert [d.layers[i].first_normalized_unit_index for i in range(4)] == [0, 6, 14, 19]
    assert d.total_parameters == d.total_weights + 16 + 2 * 22
    d0 = oracle_desc([dict(units=6), dict(units=8, activation="RELU"), dict(units=3, activation="SOFTMAX")], 4)
    assert d0.total_normalized_units == 0


def test_layout_lstm_interleaved_blocks_and_bias_quirk():
    """per block: cells x [In | cells_per_layer], then i/f/o input rows, i/f/o recurrent rows, 3 x cells_per_block
    peepholes (Prepare__Connections__LSTM); biases: cells + 3 blocks, with first_bias_connection_index left one
    cell-count past the start of the slice (Prepare__Bias__LSTM)."""
    T = 3
    d = oracle_desc([dict(units=5), dict(type="lstm", units=4, cells_per_block=2), dict(type="lstm", units=3),
                     dict(units=2, activation="LINEAR")], 2, T)
    In, K, cpb = 5, 4, 2
    C_ = K * cpb
    per_block = cpb * (In + C_) + 3 * In + 3 * C_ + 3 * cpb
    assert d.layers[1].first_connection_index == 0 and d.layers[1].last_connection_index == K * per_block
    per_block2 = 1 * (C_ + 3) + 3 * C_ + 3 * 3 + 3
    assert d.layers[2].last_connection_index - d.layers[2].first_connection_index == 3 * per_block2
    assert d.layers[3].last_connection_index - d.layers[3].first_connection_index == 3 * 2
    W = d.total_weights
    assert d.total_bias == (C_ + 3 * K) + (3 + 3 * 3) + 2
    assert d.layers[1].first_bias_connection_index == W + C_
    assert d.layers[2].first_bias_connection_index == W + (C_ + 3 * K) + 3
    assert d.layers[3].first_bias_connection_index == W + (C_ + 3 * K) + (3 + 9)
    # LSTM layers own no AF unit: no mask slots; normalised-unit count is 3 cells + 6 blocks
    assert d.total_mask_units == (5 + 2) * T
    assert d.layers[2].first_normalized_unit_index == 5 + 3 * C_ + 6 * K


def test_layout_rejects_bad_descriptors():
    with pytest.raises(ValueError):
        oracle_desc([dict(units=4)], 2)
    with pytest.raises(ValueError):
        oracle_desc([dict(units=4), dict(units=0, activation="TANH")], 2)
    with pytest.raises(ValueError):
        oracle_desc([dict(units=4), dict(units=2, activation="TANH")], 0)


def test_library_exports_every_declared_symbol():
    """the HIP library must be built (python -m myea_amd.build); dlopen works without a GPU"""
    header = open(os.path.join(ROOT, "include", "myea_hip.h")).read()
    declared = set(re.findall(r"\b(myea_(?:hip_|net_desc_|hyper_)\w+)\s*\(", header))
    assert declared, "no declarations found"
    assert declared == set(mb.ABI_SYMBOLS)
    lib = C.CDLL(mb.LIB_PATH)
    for name in sorted(declared):
        assert hasattr(lib, name), name


def test_struct_sizes_match_the_header():
    """ctypes mirrors are laid out as the C structs (checked through the layout function writing the far end)"""
    d = oracle_desc([dict(units=3)] + [dict(units=2, activation="TANH")] * 63, 1)
    assert d.n_layers == 64 and d.layers[63].first_bias_connection_index == d.total_weights + 2 * 62
    assert C.sizeof(mb.LayerDesc) == 128 and C.sizeof(mb.Hyper) == 42 * 4 and C.sizeof(mb.LossState) == 64
