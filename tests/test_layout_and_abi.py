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


def test_layout_two_direction_lstm_config5_shape_by_hand():
    """Config 5's shape: input 256, a two-direction LSTM of 1024 blocks x 1 cell, a 32-way head, T = 512, counted by hand
    from Prepare__Connections__LSTM (NN/Neural_Network__Prepare_Connections.cpp:79-222) and Prepare__Bias__LSTM (:238-252).
    Per block and direction: 1 cell row over [In | cells] = 256 + 1024, three gate rows over the inputs = 3 x 256, three over
    the cell outputs = 3 x 1024, 3 peepholes -> 5123; 1024 blocks x 2 directions.  Biases: per direction 1024 cells + 3 x 1024
    gates = 4096; the two directions' halves lie one after the other from the slice's start."""
    d = oracle_desc([dict(units=256), dict(type="lstm", units=1024, bidirectional=True), dict(units=32, activation="SOFTMAX")], 64, 512)
    per_block = 1 * (256 + 1024) + 3 * 256 + 3 * 1024 + 3
    assert per_block == 5123
    lstm_weights = 2 * 1024 * per_block
    assert lstm_weights == 10491904
    assert (d.layers[1].first_connection_index, d.layers[1].last_connection_index) == (0, lstm_weights)
    # the head reads the summed outputs of the two directions: 1024 wide, not 2048
    assert (d.layers[2].first_connection_index, d.layers[2].last_connection_index) == (lstm_weights, lstm_weights + 32 * 1024)
    assert d.total_weights == 10491904 + 32768 == 10524672
    assert d.total_bias == 2 * 4096 + 32 == 8224
    assert d.layers[1].first_bias_connection_index == d.total_weights              # forward half: [W, W + 4096)
    assert d.layers[2].first_bias_connection_index == d.total_weights + 2 * 4096   # backward half: [W + 4096, W + 8192)
    assert d.total_normalized_units == 0 and d.total_parameters == 10524672 + 8224
    # masks: input units and head units per time step; the LSTM layer owns no activation unit
    assert d.total_mask_units == (256 + 32) * 512 and [d.layers[i].first_mask_index for i in range(3)] == [0, 256 * 512, 256 * 512]


def test_layout_normalised_dense_layers_around_lstm_layers_by_hand():
    """Scale / shift offsets of a normalised dense layer below and above LSTM layers: every layer owns entries in layer order
    (Prepare__Normalized__Layers, NN/Neural_Network__Layer_Normalization.cpp:20-78) - a dense layer one per unit, an LSTM
    layer 3 per cell and 6 per block and direction."""
    d = oracle_desc([dict(units=7),
                     dict(units=6, activation="TANH", normalization="BATCH_NORMALIZATION"),
                     dict(type="lstm", units=4, cells_per_block=2),
                     dict(type="lstm", units=3, bidirectional=True),
                     dict(units=5, activation="RELU", normalization="BATCH_RENORMALIZATION"),
                     dict(units=2, activation="LINEAR")], 3, 4)
    owned = [7, 6, 3 * 8 + 6 * 4, 2 * (3 * 3 + 6 * 3), 5, 2]
    assert owned == [7, 6, 48, 54, 5, 2]
    assert [d.layers[i].first_normalized_unit_index for i in range(6)] == [0, 7, 13, 61, 115, 120]
    assert d.total_normalized_units == 122
    # weights: dense 6 x 7; LSTM 4 blocks x (2 (6 + 8) + 3 x 6 + 3 x 8 + 3 x 2 = 76); two-direction LSTM 2 x 3 x (1 (8 + 3) + 3 x 8 + 3 x 3 + 3 = 47);
    # dense 5 x 3 (the directions' outputs are summed); head 2 x 5
    assert [d.layers[i].first_connection_index for i in range(1, 6)] == [0, 42, 42 + 304, 42 + 304 + 282, 42 + 304 + 282 + 15]
    assert d.total_weights == 42 + 304 + 282 + 15 + 10 == 653
    # biases: 6 | 8 cells + 12 gates (field left 8 past the slice's start) | 2 x (3 + 9) from the slice's start | 5 | 2
    assert d.total_bias == 6 + 20 + 24 + 5 + 2 == 57
    assert [d.layers[i].first_bias_connection_index - d.total_weights for i in range(1, 6)] == [0, 6 + 8, 26, 50, 55]
    # scale and shift of layer 4 in the flat parameter vector
    scale0 = d.total_weights + d.total_bias
    assert scale0 + d.layers[4].first_normalized_unit_index == 653 + 57 + 115
    assert d.total_parameters == 653 + 57 + 2 * 122


def test_layout_pooling_and_residual_mix_by_hand():
    """A max-pooling layer (owns no weights, biases, normalised units or masks; width from Assign__Post__Layer,
    NN/Neural_Network__Compile.cpp:250-271) in front of a residual block of two members whose normalised units and masks sit
    on their input sides (Prepare__Normalized__Residual_Layer; Assign__Post__Residual_Layer, :378-384)."""
    layers = [dict(units=20),
              dict(units=16, activation="RELU"),
              dict(type="max_pooling", kernel=2, stride=2),                     # floor((16 - 1 (2 - 1) - 1) / 2 + 1) = 8
              dict(type="residual", block_depth=2),
              dict(units=8, activation="RELU", normalization="BATCH_NORMALIZATION"),
              dict(units=8, activation="RELU", normalization="BATCH_NORMALIZATION"),
              dict(units=4, activation="SOFTMAX")]
    d = oracle_desc(layers, 5)
    W = [20 * 16, 0, 0, 8 * 8, 8 * 8, 8 * 4]
    assert [d.layers[i].last_connection_index - d.layers[i].first_connection_index for i in range(1, 7)] == W
    assert d.total_weights == 320 + 64 + 64 + 32 == 480
    assert d.total_bias == 16 + 8 + 8 + 4 == 36
    assert [d.layers[i].first_bias_connection_index - 480 for i in (1, 4, 5, 6)] == [0, 16, 24, 32]
    # normalised units: input 20 | dense 16 | pooling 0 | residual layer = its last member's width 8 | members: fan-in wide 8, 8 | head 4
    assert [d.layers[i].first_normalized_unit_index for i in range(7)] == [0, 20, 36, 36, 44, 52, 60]
    assert d.total_normalized_units == 64 and d.total_parameters == 480 + 36 + 128
    # masks: 20 | 16 | - | - | first member none | second member its fan-in 8 | head 4
    assert [d.layers[i].first_mask_index for i in range(7)] == [0, 20, 36, 36, 36, 36, 44] and d.total_mask_units == 48


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


def test_adaptor_dropout_bernoulli_draws_on_the_host():
    """Neural_Network_HIP::Dropout_Bernoulli (host only, no device object): BERNOULLI layers get new draws in the reference's
    order from a std::mt19937 / std::bernoulli_distribution pair, BERNOULLI_INVERTED layers keep their masks, a retention
    probability of 0 clears the layer (NN/Neural_Network__Dropout__Bernoulli__Loop.cpp:33-97).  The check program makes the same
    draws itself and compares."""
    import subprocess
    binary = os.path.join(ROOT, "tests", "cpp", "adaptor_check")
    if not os.path.exists(binary):
        pytest.skip("tests/cpp/adaptor_check is not built (python -m myea_amd.build)")
    out = subprocess.run([binary, "/tmp", "dropout"], capture_output=True, text=True, timeout=60)
    assert out.returncode == 0 and "dropout ok" in out.stdout, out.stdout + out.stderr
