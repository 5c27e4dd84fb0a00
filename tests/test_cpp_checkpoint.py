"""The reference's checkpoint text files written and read by the C++ adaptor (include/myea_nn_hip_io.hpp), driven by the host
program tests/cpp/checkpoint_check.cpp.  Without a device object (CPU): write, read into a second object, write again -
the files must be identical - and the key order of both files is held against the order the reference's loader consumes
(Neural_Network__Load.cpp, `tmp_line.find("...")` calls in sequence).  With a device (GPU): two training steps first, so
the parameters and the normalisation running statistics come from the device, and both objects' inference outputs must
agree bit for bit.  The reference ships no checkpoint file: the format itself is followed by reading, parity unpinned."""
import os
import subprocess

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
BIN = os.path.join(HERE, "cpp", "checkpoint_check")

# Load_Parameters (Neural_Network__Load.cpp:82-2321): the keys in the order they are read
GENERAL_KEYS = """learning_rate learning_rate_final learning_momentum learning_gamma use_Nesterov quickprop_decay quickprop_mu rprop_increase_factor
rprop_decrease_factor rprop_delta_min rprop_delta_max rprop_delta_zero sarprop_weight_decay_shift sarprop_step_error_threshold_factor sarprop_step_error_shift
sarprop_temperature sarprop_epoch adam_learning_rate adam_beta1 adam_beta2 adam_epsilon adam_bias_correction adam_gamma use_Warm_Restarts
warm_restarts_decay_learning_rate warm_restarts_maximum_learning_rate warm_restarts_minimum_learning_rate warm_restarts_initial_T_i warm_restarts_multiplier
type_optimizer_function type_loss_function type_accuracy_function bit_fail_limit pre_training_level use_clip_gradient clip_gradient
regularization__max_norm_constraints regularization__l1 regularization__l2 regularization__srip regularization__weight_decay use_normalized_weight_decay
normalization_momentum_average normalization_epsilon batch_renormalization_r_correction_maximum batch_renormalization_d_correction_maximum loss_training
loss_validating loss_testing accuracy_variance accuracy_training accuracy_validating accuracy_testing use_CUDA use_OpenMP percentage_maximum_thread_usage
maximum_batch_size""".split()
# Load (:2323-3460): the header of the dimension file and the input layer
DIMENSION_HEAD = """type_network number_layers number_recurrent_depth number_time_delays use_first_layer_as_input use_last_layer_as_output total_basic_units
total_basic_indice_units total_neuron_units total_AF_units total_AF_Ind_recurrent_units total_block_units total_cell_units total_normalized_units total_parameters
total_weights total_bias type_layer type_activation type_dropout dropout_values[0] dropout_values[1] dropout_values[2] number_inputs""".split()
# a hidden fully-connected layer up to its neurons (:3488-4480)
HIDDEN_FC = """type_layer use_bidirectional type_activation type_dropout use_coded_dropout dropout_values[0] dropout_values[1] dropout_values[2] type_normalization
use_layer_normalization_before_activation number_normalized_units""".split()
HIDDEN_FC_TAIL = "use_tied_parameter k_sparsity alpha_sparsity constraint_recurrent_weight_lower_bound constraint_recurrent_weight_upper_bound number_neuron_units".split()


def _run(tmp_path, kind, device):
    out = subprocess.run([BIN, str(tmp_path), kind] + (["device"] if device else []), capture_output=True, text=True, timeout=120)
    assert out.returncode == 0 and "OK" in out.stdout, out.stdout + out.stderr
    return out.stdout


def _keys(path):
    """first token of every 'key value' line"""
    keys = []
    for line in open(path):
        parts = line.split()
        if len(parts) == 2 and not parts[0].startswith("|") and not parts[1].endswith(":"):
            keys.append(parts[0])
    return keys


def _check_files(tmp_path, kind):
    assert _keys(tmp_path / "a.nn") == GENERAL_KEYS
    text = open(tmp_path / "a.nn").read()
    assert text.startswith("|===| GRADIENT DESCENT PARAMETERS |===|\n") and text.endswith("|END| COMPUTATION PARAMETERS |END|\n")
    keys = _keys(tmp_path / "a.net")
    assert keys[:len(DIMENSION_HEAD)] == DIMENSION_HEAD
    lines = open(tmp_path / "a.net").read().split("\n")
    assert lines[0] == "|===| DIMENSION |===|" and lines[-2] == "|END| DIMENSION |END|" and "  Input layer:" in lines and "  Output layer:" in lines
    if kind == "mlp":
        at = lines.index("  Hidden layer 1:")
        got = [l.split()[0] for l in lines[at + 1:] if len(l.split()) == 2]
        assert got[:len(HIDDEN_FC)] == HIDDEN_FC
        rest = [k for k in got[len(HIDDEN_FC):] if k not in ("scale", "shift", "mean_average[0]", "variance_average[0]")]
        assert rest[:len(HIDDEN_FC_TAIL)] == HIDDEN_FC_TAIL
        # a Gaussian layer's value is written as the probability it was set with (0.2), not the spread kept in memory
        assert any(l.startswith("      dropout_values[0] 0.2") for l in lines[at:at + 10])
        assert "    number_basic_indice_units 9" in lines            # ceil mode is not in the file; the width is
        assert "    k_sparsity 4" in lines and "    alpha_sparsity 2" in lines
    if kind == "recurrent":
        assert "          connected_to_cell 0" in lines and "        connected_to_AF_Ind_R 0" in lines and "    number_block_units 4" in lines and "    number_cell_units 8" in lines
        assert "    constraint_recurrent_weight_upper_bound 0.75" in lines and "number_time_delays 1" in lines
        assert "    number_bias_parameters 12" in lines              # an LSTM layer writes its 3 x blocks gate biases
    if kind == "normalised":
        # 6 blocks of one cell: 54 normalised units, written block by block (the cell's three, then the block's six)
        assert "      number_normalized_units 54" in lines and "        NormU[53]" in lines and sum(l.split()[:1] == ["mean_average[2]"] for l in lines) == 54
        at = lines.index("        NormU[0]")
        p = np.fromfile(str(tmp_path / "params.bin"), dtype=np.float32)
        head = [l.split() for l in lines if l.startswith("total_weights") or l.startswith("total_bias")]
        base = int(head[0][1]) + int(head[1][1]) + 5   # the input layer's five units come first in the scale region
        scales = [np.float32(l.split()[1]) for l in lines[at:] if l.split()[:1] == ["scale"]]
        assert len(scales) == 54
        for u, v in enumerate(scales):   # unit u = 9 * block + group keeps its scale at group * 6 + block
            assert v == p[base + (u % 9) * 6 + u // 9], u
    if kind == "recurrent_residual":
        # a member's recurrent units sit on its input side; the block's first member owns none
        assert "    block_depth 3" in lines and "    number_block_units 8" in lines and sum(l.strip().startswith("connected_to_AF_Ind_R") for l in lines) >= 8
    if kind == "residual":
        assert "    block_depth 2" in lines and "    padding 1" in lines and "    number_basic_units 14" in lines and "          connected_to_basic 0" in lines
    # every weight line carries its flat index: the values are the parameters at those indices
    p = np.fromfile(str(tmp_path / "params.bin"), dtype=np.float32)
    seen = 0
    for l in lines:
        parts = l.split()
        if len(parts) == 2 and parts[0].startswith("weight["):
            i = int(parts[0][7:-1])
            assert np.float32(parts[1]) == p[i], (i, parts[1], p[i])
            seen += 1
    assert seen > 100


@pytest.mark.parametrize("kind", ["mlp", "recurrent", "normalised", "residual", "recurrent_residual"])
def test_checkpoint_round_trip_on_the_host(tmp_path, kind):
    _run(tmp_path, kind, device=False)
    _check_files(tmp_path, kind)


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["mlp", "recurrent", "normalised", "residual", "recurrent_residual"])
def test_checkpoint_round_trip_through_the_device(tmp_path, kind):
    out = _run(tmp_path, kind, device=True)
    assert "inference outputs" in out and "differing 0 magnitude" in out
    _check_files(tmp_path, kind)
    if kind != "recurrent":      # the running statistics moved away from their initial 0 / 1 and were written
        means = [float(l.split()[1]) for l in open(tmp_path / "a.net") if l.split()[:1] == ["mean_average[0]"]]
        assert means and any(m != 0 for m in means)
