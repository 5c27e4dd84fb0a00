"""ctypes view of include/myea_hip.h: the structs, enum values and a thin handle class.

This is plumbing for Python callers (tests, the benchmark); the product is the shared library
`csrc/libmyea_hip.so`.  Loading fails loudly when the library has not been built: there is no
CPU fallback on this path.
"""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "csrc", "libmyea_hip.so")

MAX_LAYERS = 64

# ---- enum values (Common_Library/include/Enums of the reference) ----
LAYER_FULLY_CONNECTED, LAYER_LSTM, LAYER_RESIDUAL = 4, 8, 10
LAYER_AVERAGE_POOLING, LAYER_MAX_POOLING = 1, 9
LAYER_FULLY_CONNECTED_INDEPENDENTLY_RECURRENT = 5
NETWORK_FEEDFORWARD, NETWORK_RECURRENT = 3, 4
AF = dict(NONE=0, COSINE=1, COSINE_SYMMETRIC=2, ELU=3, ELLIOT=4, ELLIOT_SYMMETRIC=5, GAUSSIAN=6,
          GAUSSIAN_STEPWISE=7, GAUSSIAN_SYMMETRIC=8, ISRU=9, ISRLU=10, LINEAR=11, LINEAR_PIECE=12,
          LINEAR_PIECE_SYMMETRIC=13, LEAKY_RELU=14, PARAMETRIC_RELU=15, RELU=16, SELU=17, SIGMOID=18,
          SINE=19, SIGMOID_STEPWISE=20, SINE_SYMMETRIC=21, SOFTMAX=22, TANH=23, TANH_STEPWISE=24,
          THRESHOLD=25, THRESHOLD_SYMMETRIC=26)
OPTIMIZER = dict(NONE=0, ADABOUND=1, ADAM=2, AMSBOUND=4, AMSGRAD=5, GD=6, IRPROP_MINUS=7, IRPROP_PLUS=8, NOSADAM=9)
DROPOUT = dict(NONE=0, BERNOULLI=2, BERNOULLI_INVERTED=3, GAUSSIAN=4, SHAKEDROP=5, UOUT=6, ZONEOUT=7)
NORMALIZATION = dict(NONE=0, BATCH_NORMALIZATION=1, BATCH_RENORMALIZATION=2)
LOSS = dict(NONE=0, BIT=1, CROSS_ENTROPY=2, L1=3, L2=4, MAE=5, MAPE=6, ME=9, MSE=10, RMSE=11, SMAPE=12)
ACCURACY = dict(NONE=0, CROSS_ENTROPY=1, DIRECTIONAL=2, DISTANCE=3, R=4, SIGN=5)
STATE_INFERENCE, STATE_TRAINING = 0, 1
OPT_STATE = dict(PREVIOUS_DELTA=0, FIRST_MOMENT=1, SECOND_MOMENT=2, SECOND_MOMENT_HAT=3, PREVIOUS_STEPS=4, PREVIOUS_DERIVATIVES=5)
TENSOR = dict(OUTPUTS=0, SUMMATIONS=1, ERRORS=2, NORM_HATS=3, NORM_MEANS=4, NORM_VARIANCES=5,
              NORM_MEANS_AVERAGES=6, NORM_VARIANCES_AVERAGES=7, INPUT_SIDE_ERRORS=8, DROPOUT_NOISE=9,
              LSTM_CELL_INPUT=16, LSTM_CELL_STATE=17, LSTM_INPUT_GATE=18, LSTM_FORGET_GATE=19,
              LSTM_OUTPUT_GATE=20, LSTM_DELTA_CELL_INPUT=21, LSTM_DELTA_CELL_STATE=22,
              LSTM_DELTA_INPUT_GATE=23, LSTM_DELTA_FORGET_GATE=24, LSTM_DELTA_OUTPUT_GATE=25, LSTM_CELL_OUTPUT=26, LSTM_DELTA_CELL_OUTPUT=27,
              DIRECTION_BACKWARD=0x100)


def TENSOR_LSTM_NORM_GROUP(group):
    """OR-ed onto a NORM_* kind (or ERRORS) of a normalised LSTM layer: one of its nine groups of normalised units, 0 block
    input from below, 1 block input recurrent, 2 cell state, 3 / 4 input gate, 5 / 6 forget gate, 7 / 8 output gate"""
    return (group + 1) << 12
E_INVALID, E_UNSUPPORTED, E_BATCH, E_STATE, E_NOMEM, E_DEVICE = -1, -2, -3, -4, -5, -6


class LayerDesc(C.Structure):
    _fields_ = [
        ("type_layer", C.c_uint32), ("n_units", C.c_uint32), ("n_cells_per_block", C.c_uint32),
        ("use_bidirectional", C.c_uint32), ("type_activation_function", C.c_uint32),
        ("activation_steepness", C.c_float), ("type_dropout", C.c_uint32), ("dropout_values", C.c_float * 2),
        ("type_normalization", C.c_uint32), ("use_layer_normalization_before_activation", C.c_uint32),
        ("block_depth", C.c_uint32), ("pooling_values", C.c_uint32 * 5),
        ("constraint_recurrent_weight_lower_bound", C.c_float), ("constraint_recurrent_weight_upper_bound", C.c_float),
        ("k_sparsity", C.c_uint32), ("alpha_sparsity", C.c_float),
        ("first_connection_index", C.c_uint64), ("last_connection_index", C.c_uint64),
        ("first_bias_connection_index", C.c_uint64), ("first_normalized_unit_index", C.c_uint64),
        ("first_mask_index", C.c_uint64),
    ]


class NetDesc(C.Structure):
    _fields_ = [
        ("type_network", C.c_uint32), ("n_layers", C.c_uint32), ("number_recurrent_depth", C.c_uint32),
        ("batch_size", C.c_uint32), ("total_weights", C.c_uint64), ("total_bias", C.c_uint64),
        ("total_normalized_units", C.c_uint64), ("total_parameters", C.c_uint64),
        ("total_mask_units", C.c_uint64), ("layers", LayerDesc * MAX_LAYERS),
    ]


class Hyper(C.Structure):
    _fields_ = [
        ("type_optimizer_function", C.c_uint32), ("type_loss_function", C.c_uint32),
        ("type_accuracy_function", C.c_uint32), ("use_Nesterov", C.c_uint32),
        ("use_adam_bias_correction", C.c_uint32), ("use_clip_gradient", C.c_uint32),
        ("learning_rate", C.c_float), ("learning_rate_final", C.c_float), ("learning_momentum", C.c_float),
        ("learning_gamma", C.c_float), ("adam_learning_rate", C.c_float), ("adam_beta1", C.c_float),
        ("adam_beta2", C.c_float), ("adam_epsilon", C.c_float), ("regularization__weight_decay", C.c_float),
        ("clip_gradient", C.c_float), ("accuracy_variance", C.c_float), ("bit_fail_limit", C.c_float),
        ("normalization_momentum_average", C.c_float), ("normalization_epsilon", C.c_float),
        ("batch_renormalization_r_correction_maximum", C.c_float),
        ("batch_renormalization_d_correction_maximum", C.c_float),
        ("optimizer_time_step", C.c_float), ("number_time_delays", C.c_uint32),
        ("use_normalized_weight_decay", C.c_uint32), ("epoch_time_step", C.c_float),
        ("adam_gamma", C.c_float), ("adam_previous_beta2", C.c_float),
        ("rprop_increase_factor", C.c_float), ("rprop_decrease_factor", C.c_float), ("rprop_delta_min", C.c_float),
        ("rprop_delta_max", C.c_float), ("rprop_delta_zero", C.c_float), ("loss_rprop", C.c_float),
        ("previous_loss_rprop", C.c_float), ("regularization__max_norm_constraints", C.c_float),
        ("use_Warm_Restarts", C.c_uint32), ("warm_restarts_decay_learning_rate", C.c_float),
        ("warm_restarts_maximum_learning_rate", C.c_float), ("warm_restarts_minimum_learning_rate", C.c_float),
        ("warm_restarts_T_i", C.c_float), ("warm_restarts_multiplier", C.c_float),
    ]


class LossState(C.Structure):
    _fields_ = [("loss_values", C.c_double), ("number_loss", C.c_uint64), ("accuracy_value", C.c_double),
                ("number_bit_fail", C.c_uint64), ("accuracy_r", C.c_double * 4)]


# every symbol include/myea_hip.h declares
ABI_SYMBOLS = [
    "myea_hyper_default", "myea_net_desc_layout", "myea_net_desc_previous_layer", "myea_net_desc_number_outputs", "myea_hip_create", "myea_hip_destroy", "myea_hip_set_stream",
    "myea_hip_synchronize", "myea_hip_last_error", "myea_hip_set_hyper", "myea_hip_get_hyper",
    "myea_hip_set_state_propagation", "myea_hip_upload_parameters", "myea_hip_download_parameters",
    "myea_hip_upload_optimizer_state", "myea_hip_download_optimizer_state", "myea_hip_upload_masks", "myea_hip_set_unit_activations",
    "myea_hip_upload_zoneout_masks", "myea_hip_set_dropout_seed", "myea_hip_upload_dropout_noise", "myea_hip_compute_loss", "myea_hip_compute_accuracy_r", "myea_hip_gather_examples", "myea_hip_device_buffer_create", "myea_hip_device_buffer_destroy",
    "myea_hip_clear_training_arrays", "myea_hip_forward_pass", "myea_hip_compute_error", "myea_hip_backward_pass",
    "myea_hip_update_derivative_weight", "myea_hip_update_derivative_weight_no_alloc", "myea_hip_backward_pass_and_update_derivative_weight", "myea_hip_update_parameter",
    "myea_hip_backward_pass_update_derivative_weight_and_update_parameter", "myea_hip_reset_loss", "myea_hip_get_loss",
    "myea_hip_download_gradient", "myea_hip_upload_gradient", "myea_hip_download_tensor", "myea_hip_upload_tensor",
    "myea_hip_profile_enable", "myea_hip_profile_read", "myea_hip_gemm_f32", "myea_hip_optimizer_update",
    "myea_hip_ceiling_mfma_f32", "myea_hip_ceiling_hbm_triad",
]

_lib = None


def load_library(path=LIB_PATH):
    """dlopen the HIP library; raises if it is not built (never falls back to anything else)."""
    global _lib
    if _lib is not None and path == LIB_PATH:
        return _lib
    if not os.path.exists(path):
        raise RuntimeError("%s is missing: build it with `python -m myea_amd.build`" % path)
    lib = C.CDLL(path)
    P, sz, i32, u32, f32p, vp = C.POINTER, C.c_size_t, C.c_int, C.c_uint32, C.POINTER(C.c_float), C.c_void_p
    lib.myea_hyper_default.argtypes = [P(Hyper)]
    lib.myea_hyper_default.restype = None
    lib.myea_net_desc_layout.argtypes = [P(NetDesc)]
    lib.myea_net_desc_previous_layer.argtypes = [P(NetDesc), u32]
    lib.myea_net_desc_previous_layer.restype = u32
    lib.myea_net_desc_number_outputs.argtypes = [P(NetDesc), u32]
    lib.myea_net_desc_number_outputs.restype = C.c_uint64
    lib.myea_hip_create.argtypes = [P(NetDesc), P(vp)]
    lib.myea_hip_destroy.argtypes = [vp]
    lib.myea_hip_set_stream.argtypes = [vp, vp]
    lib.myea_hip_synchronize.argtypes = [vp]
    lib.myea_hip_last_error.argtypes = []
    lib.myea_hip_last_error.restype = C.c_char_p
    lib.myea_hip_set_hyper.argtypes = [vp, P(Hyper)]
    lib.myea_hip_get_hyper.argtypes = [vp, P(Hyper)]
    lib.myea_hip_set_state_propagation.argtypes = [vp, u32]
    for name in ("myea_hip_upload_parameters", "myea_hip_download_parameters", "myea_hip_download_gradient",
                 "myea_hip_upload_gradient"):
        getattr(lib, name).argtypes = [vp, vp, sz]
    lib.myea_hip_upload_optimizer_state.argtypes = [vp, i32, vp, sz]
    lib.myea_hip_download_optimizer_state.argtypes = [vp, i32, vp, sz]
    lib.myea_hip_upload_masks.argtypes = [vp, vp, sz]
    lib.myea_hip_set_unit_activations.argtypes = [vp, sz, vp, vp, sz]
    lib.myea_hip_clear_training_arrays.argtypes = [vp]
    lib.myea_hip_forward_pass.argtypes = [vp, sz, vp, i32]
    lib.myea_hip_compute_error.argtypes = [vp, sz, vp, i32]
    lib.myea_hip_backward_pass.argtypes = [vp, sz]
    lib.myea_hip_backward_pass_and_update_derivative_weight.argtypes = [vp, sz]
    lib.myea_hip_backward_pass_update_derivative_weight_and_update_parameter.argtypes = [vp, sz, sz]
    lib.myea_hip_update_derivative_weight.argtypes = [vp, sz, sz, sz]
    lib.myea_hip_update_derivative_weight_no_alloc.argtypes = [vp, sz, sz, sz]
    lib.myea_hip_update_parameter.argtypes = [vp, sz, sz]
    lib.myea_hip_reset_loss.argtypes = [vp]
    lib.myea_hip_get_loss.argtypes = [vp, P(LossState)]
    lib.myea_hip_upload_zoneout_masks.argtypes = [vp, vp, sz]
    lib.myea_hip_set_dropout_seed.argtypes = [vp, C.c_uint64]
    lib.myea_hip_upload_dropout_noise.argtypes = [vp, sz, vp, sz, i32]
    lib.myea_hip_compute_loss.argtypes = [vp, sz, vp, i32]
    lib.myea_hip_compute_accuracy_r.argtypes = [vp, sz, vp, i32, C.c_float, C.c_float]
    lib.myea_hip_gather_examples.argtypes = [vp, vp, vp, sz, sz, vp, i32, sz]
    lib.myea_hip_device_buffer_create.argtypes = [sz, vp, P(vp)]
    lib.myea_hip_device_buffer_destroy.argtypes = [vp]
    lib.myea_hip_download_tensor.argtypes = [vp, sz, i32, vp, sz]
    lib.myea_hip_upload_tensor.argtypes = [vp, sz, i32, vp, sz]
    lib.myea_hip_profile_enable.argtypes = [vp, i32]
    lib.myea_hip_profile_read.argtypes = [vp, i32, P(C.c_uint64), P(C.c_double), P(C.c_double)]
    lib.myea_hip_gemm_f32.argtypes = [vp, i32, i32, i32, sz, sz, sz, vp, sz, vp, sz, vp, sz]
    lib.myea_hip_optimizer_update.argtypes = [vp, P(Hyper), sz, sz, C.c_float, vp, vp, vp, vp, vp]
    lib.myea_hip_ceiling_mfma_f32.argtypes = [vp, i32, i32, P(C.c_double)]
    lib.myea_hip_ceiling_hbm_triad.argtypes = [vp, sz, i32, P(C.c_double)]
    for name in ABI_SYMBOLS:
        if name not in ("myea_hyper_default", "myea_hip_last_error"):
            getattr(lib, name).restype = i32
    if path == LIB_PATH:
        _lib = lib
    return lib


def default_hyper(lib=None, **overrides):
    lib = lib or load_library()
    h = Hyper()
    lib.myea_hyper_default(C.byref(h))
    for k, v in overrides.items():
        setattr(h, k, v)
    return h


# Activation_Function__To__Class_Activation_Function (NN/Train.cpp:453-500): the functions of the symmetric class
_SYMMETRIC_AF = ("COSINE_SYMMETRIC", "ELLIOT_SYMMETRIC", "GAUSSIAN_SYMMETRIC", "LINEAR_PIECE_SYMMETRIC", "SINE_SYMMETRIC",
                 "TANH", "TANH_STEPWISE", "THRESHOLD_SYMMETRIC")


def constraint_recurrent_weight_default(activation, recurrent_depth, clip_gradient=1.0):
    """Compute__Regularization__Constraint_Recurrent_Weight__Default
    (NN/Neural_Network__Regularization__Constraint_Recurrent_Weight.cpp:33-75): the bounds Compile gives an
    independently recurrent layer, in the reference's float arithmetic."""
    f = np.float32
    mag = f(min(max(f(clip_gradient), f(2)), f(10)))
    T = f(recurrent_depth)
    if activation in _SYMMETRIC_AF:
        hi = np.power(f(mag / np.power(f(0.9), f(T / f(10)), dtype=f)), f(f(1) / T), dtype=f)
    else:
        hi = np.power(mag, f(f(1) / T), dtype=f)
    return float(-hi), float(hi)


def make_desc(layers, batch_size, recurrent_depth=1, network=None, lib=None):
    """layers: list of dicts (first = input layer).  Keys: units, type ('fc'|'ind_rnn'|'lstm'|...), cells_per_block,
    bidirectional, activation (name), steepness, dropout (name), keep, normalization (name), norm_before,
    recurrent_bounds ((lower, upper) clip of an ind_rnn layer's self weights; default: the reference's),
    k_sparsity / alpha_sparsity (k-sparse filter on a hidden fc layer's outputs)."""
    lib = lib or load_library()
    d = NetDesc()
    d.n_layers = len(layers)
    d.number_recurrent_depth = recurrent_depth
    d.batch_size = batch_size
    d.type_network = network if network is not None else (NETWORK_RECURRENT if recurrent_depth > 1 else NETWORK_FEEDFORWARD)
    for i, spec in enumerate(layers):
        l = d.layers[i]
        kind = spec.get("type", "fc")
        l.type_layer = {"fc": LAYER_FULLY_CONNECTED, "ind_rnn": LAYER_FULLY_CONNECTED_INDEPENDENTLY_RECURRENT, "lstm": LAYER_LSTM, "residual": LAYER_RESIDUAL,
                        "average_pooling": LAYER_AVERAGE_POOLING, "max_pooling": LAYER_MAX_POOLING}[kind]
        if kind.endswith("pooling"):   # units is computed by the layout
            for k, name in enumerate(("kernel", "stride", "padding", "dilation", "ceil_mode")):
                l.pooling_values[k] = int(spec.get(name, 1 if name in ("stride", "dilation") else 0))
        l.n_units = spec.get("units", 0)
        l.n_cells_per_block = spec.get("cells_per_block", 1 if kind == "lstm" else 0)
        l.use_bidirectional = int(spec.get("bidirectional", False))
        l.type_activation_function = AF[spec.get("activation", "SIGMOID")] if (kind in ("fc", "ind_rnn") and i > 0) else 0
        if kind == "ind_rnn":
            lo, hi = spec.get("recurrent_bounds") or constraint_recurrent_weight_default(spec.get("activation", "SIGMOID"), recurrent_depth)
            l.constraint_recurrent_weight_lower_bound, l.constraint_recurrent_weight_upper_bound = lo, hi
        l.activation_steepness = spec.get("steepness", 1.0)
        l.type_dropout = DROPOUT[spec.get("dropout", "NONE")]
        l.dropout_values[0] = spec.get("keep", 1.0)
        l.dropout_values[1] = spec.get("keep_output", 0.0)
        l.type_normalization = NORMALIZATION[spec.get("normalization", "NONE")]
        l.use_layer_normalization_before_activation = int(spec.get("norm_before", True))
        l.block_depth = spec.get("block_depth", 0)
        l.k_sparsity = spec.get("k_sparsity", 0)
        l.alpha_sparsity = spec.get("alpha_sparsity", 1.0)
    rc = lib.myea_net_desc_layout(C.byref(d))
    if rc != 0:
        raise ValueError("myea_net_desc_layout failed with %d" % rc)
    return d


def _ptr(a):
    """pointer of a numpy array, a torch tensor (host or device) or a raw integer address"""
    if a is None:
        return None
    if isinstance(a, int):
        return C.c_void_p(a)
    if isinstance(a, np.ndarray):
        return C.c_void_p(a.ctypes.data)
    return C.c_void_p(a.data_ptr())  # torch tensor


class MyeaError(RuntimeError):
    def __init__(self, code, text):
        super().__init__("myea_hip error %d: %s" % (code, text))
        self.code = code


class HipNetwork:
    """Handle over myea_hip_create(); method names follow the reference's Neural_Network entry points."""

    def __init__(self, desc, hyper=None):
        self.lib = load_library()
        self.desc = desc
        self.handle = C.c_void_p()
        self._check(self.lib.myea_hip_create(C.byref(desc), C.byref(self.handle)))
        if hyper is not None:
            self.set_hyper(hyper)

    def _check(self, rc):
        if rc != 0:
            raise MyeaError(rc, (self.lib.myea_hip_last_error() or b"").decode())

    def close(self):
        if self.handle:
            self.lib.myea_hip_destroy(self.handle)
            self.handle = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # configuration
    def set_stream(self, stream_ptr): self._check(self.lib.myea_hip_set_stream(self.handle, C.c_void_p(stream_ptr)))
    def synchronize(self): self._check(self.lib.myea_hip_synchronize(self.handle))
    def set_hyper(self, h): self._check(self.lib.myea_hip_set_hyper(self.handle, C.byref(h)))

    def get_hyper(self):
        h = Hyper()
        self._check(self.lib.myea_hip_get_hyper(self.handle, C.byref(h)))
        return h

    def set_state_propagation(self, s): self._check(self.lib.myea_hip_set_state_propagation(self.handle, s))

    # parameter / state movement
    def upload_parameters(self, w):
        w = np.ascontiguousarray(w, dtype=np.float32)
        self._check(self.lib.myea_hip_upload_parameters(self.handle, _ptr(w), w.size))

    def download_parameters(self):
        out = np.empty(self.desc.total_parameters, dtype=np.float32)
        self._check(self.lib.myea_hip_download_parameters(self.handle, _ptr(out), out.size))
        return out

    def upload_optimizer_state(self, kind, v):
        v = np.ascontiguousarray(v, dtype=np.float32)
        self._check(self.lib.myea_hip_upload_optimizer_state(self.handle, kind, _ptr(v), v.size))

    def download_optimizer_state(self, kind):
        out = np.empty(self.desc.total_parameters, dtype=np.float32)
        self._check(self.lib.myea_hip_download_optimizer_state(self.handle, kind, _ptr(out), out.size))
        return out

    def set_unit_activations(self, layer, types=None, steepness=None):
        t = None if types is None else np.ascontiguousarray(types, dtype=np.uint32)
        st = None if steepness is None else np.ascontiguousarray(steepness, dtype=np.float32)
        n = len(t) if t is not None else (len(st) if st is not None else 0)
        self._check(self.lib.myea_hip_set_unit_activations(self.handle, layer, _ptr(t), _ptr(st), n))

    def upload_masks(self, m):
        m = np.ascontiguousarray(m, dtype=np.uint8)
        self._check(self.lib.myea_hip_upload_masks(self.handle, _ptr(m), m.size))

    def download_gradient(self):
        out = np.empty(self.desc.total_parameters, dtype=np.float32)
        self._check(self.lib.myea_hip_download_gradient(self.handle, _ptr(out), out.size))
        return out

    def upload_gradient(self, g):
        g = np.ascontiguousarray(g, dtype=np.float32)
        self._check(self.lib.myea_hip_upload_gradient(self.handle, _ptr(g), g.size))

    def download_tensor(self, layer, kind, count=None):
        if count is None:   # a [T][batch_size][width] tensor of the layer, whole
            count = self.desc.number_recurrent_depth * self.desc.batch_size * self.lib.myea_net_desc_number_outputs(C.byref(self.desc), layer)
        out = np.empty(count, dtype=np.float32)
        self._check(self.lib.myea_hip_download_tensor(self.handle, layer, kind, _ptr(out), out.size))
        return out

    def upload_tensor(self, layer, kind, values):
        """running means / variances of a normalised layer, [T][units]"""
        v = np.ascontiguousarray(values, dtype=np.float32)
        self._check(self.lib.myea_hip_upload_tensor(self.handle, layer, kind, _ptr(v), v.size))

    def set_dropout_seed(self, seed):
        self._check(self.lib.myea_hip_set_dropout_seed(self.handle, seed))

    def upload_dropout_noise(self, layer, noise, on_device=False):
        """[T][batch_size][width] draws for a Gaussian / Uout layer; None returns the layer to the device generator"""
        if noise is None:
            self._check(self.lib.myea_hip_upload_dropout_noise(self.handle, layer, None, 0, 0))
            return
        if isinstance(noise, np.ndarray):
            noise = np.ascontiguousarray(noise, dtype=np.float32)
            count = noise.size
        else:
            count = noise.numel()
        self._check(self.lib.myea_hip_upload_dropout_noise(self.handle, layer, _ptr(noise), count, int(on_device)))

    def upload_zoneout_masks(self, m):
        m = np.ascontiguousarray(m, dtype=np.uint8)
        self._check(self.lib.myea_hip_upload_zoneout_masks(self.handle, _ptr(m), m.size))

    def Clear_Training_Arrays(self): self._check(self.lib.myea_hip_clear_training_arrays(self.handle))

    # the five step entry points
    def Forward_Pass(self, batch_size, inputs, on_device=False):
        if isinstance(inputs, np.ndarray):
            inputs = np.ascontiguousarray(inputs, dtype=np.float32)
        self._check(self.lib.myea_hip_forward_pass(self.handle, batch_size, _ptr(inputs), int(on_device)))

    def Compute__Error(self, batch_size, desired, on_device=False):
        if isinstance(desired, np.ndarray):
            desired = np.ascontiguousarray(desired, dtype=np.float32)
        self._check(self.lib.myea_hip_compute_error(self.handle, batch_size, _ptr(desired), int(on_device)))

    def Compute__Loss(self, batch_size, desired, on_device=False):
        if isinstance(desired, np.ndarray):
            desired = np.ascontiguousarray(desired, dtype=np.float32)
        self._check(self.lib.myea_hip_compute_loss(self.handle, batch_size, _ptr(desired), int(on_device)))

    def Compute__Accuracy__R(self, batch_size, desired, desired_mean, predicted_mean, on_device=False):
        if isinstance(desired, np.ndarray):
            desired = np.ascontiguousarray(desired, dtype=np.float32)
        self._check(self.lib.myea_hip_compute_accuracy_r(self.handle, batch_size, _ptr(desired), int(on_device), desired_mean, predicted_mean))

    def gather_examples(self, device_batch, device_dataset, dataset_examples, row_floats, index, batch_size, index_on_device=False):
        """device_batch / device_dataset: device pointers (int or an object with data_ptr()); index: uint64 array (host) or device pointer"""
        if isinstance(index, np.ndarray):
            index = np.ascontiguousarray(index, dtype=np.uint64)
        self._check(self.lib.myea_hip_gather_examples(self.handle, _ptr(device_batch), _ptr(device_dataset), dataset_examples, row_floats,
                                                      _ptr(index), int(index_on_device), batch_size))

    def Backward_Pass(self, batch_size): self._check(self.lib.myea_hip_backward_pass(self.handle, batch_size))

    def Backward_Pass__Update_Derivative_Weight(self, batch_size):
        """Backward_Pass then Update_Derivative_Weight over all layers, as one call"""
        self._check(self.lib.myea_hip_backward_pass_and_update_derivative_weight(self.handle, batch_size))

    def Backward_Pass__Update_Derivative_Weight__Update_Parameter(self, batch_size, training_size):
        """Backward_Pass, Update_Derivative_Weight over all layers and Update_Parameter, as one call"""
        self._check(self.lib.myea_hip_backward_pass_update_derivative_weight_and_update_parameter(self.handle, batch_size, training_size))

    def Update_Derivative_Weight(self, batch_size, first_layer=1, end_layer=None):
        end_layer = self.desc.n_layers if end_layer is None else end_layer
        self._check(self.lib.myea_hip_update_derivative_weight(self.handle, batch_size, first_layer, end_layer))

    def Update_Derivative_Weight__No_Alloc(self, batch_size, first_layer=1, end_layer=None):
        """Update_Derivative_Weight with its kernels' scratch memory in the library's static device array"""
        end_layer = self.desc.n_layers if end_layer is None else end_layer
        self._check(self.lib.myea_hip_update_derivative_weight_no_alloc(self.handle, batch_size, first_layer, end_layer))

    def Update_Parameter(self, batch_size, training_size):
        self._check(self.lib.myea_hip_update_parameter(self.handle, batch_size, training_size))

    def Reset__Loss(self): self._check(self.lib.myea_hip_reset_loss(self.handle))

    def get_loss(self):
        s = LossState()
        self._check(self.lib.myea_hip_get_loss(self.handle, C.byref(s)))
        return s

    # profiling taps
    def profile_enable(self, on): self._check(self.lib.myea_hip_profile_enable(self.handle, int(on)))

    def profile_read(self, family):
        n, ms, work = C.c_uint64(), C.c_double(), C.c_double()
        self._check(self.lib.myea_hip_profile_read(self.handle, family, C.byref(n), C.byref(ms), C.byref(work)))
        return n.value, ms.value, work.value
