"""ctypes wrapper over oracle/libmyea_oracle.so (the CPU checker) with the same method names as
myea_amd.binding.HipNetwork, so a parity test drives both sides with identical calls."""
import ctypes as C
import os

import numpy as np

from myea_amd import binding as mb

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_PATH = os.path.join(ROOT, "oracle", "libmyea_oracle.so")

_lib = None


def load_oracle():
    global _lib
    if _lib is not None:
        return _lib
    lib = C.CDLL(ORACLE_PATH)
    P, sz, vp, i32 = C.POINTER, C.c_size_t, C.c_void_p, C.c_int
    lib.myea_oracle_create.argtypes = [P(mb.NetDesc), P(vp)]
    lib.myea_net_desc_previous_layer.argtypes = [P(mb.NetDesc), C.c_uint32]
    lib.myea_net_desc_previous_layer.restype = C.c_uint32
    lib.myea_net_desc_number_outputs.argtypes = [P(mb.NetDesc), C.c_uint32]
    lib.myea_net_desc_number_outputs.restype = C.c_uint64
    lib.myea_oracle_destroy.argtypes = [vp]
    lib.myea_oracle_set_hyper.argtypes = [vp, P(mb.Hyper)]
    lib.myea_oracle_get_hyper.argtypes = [vp, P(mb.Hyper)]
    lib.myea_oracle_set_state_propagation.argtypes = [vp, C.c_uint32]
    lib.myea_oracle_set_threads.argtypes = [vp, i32]
    lib.myea_oracle_set_unit_activations.argtypes = [vp, C.c_size_t, vp, vp, C.c_size_t]
    for name in ("myea_oracle_parameters", "myea_oracle_gradient"):
        getattr(lib, name).argtypes = [vp]
        getattr(lib, name).restype = P(C.c_float)
    lib.myea_oracle_optimizer_state.argtypes = [vp, i32]
    lib.myea_oracle_optimizer_state.restype = P(C.c_float)
    lib.myea_oracle_masks.argtypes = [vp]
    lib.myea_oracle_masks.restype = P(C.c_uint8)
    lib.myea_oracle_zoneout_masks.argtypes = [vp, P(sz)]
    lib.myea_oracle_zoneout_masks.restype = P(C.c_uint8)
    lib.myea_oracle_dropout_noise.argtypes = [vp, sz, P(sz)]
    lib.myea_oracle_dropout_noise.restype = P(C.c_float)
    lib.myea_oracle_clear_training_arrays.argtypes = [vp]
    lib.myea_oracle_forward_pass.argtypes = [vp, sz, vp]
    lib.myea_oracle_compute_error.argtypes = [vp, sz, vp]
    lib.myea_oracle_compute_loss.argtypes = [vp, sz, vp]
    lib.myea_oracle_compute_accuracy_r.argtypes = [vp, sz, vp, C.c_float, C.c_float]
    lib.myea_oracle_backward_pass.argtypes = [vp, sz]
    lib.myea_oracle_update_derivative_weight.argtypes = [vp, sz, sz, sz]
    lib.myea_oracle_update_parameter.argtypes = [vp, sz, sz]
    lib.myea_oracle_reset_loss.argtypes = [vp]
    lib.myea_oracle_get_loss.argtypes = [vp, P(mb.LossState)]
    lib.myea_oracle_tensor.argtypes = [vp, sz, i32, P(sz)]
    lib.myea_oracle_tensor.restype = P(C.c_float)
    lib.myea_oracle_activation.argtypes = [C.c_uint32, C.c_float]
    lib.myea_oracle_activation.restype = C.c_float
    lib.myea_oracle_activation_derive.argtypes = [C.c_uint32, C.c_float, C.c_float, C.c_float]
    lib.myea_oracle_activation_derive.restype = C.c_float
    lib.myea_oracle_irprop_minus.argtypes = [P(mb.Hyper), sz, vp, vp, vp, vp]
    lib.myea_oracle_irprop_minus.restype = None
    lib.myea_hyper_default.argtypes = [P(mb.Hyper)]
    lib.myea_hyper_default.restype = None
    lib.myea_net_desc_layout.argtypes = [P(mb.NetDesc)]
    _lib = lib
    return lib


class OracleError(RuntimeError):
    def __init__(self, code):
        super().__init__("oracle error %d" % code)
        self.code = code


class OracleNetwork:
    def __init__(self, desc, hyper=None, threads=1):
        self.lib = load_oracle()
        self.desc = desc
        self.handle = C.c_void_p()
        self._check(self.lib.myea_oracle_create(C.byref(desc), C.byref(self.handle)))
        if hyper is not None:
            self.set_hyper(hyper)
        if threads != 1:
            self._check(self.lib.myea_oracle_set_threads(self.handle, threads))

    def _check(self, rc):
        if rc != 0:
            raise OracleError(rc)

    def close(self):
        if self.handle:
            self.lib.myea_oracle_destroy(self.handle)
            self.handle = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def _view(self, ptr, n, dtype=np.float32):
        return np.ctypeslib.as_array(ptr, shape=(n,)) if n else np.zeros(0, dtype)

    def set_hyper(self, h): self._check(self.lib.myea_oracle_set_hyper(self.handle, C.byref(h)))

    def get_hyper(self):
        h = mb.Hyper()
        self._check(self.lib.myea_oracle_get_hyper(self.handle, C.byref(h)))
        return h

    def set_state_propagation(self, s): self._check(self.lib.myea_oracle_set_state_propagation(self.handle, s))

    def parameters_view(self): return self._view(self.lib.myea_oracle_parameters(self.handle), self.desc.total_parameters)
    def gradient_view(self): return self._view(self.lib.myea_oracle_gradient(self.handle), self.desc.total_parameters)
    def upload_parameters(self, w): self.parameters_view()[: len(w)] = np.asarray(w, dtype=np.float32)
    def download_parameters(self): return self.parameters_view().copy()
    def download_gradient(self): return self.gradient_view().copy()
    def upload_gradient(self, g): self.gradient_view()[: len(g)] = np.asarray(g, dtype=np.float32)

    def upload_optimizer_state(self, kind, v):
        self._view(self.lib.myea_oracle_optimizer_state(self.handle, kind), self.desc.total_parameters)[: len(v)] = v

    def download_optimizer_state(self, kind):
        return self._view(self.lib.myea_oracle_optimizer_state(self.handle, kind), self.desc.total_parameters).copy()

    def set_unit_activations(self, layer, types=None, steepness=None):
        t = None if types is None else np.ascontiguousarray(types, dtype=np.uint32)
        st = None if steepness is None else np.ascontiguousarray(steepness, dtype=np.float32)
        n = len(t) if t is not None else (len(st) if st is not None else 0)
        self._keep = (t, st)
        self._check(self.lib.myea_oracle_set_unit_activations(self.handle, layer, None if t is None else t.ctypes.data_as(C.c_void_p),
                                                              None if st is None else st.ctypes.data_as(C.c_void_p), n))

    def upload_masks(self, m):
        m = np.asarray(m, dtype=np.uint8)
        self._view(self.lib.myea_oracle_masks(self.handle), self.desc.total_mask_units, np.uint8)[: len(m)] = m

    def upload_dropout_noise(self, layer, noise):
        n = C.c_size_t()
        p = self.lib.myea_oracle_dropout_noise(self.handle, layer, C.byref(n))
        noise = np.asarray(noise, dtype=np.float32).ravel()
        assert p and len(noise) == n.value, "dropout noise count %d != %d" % (len(noise), n.value)
        self._view(p, n.value)[:] = noise

    def upload_zoneout_masks(self, m):
        m = np.asarray(m, dtype=np.uint8)
        n = C.c_size_t()
        p = self.lib.myea_oracle_zoneout_masks(self.handle, C.byref(n))
        assert len(m) == n.value, "zoneout mask count %d != %d" % (len(m), n.value)
        self._view(p, n.value, np.uint8)[:] = m

    def download_tensor(self, layer, kind, count=None):
        n = C.c_size_t()
        p = self.lib.myea_oracle_tensor(self.handle, layer, kind, C.byref(n))
        if not p:
            raise OracleError(-1)
        a = self._view(p, n.value).copy()
        return a if count is None else a[:count]

    def Clear_Training_Arrays(self): self._check(self.lib.myea_oracle_clear_training_arrays(self.handle))

    def Forward_Pass(self, batch_size, inputs, on_device=False):
        x = np.ascontiguousarray(inputs, dtype=np.float32)
        self._check(self.lib.myea_oracle_forward_pass(self.handle, batch_size, C.c_void_p(x.ctypes.data)))

    def Compute__Error(self, batch_size, desired, on_device=False):
        y = np.ascontiguousarray(desired, dtype=np.float32)
        self._check(self.lib.myea_oracle_compute_error(self.handle, batch_size, C.c_void_p(y.ctypes.data)))

    def Compute__Loss(self, batch_size, desired, on_device=False):
        y = np.ascontiguousarray(desired, dtype=np.float32)
        self._check(self.lib.myea_oracle_compute_loss(self.handle, batch_size, C.c_void_p(y.ctypes.data)))

    def Compute__Accuracy__R(self, batch_size, desired, desired_mean, predicted_mean, on_device=False):
        y = np.ascontiguousarray(desired, dtype=np.float32)
        self._check(self.lib.myea_oracle_compute_accuracy_r(self.handle, batch_size, C.c_void_p(y.ctypes.data), desired_mean, predicted_mean))

    def Backward_Pass(self, batch_size): self._check(self.lib.myea_oracle_backward_pass(self.handle, batch_size))

    def Update_Derivative_Weight(self, batch_size, first_layer=1, end_layer=None):
        end_layer = self.desc.n_layers if end_layer is None else end_layer
        self._check(self.lib.myea_oracle_update_derivative_weight(self.handle, batch_size, first_layer, end_layer))

    def Update_Parameter(self, batch_size, training_size):
        self._check(self.lib.myea_oracle_update_parameter(self.handle, batch_size, training_size))

    def Reset__Loss(self): self._check(self.lib.myea_oracle_reset_loss(self.handle))

    def get_loss(self):
        s = mb.LossState()
        self._check(self.lib.myea_oracle_get_loss(self.handle, C.byref(s)))
        return s
