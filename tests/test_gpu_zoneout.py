"""GPU parity of zoneout on LSTM layers (masks uploaded by the caller, acting in the training state's forward pass only):
the HIP library (through its C ABI) against the CPU oracle - generic step kernels, the fused time step, two directions.
Tolerance rel 1e-4 / abs 1e-5; zoned-out units repeat their previous value bit for bit."""
import numpy as np
import pytest

from myea_amd import binding as mb
from tests.common import assert_close, glorot_parameters, run_step
from tests.oracle_lib import OracleNetwork
from tests.test_gpu_lstm import LSTM_TAPS, _rows, _width

pytestmark = pytest.mark.gpu
REL, ABS = 1e-4, 1e-5

zone = lambda units, cpb=1, **kw: dict(type="lstm", units=units, cells_per_block=cpb, dropout="ZONEOUT", keep=0.3, keep_output=0.2, **kw)
CASES = [
    ("generic-two-cells-per-block", [dict(units=6), zone(5, 2), dict(units=10, activation="LINEAR")], 5, 4, 4),
    ("fused-step-64-cells-partial-batch", [dict(units=12), zone(64), dict(units=64, activation="TANH")], 6, 35, 40),
    ("stacked-zoned-plain-zoned", [dict(units=8), zone(32), dict(type="lstm", units=12), zone(7, 3), dict(units=21, activation="LINEAR")], 4, 6, 6),
    ("two-directions", [dict(units=5), zone(32, 1, bidirectional=True), dict(units=32, activation="LINEAR")], 5, 9, 9),
]


@pytest.mark.parametrize("name,specs,T,B,Bmax", CASES, ids=[c[0] for c in CASES])
def test_zoneout_parity(name, specs, T, B, Bmax):
    desc = mb.make_desc(specs, Bmax, T)
    h = mb.default_hyper(type_optimizer_function=mb.OPTIMIZER["ADAM"], type_loss_function=mb.LOSS["MSE"])
    gpu, cpu = mb.HipNetwork(desc, h), OracleNetwork(desc, h)
    w = glorot_parameters(desc, 9, bias_range=0.3)
    rng = np.random.default_rng(9)
    cells = sum(_width(desc.layers[i]) * (2 if desc.layers[i].use_bidirectional else 1) for i in range(desc.n_layers) if desc.layers[i].type_layer == mb.LAYER_LSTM)
    masks = (rng.uniform(0, 1, 2 * T * cells) < 0.6).astype(np.uint8)
    X = rng.normal(0, 1, (B, T * specs[0]["units"])).astype(np.float32)
    Y = rng.normal(0, 1, (B, T * specs[-1]["units"])).astype(np.float32)
    for n in (gpu, cpu):
        n.set_state_propagation(mb.STATE_TRAINING)
        n.upload_parameters(w)
        n.upload_zoneout_masks(masks)
        n.Clear_Training_Arrays()
    for step in range(2):
        for n in (gpu, cpu):
            n.Reset__Loss()
            run_step(n, B, X, Y, update=False)
        for li in range(1, desc.n_layers):
            l = desc.layers[li]
            W = _width(l)
            lstm = l.type_layer == mb.LAYER_LSTM
            dirs = [0, mb.TENSOR["DIRECTION_BACKWARD"]] if (lstm and l.use_bidirectional) else [0]
            for kind in ["OUTPUTS", "ERRORS"] + (LSTM_TAPS + ["LSTM_CELL_OUTPUT"] if lstm else []):
                for flag in (dirs if kind.startswith("LSTM") else [0]):
                    Wk = l.n_units if kind.endswith("_GATE") else W
                    a = gpu.download_tensor(li, mb.TENSOR[kind] | flag, T * Bmax * Wk)
                    b = cpu.download_tensor(li, mb.TENSOR[kind] | flag, T * Bmax * Wk)
                    assert_close(_rows(a, T, Bmax, B, Wk), _rows(b, T, Bmax, B, Wk), REL, ABS, what="step %d layer %d %s/%d" % (step, li, kind, flag))
        assert_close(gpu.download_gradient(), cpu.download_gradient(), REL, ABS, what="gradient step %d" % step)
        for n in (gpu, cpu):
            n.Update_Parameter(B, B)
        gpu.upload_parameters(cpu.download_parameters())
    # a zoned-out cell output is the previous step's, bit for bit (first zoned layer, forward direction)
    li = 1
    C = _width(desc.layers[li])
    stride = C * (2 if desc.layers[li].use_bidirectional else 1)
    out_masks = masks[T * cells:][:T * stride].reshape(T, stride)[:, :C]
    hcell = _rows(gpu.download_tensor(li, mb.TENSOR["LSTM_CELL_OUTPUT"], T * Bmax * C), T, Bmax, B, C)
    for t in range(1, T):
        held = out_masks[t] == 0
        assert held.any() and np.array_equal(hcell[t][:, held], hcell[t - 1][:, held])
    assert np.all(hcell[0][:, out_masks[0] == 0] == 0)
    # inference: the masks do not act
    plain = [dict(s, dropout="NONE") if s.get("dropout") == "ZONEOUT" else s for s in specs]
    ref = OracleNetwork(mb.make_desc(plain, Bmax, T), h)
    ref.upload_parameters(cpu.download_parameters())
    gpu.set_state_propagation(mb.STATE_INFERENCE)
    gpu.Forward_Pass(B, X); ref.Forward_Pass(B, X)
    last = desc.n_layers - 1
    Wl = _width(desc.layers[last])
    assert_close(_rows(gpu.download_tensor(last, mb.TENSOR["OUTPUTS"], T * Bmax * Wl), T, Bmax, B, Wl),
                 _rows(ref.download_tensor(last, mb.TENSOR["OUTPUTS"], T * Bmax * Wl), T, Bmax, B, Wl), REL, ABS, what="inference")


def test_zoneout_error_paths():
    desc = mb.make_desc([dict(units=4), zone(6), dict(units=6, activation="LINEAR")], 2, 3)
    gpu = mb.HipNetwork(desc)
    with pytest.raises(mb.MyeaError) as e:
        gpu.upload_zoneout_masks(np.ones(5, dtype=np.uint8))
    assert e.value.code == mb.E_INVALID
    gpu.upload_zoneout_masks(np.ones(2 * 3 * 6, dtype=np.uint8))
    with pytest.raises(mb.MyeaError) as e:    # zoneout belongs to LSTM layers
        mb.HipNetwork(mb.make_desc([dict(units=4), dict(units=6, activation="TANH", dropout="ZONEOUT"), dict(units=6, activation="LINEAR")], 2))
    assert e.value.code == mb.E_UNSUPPORTED
