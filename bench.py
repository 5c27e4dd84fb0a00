#!/usr/bin/env python3
"""Benchmark of the training hot path on one MI355X.

One "step" = Forward_Pass + Compute__Error + Backward_Pass, Update_Derivative_Weight and Update_Parameter (the last three as
one call; --separate-update: Update_Parameter as a call of its own) on one batch of synthetic data already resident in HBM.  Default workload: BASELINE config 2, the deep fully-connected
stack 4096-4096-4096-4096-4096-1000 (ReLU, softmax + cross-entropy, Adam) at batch 1024, fp32.

Prints ONE JSON line.  The timed block of exactly `steps` steps is run `--repeats` times; `value` and `ms_per_step` are the
median block's, every block's figure is listed (`ms_per_step_blocks`).  `roofline` covers the dominant kernel family — the
FP32 MFMA contractions (forward X W^T, dX = delta W, dW += delta^T X): algorithmic FLOPs of all their launches over their
summed HIP-event durations on the stream they run on, taken in a second pass of `steps` steps (`events_pass`), because a
pair of timing events around every launch slows the step it measures.  `cpu_baseline` times the CPU restatement of the
reference (oracle/, OpenMP) on this host on a bounded sample of the same workload.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# HBM bytes per contraction launch (mean over the launches of one step): NOT measured by this script's run.  Recorded
# from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this script, scaled by what the same counters read for copies of
# known size (FETCH_SIZE x2, WRITE_SIZE x1); the line names the file the figure comes from.
RECORDED_TRAFFIC = {"fc4096x4_b1024_adam": dict(bytes_per_launch=2951372 * 1024 / 10,
                                                source="recorded constant, not measured in this run: profiles/hbm_traffic__fc4096x4_b1024_adam__pmc.txt"),
                    # the two resident time loops of one layer (forward + backward launch), mean per launch
                    "lstm512x2_t64_b256_amsgrad": dict(bytes_per_launch=(2 * 98055.1 + 230411.5 + 2 * 203936.9 + 197795.6) * 1024 / 2,
                                                       source="recorded constant, not measured in this run: profiles/lstm_resident__lstm512x2_t64_b256_amsgrad__pmc.txt")}
from myea_amd.synthetic import simple_debug_layers  # noqa: E402  (no device is touched by the import)

PEAK_FP32_MFMA_TFLOPS = 157.3   # MI355X dense FP32 matrix
PEAK_HBM_GBS = 8000.0           # MI355X HBM3E

WORKLOADS = {
    # BASELINE.json configs[1]
    "fc4096x4_b1024_adam": dict(
        layers=[dict(units=4096)] + [dict(units=4096, activation="RELU")] * 4 + [dict(units=1000, activation="SOFTMAX")],
        batch=1024, head="SOFTMAX", optimizer="ADAM", loss="CROSS_ENTROPY", data="normal", hyper={}),
    # BASELINE.json configs[2]: 2 x LSTM-512 with peepholes, input 128, T = 64, batch 256, linear FC-512 head, MSE, AMSGrad
    "lstm512x2_t64_b256_amsgrad": dict(
        layers=[dict(units=128), dict(type="lstm", units=512), dict(type="lstm", units=512), dict(units=512, activation="LINEAR")],
        batch=256, depth=64, head="LINEAR", optimizer="AMSGRAD", loss="MSE", data="normal", hyper={}),
    # BASELINE.json configs[0] (the reference's own CPU-sized case)
    "mlp784_256_10_b128_sgd": dict(
        layers=[dict(units=784), dict(units=256, activation="TANH"), dict(units=10, activation="SIGMOID")],
        batch=128, head="SIGMOID", optimizer="GD", loss="MSE", data="uniform", hyper=dict(learning_rate=0.01, learning_momentum=0.9)),
    # BASELINE.json configs[3] (input width 2048)
    "fc2048x8_bn_relu_dropout_b512_nesterov": dict(
        layers=[dict(units=2048)] + [dict(units=2048, activation="RELU", normalization="BATCH_NORMALIZATION", norm_before=True,
                                          dropout="BERNOULLI_INVERTED", keep=0.5)] * 8 + [dict(units=100, activation="SOFTMAX")],
        batch=512, head="SOFTMAX", optimizer="GD", loss="CROSS_ENTROPY", data="normal",
        hyper=dict(learning_rate=0.01, learning_momentum=0.9, use_Nesterov=1)),
    # BASELINE.json configs[4]: bidirectional LSTM with peepholes, input 256, 1024 cells per direction, T = 512, batch 64,
    # per-step 32-class softmax + cross-entropy, clip at norm 1, AdaBound
    "bilstm1024_t512_b64_adabound": dict(
        layers=[dict(units=256), dict(type="lstm", units=1024, bidirectional=True), dict(units=32, activation="SOFTMAX")],
        batch=64, depth=512, head="SOFTMAX", optimizer="ADABOUND", loss="CROSS_ENTROPY", data="uniform_pm1",
        hyper=dict(use_clip_gradient=1, clip_gradient=1.0)),
    # configs[3] as residual blocks: 4 blocks of 2 pre-activation members [BN -> ReLU -> inverted dropout -> FC 2048]
    "resfc2048x8_bn_relu_dropout_b512_nesterov": dict(
        layers=[dict(units=2048), dict(units=2048, activation="RELU")]
               + sum(([dict(type="residual", block_depth=2),
                       dict(units=2048, activation="RELU", normalization="BATCH_NORMALIZATION"),
                       dict(units=2048, activation="RELU", normalization="BATCH_NORMALIZATION", dropout="BERNOULLI_INVERTED", keep=0.5)]
                      for _ in range(4)), [])
               + [dict(units=100, activation="SOFTMAX")],
        batch=512, head="SOFTMAX", optimizer="GD", loss="CROSS_ENTROPY", data="normal",
        hyper=dict(learning_rate=0.01, learning_momentum=0.9, use_Nesterov=1)),
    # LSTM layers normalised inside (batch normalisation of the eight gate sums and of the cell state at every time step)
    "lstm256x2_bn_t32_b128_adam": dict(
        layers=[dict(units=64), dict(type="lstm", units=256, normalization="BATCH_NORMALIZATION"),
                dict(type="lstm", units=256, normalization="BATCH_NORMALIZATION"), dict(units=256, activation="LINEAR")],
        batch=128, depth=32, head="LINEAR", optimizer="ADAM", loss="MSE", data="normal", hyper={}),
    # the reference's worked example (Neural_Network_Launcher_Windows/Source_Files/debug.cpp:36-1555): sMNIST rows (28 inputs x 28
    # time steps, the label read at the last one), residual blocks of independently recurrent ISRLU members with batch
    # normalisation, max pooling between the groups, softmax head, AMSGrad at 1e-3, max-norm constraint 8
    "resindrnn_smnist28_t28_b256_amsgrad": dict(
        layers=simple_debug_layers(), batch=256, depth=28, head="SOFTMAX", optimizer="AMSGRAD", loss="CROSS_ENTROPY", data="uniform",
        hyper=dict(adam_learning_rate=1e-3, regularization__max_norm_constraints=8.0, normalization_momentum_average=1.0,
                   normalization_epsilon=0.1, number_time_delays=27)),
}


def gemm_flops_per_step(layers, batch, depth=1):
    """2*M*N*K of forward, dX (every layer whose producer is not the input layer) and dW; LSTM layers: 4 gate rows per cell, input
    contraction at every step, recurrent contraction at T-1 steps.  Widths come from the laid-out description (pooling layers
    and residual blocks change them and own no contraction)."""
    from myea_amd import binding as mb
    lib = mb.load_library()
    desc = mb.make_desc(layers, batch, depth)
    fwd = dx = 0.0
    for i in range(1, desc.n_layers):
        l = desc.layers[i]
        if l.type_layer in (mb.LAYER_RESIDUAL, mb.LAYER_AVERAGE_POOLING, mb.LAYER_MAX_POOLING):
            continue
        prev = lib.myea_net_desc_previous_layer(desc, i)
        fan_in, width = lib.myea_net_desc_number_outputs(desc, prev), lib.myea_net_desc_number_outputs(desc, i)
        if l.type_layer == mb.LAYER_LSTM:
            dirs = 2 if l.use_bidirectional else 1
            cells = l.n_units * l.n_cells_per_block
            gates = cells + 3 * l.n_units
            f_in, f_rec = 2.0 * dirs * batch * depth * gates * fan_in, 2.0 * dirs * batch * (depth - 1) * gates * cells
            fwd += f_in + f_rec
            dx += f_rec + (f_in if prev != 0 else 0.0)
        else:
            f = 2.0 * batch * depth * width * fan_in
            fwd += f
            dx += f if prev != 0 else 0.0
    return fwd + dx + fwd


def make_inputs(np, wl, seed):
    rng = np.random.default_rng(seed)
    T = wl.get("depth", 1)
    B, n_in, n_out = wl["batch"], wl["layers"][0]["units"] * T, wl["layers"][-1]["units"]
    X = (rng.normal(0, 1, (B, n_in)) if wl["data"] == "normal" else
         rng.uniform(-1, 1, (B, n_in)) if wl["data"] == "uniform_pm1" else rng.uniform(0, 1, (B, n_in))).astype(np.float32)
    if wl["loss"] == "MSE" and T > 1:
        return X, rng.normal(0, 1, (B, T * n_out)).astype(np.float32)
    if T > 1:   # one label per time step
        Y = np.zeros((B, T, n_out), dtype=np.float32)
        np.put_along_axis(Y, rng.integers(0, n_out, (B, T))[..., None], 1.0, axis=2)
        return X, Y.reshape(B, T * n_out)
    Y = np.zeros((B, n_out), dtype=np.float32)
    Y[np.arange(B), rng.integers(0, n_out, B)] = 1.0
    return X, Y


def cpu_baseline(wl, sample_rows, threads):
    """The oracle (a port of the reference's CPU path) on `sample_rows` examples of the same network: forward +
    error + backward + dW are timed on the sample and scaled to the full batch; the weight update is timed over the
    full parameter vector; samples/s = batch / (t_sample * batch / sample_rows + t_update)."""
    import numpy as np
    from myea_amd import binding as mb
    from myea_amd.synthetic import glorot_parameters
    from tests.oracle_lib import OracleNetwork, load_oracle
    lib = load_oracle()
    desc = mb.make_desc(wl["layers"], sample_rows, wl.get("depth", 1), lib=lib)
    h = mb.default_hyper(lib=lib, type_optimizer_function=mb.OPTIMIZER[wl["optimizer"]], type_loss_function=mb.LOSS[wl["loss"]], **wl["hyper"])
    net = OracleNetwork(desc, h, threads=threads)
    net.set_state_propagation(mb.STATE_TRAINING)
    net.upload_parameters(glorot_parameters(desc, 2))
    if desc.total_mask_units:
        net.upload_masks((np.random.default_rng(4).uniform(0, 1, desc.total_mask_units) < 0.5).astype(np.uint8))
    X, Y = make_inputs(np, dict(wl, batch=sample_rows), 2)
    t_sample, t_update, reps = 0.0, 0.0, 0
    while reps < 1 or (t_sample + t_update < 10.0 and reps < 8):   # about 10-30 s of CPU work
        t0 = time.perf_counter()
        net.Forward_Pass(sample_rows, X)
        net.Compute__Error(sample_rows, Y)
        net.Backward_Pass(sample_rows)
        net.Update_Derivative_Weight(sample_rows)
        t1 = time.perf_counter()
        net.Update_Parameter(sample_rows, sample_rows)
        t2 = time.perf_counter()
        t_sample += t1 - t0
        t_update += t2 - t1
        reps += 1
    t_sample /= reps
    t_update /= reps
    t_step = t_sample * wl["batch"] / sample_rows + t_update
    return dict(value=wl["batch"] / t_step, unit="samples/s", cores=threads, kind="port",
                sample="%d of %d examples through the full-width network (%.2f s per pass, %d passes) scaled to the batch, plus the full weight update (%.2f s)"
                       % (sample_rows, wl["batch"], t_sample, reps, t_update))


# profile families of the library (myea_hip_profile_read): name, what its `work` counts
FAMILIES = (("forward", "flop"), ("dx", "flop"), ("dw", "flop"), ("update", "byte"), ("dx_dw_pair", "flop"),
            ("lstm_forward_loop", "flop"), ("lstm_backward_loop", "flop"),
            ("normalization", "byte"), ("bias_gradient", "byte"), ("output_error", "byte"), ("softmax", "byte"))
KERNEL_NAMES = {"forward": "gemm_forward", "dx": "gemm_dx", "dw": "gemm_dw", "dx_dw_pair": "gemm_dx_dw_pair", "update": "optimizer_update"}


def run_workload(name, steps, warmup, separate_update=False, repeats=1):
    """Times `steps` training steps of one workload on cuda:0 (inputs resident in HBM): that is the throughput.  Then runs
    `steps` more with the library's per-family HIP-event timers on for the per-kernel figures - a pair of timing events around
    every launch keeps launches from overlapping their neighbours' tails and costs 3 % (the wide dense stack) to 16 % (the
    normalised stack of 43 short launches) of a step, so the two are not measured in one pass; both step times are reported.
    Returns the measurements as a dict."""
    import numpy as np
    import torch
    from myea_amd import binding as mb
    from myea_amd.synthetic import glorot_parameters

    wl = WORKLOADS[name]
    B = wl["batch"]
    desc = mb.make_desc(wl["layers"], B, wl.get("depth", 1))
    h = mb.default_hyper(type_optimizer_function=mb.OPTIMIZER[wl["optimizer"]], type_loss_function=mb.LOSS[wl["loss"]], **wl["hyper"])
    net = mb.HipNetwork(desc, h)
    net.set_stream(torch.cuda.current_stream().cuda_stream)
    net.set_state_propagation(mb.STATE_TRAINING)
    net.upload_parameters(glorot_parameters(desc, 2))
    net.Clear_Training_Arrays()
    if desc.total_mask_units:
        net.upload_masks((np.random.default_rng(4).uniform(0, 1, desc.total_mask_units) < 0.5).astype(np.uint8))
    X, Y = make_inputs(np, wl, 2)
    xd, yd = torch.from_numpy(X).cuda(), torch.from_numpy(Y).cuda()   # inputs resident in HBM before the timed region

    def step(separate=separate_update):
        net.Forward_Pass(B, xd, on_device=True)
        net.Compute__Error(B, yd, on_device=True)
        if separate:
            net.Backward_Pass__Update_Derivative_Weight(B)     # the two calls of Train_Batch_BP as one entry point
            net.Update_Parameter(B, B)
        else:   # and the update that follows them: a layer's weights step as soon as their gradient is complete
            net.Backward_Pass__Update_Derivative_Weight__Update_Parameter(B, B)

    for _ in range(warmup):
        step()
    blocks = []
    for _ in range(max(1, repeats)):      # every block: exactly `steps` steps between two synchronisations
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            step()
        torch.cuda.synchronize()
        blocks.append((time.perf_counter() - t0) * 1e3 / steps)
    ms_per_step = sorted(blocks)[(len(blocks) - 1) // 2]   # the median block (the lower middle one of an even count)
    net.profile_enable(True)
    for f in range(len(FAMILIES)):
        net.profile_read(f)            # drop anything recorded so far
    t2 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    t3 = time.perf_counter()
    ms_per_step_events = (t3 - t2) * 1e3 / steps
    fam = {fname: net.profile_read(i) for i, (fname, _) in enumerate(FAMILIES)}
    # When layers took their update beside the contractions below them (more update launches than steps), the contractions'
    # durations above include what the update took from them: a third pass with Update_Parameter as a call of its own times
    # the contractions alone on the device.
    fam_alone, ms_per_step_alone = None, None
    if not separate_update and fam["update"][0] > steps:
        t4 = time.perf_counter()
        for _ in range(steps):
            step(separate=True)
        torch.cuda.synchronize()
        ms_per_step_alone = (time.perf_counter() - t4) * 1e3 / steps
        fam_alone = {fname: net.profile_read(i) for i, (fname, _) in enumerate(FAMILIES)}
    net.profile_enable(False)
    loss = net.get_loss()
    net.close()

    kernels = {}
    for fname, unit in FAMILIES:
        n, ms, work = fam[fname]
        if n == 0:
            continue
        rate = work / max(ms * 1e-3, 1e-12)
        entry = dict(launches=n, avg_ms=ms / n, ms_per_step=ms / steps)
        if unit == "flop":
            entry.update(tflops=rate / 1e12, frac_mfma_peak=rate / 1e12 / PEAK_FP32_MFMA_TFLOPS)
        else:
            entry.update(gbs=rate / 1e9, frac_hbm_peak=rate / 1e9 / PEAK_HBM_GBS)
        kernels[KERNEL_NAMES.get(fname, fname)] = entry

    def mfma_aggregate(names, fam=fam):
        n = sum(fam[k][0] for k in names)
        ms = sum(fam[k][1] for k in names)
        flop = sum(fam[k][2] for k in names)
        achieved = flop / (ms * 1e-3) / 1e12 if ms > 0 else 0.0
        return dict(bound="mfma", achieved=achieved, peak=PEAK_FP32_MFMA_TFLOPS, unit="TFLOP/s", frac=achieved / PEAK_FP32_MFMA_TFLOPS,
                    launches=n, avg_launch_ms=ms / max(n, 1), flops_per_launch=flop / max(n, 1), ms_per_step=ms / steps)

    return dict(workload=name, wl=wl, desc_parameters=int(desc.total_parameters), batch=B, ms_per_step=ms_per_step, value=B / (ms_per_step * 1e-3),
                ms_per_step_blocks=blocks,
                ms_per_step_events=ms_per_step_events,
                kernels=kernels, loss_per_output=loss.loss_values / max(loss.number_loss, 1),
                contractions=mfma_aggregate(("forward", "dx", "dw", "dx_dw_pair")),
                contractions_alone=mfma_aggregate(("forward", "dx", "dw", "dx_dw_pair"), fam_alone) if fam_alone else None,
                ms_per_step_events_alone=ms_per_step_alone,
                time_loops=mfma_aggregate(("lstm_forward_loop", "lstm_backward_loop")))


def config_of(r):
    wl = r["wl"]
    return {"workload": r["workload"], "batch": r["batch"], "sequence_length": wl.get("depth", 1),
            "layers": ["res%d" % l["block_depth"] if l.get("type") == "residual" else
                       "%s_k%d_s%d" % (l["type"], l["kernel"], l["stride"]) if "pooling" in l.get("type", "") else
                       ("bilstm%d" if l.get("bidirectional") else "lstm%d" if l.get("type") == "lstm" else
                        "indrnn%d" if l.get("type") == "ind_rnn" else "fc%d") % l["units"] for l in wl["layers"]],
            "optimizer": wl["optimizer"], "parameters": r["desc_parameters"],
            "gemm_flops_per_step": gemm_flops_per_step(wl["layers"], r["batch"], wl.get("depth", 1))}


SECONDARY = "lstm512x2_t64_b256_amsgrad"   # the metric's other half
OTHERS = ("fc2048x8_bn_relu_dropout_b512_nesterov", "bilstm1024_t512_b64_adabound")
EXAMPLE = "resindrnn_smnist28_t28_b256_amsgrad"   # the reference's own worked example: a leg of the default line too


def timed_blocks(stream_call):
    """stream_call() enqueues one launch on torch's current stream; returns the mean duration in ms of a launch inside a block
    of 20 back-to-back launches between two events on that stream (best of 3 blocks, after a warm-up launch)"""
    import torch
    stream_call()
    best = None
    for _ in range(3):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(20):
            stream_call()
        b.record()
        b.synchronize()
        ms = a.elapsed_time(b) / 20
        best = ms if best is None or ms < best else best
    return best


def optimizer_update_alone(parameters):
    """myea_hip_optimizer_update alone on the device over `parameters` floats (the headline configuration's vector), per
    optimizer: algorithmic bytes (every vector the update reads or writes, once) over the launch's duration."""
    import ctypes as C
    import torch
    from myea_amd import binding as mb
    lib = mb.load_library()
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    vec = [torch.zeros(parameters, dtype=torch.float32, device="cuda") for _ in range(5)]
    vec[1].normal_(0, 1e-2)
    legs = {}
    for name, kw, bytes_per in (("adam", dict(type_optimizer_function=mb.OPTIMIZER["ADAM"]), 32), ("amsgrad", dict(type_optimizer_function=mb.OPTIMIZER["AMSGRAD"]), 40),
                                ("adabound", dict(type_optimizer_function=mb.OPTIMIZER["ADABOUND"]), 32),
                                ("nesterov", dict(type_optimizer_function=mb.OPTIMIZER["GD"], use_Nesterov=1, learning_momentum=0.9), 24)):
        h = mb.default_hyper(optimizer_time_step=1.0, **kw)

        def call():
            rc = lib.myea_hip_optimizer_update(stream, C.byref(h), parameters, parameters, 1.0, *(C.c_void_p(v.data_ptr()) for v in vec))
            if rc != 0:
                raise RuntimeError((lib.myea_hip_last_error() or b"").decode())
        ms = timed_blocks(call)
        gbs = bytes_per * parameters / (ms * 1e-3) / 1e9
        legs[name] = dict(avg_ms=ms, bytes_per_parameter=bytes_per, gbs=gbs, frac_hbm_peak=gbs / PEAK_HBM_GBS)
    return dict(kernel="update_kernel (myea_hip_optimizer_update alone on the device)", parameters=parameters, optimizers=legs)


def measured_ceilings():
    """What this device reaches on a kernel of nothing but FP32 MFMAs and on a streaming triad, beside the published peaks."""
    import ctypes as C
    import torch
    from myea_amd import binding as mb
    lib = mb.load_library()
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    tf, gb = C.c_double(), C.c_double()
    if lib.myea_hip_ceiling_mfma_f32(stream, 20000, 3, C.byref(tf)) != 0 or lib.myea_hip_ceiling_hbm_triad(stream, 1 << 30, 5, C.byref(gb)) != 0:
        raise RuntimeError((lib.myea_hip_last_error() or b"").decode())
    return {"mfma_f32_tflops": tf.value, "mfma_f32_published": PEAK_FP32_MFMA_TFLOPS, "hbm_triad_gbs": gb.value, "hbm_published": PEAK_HBM_GBS,
            "how": "myea_hip_ceiling_mfma_f32 (independent v_mfma_f32_32x32x2_f32, 2 wavefronts per SIMD) and myea_hip_ceiling_hbm_triad (3 x 1 GiB)"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--repeats", type=int, default=10, help="timed blocks of exactly --steps steps; value = the median block")
    ap.add_argument("--workload", default="fc4096x4_b1024_adam", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-secondary", action="store_true", help="skip the LSTM-512 leg and the two short legs of the other configurations that the default workload's line also carries")
    ap.add_argument("--no-ceilings", action="store_true", help="skip the measured MFMA / HBM ceilings")
    ap.add_argument("--separate-update", action="store_true", help="Update_Parameter as a call of its own behind the backward pass")
    ap.add_argument("--cpu-sample-rows", type=int, default=0, help="examples in the CPU sample (default: sized for ~20 s)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py: this build runs on one GPU only (--gpus 1); no multi-GPU path exists")

    import torch

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    r = run_workload(args.workload, args.steps, args.warmup, args.separate_update, args.repeats)
    wl, B = r["wl"], r["batch"]
    has_loops = r["time_loops"]["launches"] > 0
    alone = r["contractions_alone"]
    roofline = dict(alone or r["contractions"])
    roofline["kernel"] = "gemm_f32_mfma_kernel / gemm_pair_kernel (forward, dX, dW and paired dX + dW launches)"
    roofline["gemm_ms_per_step"] = roofline.pop("ms_per_step")
    roofline["measured_in"] = "events_pass"
    if alone:
        # the timed steps run the optimizer update of a layer on a second stream beside the contractions of the layers below it;
        # what a contraction's events then span includes the update's share of the device.  The figures above are the
        # contractions alone (Update_Parameter as a call of its own); these are the same launches beside the update.
        roofline["measured_in"] = "events_pass_update_apart"
        roofline["beside_update"] = {k: r["contractions"][k] for k in ("achieved", "frac", "avg_launch_ms")}
        roofline["beside_update"]["gemm_ms_per_step"] = r["contractions"]["ms_per_step"]
    traffic = RECORDED_TRAFFIC.get(args.workload)
    roofline["traffic"] = traffic["bytes_per_launch"] if traffic else None
    if traffic:
        roofline["traffic_source"] = traffic["source"]

    out = {
        "metric": "train samples/s (fwd+bwd+Adam) FC-4096x4 & LSTM-512; % FP32 MFMA/HBM peak",
        "value": r["value"],
        "unit": "samples/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": r["ms_per_step"],
        # the timed block (exactly `steps` steps between two synchronisations) was run `repeats` times: value and ms_per_step are the
        # median block's, the others are listed
        "repeats": len(r["ms_per_step_blocks"]), "ms_per_step_blocks": [round(x, 4) for x in r["ms_per_step_blocks"]],
        "ms_per_step_spread": {"min": min(r["ms_per_step_blocks"]), "max": max(r["ms_per_step_blocks"])},
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": config_of(r),
        "roofline": roofline,
        "kernels": r["kernels"],
        # the per-kernel figures (roofline, kernels, time_loops) come from a second pass of `steps` steps with a pair of HIP timing
        # events around every launch; those events slow the step itself, so `value` is from the pass without them
        "events_pass": {"steps": args.steps, "ms_per_step": r["ms_per_step_events"]},
        "update": "separate call" if args.separate_update else "with the backward pass (one call)",
        "loss_per_output": r["loss_per_output"],
    }
    if alone:
        out["events_pass_update_apart"] = {"steps": args.steps, "ms_per_step": r["ms_per_step_events_alone"]}
    if has_loops:
        out["time_loops"] = dict(r["time_loops"], kernel="lstm_resident_forward_kernel / lstm_resident_backward_kernel (or one lstm_fused_* launch per step)")
    if args.workload != SECONDARY and args.workload == "fc4096x4_b1024_adam" and not args.no_secondary:
        sec_steps = max(5, 2 * args.steps // 3)
        s = run_workload(SECONDARY, sec_steps, max(2, args.warmup), args.separate_update, args.repeats)
        loops = dict(s["time_loops"], kernel="lstm_resident_forward_kernel + lstm_resident_backward_kernel: the recurrent contractions and gate math of steps 1 .. T-1, one launch per layer and pass")
        sec_traffic = RECORDED_TRAFFIC.get(SECONDARY)
        loops["traffic"] = sec_traffic["bytes_per_launch"] if sec_traffic else None
        if sec_traffic:
            loops["traffic_source"] = sec_traffic["source"]
        out["secondary"] = {"workload": SECONDARY, "value": s["value"], "unit": "samples/s", "ms_per_step": s["ms_per_step"],
                            "repeats": len(s["ms_per_step_blocks"]), "ms_per_step_blocks": [round(x, 4) for x in s["ms_per_step_blocks"]],
                            "steps": sec_steps, "events_pass": {"steps": sec_steps, "ms_per_step": s["ms_per_step_events"]}, "config": config_of(s), "roofline": loops,
                            "contractions": s["contractions"], "kernels": s["kernels"], "loss_per_output": s["loss_per_output"]}
        # the other two configurations of the baseline that are timed on the GPU, a few steps each, so that one run records all four
        out["other_configurations"] = []
        for name in OTHERS + (EXAMPLE,):
            # timed like the headline: the same warm-up, the median of `repeats` blocks of exactly `steps` steps each
            o = run_workload(name, max(5, args.steps // 3), max(2, args.warmup), args.separate_update, repeats=args.repeats)
            leg = {"workload": name, "value": o["value"], "unit": "samples/s", "ms_per_step": o["ms_per_step"], "steps": max(5, args.steps // 3),
                   "warmup": max(2, args.warmup), "repeats": args.repeats, "ms_per_step_blocks": [round(x, 4) for x in o["ms_per_step_blocks"]],
                   "config": config_of(o), "contractions": o["contractions_alone"] or o["contractions"], "kernels": o["kernels"], "loss_per_output": o["loss_per_output"]}
            if o["time_loops"]["launches"] > 0:
                leg["time_loops"] = o["time_loops"]
            out["other_configurations"].append(leg)
        # the memory-bound update alone on the device, per optimizer, over the headline configuration's parameter vector
        out["optimizer_update_alone"] = optimizer_update_alone(r["desc_parameters"])
    if not args.no_ceilings:
        out["ceilings"] = measured_ceilings()
    if not args.no_cpu_baseline:
        threads = min(16, os.cpu_count() or 1)
        rows = args.cpu_sample_rows
        if rows <= 0:
            # sized from the layer widths for ~20 s at ~15 GFLOP/s per thread (gcc -O2 vectorises the inner loops)
            flop_per_row = gemm_flops_per_step(wl["layers"], 1, wl.get("depth", 1))
            rows = int(max(4, min(B, 20.0 * threads * 15.0e9 / flop_per_row)))
            rows = max(threads, rows - rows % threads)
        out["cpu_baseline"] = cpu_baseline(wl, rows, threads)
        if "secondary" in out:   # the metric's other half on the same host cores: whole sequences through the oracle
            swl = WORKLOADS[SECONDARY]
            flop_per_row = gemm_flops_per_step(swl["layers"], 1, swl.get("depth", 1))
            rows = int(max(4, min(swl["batch"], 20.0 * threads * 15.0e9 / flop_per_row)))
            rows = max(threads, rows - rows % threads)
            out["secondary"]["cpu_baseline"] = cpu_baseline(swl, min(rows, swl["batch"]), threads)
            for leg in out.get("other_configurations", []):   # the example network is small enough to walk whole on the host
                if leg["workload"] == EXAMPLE:
                    leg["cpu_baseline"] = cpu_baseline(WORKLOADS[EXAMPLE], WORKLOADS[EXAMPLE]["batch"], threads)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
