"""Kernel-level GPU checks through the C ABI: the FP32 MFMA contraction in all operand layouts against float64
matmul (brute force) on ragged shapes, at BASELINE config 2's full shapes against torch.matmul (library routine)
and through linearity; the fused optimizer kernel at an odd length against a float64 restatement."""
import ctypes as C

import numpy as np
import pytest
import torch

from myea_amd import binding as mb
from tests.common import assert_close

pytestmark = pytest.mark.gpu


def _gemm(lib, a_kc, b_kc, acc, M, N, K, A, B, Cc, lda=None, ldb=None, ldc=None):
    lda = lda or (K if a_kc else M)
    ldb = ldb or (K if b_kc else N)
    ldc = ldc or N
    rc = lib.myea_hip_gemm_f32(None, int(a_kc), int(b_kc), int(acc), M, N, K, C.c_void_p(A.data_ptr()), lda,
                               C.c_void_p(B.data_ptr()), ldb, C.c_void_p(Cc.data_ptr()), ldc)
    assert rc == 0, lib.myea_hip_last_error()
    torch.cuda.synchronize()


SHAPES = [(1, 1, 1), (3, 5, 7), (64, 64, 32), (65, 63, 33), (128, 256, 100), (130, 70, 257), (256, 128, 64),
          (1000, 36, 20), (17, 1000, 520), (512, 1024, 96), (1024, 1000, 128),
          # at most 32 columns over at most 64 k's and 256 rows or more: the kernel that feeds the matrix unit straight from memory
          (256, 32, 32), (300, 31, 31), (257, 10, 64), (7168, 23, 29), (1000, 1, 33)]


@pytest.mark.parametrize("a_kc,b_kc", [(1, 1), (1, 0), (0, 0), (0, 1)])
@pytest.mark.parametrize("M,N,K", SHAPES)
def test_gemm_layouts_against_float64_matmul(a_kc, b_kc, M, N, K):
    lib = mb.load_library()
    rng = np.random.default_rng(M * 31 + N * 7 + K)
    A = rng.normal(0, 1, (M, K)).astype(np.float32)
    B = rng.normal(0, 1, (K, N)).astype(np.float32)
    C0 = rng.normal(0, 1, (M, N)).astype(np.float32)
    want = A.astype(np.float64) @ B.astype(np.float64)
    Ad = torch.from_numpy(np.ascontiguousarray(A if a_kc else A.T)).cuda()
    Bd = torch.from_numpy(np.ascontiguousarray(B.T if b_kc else B)).cuda()
    Cd = torch.from_numpy(C0.copy()).cuda()
    _gemm(lib, a_kc, b_kc, 0, M, N, K, Ad, Bd, Cd)
    tol = 2e-6 * np.sqrt(K) * np.abs(A).max() * np.abs(B).max() + 1e-6
    assert np.max(np.abs(Cd.cpu().numpy() - want)) <= tol * 4
    _gemm(lib, a_kc, b_kc, 1, M, N, K, Ad, Bd, Cd)      # accumulate: C = C + AB
    assert np.max(np.abs(Cd.cpu().numpy() - 2 * want)) <= tol * 8


def test_gemm_unaligned_pointers_and_leading_dimensions():
    lib = mb.load_library()
    M, N, K = 70, 50, 45
    rng = np.random.default_rng(0)
    big_a = torch.from_numpy(rng.normal(0, 1, (M, K + 3)).astype(np.float32)).cuda()
    big_b = torch.from_numpy(rng.normal(0, 1, (N, K + 5)).astype(np.float32)).cuda()
    big_c = torch.zeros((M, N + 2), dtype=torch.float32).cuda()
    A, B = big_a[:, 1:K + 1], big_b[:, 2:K + 2]
    rc = lib.myea_hip_gemm_f32(None, 1, 1, 0, M, N, K, C.c_void_p(big_a.data_ptr() + 4), K + 3, C.c_void_p(big_b.data_ptr() + 8), K + 5,
                               C.c_void_p(big_c.data_ptr() + 4), N + 2)
    assert rc == 0
    torch.cuda.synchronize()
    want = A.double().cpu().numpy() @ B.double().cpu().numpy().T
    got = big_c.cpu().numpy()
    assert_close(got[:, 1:N + 1], want, 1e-4, 1e-4)
    assert np.all(got[:, 0] == 0) and np.all(got[:, N + 1] == 0)        # nothing written outside the tile
    assert lib.myea_hip_gemm_f32(None, 1, 1, 0, M, N, K, C.c_void_p(big_a.data_ptr()), K - 1, C.c_void_p(big_b.data_ptr()), K + 5,
                                 C.c_void_p(big_c.data_ptr()), N + 2) == mb.E_INVALID


@pytest.mark.parametrize("a_kc,b_kc,M,N,K", [(1, 1, 1024, 4096, 4096), (1, 0, 1024, 4096, 4096), (0, 0, 4096, 4096, 1024),
                                             (1, 1, 1024, 1000, 4096), (1, 0, 1024, 4096, 1000), (0, 0, 1000, 4096, 1024)])
def test_gemm_full_size_config2_shapes(a_kc, b_kc, M, N, K):
    """forward / dX / dW contractions of the 4096-wide stack at batch 1024: against torch.matmul in fp32, and
    linearity C(A1 + A2) = C(A1) + C(A2)."""
    lib = mb.load_library()
    g = torch.Generator(device="cuda").manual_seed(M + N + K)
    A1 = torch.randn((M, K) if a_kc else (K, M), generator=g, device="cuda")
    A2 = torch.randn_like(A1)
    B = torch.randn((N, K) if b_kc else (K, N), generator=g, device="cuda")
    outs = []
    for A in (A1, A2, A1 + A2):
        Cd = torch.empty((M, N), device="cuda")
        _gemm(lib, a_kc, b_kc, 0, M, N, K, A, B, Cd)
        outs.append(Cd)
    ref = (A1 if a_kc else A1.t()).double() @ (B.t() if b_kc else B).double()
    err = (outs[0].double() - ref).abs().max().item()
    assert err <= 5e-6 * np.sqrt(K) * 16 + 1e-5, err
    lin = (outs[0] + outs[1] - outs[2]).abs().max().item()
    assert lin <= 5e-6 * np.sqrt(K) * 32 + 1e-4, lin


@pytest.mark.parametrize("kind,extra", [("GD", dict(learning_momentum=0.0)), ("GD", {}), ("GD", dict(use_Nesterov=1)), ("ADAM", {}),
                                        ("AMSGRAD", {}), ("ADABOUND", {}), ("ADAM", dict(regularization__weight_decay=1e-2))])
def test_optimizer_kernel_odd_length(kind, extra):
    lib = mb.load_library()
    n, n_w = 1_000_003, 700_001
    rng = np.random.default_rng(5)
    w = rng.normal(0, 1, n).astype(np.float32)
    g = rng.normal(0, 1, n).astype(np.float32)
    s = [np.abs(rng.normal(0, 0.1, n)).astype(np.float32) for _ in range(3)]
    h = mb.default_hyper(type_optimizer_function=mb.OPTIMIZER[kind], optimizer_time_step=3.0, **extra)
    wd, gd = torch.from_numpy(w.copy()).cuda(), torch.from_numpy(g.copy()).cuda()
    sd = [torch.from_numpy(x.copy()).cuda() for x in s]
    rc = lib.myea_hip_optimizer_update(None, C.byref(h), n, n_w, 0.5, *[C.c_void_p(t.data_ptr()) for t in (wd, gd, *sd)])
    assert rc == 0, lib.myea_hip_last_error()
    torch.cuda.synchronize()
    assert torch.count_nonzero(gd).item() == 0
    W, G = w.astype(np.float64), 0.5 * g.astype(np.float64)
    a, b, c = (x.astype(np.float64) for x in s)
    lr, mu, t = 0.01, (0.0 if extra.get("learning_momentum") == 0.0 else 0.9), 3.0
    reg = extra.get("regularization__weight_decay", 0.0) * W * (np.arange(n) < n_w)
    if kind == "GD":
        if mu == 0.0: step = lr * G
        else:
            a = lr * G + mu * a
            step = (mu * a - lr * G) if extra.get("use_Nesterov") else a
    else:
        a = 0.9 * a + 0.1 * G
        b = 0.999 * b + 0.001 * G * G
        lr_t = 1e-3 * np.sqrt(1 - 0.999 ** t) / (1 - 0.9 ** t)
        if kind == "ADAM": step = lr_t * a / (np.sqrt(b) + 1e-8)
        elif kind == "AMSGRAD":
            c = np.maximum(c, b); step = lr_t * a / (np.sqrt(c) + 1e-8)
        else: step = np.clip(lr_t / (np.sqrt(b) + 1e-8), 0.1 * (1 - 1 / (1e-3 * t + 1)), 0.1 * (1 + 1 / (1e-3 * t))) * a
    assert_close(wd.cpu().numpy(), W - step - reg, 1e-5, 1e-6, what="parameters")
    if kind != "GD" or mu != 0.0:
        assert_close(sd[0].cpu().numpy(), a, 1e-5, 1e-7, what="state 0")
    if kind != "GD":
        assert_close(sd[1].cpu().numpy(), b, 1e-5, 1e-7, what="state 1")
    if kind == "AMSGRAD":
        assert_close(sd[2].cpu().numpy(), c, 1e-5, 1e-7, what="state 2")
