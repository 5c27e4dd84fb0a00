import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")
    # the CPU checker is built on demand; the HIP library is never built from inside a test
    lib = os.path.join(ROOT, "oracle", "libmyea_oracle.so")
    if not os.path.exists(lib):
        subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle")])
    _cross_checked_make_desc()


def _cross_checked_make_desc():
    """Every description any test lays out goes through BOTH implementations of the index table - the product's
    (myea_amd/csrc/myea_layout.c, inside libmyea_hip.so) and the checker's own restatement of the reference's Compile sequence
    (oracle/myea_oracle_layout.c) - and the two must agree on the outcome and, field by field, on the table."""
    import ctypes as C
    from myea_amd import binding as mb
    original = mb.make_desc
    if getattr(original, "cross_checked", False):
        return

    def make_desc(layers, batch_size, recurrent_depth=1, network=None, lib=None):
        from tests.oracle_lib import load_oracle
        libs = [lib] if lib is not None else []
        try:
            libs.append(mb.load_library())
        except (RuntimeError, OSError):
            pass   # the HIP library is not built: the caller finds out where it needs it
        libs.append(load_oracle())
        results = []
        for l in libs:
            try:
                results.append(original(layers, batch_size, recurrent_depth, network, lib=l))
            except ValueError as e:
                results.append(str(e))
        first = results[0]
        for other in results[1:]:
            if isinstance(first, str) or isinstance(other, str):
                assert isinstance(first, str) and isinstance(other, str), "the two layouts disagree on whether %r can be laid out: %r / %r" % (layers, first, other)
                continue
            for name, _ in mb.NetDesc._fields_:
                if name != "layers":
                    assert getattr(first, name) == getattr(other, name), "layout of %r: %s differs: %r / %r" % (layers, name, getattr(first, name), getattr(other, name))
            for i in range(first.n_layers):
                for name, _ in mb.LayerDesc._fields_:
                    a, b = getattr(first.layers[i], name), getattr(other.layers[i], name)
                    a, b = (list(a), list(b)) if hasattr(a, "__len__") else (a, b)
                    assert a == b, "layout of %r: layer %d %s differs: %r / %r" % (layers, i, name, a, b)
        if isinstance(first, str):
            raise ValueError(first)
        return first

    make_desc.cross_checked = True
    mb.make_desc = make_desc


@pytest.fixture(scope="session")
def hip_available():
    import torch
    return torch.cuda.is_available()
