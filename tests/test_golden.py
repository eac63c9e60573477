"""Committed golden vectors (tests/golden/tq8_cases.npz, written by tests/golden/make_golden.py):
the oracle must keep reproducing them on the CPU, and the HIP path must reproduce them on the GPU
without the oracle in the loop."""
import os

import numpy as np
import pytest

import __graft_entry__ as entry

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "tq8_cases.npz")


def _cases():
    data = np.load(GOLDEN, allow_pickle=False)
    names = sorted({k.split("/")[0] for k in data.files})
    return data, names


class _Obj:
    def __init__(self, **kw):
        self.__dict__.update(kw)


@pytest.mark.parametrize("name", _cases()[1])
def test_oracle_reproduces_golden(oracle, name):
    d, _ = _cases()
    g = lambda k: d[f"{name}/{k}"]
    qw = oracle.QuantizedWeight(g("pp"), g("pr"), g("norms"), g("seeds"))
    pb = 5 if len(g("cbp")) == 32 else 4
    cbp = oracle.Codebook(g("cbp"), pb)
    cbr = oracle.Codebook(g("cbr"), 4 if len(g("cbr")) == 16 else 3)
    bs = int(g("bs")[0])
    W = oracle.dequantize_weight_cpu(qw, cbp, cbr, bs)
    assert np.array_equal(W, g("W"))
    assert np.array_equal(oracle.matmul_xwT(g("x"), W, acc_double=True), g("y"))
    # the quantiser regenerates the packed planes from the LCG weights bit for bit
    rows, cols = g("W").shape
    rb = 0 if not g("pr").any() else (4 if len(g("cbr")) == 16 else 3)
    shared = bool(g("seeds")[1] == 0 and rb)
    q2 = oracle.quantize_weight(oracle.lcg_matrix(rows, cols, 42), cbp, cbr, pb, rb, bs, shared)
    assert np.array_equal(q2.packed_primary, g("pp")) and np.array_equal(q2.packed_residual, g("pr"))
    assert np.array_equal(q2.norms, g("norms")) and np.array_equal(q2.seeds, g("seeds"))


@pytest.mark.gpu
@pytest.mark.parametrize("name", _cases()[1])
def test_hip_path_reproduces_golden(name):
    tq = entry.load_package()
    d, _ = _cases()
    g = lambda k: d[f"{name}/{k}"]
    qw = _Obj(packed_primary=g("pp"), packed_residual=g("pr"), norms=g("norms"), seeds=g("seeds"))
    cbp, cbr = _Obj(centroids=g("cbp")), _Obj(centroids=g("cbr"))
    bs = int(g("bs")[0])
    rows, cols = g("W").shape
    layer = tq.TurboQuantLinear(cols, rows, qw, cbp, cbr, bs)
    assert np.array_equal(layer.dequantize(), g("W"))           # bit-exact weights
    if len(g("cbp")) == 16:                                      # fused forward: 4-bit primaries
        y = layer.forward(g("x"))
        rel = np.linalg.norm(y - g("y")) / np.linalg.norm(g("y"))
        assert rel < 1e-3
    layer.close()
