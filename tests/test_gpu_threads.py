"""Host threads: tq_linear_forward on different layers from several threads at once (each thread its own
stream and buffers), and on ONE layer from several threads for the paths that use no per-layer workspace
(one row per call).  Results must equal the single-threaded ones bit for bit; tq_last_error is per thread."""
import ctypes
import threading

import numpy as np
import pytest

from test_gpu_graph import _Hip, _bits, _layer

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def tq():
    import __graft_entry__ as entry
    pkg = entry.load_package()
    pkg.lib()
    return pkg


def test_forward_from_four_threads(tq, oracle):
    o = oracle
    shapes = [(384, 1024, 512, "shared"), (200, 2048, 256, "dual"), (96, 5120, 512, "shared"), (130, 1536, 512, "primary_only")]
    layers = [_layer(tq, o, out, inf, bs, mode, seed=20 + i)[0] for i, (out, inf, bs, mode) in enumerate(shapes)]
    shared_layer = layers[0]
    rng = np.random.default_rng(9)
    xb = [{b: _bits(o, rng, b, inf) for b in (1, 4)} for (_, inf, _, _) in shapes]
    hips = [_Hip() for _ in shapes]
    # single-threaded results first
    want, xs, ys = [], [], []
    for i, (out, inf, bs, mode) in enumerate(shapes):
        h = hips[i]
        layers[i].reserve(4)
        xs.append({b: h.upload(xb[i][b]) for b in (1, 4)})
        ys.append({b: h.alloc(b * out * 4) for b in (1, 4)})
        w = {}
        for b in (1, 4):
            layers[i].forward_device(xs[i][b], tq.BF16, b, ys[i][b], tq.F32, h.stream)
            w[b] = h.download(ys[i][b], (b, out))
        want.append(w)
    y_shared = [h.alloc(shapes[0][0] * 4) for h in hips]
    failures = []

    def work(i):
        try:
            h, (out, inf, bs, mode) = hips[i], shapes[i]
            for turn in range(40):
                b = (1, 4)[turn % 2]
                layers[i].forward_device(xs[i][b], tq.BF16, b, ys[i][b], tq.F32, h.stream)
                # one row of the layer every thread shares: no per-layer workspace involved
                shared_layer.forward_device(xs[0][1], tq.BF16, 1, y_shared[i], tq.F32, h.stream)
                if turn % 10 == 9:
                    assert h.rt.hipStreamSynchronize(h.stream) == 0
                    got = np.empty((b, out), np.float32)
                    assert h.rt.hipMemcpy(got.ctypes.data_as(ctypes.c_void_p), ys[i][b], got.nbytes, 2) == 0
                    if not np.array_equal(got, want[i][b]):
                        failures.append((i, turn, "own layer"))
                    got = np.empty((1, shapes[0][0]), np.float32)
                    assert h.rt.hipMemcpy(got.ctypes.data_as(ctypes.c_void_p), y_shared[i], got.nbytes, 2) == 0
                    if not np.array_equal(got, want[0][1]):
                        failures.append((i, turn, "shared layer"))
            # an error in this thread is this thread's message
            rc = tq.lib().tq_linear_forward(layers[i]._h, None, tq.BF16, 1, ys[i][1], tq.F32, None)
            if rc == 0 or "NULL" not in tq.last_error():
                failures.append((i, "error message", tq.last_error()))
        except Exception as e:                                 # noqa: BLE001 - reported through the list
            failures.append((i, repr(e)))

    threads = [threading.Thread(target=work, args=(i,)) for i in range(len(shapes))]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not any(t.is_alive() for t in threads)
    assert not failures, failures
    for layer in layers:
        layer.close()
    for h in hips:
        h.close()
