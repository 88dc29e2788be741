"""Recorded chains of dispatches replay with the same results as eager submission."""
import numpy as np
import pytest

from conftest import peak_err

pytestmark = pytest.mark.gpu
Q4_K = 12


def test_recorded_step_replays_identically(gpu, orc, pkg):
    n, k = 300, 1024
    w = pkg.synth.q4k_weights(n, k, "graph", "w")
    lin = gpu.lin(Q4_K, n, k, w)
    xs = [pkg.synth.normal_f32(k, "graph", "x", i) for i in range(4)]
    xd, yd = gpu.upload(xs[0]), gpu.alloc(n)
    xq, xsc = gpu.alloc_bytes(k), gpu.alloc(k // 256)

    def chain():
        gpu.quant_q8k(xd, 1, k, xq, xsc)
        gpu.mm_q8k(xq, xsc, lin, yd)

    chain()                      # eager once: loads the families, sizes nothing lazily later
    eager = gpu.read(yd, n)
    gpu.capture_begin()
    chain()
    with pytest.raises(pkg.OjasHipError, match="recording"):
        gpu.submit()
    with pytest.raises(pkg.OjasHipError, match="recording"):
        gpu.alloc(16)
    graph = gpu.capture_end()
    # replay several times with eager work and synchronisations in between; every replay is checked
    for i, x in enumerate(xs):
        gpu.write_bytes(xd, 0, x)
        gpu.memset0(yd)
        graph.launch()
        got = gpu.read(yd, n)
        want = orc.matvec_kq(w, Q4_K, n, k, x)
        assert peak_err(got, want) <= 2e-5, i
        if i == 0:
            assert np.array_equal(got, eager)
    graph.free()
