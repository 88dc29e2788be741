"""Recorded chains of dispatches replay with the same results as eager submission."""
import numpy as np
import pytest

from conftest import peak_err

pytestmark = pytest.mark.gpu
Q4_K = 12


@pytest.fixture(params=["list", "graph"])
def replay_mode(request, monkeypatch):
    """The two replay engines: the library's own command list (default) and an instantiated hipGraph."""
    if request.param == "graph":
        monkeypatch.setenv("OJAS_HIP_REPLAY", "graph")     # read by capture_begin
    else:
        monkeypatch.delenv("OJAS_HIP_REPLAY", raising=False)
    return request.param


def test_recorded_step_replays_identically(gpu, orc, pkg, replay_mode):
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


def test_replay_survives_a_scratch_buffer_that_grows(gpu, orc, pkg, replay_mode):
    """`ojh_mm` stages quantized activations in the library's scratch; a chain recorded at m = 1 keeps that address.
    A later eager call with more tokens outgrows the buffer: the old one must stay alive for the chain."""
    n, k = 256, 2048
    w = pkg.synth.q4k_weights(n, k, "graph", "w2")
    lin = gpu.lin(Q4_K, n, k, w)
    x1 = pkg.synth.normal_f32(k, "graph", "x1")
    xd, yd = gpu.upload(x1), gpu.alloc(n)
    gpu.mm(xd, lin, yd, 1, act_mode=pkg.ACT_Q8K)     # eager once: families loaded, scratch sized for one token
    want = gpu.read(yd, n)
    gpu.capture_begin()
    gpu.mm(xd, lin, yd, 1, act_mode=pkg.ACT_Q8K)
    graph = gpu.capture_end()
    m_big = 4096                                        # 8 MB of int8 activations: far beyond the recorded buffer
    xb, yb = gpu.upload(pkg.synth.normal_f32(m_big * k, "graph", "xbig")), gpu.alloc(m_big * n)
    gpu.mm(xb, lin, yb, m_big, act_mode=pkg.ACT_Q8K)
    big = [gpu.alloc_bytes(m_big * k) for _ in range(4)]   # allocations that would reuse freed scratch addresses
    for b in big:
        gpu.memset0(b)
    for _ in range(3):
        gpu.memset0(yd)
        graph.launch()
        assert np.array_equal(gpu.read(yd, n), want)
    assert peak_err(want, orc.matvec_kq(w, Q4_K, n, k, x1)) <= 2e-5
    graph.free()


def test_a_failed_call_while_recording_leaves_the_device_usable(gpu, pkg, replay_mode):
    n, k = 64, 512
    lin = gpu.lin(Q4_K, n, k, pkg.synth.q4k_weights(n, k, "graph", "w3"))
    xd, yd, small = gpu.upload(pkg.synth.normal_f32(k, "graph", "x3")), gpu.alloc(n), gpu.alloc(n // 2)
    gpu.mm(xd, lin, yd, 1, act_mode=pkg.ACT_Q8K)
    want = gpu.read(yd, n)
    gpu.capture_begin()
    with pytest.raises(pkg.OjasHipError) as e:
        gpu.mm(xd, lin, small, 1, act_mode=pkg.ACT_Q8K)        # y too small: refused before anything is queued
    assert e.value.code == -5
    try:
        gpu.capture_end().free()
    except pkg.OjasHipError:
        pass                                                     # the recording is over either way
    gpu.memset0(yd)
    gpu.mm(xd, lin, yd, 1, act_mode=pkg.ACT_Q8K)
    assert np.array_equal(gpu.read(yd, n), want)
