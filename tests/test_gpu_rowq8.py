"""The CPU models' row-int8 matmul on the GPU, bit for bit against the CPU oracle.

Reference: `W::Q8` / `quant_row_i8` / `matmul` / `dot_i8` (crates/ojas-cpu/src/cpu_math.rs:14-23,
174-179, 187-289, 404-415) and the load-time requantization `q8_rows_from_f16`
(crates/ojas-formats/src/quant.rs:16-39).  Integer sums are exact and the epilogue's three f32
operations are rounded one by one in the reference's order, so the bar is equality of bits.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _weights_f16(pkg, n, k, tag):
    return (pkg.synth.normal_f32(n * k, "rowq8", tag, n, k) * 0.05).astype(np.float16)


@pytest.mark.parametrize("n,k", [(5, 16), (64, 4096), (300, 2560), (1, 14336)])
def test_requantization_is_bit_exact(gpu, orc, pkg, n, k):
    w = _weights_f16(pkg, n, k, "w").reshape(n, k)
    w[n // 2] = 0                       # an all-zero row takes scale 1
    w[0, :4] = [0.5, -0.5, 1.5, -2.5]   # ties round away from zero
    wd = gpu.upload_bytes(w.view(np.uint16))
    q, s = gpu.alloc_bytes(n * k), gpu.alloc(n)
    gpu.q8rows_from_f16(wd, n, k, q, s)
    wq, ws = orc.q8_rows_from_f16(w.view(np.uint16).reshape(-1), n, k)
    assert np.array_equal(gpu.read(s, n).view(np.uint32), ws.view(np.uint32))
    assert np.array_equal(gpu.read(q, n * k, np.int8), wq)


@pytest.mark.parametrize("m,n,k,bias", [(1, 64, 256, False), (1, 4096, 4096, True), (3, 333, 2560, True),
                                        (8, 96, 14336, False), (19, 130, 512, True), (64, 256, 1024, False)])
def test_matmul_is_bit_exact(gpu, orc, pkg, m, n, k, bias):
    w = _weights_f16(pkg, n, k, "mw").reshape(n, k)
    wq, ws = orc.q8_rows_from_f16(w.view(np.uint16).reshape(-1), n, k)
    x = pkg.synth.normal_f32(m * k, "rowq8", "x", m, k).reshape(m, k)
    x[0, :3] = [0.0, 1e-30, -3.0]
    if m > 1:
        x[1] = 0.0                      # an all-zero token takes scale 1
    b = pkg.synth.normal_f32(n, "rowq8", "b", n) if bias else None
    guard = np.float32(777.25)
    yd = gpu.upload(np.full(m * n + 8, guard, np.float32))
    gpu.matmul_q8(gpu.upload(x), gpu.upload_bytes(wq), gpu.upload(ws), yd, n, k, m,
                  bias=gpu.upload(b) if bias else None)
    got = gpu.read(yd, m * n + 8)
    assert np.all(got[m * n:] == guard)
    want = orc.matmul_q8(wq, ws, n, k, x, bias=b)
    assert np.array_equal(got[:m * n].reshape(m, n).view(np.uint32), want.view(np.uint32))


def test_kernel_seam_and_errors(gpu, orc, pkg):
    gpu.ensure_family("rowq8")
    m, n, k = 2, 40, 64
    x = pkg.synth.normal_f32(m * k, "rowq8", "sx").reshape(m, k)
    xd, q, s = gpu.upload(x), gpu.alloc_bytes(m * k), gpu.alloc(m)
    grid, block = gpu.launch_shape("quant_rows_i8", k, 0, m)
    gpu.dispatch(gpu.begin(), "quant_rows_i8", [(xd, 0), (q, 0), (s, 0)], [k, m], grid, block)
    for t in range(m):
        wq, ws = orc.quant_row_i8(x[t])
        assert np.array_equal(gpu.read(q, m * k, np.int8)[t * k:(t + 1) * k], wq)
        assert gpu.read(s, m)[t] == np.float32(ws)
    with pytest.raises(pkg.OjasHipError, match="multiple of 16"):
        gpu.matmul_q8(xd, q, s, gpu.alloc(8), 2, 24, 1)
    with pytest.raises(pkg.OjasHipError, match="needs"):
        gpu.matmul_q8(xd, q, s, gpu.alloc(8), n, k, m)
