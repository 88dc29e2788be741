"""MXFP4 as the reference packs it for its native matvec — { u8 e8m0 scale; u8 qs[16] }, 17 bytes per 32 weights,
synthetic type id 139 (crates/ojas-core/src/quant_src.rs:91-95, :333-353; crates/ojas-formats/src/mxfp4.rs): the
decoder bit for bit, `gemv_nat_mxfp4*` by name and through `mm`.  No CPU dot exists for the format (the CPU path widens
it), so the matvec is judged against the exact block values in double, like the other GPU-path formats."""
import numpy as np
import pytest

from conftest import peak_err

pytestmark = pytest.mark.gpu
MXFP4 = 139
LUT = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0])


def test_decoder_bit_exact(gpu, orc, pkg):
    """Every scale exponent below the reserved 255 against every code; ragged block counts; odd block addresses."""
    nb = 255 * 2 + 3
    raw = np.zeros((nb, 17), np.uint8)
    raw[:, 0] = np.arange(nb) % 255
    raw[:, 1:] = (np.arange(nb * 16).reshape(nb, 16) * 37 + np.arange(nb)[:, None]) & 0xFF
    raw = raw.reshape(-1)
    out = gpu.alloc_bytes(nb * 32 * 2)
    gpu.dequant_f16(MXFP4, gpu.upload_bytes(raw), nb * 32, out)
    got = gpu.read(out, nb * 32, np.uint16)
    assert np.array_equal(got, orc.dequant_to_f16(raw, MXFP4, nb * 32))
    blocks = raw.reshape(nb, 17)
    e = blocks[:, 0].astype(np.int64)
    scale = np.where(e == 0, 0.0, 2.0 ** (e - 127.0))                # e8m0: the exponent field alone (mxfp4.rs:44-47)
    want = (scale[:, None, None] * LUT[np.stack([blocks[:, 1:] & 0xF, blocks[:, 1:] >> 4], -1)]).reshape(-1)
    with np.errstate(over="ignore"):
        assert np.array_equal(got, want.astype(np.float16).view(np.uint16))
    gpu.dequant_f16(MXFP4, gpu.upload_bytes(raw), 7 * 32, out, raw_off=5 * 17)
    assert np.array_equal(gpu.read(out, 7 * 32, np.uint16), got[5 * 32:12 * 32])


@pytest.mark.parametrize("n,k", [(1, 32), (13, 2560), (1000, 4096), (96, 14336), (4099, 4096), (33001, 2816)])
def test_float_matvec_matches_the_exact_dot(gpu, orc, pkg, n, k):
    w = pkg.synth.weights(MXFP4, n, k, "mx", n, k)
    x = pkg.synth.normal_f32(k, "mx", "x", n, k)
    lin = gpu.lin(MXFP4, n, k, w)
    yd = gpu.upload(np.full(n + 2, 12345.0, np.float32))
    gpu.mm(gpu.upload(x), lin, yd, 1, False, y_off=4)
    got = gpu.read(yd, n + 2)
    assert got[0] == 12345.0 and got[-1] == 12345.0, "wrote outside y"
    assert peak_err(got[1:-1], orc.matmul_ref(w, MXFP4, n, k, x)[0]) <= 1e-5
    with pytest.raises(pkg.OjasHipError, match="f32 activations"):
        gpu.mm(gpu.upload(x), lin, yd, 1, act_mode=pkg.ACT_Q8K)


def test_entries_by_name(gpu, orc, pkg):
    """gemv_nat_mxfp4{,_r1,_r2,_accum,_bias,_m,_px} as a reference caller dispatches them (the format table's row)."""
    gpu.ensure_family("gemv")
    n, k, m = 203, 1056, 3
    w = pkg.synth.weights(MXFP4, n, k, "mxn")
    xs = pkg.synth.normal_f32(m * k, "mxn", "x").reshape(m, k)
    ref = orc.matmul_ref(w, MXFP4, n, k, xs).astype(np.float32)
    wd, xd = gpu.upload_bytes(np.concatenate([np.zeros(1, np.uint8), w])), gpu.upload(xs)     # rows from an odd address
    outs = {}
    for name in ("gemv_nat_mxfp4", "gemv_nat_mxfp4_r1", "gemv_nat_mxfp4_r2", "gemv_nat_mxfp4_px"):
        grid, block = gpu.launch_shape(name, k, n, 1)
        yd = gpu.upload(np.full(n + 2, 777.0, np.float32))
        gpu.dispatch(gpu.begin(), name, [(xd, 0), (wd, 1), (yd, 4)], [k, n], grid, block)
        got = gpu.read(yd, n + 2)
        assert got[0] == 777.0 and got[-1] == 777.0, name
        assert peak_err(got[1:-1], ref[0]) <= 1e-5, name
        outs[name] = got[1:-1].copy()
    first = outs["gemv_nat_mxfp4"]
    assert all(np.array_equal(first, o) for o in outs.values())
    grid, block = gpu.launch_shape("gemv_nat_mxfp4_bias", k, n, 1)
    bias = (1000.0 + np.arange(n)).astype(np.float32)
    yb = gpu.alloc(n)
    gpu.dispatch(gpu.begin(), "gemv_nat_mxfp4_bias", [(xd, 0), (wd, 1), (yb, 0), (gpu.upload(bias), 0)], [k, n], grid, block)
    assert np.array_equal(gpu.read(yb, n), first + bias)
    y0 = pkg.synth.normal_f32(n, "mxn", "y0")
    ya = gpu.upload(y0)
    gpu.dispatch(gpu.begin(), "gemv_nat_mxfp4_accum", [(xd, 0), (wd, 1), (ya, 0)], [k, n], grid, block)
    assert np.array_equal(gpu.read(ya, n), y0 + first)
    grid, block = gpu.launch_shape("gemv_nat_mxfp4_m", k, n, m)
    ym = gpu.upload(np.full(m * n + 2, 777.0, np.float32))
    gpu.dispatch(gpu.begin(), "gemv_nat_mxfp4_m", [(xd, 0), (wd, 1), (ym, 4)], [k, n, m, 0], grid, block)
    got = gpu.read(ym, m * n + 2)
    assert got[0] == 777.0 and got[-1] == 777.0
    assert peak_err(got[1:-1].reshape(m, n), ref) <= 1e-5
