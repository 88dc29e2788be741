"""Element-wise glue kernels through the kernel seam: conversions are exact restatements of IEEE
round-to-nearest-even (`copy_f32_half`, `copy_f32_bf16` of crates/ojas-cuda/src/kernels/mod.rs
naming), at ragged lengths and at offsets that defeat the 128-bit path."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _cases(pkg):
    x = pkg.synth.normal_f32(5000, "glue", "x") * 37.0
    x[:8] = [0.0, -0.0, 65504.0, 65520.0, 1e-8, -1e-8, 2049.0, 2051.0]
    return x


@pytest.mark.parametrize("n", [1, 7, 8, 9, 1000, 4099])
@pytest.mark.parametrize("shift", [0, 1])
def test_conversions(gpu, pkg, n, shift):
    gpu.ensure_family("glue")
    x = _cases(pkg)[:n]
    xb = pkg.synth.to_bf16_bits(x)
    with np.errstate(over="ignore"):   # 65520 -> inf is the expected binary16 result
        h_of_f32 = x.astype(np.float16).view(np.uint16)
        h_of_bf16 = pkg.synth.bf16_bits_to_f32(xb).astype(np.float16).view(np.uint16)
    for name, src, esz_in, esz_out, want in [
        ("copy_f32_half", x, 4, 2, h_of_f32),
        ("copy_f32_bf16", x, 4, 2, xb),
        ("copy_bf16_f32", xb, 2, 4, pkg.synth.bf16_bits_to_f32(xb).view(np.uint32)),
        ("copy_bf16_half", xb, 2, 2, h_of_bf16),
    ]:
        xin = gpu.alloc_bytes(n * esz_in + 32)
        gpu.write_bytes(xin, shift * esz_in, np.ascontiguousarray(src).view(np.uint8))
        out = gpu.upload_bytes(np.full(n * esz_out + 64, 0xA5, np.uint8))
        grid, block = gpu.launch_shape(name, 0, n, 0)
        gpu.dispatch(gpu.begin(), name, [(xin, shift * esz_in), (out, shift * esz_out)], [n], grid, block)
        raw = gpu.read(out, n * esz_out + 64, np.uint8)
        got = raw[shift * esz_out:shift * esz_out + n * esz_out].view(want.dtype)
        assert np.array_equal(got, want), name
        assert np.all(raw[:shift * esz_out] == 0xA5) and np.all(raw[shift * esz_out + n * esz_out:] == 0xA5), name


def test_fill_zero(gpu, pkg):
    gpu.ensure_family("glue")
    for n, off in [(1, 0), (5, 4), (1024, 0), (4099, 12)]:
        buf = gpu.upload_bytes(np.full(n * 4 + 64, 0xA5, np.uint8))
        grid, block = gpu.launch_shape("fill_zero_u32", 0, n, 0)
        gpu.dispatch(gpu.begin(), "fill_zero_u32", [(buf, off)], [n], grid, block)
        raw = gpu.read(buf, n * 4 + 64, np.uint8)
        assert np.all(raw[off:off + 4 * n] == 0) and np.all(raw[:off] == 0xA5) and np.all(raw[off + 4 * n:] == 0xA5)


@pytest.mark.parametrize("n,nz,shift", [(1, 1, 0), (9, 5, 1), (4099, 1024, 0), (1000, 4099, 1), (70000, 3, 0)])
def test_conversion_and_zero_fill_in_one_launch(gpu, pkg, n, nz, shift):
    """copy_{bf16,f32}_half_zero: the first CB workgroups convert, the others clear; nothing outside either range moves."""
    gpu.ensure_family("glue")
    x = np.resize(_cases(pkg), n).astype(np.float32)
    xb = pkg.synth.to_bf16_bits(x)
    with np.errstate(over="ignore"):
        wants = {"copy_f32_half_zero": (x, 4, x.astype(np.float16).view(np.uint16)),
                 "copy_bf16_half_zero": (xb, 2, pkg.synth.bf16_bits_to_f32(xb).astype(np.float16).view(np.uint16))}
    for name, (src, esz, want) in wants.items():
        xin = gpu.alloc_bytes(n * esz + 32)
        gpu.write_bytes(xin, shift * esz, np.ascontiguousarray(src).view(np.uint8))
        out = gpu.upload_bytes(np.full(n * 2 + 64, 0xA5, np.uint8))
        z = gpu.upload_bytes(np.full(nz * 4 + 64, 0xA5, np.uint8))
        grid, block = gpu.launch_shape(name, 0, n, nz)
        cb = (n // 8 + 255) // 256 + 1
        assert grid[0] > cb
        gpu.dispatch(gpu.begin(), name, [(xin, shift * esz), (out, shift * 2), (z, shift * 4)], [n, nz, cb], grid, block)
        raw = gpu.read(out, n * 2 + 64, np.uint8)
        assert np.array_equal(raw[shift * 2:shift * 2 + n * 2].view(np.uint16), want), name
        assert np.all(raw[:shift * 2] == 0xA5) and np.all(raw[shift * 2 + n * 2:] == 0xA5), name
        zr = gpu.read(z, nz * 4 + 64, np.uint8)
        assert np.all(zr[shift * 4:shift * 4 + nz * 4] == 0) and np.all(zr[:shift * 4] == 0xA5) and np.all(zr[shift * 4 + nz * 4:] == 0xA5)
        with pytest.raises(pkg.OjasHipError, match="CB"):
            gpu.dispatch(gpu.begin(), name, [(xin, shift * esz), (out, shift * 2), (z, shift * 4)], [n, nz, grid[0]], grid, block)
