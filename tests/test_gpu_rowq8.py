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


def _quantized(gpu, orc, pkg, m, n, k, tag):
    w = _weights_f16(pkg, n, k, tag).reshape(n, k)
    wq, ws = orc.q8_rows_from_f16(w.view(np.uint16).reshape(-1), n, k)
    x = pkg.synth.normal_f32(m * k, "rowq8", tag, "x", m, k).reshape(m, k)
    x[m // 2] = 0.0
    x[m - 1] *= 300.0
    return wq, ws, x


@pytest.mark.parametrize("m,n,k,bias", [(9, 100, 512, True), (33, 130, 16, False), (64, 128, 1040, True), (70, 77, 4096, False),
                                        (300, 1000, 2560, True)])
def test_matrix_tile_by_name(gpu, orc, pkg, m, n, k, bias):
    """`matmul_q8row_mt{,_sr}`: ragged tokens, rows and K (any multiple of 16), with and without a bias, nothing written
    past row M; every number of K slices gives the bits of the per-row kernel and leaves the tile counters at zero."""
    gpu.ensure_family("rowq8")
    wq, ws, x = _quantized(gpu, orc, pkg, m, n, k, "mt")
    b = pkg.synth.normal_f32(n, "rowq8", "mtb", n) if bias else None
    want = orc.matmul_q8(wq, ws, n, k, x, bias=b).view(np.uint32)
    xq, sx = gpu.alloc_bytes(m * k), gpu.alloc(m)
    gpu.dispatch(gpu.begin(), "quant_rows_i8", [(gpu.upload(x), 0), (xq, 0), (sx, 0)], [k, m], *gpu.launch_shape("quant_rows_i8", k, 0, m))
    wd, sd, bd = gpu.upload_bytes(wq), gpu.upload(ws), (gpu.upload(b) if bias else None)
    grid = [(n + 127) // 128, (m + 63) // 64, 1]
    guard = np.float32(777.25)

    def run(name, extra_bufs, consts, g):
        yd = gpu.upload(np.full(m * n + n, guard, np.float32))
        gpu.dispatch(gpu.begin(), name, [(xq, 0), (sx, 0), (wd, 0), (sd, 0), (yd, 0), (bd, 0)] + extra_bufs, consts, g, [256, 1, 1])
        got = gpu.read(yd, m * n + n)
        assert np.all(got[m * n:] == guard), "wrote past the last token"
        assert np.array_equal(got[:m * n].reshape(m, n).view(np.uint32), want), name

    run("matmul_q8row_mt", [], [k, n, m], grid)
    run("matmul_q8row_mt128", [], [k, n, m], [grid[0], (m + 127) // 128, 1])
    tiles, nks = grid[0] * grid[1], (k + 127) // 128
    cnt = gpu.alloc_bytes(tiles * 4)
    gpu.memset0(cnt)
    for nsplit in sorted({min(s, nks) for s in (1, 2, 3, 5, nks)}):
        per = (nks + nsplit - 1) // nsplit
        slices = (nks + per - 1) // per
        part = gpu.alloc(tiles * slices * 8192)
        for _ in range(2):
            run("matmul_q8row_mt_sr", [(part, 0), (cnt, 0)], [k, n, m, nsplit], [grid[0], grid[1], slices])
            assert not gpu.read(cnt, tiles, np.uint32).any()
    with pytest.raises(pkg.OjasHipError, match="grid must be"):
        gpu.dispatch(gpu.begin(), "matmul_q8row_mt", [(xq, 0), (sx, 0), (wd, 0), (sd, 0), (gpu.alloc(m * n), 0), (bd, 0)],
                     [k, n, m], [grid[0] + 1, grid[1], 1], [256, 1, 1])


@pytest.mark.parametrize("m,n,k,bias", [(9, 4096, 4096, False), (40, 333, 14336, True), (129, 2000, 2048, False), (512, 640, 1536, True)])
def test_batches_take_the_matrix_tile_with_the_same_bits(gpu, orc, pkg, m, n, k, bias):
    """Through `ojh_matmul_q8`: whole tiles and K slices as the library picks them — and a token's result does not depend
    on its batch (the same rows, one token at a time, on the per-row kernel)."""
    wq, ws, x = _quantized(gpu, orc, pkg, m, n, k, "route")
    b = pkg.synth.normal_f32(n, "rowq8", "rb", n) if bias else None
    wd, sd, bd = gpu.upload_bytes(wq), gpu.upload(ws), (gpu.upload(b) if bias else None)
    yd = gpu.upload(np.full(m * n + 8, 777.25, np.float32))
    gpu.matmul_q8(gpu.upload(x), wd, sd, yd, n, k, m, bias=bd)
    got = gpu.read(yd, m * n + 8)
    assert np.all(got[m * n:] == np.float32(777.25))
    got = got[:m * n].reshape(m, n).view(np.uint32)
    rows = np.unique(np.concatenate([np.arange(min(n, 40)), np.arange(n - min(n, 40), n)]))
    want = orc.matmul_q8(np.ascontiguousarray(wq.reshape(n, k)[rows]).reshape(-1), ws[rows], len(rows), k, x,
                         bias=b[rows] if bias else None)
    assert np.array_equal(got[:, rows], want.view(np.uint32))
    one = gpu.alloc(n)
    for t in (0, m // 2, m - 1):
        gpu.matmul_q8(gpu.upload(x[t]), wd, sd, one, n, k, 1, bias=bd)
        assert np.array_equal(gpu.read(one, n).view(np.uint32), got[t])


@pytest.mark.parametrize("m,n,k,bias", [(1, 64, 16, False), (1, 4097, 4096, True), (2, 333, 2560, False), (3, 50, 14336, True),
                                        (5, 1000, 1040, False), (8, 4096, 4096, True), (8, 31, 16384, False)])
def test_few_tokens_staged_in_lds_by_name(gpu, orc, pkg, m, n, k, bias):
    """`matmul_q8row_dec{,_l}`: every token count of each compiled width, an odd last row, a K that is no multiple of
    1024 and one whose 8 tokens need the larger LDS; the library's launch shape and a small one give the same bits."""
    gpu.ensure_family("rowq8")
    wq, ws, x = _quantized(gpu, orc, pkg, m, n, k, "dec")
    b = pkg.synth.normal_f32(n, "rowq8", "decb", n) if bias else None
    want = orc.matmul_q8(wq, ws, n, k, x, bias=b).view(np.uint32)
    xq, sx = gpu.alloc_bytes(m * k), gpu.alloc(m)
    gpu.dispatch(gpu.begin(), "quant_rows_i8", [(gpu.upload(x), 0), (xq, 0), (sx, 0)], [k, m], *gpu.launch_shape("quant_rows_i8", k, 0, m))
    wd, sd, bd = gpu.upload_bytes(wq), gpu.upload(ws), (gpu.upload(b) if bias else None)
    names = ["matmul_q8row_dec_l"] + (["matmul_q8row_dec"] if m * k <= 65536 else [])
    for name in names:
        g, blk = gpu.launch_shape(name, k, n, m)
        for grid, block in ((list(g), list(blk)), ([3, 1, 1], [128, 1, 1])):
            yd = gpu.upload(np.full(m * n + n, 777.25, np.float32))
            gpu.dispatch(gpu.begin(), name, [(xq, 0), (sx, 0), (wd, 0), (sd, 0), (yd, 0), (bd, 0)], [k, n, m], grid, block)
            got = gpu.read(yd, m * n + n)
            assert np.all(got[m * n:] == np.float32(777.25))
            assert np.array_equal(got[:m * n].reshape(m, n).view(np.uint32), want), (name, grid, block)
    if m * k > 65536:
        with pytest.raises(pkg.OjasHipError, match="exceeds"):
            gpu.dispatch(gpu.begin(), "matmul_q8row_dec", [(xq, 0), (sx, 0), (wd, 0), (sd, 0), (gpu.alloc(m * n), 0), (bd, 0)],
                         [k, n, m], [3, 1, 1], [128, 1, 1])


@pytest.mark.parametrize("m,k,off", [(1, 4096, 0), (3, 14336, 0), (2, 20000, 0), (5, 100, 0), (2, 18, 0), (2, 4096, 1), (4, 16384, 0)])
def test_token_quantizer_bit_exact_at_every_block_size(gpu, orc, pkg, m, k, off):
    """`quant_rows_i8`: rows held in registers (up to 16 values a thread), rows read twice (longer, K no multiple of 4, or
    a start that is not 16-byte aligned), with the library's block and with one and sixteen waves."""
    gpu.ensure_family("rowq8")
    x = pkg.synth.normal_f32(m * k + off, "rowq8", "tq", m, k)
    x[off:off + 4] = np.float32(np.abs(x).max()) * np.float32([0.5, 1.5, -2.5, 3.5]) / np.float32(127.0)
    if m > 1:
        x[off + k:off + 2 * k] = 0.0
    xd = gpu.upload(x)
    want = [orc.quant_row_i8(x[off + t * k:off + (t + 1) * k]) for t in range(m)]
    g, b = gpu.launch_shape("quant_rows_i8", k, 0, m)
    assert list(g) == [m, 1, 1]
    for block in sorted({b[0], 64, 1024}):
        q, s = gpu.alloc_bytes(m * k + 16), gpu.alloc(m)
        gpu.memset0(q)
        gpu.dispatch(gpu.begin(), "quant_rows_i8", [(xd, 4 * off), (q, 0), (s, 0)], [k, m], [m, 1, 1], [block, 1, 1])
        got = gpu.read(q, m * k + 16, np.int8)
        assert not got[m * k:].any()
        for t in range(m):
            assert np.array_equal(got[t * k:(t + 1) * k], want[t][0]), (block, t)
            assert gpu.read(s, m)[t] == np.float32(want[t][1])
