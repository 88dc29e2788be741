"""Prefill / verify matmul on the MFMA tiles against the CPU oracle.

Oracle: x . W^T accumulated in double (crates/ojas-cuda/tests/prefill_gemm_q.rs:116-130), once
with x rounded to f16 and W as the f16 bits the tile is specified to hold (the kernel's own
error) and once with x and W unrounded.  Metrics and the reference's bounds:
(max|d| / rms, rms(d) / rms) < (5e-3, 5e-4) against the rounded oracle and < (2e-2, 3e-3) against
the unrounded one (prefill_gemm_q.rs:288-343).  Every tile here feeds the MFMA exactly the
specified f16 bits, so the first pair is held to (2e-5, 5e-6).

The specified bits: `dequant_to_f16` for Q5_K, Q6_K, Q8_0 and for Q4_K under ACT_FLOAT_EXACT ("x4"
below); for Q4_K under ACT_FLOAT the binary16 fma qa*q + qb of the reference's `gemm_mm_q4l`
(crates/ojas-cuda/src/kernels/gemm_q.rs:104-140), oracle weight mode 2.
"""
import numpy as np
import pytest

from conftest import peak_err, rms_errs

pytestmark = pytest.mark.gpu
Q8_0, Q4_K, Q5_K, Q6_K = 8, 12, 13, 14
X4 = "q4k-exact"   # Q4_K through the tile that holds dequant_to_f16 bits
TIGHT = (2e-5, 5e-6)


def _mode(pkg, ty):
    """(GGUF type, act_mode, oracle weight mode) of a test case label."""
    if ty == X4:
        return Q4_K, pkg.ACT_FLOAT_EXACT, 1
    return ty, pkg.ACT_FLOAT, 2 if ty == Q4_K else 1


def _run(gpu, pkg, orc, ty, m, k, n, accum=False, x_dtype="f32", split=None):
    ty, act, wmode = _mode(pkg, ty)
    w = pkg.synth.weights(ty, n, k, "gemm", ty, n, k)
    x = pkg.synth.normal_f32(m * k, "gemm", "x", m, k).reshape(m, k)
    if x_dtype == "bf16":
        xb = pkg.synth.to_bf16_bits(x)
        x = pkg.synth.bf16_bits_to_f32(xb).reshape(m, k)
        xd = gpu.upload_bytes(xb)
    else:
        xd = gpu.upload(x)
    y0 = pkg.synth.normal_f32(m * n, "gemm", "y0").reshape(m, n) if accum else np.zeros((m, n), np.float32)
    sent = np.full(n, 12345.5, np.float32)
    yd = gpu.upload(np.concatenate([y0.ravel(), sent]))
    lin = gpu.lin(ty, n, k, w)
    gpu.mm(xd, lin, yd, m, accum, act_mode=act, x_dtype=pkg.X_BF16 if x_dtype == "bf16" else pkg.X_F32)
    got = gpu.read(yd, m * n + n)
    assert np.all(got[m * n:] == 12345.5), "wrote past row M"
    got = got[:m * n].reshape(m, n)
    want16 = orc.matmul_ref(w, ty, n, k, x, wmode=wmode, xmode=1) + y0
    want32 = orc.matmul_ref(w, ty, n, k, x) + y0
    return rms_errs(got, want16), rms_errs(got, want32)


# the reference's sweep: ragged M and N, accumulate, short and long K (prefill_gemm_q.rs:346-380)
SWEEP = [(64, 256, 128, False), (33, 512, 130, False), (100, 1024, 200, True), (256, 4096, 256, False),
         (300, 2048, 72, True), (512, 1024, 384, False), (77, 14336, 64, False), (129, 768, 513, False),
         (700, 768, 300, True)]


@pytest.mark.parametrize("ty", [Q4_K, X4, Q5_K, Q6_K, Q8_0])
@pytest.mark.parametrize("m,k,n,accum", SWEEP)
def test_gemm_sweep(gpu, orc, pkg, ty, m, k, n, accum):
    e16, e32 = _run(gpu, pkg, orc, ty, m, k, n, accum)
    assert e16[0] < TIGHT[0] and e16[1] < TIGHT[1], (e16, "vs the rounded oracle")
    assert e32[0] < 2e-2 and e32[1] < 3e-3, (e32, "vs the unrounded oracle")


@pytest.mark.parametrize("ty", [Q4_K, X4, Q5_K, Q6_K])
def test_gemm_bf16_activations(gpu, orc, pkg, ty):
    """bf16 activations (the prefill / verify input type) convert to f16 exactly in range."""
    e16, e32 = _run(gpu, pkg, orc, ty, 128, 2048, 256, x_dtype="bf16")
    assert e16[0] < TIGHT[0] and e16[1] < TIGHT[1], e16
    assert e32[0] < 2e-2 and e32[1] < 3e-3, e32


@pytest.mark.parametrize("ty", [Q4_K, X4, Q5_K, Q6_K, Q8_0])
def test_tile_holds_the_reference_decoders_bits(gpu, orc, pkg, ty):
    """One-hot activations read the tile back: y[m][n] must be the specified f16 weight [n][m]
    exactly, for every weight of two super-blocks per row and for extreme scales."""
    k, n = 512, 160
    ty, act, wmode = _mode(pkg, ty)
    bb, wpb = pkg.synth.BLOCK_SHAPE[ty]
    raw = orc.synth_blocks(ty, n * k // wpb).reshape(-1, bb).copy()
    scales = np.array([0x0001, 0x03FF, 0x0400, 0x8001, 0xBC00, 0x3555, 0x1234, 0x2E66], np.uint16)
    off = 208 if ty == Q6_K else 0
    for i in range(raw.shape[0]):
        raw[i, off:off + 2] = scales[i % 8:i % 8 + 1].view(np.uint8)
        if ty in (Q4_K, Q5_K):
            raw[i, 2:4] = scales[(i * 3 + 1) % 8:(i * 3 + 1) % 8 + 1].view(np.uint8)
    raw = raw.reshape(-1)
    bits = orc.q4l_weights_f16(raw, k, n) if wmode == 2 else orc.dequant_to_f16(raw, ty, n * k)
    want = bits.view(np.float16).astype(np.float32).reshape(n, k)
    lin = gpu.lin(ty, n, k, raw)
    x = np.eye(k, dtype=np.float32)
    yd = gpu.alloc(k * n)
    gpu.mm(gpu.upload(x), lin, yd, k, act_mode=act)
    got = gpu.read(yd, k * n).reshape(k, n)
    # value equality: a -0 weight reads back as +0 through the accumulator, every other bit must match
    assert np.array_equal(got, want.T)
    nz = want.T != 0
    assert np.array_equal(got.view(np.uint32)[nz], want.T.copy().view(np.uint32)[nz])


@pytest.mark.parametrize("kernel,family,bm,bn,wmode", [("gemm_mm_q4k_sk", "gemm", 256, 128, 1),
                                                       ("gemm_mm_q4kl_sk", "gemm_xl", 256, 256, 2),
                                                       ("gemm_mm_q4kl_bd_sk", "gemm_xl", 128, 256, 2),
                                                       ("gemm_mm_q4kl_bd256_sk", "gemm_xl", 256, 256, 2),
                                                       ("gemm_mm_q4kl_bdk_sk", "gemm_xl", 128, 64, 2)])
def test_split_k_entry_through_the_kernel_seam(gpu, orc, pkg, kernel, family, bm, bn, wmode):
    """Split-K entries dispatched by name with several K slices; y holds what is accumulated into."""
    gpu.ensure_family(family)
    gpu.ensure_family("glue")
    m, k, n = 140, 2048, 300
    w = pkg.synth.q4k_weights(n, k, "gemmsk", "w")
    x = pkg.synth.normal_f32(m * k, "gemmsk", "x").reshape(m, k)
    xh = gpu.upload_bytes(x.astype(np.float16))
    wd = gpu.upload_bytes(w)
    want = orc.matmul_ref(w, Q4_K, n, k, x, wmode=wmode, xmode=1)
    for nsplit in (1, 3, 8):
        y0 = pkg.synth.normal_f32(m * n, "gemmsk", "y0", nsplit).reshape(m, n)
        yd = gpu.upload(y0)
        enc = gpu.begin()
        gpu.dispatch(enc, kernel, [(xh, 0), (wd, 0), (yd, 0)], [k, n, m, nsplit],
                     [(n + bn - 1) // bn, (m + bm - 1) // bm, nsplit], [256, 1, 1])
        gpu.submit(enc)
        e = rms_errs(gpu.read(yd, m * n).reshape(m, n), want + y0)
        assert e[0] < 1e-4 and e[1] < 2e-5, (nsplit, e)
    with pytest.raises(pkg.OjasHipError, match="grid must be"):
        gpu.dispatch(enc, kernel, [(xh, 0), (wd, 0), (yd, 0)], [k, n, m, 2], [3, 1, 1], [256, 1, 1])


@pytest.mark.parametrize("kernel,bm", [("gemm_mm_q4kl_bd_sr", 128), ("gemm_mm_q4kl_bd256_sr", 256)])
def test_split_k_slices_meeting_in_scratch(gpu, orc, pkg, kernel, bm):
    """`_sr`: K slices leave partial tiles in a scratch buffer and the last to arrive adds them in slice order — store
    or accumulate, no zero fill, the counters back at zero for the next launch, the same bits on every run and the bits
    of the unsplit tile when there is one slice; more slices than super-blocks leave the surplus empty."""
    gpu.ensure_family("gemm_xl")
    m, k, n = 300, 2048, 520
    w = pkg.synth.q4k_weights(n, k, "gemmsr", "w")
    x = pkg.synth.normal_f32(m * k, "gemmsr", "x").reshape(m, k)
    xh, wd = gpu.upload_bytes(x.astype(np.float16)), gpu.upload_bytes(w)
    want = orc.matmul_ref(w, Q4_K, n, k, x, wmode=2, xmode=1)
    tiles = ((n + 255) // 256) * ((m + bm - 1) // bm)
    cnt = gpu.upload_bytes(np.zeros(tiles, np.uint32))
    sent = np.full(n, 12345.5, np.float32)
    plain = kernel[:-3]
    yp = gpu.alloc(m * n)
    gpu.dispatch(gpu.begin(), plain, [(xh, 0), (wd, 0), (yp, 0)], [k, n, 0, m], [(n + 255) // 256, (m + bm - 1) // bm, 1], [256, 1, 1])
    unsplit = gpu.read(yp, m * n)
    for nsplit in (1, 2, 3, 8):
        slices = -(-(k // 256) // -(-(k // 256) // nsplit))
        part = gpu.upload(np.full(tiles * slices * bm * 256, np.nan, np.float32))
        grid = [(n + 255) // 256, (m + bm - 1) // bm, nsplit]
        runs = []
        for accum in (0, 1, 0):
            y0 = pkg.synth.normal_f32(m * n, "gemmsr", "y0", nsplit, accum).reshape(m, n)
            yd = gpu.upload(np.concatenate([y0.ravel(), sent]))
            gpu.dispatch(gpu.begin(), kernel, [(xh, 0), (wd, 0), (yd, 0), (part, 0), (cnt, 0)], [k, n, m, nsplit, accum], grid, [256, 1, 1])
            got = gpu.read(yd, m * n + n)
            assert np.array_equal(got[m * n:], sent), "wrote past row M"
            e = rms_errs(got[:m * n].reshape(m, n), want + (y0 if accum else 0.0))
            assert e[0] < 1e-4 and e[1] < 2e-5, (nsplit, accum, e)
            assert not np.any(gpu.read(cnt, tiles, np.uint32)), "a tile counter was left non-zero"
            if not accum:
                runs.append(got[:m * n].copy())
        assert np.array_equal(runs[0], runs[1]), "slices added in an order that depends on arrival"
        if nsplit == 1:
            assert np.array_equal(runs[0], unsplit)
    with pytest.raises(pkg.OjasHipError, match="needs"):
        gpu.dispatch(gpu.begin(), kernel, [(xh, 0), (wd, 0), (yp, 0), (cnt, 0), (cnt, 0)], [k, n, m, 2, 0],
                     [(n + 255) // 256, (m + bm - 1) // bm, 2], [256, 1, 1])


def test_mm_with_reproducible_split_k(gpu, orc, pkg, monkeypatch):
    """A device handle opened under OJAS_HIP_GEMM_SR=1 routes the split-K launches of `mm` to the `_sr` entries: the
    same result to the order of the f32 sums as the default handle's atomics, and the same bits on every run."""
    m, k, n = 128, 4096, 1536          # 6 tiles of 256 rows: split into K slices on any GPU with more than 6 CUs
    w = pkg.synth.q4k_weights(n, k, "gemmsr", "mm")
    xb = pkg.synth.to_bf16_bits(pkg.synth.normal_f32(m * k, "gemmsr", "mmx"))
    gpu.ensure_family("gemm_xl")
    assert gpu.launch_shape("gemm_mm_q4kl_bd_sk", k, n, m)[0][2] > 1
    yd = gpu.alloc(m * n)
    gpu.mm(gpu.upload_bytes(xb), gpu.lin(12, n, k, w), yd, m, x_dtype=pkg.X_BF16, act_mode=pkg.ACT_FLOAT)
    base = gpu.read(yd, m * n)
    monkeypatch.setenv("OJAS_HIP_GEMM_SR", "1")
    g2 = pkg.HipGpu(0)
    try:
        lin, xd = g2.lin(12, n, k, w), g2.upload_bytes(xb)
        runs = []
        for accum in (False, False, True):
            y2 = g2.upload(np.full(m * n, 3.0, np.float32))
            g2.mm(xd, lin, y2, m, accum, x_dtype=pkg.X_BF16, act_mode=pkg.ACT_FLOAT)
            runs.append(g2.read(y2, m * n))
        assert np.array_equal(runs[0], runs[1])
        assert peak_err(runs[0], base) <= 2e-6
        assert peak_err(runs[2] - 3.0, base) <= 1e-5
    finally:
        g2.close()


@pytest.mark.parametrize("m,k,n", [(140, 2048, 300), (128, 256, 256), (77, 512, 64), (260, 1024, 513)])
def test_tile_with_weights_dequantized_into_registers(gpu, orc, pkg, m, k, n):
    """`gemm_mm_q4kl_bd`, `gemm_mm_q4kl_bd256` and `gemm_mm_q4kl_bdk` by name: the 128 x 256 and 256 x 256 tiles whose waves
    dequantize their own 64 rows into the B operand, and the 128 x 64 tile whose waves share 64 rows and split K.  Ragged
    M and N, store and accumulate, sentinels behind row M; the oracle holds the tile's specified f16 weights."""
    gpu.ensure_family("gemm_xl")
    w = pkg.synth.q4k_weights(n, k, "bd", "w", n, k)
    x = pkg.synth.normal_f32(m * k, "bd", "x", m, k).reshape(m, k)
    xh, wd = gpu.upload_bytes(x.astype(np.float16)), gpu.upload_bytes(w)
    want = orc.matmul_ref(w, Q4_K, n, k, x, wmode=2, xmode=1)
    sent = np.full(n, 12345.5, np.float32)
    outs = {}
    for kernel, bm in (("gemm_mm_q4kl_bd", 128), ("gemm_mm_q4kl_bd256", 256), ("gemm_mm_q4kl_bdk", 128)):
        grid = [(n + 63) // 64 if kernel.endswith("bdk") else (n + 255) // 256, (m + bm - 1) // bm, 1]
        for accum in (0, 1):
            y0 = pkg.synth.normal_f32(m * n, "bd", "y0", accum).reshape(m, n)
            yd = gpu.upload(np.concatenate([y0.ravel(), sent]))
            gpu.dispatch(gpu.begin(), kernel, [(xh, 0), (wd, 0), (yd, 0)], [k, n, accum, m], grid, [256, 1, 1])
            got = gpu.read(yd, m * n + n)
            assert np.array_equal(got[m * n:], sent), "wrote past row M"
            got = got[:m * n].reshape(m, n)
            e = rms_errs(got, want + (y0 if accum else 0.0))
            assert e[0] < 1e-4 and e[1] < 2e-5, (kernel, accum, e)
            outs[kernel, accum] = got
    assert np.array_equal(outs["gemm_mm_q4kl_bd256", 0], outs["gemm_mm_q4kl_bd", 0])      # the same sums in the same order
    # 64-row tiles whose four waves split K: the same products, the K quarters added at the end
    assert peak_err(outs["gemm_mm_q4kl_bdk", 0], outs["gemm_mm_q4kl_bd", 0]) <= 2e-6


def test_q4l_entries_by_their_reference_names(gpu, orc, pkg):
    """`gemm_mm_q4l` (f32 x), `gemm_mm_q4l_hb` (f16 x) and `gemm_mm_q4l_sk` with the reference's argument lists
    (crates/ojas-cuda/src/kernels/gemm_q.rs:26-38: x, w4, y, qa, qb; K, N, accum, M | K, N, M, nsplit) on weights relaid
    by `relayout_q4k_q4l` — on the device here, checked bit for bit elsewhere.  Ragged M and N, accumulate, sentinels
    behind row M, and a one-hot read-back of the tile's bits."""
    gpu.ensure_family("gemm")
    gpu.ensure_family("dequant")
    for m, k, n in ((140, 2048, 300), (64, 256, 128), (300, 512, 72)):
        w = pkg.synth.q4k_weights(n, k, "q4l", "w", n, k)
        x = pkg.synth.normal_f32(m * k, "q4l", "x", m, k).reshape(m, k)
        raw = gpu.upload_bytes(w)
        nib, qa, qb = gpu.alloc_bytes(n * k // 2), gpu.alloc_bytes(n * k // 32 * 2), gpu.alloc_bytes(n * k // 32 * 2)
        gpu.relayout_q4k_q4l(raw, n, k, nib, qa, qb)
        xf, xh = gpu.upload(x), gpu.upload_bytes(x.astype(np.float16))
        want = orc.matmul_ref(w, Q4_K, n, k, x, wmode=2, xmode=1)
        grid = [(n + 127) // 128, (m + 255) // 256, 1]
        sent = np.full(n, 12345.5, np.float32)
        for kernel, xbuf in (("gemm_mm_q4l", xf), ("gemm_mm_q4l_hb", xh)):
            for accum in (0, 1):
                y0 = pkg.synth.normal_f32(m * n, "q4l", "y0", accum).reshape(m, n)
                yd = gpu.upload(np.concatenate([y0.ravel(), sent]))
                gpu.dispatch(gpu.begin(), kernel, [(xbuf, 0), (nib, 0), (yd, 0), (qa, 0), (qb, 0)], [k, n, accum, m], grid, [256, 1, 1])
                got = gpu.read(yd, m * n + n)
                assert np.all(got[m * n:] == 12345.5), "wrote past row M"
                e = rms_errs(got[:m * n].reshape(m, n), want + (y0 if accum else 0))
                assert e[0] < TIGHT[0] and e[1] < TIGHT[1], (kernel, accum, m, k, n, e)
        for nsplit in (1, 3):
            if k // 64 < nsplit:
                continue
            y0 = pkg.synth.normal_f32(m * n, "q4l", "y0sk", nsplit).reshape(m, n)
            yd = gpu.upload(y0)
            gpu.dispatch(gpu.begin(), "gemm_mm_q4l_sk", [(xh, 0), (nib, 0), (yd, 0), (qa, 0), (qb, 0)], [k, n, m, nsplit],
                         [grid[0], grid[1], nsplit], [256, 1, 1])
            e = rms_errs(gpu.read(yd, m * n).reshape(m, n), want + y0)
            assert e[0] < 1e-4 and e[1] < 2e-5, (nsplit, e)
    # the tile's bits: one-hot activations read every weight back
    k, n = 512, 160
    w = orc.synth_blocks(Q4_K, n * k // 256)
    raw = gpu.upload_bytes(w)
    nib, qa, qb = gpu.alloc_bytes(n * k // 2), gpu.alloc_bytes(n * k // 32 * 2), gpu.alloc_bytes(n * k // 32 * 2)
    gpu.relayout_q4k_q4l(raw, n, k, nib, qa, qb)
    yd = gpu.alloc(k * n)
    gpu.dispatch(gpu.begin(), "gemm_mm_q4l", [(gpu.upload(np.eye(k, dtype=np.float32)), 0), (nib, 0), (yd, 0), (qa, 0), (qb, 0)],
                 [k, n, 0, k], [(n + 127) // 128, (k + 255) // 256, 1], [256, 1, 1])
    want = orc.q4l_weights_f16(w, k, n).view(np.float16).astype(np.float32).reshape(n, k)
    assert np.array_equal(gpu.read(yd, k * n).reshape(k, n), want.T)
    with pytest.raises(pkg.OjasHipError, match="takes 5 buffers"):
        gpu.dispatch(gpu.begin(), "gemm_mm_q4l", [(xh, 0), (nib, 0), (yd, 0)], [k, n, 0, k], [2, 2, 1], [256, 1, 1])


def test_router_prefers_the_tile_only_above_the_crossover(gpu, orc, pkg):
    """ACT_AUTO: small M keeps the CPU-reference arithmetic (int8 activations); large M takes the
    f16 tile.  Both must sit within their own oracle's bound."""
    n, k = 256, 1024
    w = pkg.synth.q4k_weights(n, k, "xover", "w")
    lin = gpu.lin(Q4_K, n, k, w)
    for m in (4, 64):
        x = pkg.synth.normal_f32(m * k, "xover", "x", m).reshape(m, k)
        yd = gpu.alloc(m * n)
        gpu.mm(gpu.upload(x), lin, yd, m)
        got = gpu.read(yd, m * n).reshape(m, n)
        if m < 32:
            want = np.stack([orc.matvec_kq(w, Q4_K, n, k, x[t]) for t in range(m)])
            assert np.max(np.abs(got - want)) <= 2e-5 * np.max(np.abs(want))
        else:
            e = rms_errs(got, orc.matmul_ref(w, Q4_K, n, k, x, wmode=2, xmode=1))
            assert e[0] < TIGHT[0] and e[1] < TIGHT[1], e


@pytest.mark.parametrize("ty", ["iq4xs", "iq4nl", "q40", "q51", "q2k", "q3k", "mxfp4", "iq2xxs", "iq2s", "iq3s", "iq1m"])
@pytest.mark.parametrize("m,k,n,accum", [(40, 1024, 200, False), (300, 2048, 130, True)])
def test_formats_without_a_tile_are_decoded_into_scratch_for_a_batch(gpu, orc, pkg, ty, m, k, n, accum):
    """A batch on a format that has only matvecs: `ojh_mm` decodes the rows once (`dequant_<fmt>_f16`, dequant_to_f16's
    bits) into library scratch and runs the f16 tile — the contract of the Q6_K / Q8_0 tiles: activations rounded to
    f16, f32 accumulation, held to the tile's own bound against the rounded oracle and to the reference's bound against
    the unrounded one.  Below the crossover the per-token matvec still answers (f32 activations, the dequantized dot)."""
    S = pkg.synth
    types = {"iq4xs": S.IQ4_XS, "iq4nl": S.IQ4_NL, "q40": S.Q4_0, "q51": S.Q5_1, "q2k": S.Q2_K, "q3k": S.Q3_K, "mxfp4": pkg.MXFP4,
             "iq2xxs": S.IQ2_XXS, "iq2s": S.IQ2_S, "iq3s": S.IQ3_S, "iq1m": S.IQ1_M}
    t = types[ty]
    w = S.mxfp4_weights(n, k, "deq", ty) if ty == "mxfp4" else S.grid_weights(t, n, k, "deq", ty) if t in S.GRID_TYPES else S.weights(t, n, k, "deq", ty)
    x = S.normal_f32(m * k, "deq", "x", m, k).reshape(m, k)
    y0 = S.normal_f32(m * n, "deq", "y0").reshape(m, n) if accum else np.zeros((m, n), np.float32)
    yd = gpu.upload(np.concatenate([y0.ravel(), np.full(n, 12345.5, np.float32)]))
    lin = gpu.lin(t, n, k, w)
    gpu.mm(gpu.upload(x), lin, yd, m, accum)
    got = gpu.read(yd, m * n + n)
    assert np.all(got[m * n:] == 12345.5), "wrote past row M"
    got = got[:m * n].reshape(m, n)
    e16 = rms_errs(got, orc.matmul_ref(w, t, n, k, x, wmode=1, xmode=1) + y0)
    e32 = rms_errs(got, orc.matmul_ref(w, t, n, k, x) + y0)
    assert e16[0] < TIGHT[0] and e16[1] < TIGHT[1], e16
    assert e32[0] < 2e-2 and e32[1] < 3e-3, e32
    # four tokens: the matvec path, within its own (tighter) bound of the same oracle
    y4 = gpu.alloc(4 * n)
    gpu.mm(gpu.upload(x[:4].copy()), lin, y4, 4, act_mode=pkg.ACT_FLOAT)
    assert peak_err(gpu.read(y4, 4 * n).reshape(4, n), orc.matmul_ref(w, t, n, k, x[:4])) <= 1e-5
    lin.free()


@pytest.mark.parametrize("ty,m", [(Q6_K, 1024), (Q8_0, 2048)])
def test_long_batches_decode_the_rows_ahead_of_the_tile(gpu, orc, pkg, ty, m):
    """Q6_K rows from 1024 tokens (Q5_K / Q8_0 from 2048) of a matrix of 32 Mi weights: `ojh_mm` decodes them into
    scratch and runs the plain-f16 tile — the same weights (dequant_to_f16's bits) as the tile that dequantizes on the
    way into LDS, so the two agree to the last bits of an f32 sum; sampled rows against the oracle at the tile's bound."""
    n, k = 8192, 4096
    gen = {Q6_K: pkg.synth.q6k_weights, Q8_0: pkg.synth.q80_weights}[ty]
    w = gen(n, k, "big", ty)
    x = pkg.synth.normal_f32(m * k, "big", "x", m).reshape(m, k)
    outs = {}
    for big in ("1024", "0"):
        monkey = pytest.MonkeyPatch()
        monkey.setenv("OJAS_HIP_DEQ_BIG_M", big)
        g = pkg.HipGpu(0)
        try:
            yd = g.upload(np.full(m * n + n, 12345.5, np.float32))
            g.mm(g.upload(x), g.lin(ty, n, k, w), yd, m, act_mode=pkg.ACT_FLOAT)
            got = g.read(yd, m * n + n)
            assert np.all(got[m * n:] == 12345.5), "wrote past row M"
            outs[big] = got[:m * n].reshape(m, n)
            if big != "0":
                assert g.has_kernel("dequant_%s_f16" % {Q6_K: "q6k", Q8_0: "q80"}[ty]), "the rows were not decoded first"
        finally:
            g.close()
            monkey.undo()
    assert peak_err(outs["1024"], outs["0"]) <= 2e-6
    rows = np.r_[0:16, n // 2:n // 2 + 16, n - 16:n]
    rb = len(w) // n
    wr = np.concatenate([w[r * rb:(r + 1) * rb] for r in rows])
    toks = np.r_[0:8, m // 2:m // 2 + 8, m - 8:m]
    want = orc.matmul_ref(wr, ty, len(rows), k, x[toks], wmode=1, xmode=1)
    e = rms_errs(outs["1024"][np.ix_(toks, rows)], want)
    assert e[0] < TIGHT[0] and e[1] < TIGHT[1], e


@pytest.mark.parametrize("ty,tag", [(20, "iq4nl"), (23, "iq4xs"), (2, "q40"), (3, "q41"), (6, "q50"), (7, "q51"), (139, "mxfp4"), (10, "q2k"), (11, "q3k")])
def test_iq4_rows_on_the_tile_by_name(gpu, orc, pkg, ty, tag):
    """`gemm_mm_<fmt>{,_m128}` read IQ4_NL / IQ4_XS, Q4_0 / Q4_1 / Q5_0 / Q5_1, MXFP4, Q2_K and Q3_K rows through loaders of their own: one-hot activations read back
    `dequant_to_f16`'s bits of every weight, and a product equals, bit for bit, the plain-f16 tile on the decoded rows
    (`dequant_<fmt>_f16` + `gemm_mm_f16`: the same weights meet the same sums in the same order)."""
    k, n, m = 512, 200, 150
    bb, wpb = pkg.synth.BLOCK_SHAPE[ty]
    raw = pkg.synth.weights(ty, n, k, "iq4tile", tag)
    want = orc.dequant_to_f16(raw, ty, n * k).view(np.float16).astype(np.float32).reshape(n, k)
    gpu.ensure_family("gemm")
    gpu.ensure_family("dequant")
    wd = gpu.upload_bytes(raw)
    eye = gpu.upload_bytes(np.eye(k, dtype=np.float16).view(np.uint8))
    yd = gpu.upload(np.full(k * n + 64, 777.25, np.float32))
    gpu.dispatch(gpu.begin(), "gemm_mm_" + tag, [(eye, 0), (wd, 0), (yd, 0)], [k, n, 0, k], [(n + 127) // 128, (k + 255) // 256, 1], [256, 1, 1])
    got = gpu.read(yd, k * n + 64)
    assert np.all(got[k * n:] == np.float32(777.25))
    assert np.array_equal(got[:k * n].reshape(k, n), want.T)
    x = pkg.synth.normal_f32(m * k, "iq4tile", "x").astype(np.float16)
    xd = gpu.upload_bytes(x.view(np.uint8))
    w16 = gpu.alloc_bytes(n * k * 2)
    grid, block = gpu.launch_shape("dequant_%s_f16" % tag, 0, n * k // wpb, 0)
    gpu.dispatch(gpu.begin(), "dequant_%s_f16" % tag, [(wd, 0), (w16, 0)], [n * k // wpb], grid, block)
    outs = {}
    for kernel, src, bm in (("gemm_mm_" + tag, wd, 256), ("gemm_mm_f16", w16, 256), ("gemm_mm_%s_m128" % tag, wd, 128),
                            ("gemm_mm_f16_m128", w16, 128)):
        yk = gpu.alloc(m * n)
        gpu.dispatch(gpu.begin(), kernel, [(xd, 0), (src, 0), (yk, 0)], [k, n, 0, m], [(n + 127) // 128, (m + bm - 1) // bm, 1], [256, 1, 1])
        outs[kernel] = gpu.read(yk, m * n).view(np.uint32)
    assert np.array_equal(outs["gemm_mm_" + tag], outs["gemm_mm_f16"])
    assert np.array_equal(outs["gemm_mm_%s_m128" % tag], outs["gemm_mm_f16_m128"])
    ref = x.astype(np.float32).reshape(m, k).astype(np.float64) @ want.astype(np.float64).T
    assert peak_err(outs["gemm_mm_" + tag].view(np.float32).reshape(m, n), ref) <= 1e-5


@pytest.mark.parametrize("ty,tag", [(8, "q8_0"), (20, "iq4nl"), (23, "iq4xs"), (2, "q40"), (7, "q51"), (139, "mxfp4"), (10, "q2k"),
                                    (11, "q3k")])
@pytest.mark.parametrize("m,k,n,accum,threads", [(1, 256, 16, False, 256), (5, 384, 200, False, 256), (16, 512, 37, True, 512),
                                                 (17, 1024, 130, False, 256), (33, 2048, 64, False, 512), (64, 768, 48, True, 256)])
def test_few_token_kernel_by_name(gpu, orc, pkg, ty, tag, m, k, n, accum, threads):
    """`gemm_few_<fmt>{,_r4}_t{1,2,4}(xh, w, y, K, N, accum, M)`: 16 or 64 rows per workgroup, the K chunks dealt to its 4 or 8 waves,
    up to 16 / 32 / 64 tokens.  Every output against the f64 product of `dequant_to_f16`'s weights with the f16 activations;
    nothing written past row N or token M; more tokens than the entry holds are refused."""
    if ty in (23, 10, 11) and k % 256:
        pytest.skip("rows of this format are whole super-blocks of 256")
    raw = pkg.synth.weights(ty, n, k, "few", tag, n, k)
    wf = orc.dequant_to_f16(raw, ty, n * k).view(np.float16).astype(np.float64).reshape(n, k)
    x = pkg.synth.normal_f32(m * k, "few", "x", m, k).astype(np.float16)
    want = x.astype(np.float64).reshape(m, k) @ wf.T
    y0 = pkg.synth.normal_f32(m * n, "few", "y0", m, n) if accum else np.full(m * n, 777.25, np.float32)
    gpu.ensure_family("gemm")
    wd, xd = gpu.upload_bytes(raw), gpu.upload_bytes(x.view(np.uint8))
    tg = 1 if m <= 16 else 2 if m <= 32 else 4
    for t, rg in ((tg, 1), (4, 1), (tg, 4), (4, 4)):
        yd = gpu.upload(np.concatenate([y0, np.full(n, 4242.5, np.float32)]))
        gpu.dispatch(gpu.begin(), "gemm_few_%s%s_t%d" % (tag, "_r4" if rg == 4 else "", t), [(xd, 0), (wd, 0), (yd, 0)], [k, n, int(accum), m],
                     [(n + 16 * rg - 1) // (16 * rg), 1, 1], [threads if rg * t <= 4 else 256, 1, 1])
        got = gpu.read(yd, m * n + n)
        assert np.all(got[m * n:] == np.float32(4242.5)), "wrote past the last token"
        got = got[:m * n].reshape(m, n) - (y0.reshape(m, n) if accum else 0.0)
        assert peak_err(got, want) <= (2e-5 if accum else 2e-6), (t, rg)
    if tg < 4:
        with pytest.raises(pkg.OjasHipError, match="tokens"):
            gpu.dispatch(gpu.begin(), "gemm_few_%s_t%d" % (tag, tg), [(xd, 0), (wd, 0), (yd, 0)], [k, n, 0, 16 * tg + 1], [(n + 15) // 16, 1, 1],
                         [256, 1, 1])
