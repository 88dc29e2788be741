"""Family "gemv_q8": the reference GPU decoder's row-int8 matvecs by their own names and argument order
(crates/ojas-cuda/src/kernels/gemv_q8.rs:48-152, gemv.rs:57-74), on the shapes and generators of the reference's
conformance tests (crates/ojas-cuda/tests/conformance.rs:248-355) and on decode sizes.  The reference bounds them at
1e-4 .. 1e-3 relative per element; here 2e-6 of the peak against the f64-summed oracle (the per-element figure of the
reference is checked too)."""
import numpy as np
import pytest

from conftest import peak_err

pytestmark = pytest.mark.gpu


def max_rel_err(got, want):
    """crates/ojas-cuda/tests/conformance.rs:215-220"""
    return float(np.max(np.abs(got - want) / np.maximum(np.abs(want), 1e-6)))


def _shape(gpu, name, k, n, m=1):
    g, b = gpu.launch_shape(name, k, n, m)
    return list(g), list(b)


def _fam(gpu):
    gpu.ensure_family("gemv_q8")
    for name in ("gemv_q8", "gemv_q8_accum", "gemv_q8_bias", "gemv_q8_ksplit", "ffn_gu_q8", "qkv_q8", "embed_q8", "quantize_q8_pertoken"):
        assert gpu.has_kernel(name), name


@pytest.mark.parametrize("k,n,seed", [(512, 256, 11), (4864, 96, 21), (100, 7, 5), (4096, 4099, 3), (20480, 33, 9)])
def test_gemv_q8_plain_accum_bias_ksplit(gpu, orc, pkg, k, n, seed):
    """(512, 256, 11) and (4864, 96, 21) are the reference's own cases; K = 100 walks rows that are only 4-byte
    aligned; N = 4099 leaves an odd last row; K = 20480 is longer than the activations a workgroup stages."""
    _fam(gpu)
    x = pkg.synth.tvec(k, seed)
    w, scale = pkg.synth.q8_rows(n, k, seed + 1)
    want = orc.gemv_q8_rows(w, scale, x)
    xd, wd, sd = gpu.upload(x), gpu.upload_bytes(w.view(np.uint8)), gpu.upload(scale)
    grid, block = _shape(gpu, "gemv_q8", k, n)
    y0 = pkg.synth.normal_f32(n, "gq8", "y0", k, n)
    bias = pkg.synth.normal_f32(n, "gq8", "bias", k, n)
    yd = gpu.upload(np.concatenate([y0, [4242.5]]).astype(np.float32))
    gpu.dispatch(gpu.begin(), "gemv_q8", [(xd, 0), (wd, 0), (yd, 0), (sd, 0)], [k, n], grid, block)
    got = gpu.read(yd, n + 1)
    assert got[n] == 4242.5
    assert peak_err(got[:n], want) <= 2e-6 and max_rel_err(got[:n], want) < 1e-4 * max(1.0, k / 512)
    plain = got[:n].copy()
    # the reference's launch of it: eight rows per 256-thread block
    gpu.dispatch(gpu.begin(), "gemv_q8", [(xd, 0), (wd, 0), (yd, 0), (sd, 0)], [k, n], [(n + 7) // 8, 1, 1], [256, 1, 1])
    assert np.array_equal(gpu.read(yd, n), plain)
    ya = gpu.upload(y0)
    gpu.dispatch(gpu.begin(), "gemv_q8_accum", [(xd, 0), (wd, 0), (ya, 0), (sd, 0)], [k, n], grid, block)
    assert np.array_equal(gpu.read(ya, n), y0 + plain)
    yb = gpu.alloc(n)
    gpu.dispatch(gpu.begin(), "gemv_q8_bias", [(xd, 0), (wd, 0), (yb, 0), (sd, 0), (gpu.upload(bias), 0)], [k, n], grid, block)
    assert np.array_equal(gpu.read(yb, n), plain + bias)
    yk = gpu.upload(np.concatenate([y0, [4242.5]]).astype(np.float32))
    for threads in (256, _shape(gpu, "gemv_q8_ksplit", k, n)[1][0], 1024):
        gpu.dispatch(gpu.begin(), "gemv_q8_ksplit", [(xd, 0), (wd, 0), (yk, 0), (sd, 0)], [k, n], [n, 1, 1], [threads, 1, 1])
        got = gpu.read(yk, n + 1)
        assert got[n] == 4242.5 and peak_err(got[:n], want) <= 2e-6 and max_rel_err(got[:n], want) < 1e-3
    with pytest.raises(pkg.OjasHipError, match="multiple of 4"):
        gpu.dispatch(gpu.begin(), "gemv_q8", [(xd, 0), (wd, 0), (yd, 0), (sd, 0)], [k - 1, n], grid, block)
    with pytest.raises(pkg.OjasHipError):
        gpu.dispatch(gpu.begin(), "gemv_q8", [(xd, 0), (wd, 0), (yd, 0), (sd, 0)], [k, n + 2], grid, block)   # past w, y, scale


@pytest.mark.parametrize("k,n,act", [(512, 128, 0), (512, 128, 1), (4096, 1001, 0), (36, 5, 1)])
def test_ffn_gu_q8(gpu, orc, pkg, k, n, act):
    """(512, 128, SiLU) with seeds 31 / 32 / 33 is the reference's case (conformance.rs:312-336)."""
    _fam(gpu)
    x = pkg.synth.tvec(k, 31)
    (wg, sg), (wu, su) = pkg.synth.q8_rows(n, k, 32), pkg.synth.q8_rows(n, k, 33)
    if act == 1:
        sg = sg * np.float32(40.0)                      # gate values up to a few tens: GELU's clamp is reached
    g, u = orc.gemv_q8_rows(wg, sg, x).astype(np.float64), orc.gemv_q8_rows(wu, su, x).astype(np.float64)
    if act == 0:
        want = g / (1.0 + np.exp(-g)) * u
    else:
        inner = np.clip(0.7978845608 * (g + 0.044715 * g ** 3), -30.0, 30.0)
        want = 0.5 * g * (1.0 + np.tanh(inner)) * u
    od = gpu.upload(np.full(n + 1, 4242.5, np.float32))
    grid, block = _shape(gpu, "ffn_gu_q8", k, n)
    gpu.dispatch(gpu.begin(), "ffn_gu_q8", [(gpu.upload(x), 0), (gpu.upload_bytes(wg.view(np.uint8)), 0), (gpu.upload_bytes(wu.view(np.uint8)), 0),
                                            (od, 0), (gpu.upload(sg), 0), (gpu.upload(su), 0)], [k, n, act], grid, block)
    got = gpu.read(od, n + 1)
    assert got[n] == 4242.5
    assert peak_err(got[:n], want.astype(np.float32)) <= 5e-6 and max_rel_err(got[:n], want.astype(np.float32)) < 1e-3


@pytest.mark.parametrize("k,nq,nkv,with_bias", [(512, 64, 16, True), (512, 64, 16, False), (4096, 4096, 1024, False), (100, 5, 3, True)])
def test_qkv_q8(gpu, orc, pkg, k, nq, nkv, with_bias):
    _fam(gpu)
    x = pkg.synth.tvec(k, 41)
    ws = [pkg.synth.q8_rows(n, k, 42 + i) for i, n in enumerate((nq, nkv, nkv))]
    bs = [pkg.synth.normal_f32(n, "gq8", "qkvb", i) if with_bias else None for i, n in enumerate((nq, nkv, nkv))]
    ys = [gpu.upload(np.full(n + 1, 4242.5, np.float32)) for n in (nq, nkv, nkv)]
    bufs = [(gpu.upload(x), 0)] + [(gpu.upload_bytes(w.view(np.uint8)), 0) for w, _ in ws] + [(y, 0) for y in ys] + \
           [(gpu.upload(s), 0) for _, s in ws] + [((gpu.upload(b) if b is not None else None), 0) for b in bs]
    grid, block = _shape(gpu, "qkv_q8", k, nq + 2 * nkv)
    gpu.dispatch(gpu.begin(), "qkv_q8", bufs, [k, nq, nkv], grid, block)
    for (w, s), b, y, n in zip(ws, bs, ys, (nq, nkv, nkv)):
        got = gpu.read(y, n + 1)
        want = orc.gemv_q8_rows(w, s, x) + (b if b is not None else 0.0)
        assert got[n] == 4242.5 and peak_err(got[:n], want) <= 2e-6
    # each projection alone gives the same bits
    y1 = gpu.alloc(nkv)
    gpu.dispatch(gpu.begin(), "gemv_q8", [bufs[0], bufs[3], (y1, 0), bufs[9]], [k, nkv], *_shape(gpu, "gemv_q8", k, nkv))
    if not with_bias:
        assert np.array_equal(gpu.read(y1, nkv), gpu.read(ys[2], nkv))


def test_embed_q8(gpu, pkg):
    """conformance.rs:338-355: vocab 64, D 256, token 37, seed 41."""
    _fam(gpu)
    vocab, d, token = 64, 256, 37
    table, scale = pkg.synth.q8_rows(vocab, d, 41)
    od = gpu.upload(np.full(d + 1, 4242.5, np.float32))
    gpu.dispatch(gpu.begin(), "embed_q8", [(gpu.upload_bytes(table.view(np.uint8)), 0), (gpu.upload(scale), 0), (od, 0)], [token, d], [4, 1, 1], [128, 1, 1])
    got = gpu.read(od, d + 1)
    assert got[d] == 4242.5 and np.array_equal(got[:d], table[token].astype(np.float32) * scale[token])
    with pytest.raises(pkg.OjasHipError):
        gpu.dispatch(gpu.begin(), "embed_q8", [(gpu.upload_bytes(table.view(np.uint8)), 0), (gpu.upload(scale), 0), (od, 0)], [vocab, d], [4, 1, 1], [128, 1, 1])


@pytest.mark.parametrize("m,k", [(1, 4096), (5, 640), (33, 14336)])
def test_quantize_q8_pertoken_bit_exact(gpu, orc, pkg, m, k):
    _fam(gpu)
    x = pkg.synth.normal_f32(m * k, "gq8", "pertoken", m, k).reshape(m, k)
    x[m // 2] = 0.0
    x[0, :4] = np.float32(np.abs(x[0]).max()) * np.float32([0.5, 1.5, -2.5, 3.5]) / np.float32(127.0)
    q, d = orc.quantize_q8_pertoken(x)
    qd, dd = gpu.alloc_bytes(m * k + 16), gpu.alloc(m + 1)
    gpu.memset0(qd)
    grid, block = _shape(gpu, "quantize_q8_pertoken", k, 1, m)
    assert grid[0] == m
    gpu.dispatch(gpu.begin(), "quantize_q8_pertoken", [(gpu.upload(x), 0), (qd, 0), (dd, 0)], [k], grid, block)
    assert np.array_equal(gpu.read(qd, m * k, np.int8).reshape(m, k), q)
    assert np.array_equal(gpu.read(dd, m).view(np.uint32), d.view(np.uint32))
    assert not gpu.read(qd, m * k + 16, np.int8)[m * k:].any()
