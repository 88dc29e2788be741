"""The benchmark configurations at their full sizes.

The threaded C oracle walks a whole 128256 x 4096 head in well under a second, so the matvecs are
compared with it in full; the prefill GEMM (30 G multiply-adds per call at M = 512) is compared on
sampled weight rows against every token, and through properties that hold at any size: exact
doubling of a matvec under x -> 2x (a power of two passes through the quantizer and every f32
product and sum unchanged), a row block of the big launch equal to the same rows launched alone,
a token's outputs independent of its position in the batch.
"""
import numpy as np
import pytest

from conftest import peak_err, rms_errs

pytestmark = pytest.mark.gpu
Q8_0, Q4_K, Q5_K, Q6_K = 8, 12, 13, 14


def _rows(raw, ty, pkg, k, rows):
    rb = pkg.row_bytes(ty, k)
    return np.concatenate([raw[r * rb:(r + 1) * rb] for r in rows])


def test_q4k_decode_projection_set_at_full_size(gpu, orc, pkg):
    """Llama-3-8B shapes, batch 1, the CPU reference's arithmetic: every output of every projection."""
    for name, n, k in [("q", 4096, 4096), ("k", 1024, 4096), ("gate", 14336, 4096), ("down", 4096, 14336),
                       ("head", 128256, 4096)]:
        w = pkg.synth.q4k_weights(n, k, "full", name)
        x = pkg.synth.normal_f32(k, "full", name, "x")
        lin = gpu.lin(Q4_K, n, k, w)
        yd, y2 = gpu.alloc(n), gpu.alloc(n)
        gpu.mm(gpu.upload(x), lin, yd, 1, act_mode=pkg.ACT_Q8K)
        got = gpu.read(yd, n)
        want = orc.matvec_kq(w, Q4_K, n, k, x)
        assert peak_err(got, want) <= 2e-5, name
        # x -> 2x: the quantizer's scale doubles, its codes do not move, every f32 product doubles
        gpu.mm(gpu.upload(2.0 * x), lin, y2, 1, act_mode=pkg.ACT_Q8K)
        assert np.array_equal(gpu.read(y2, n), 2.0 * got), name
        # a block of rows launched alone (another row-count variant of the kernel): same bits
        lo, cnt = n // 3, min(1000, n // 2)
        rb = pkg.row_bytes(Q4_K, k)
        sub = gpu.lin(Q4_K, cnt, k, w[lo * rb:(lo + cnt) * rb])
        ys = gpu.alloc(cnt)
        gpu.mm(gpu.upload(x), sub, ys, 1, act_mode=pkg.ACT_Q8K)
        assert np.array_equal(gpu.read(ys, cnt), got[lo:lo + cnt]), name
        del lin, sub


def test_q80_matvec_at_full_size_doubles_exactly(gpu, orc, pkg):
    n = k = 4096
    w = pkg.synth.q80_weights(n, k, "full", "q80")
    x = pkg.synth.normal_f32(k, "full", "q80", "x")
    lin = gpu.lin(Q8_0, n, k, w)
    y1, y2 = gpu.alloc(n), gpu.alloc(n)
    gpu.mm(gpu.upload(x), lin, y1, 1)
    gpu.mm(gpu.upload(2.0 * x), lin, y2, 1)
    got = gpu.read(y1, n)
    assert peak_err(got, orc.matvec_kq(w, Q8_0, n, k, x)) <= 1e-5
    assert np.array_equal(gpu.read(y2, n), 2.0 * got)


@pytest.mark.parametrize("m", [1, 2, 4, 8, 16])
def test_q6k_verify_head_at_full_size(gpu, orc, pkg, m):
    """Q6_K 151936 x 4096 output head, bf16 activations, 1 to 16 tokens: every logit of every token."""
    n, k = 151936, 4096
    w = pkg.synth.q6k_weights(n, k, "full", "q6k-head")
    xb = pkg.synth.to_bf16_bits(pkg.synth.normal_f32(m * k, "full", "q6k-x", m))
    xf = pkg.synth.bf16_bits_to_f32(xb).reshape(m, k)
    lin = gpu.lin(Q6_K, n, k, w)
    yd = gpu.upload(np.full(m * n + 64, 12345.5, np.float32))
    gpu.mm(gpu.upload_bytes(xb), lin, yd, m, x_dtype=pkg.X_BF16, act_mode=pkg.ACT_Q8K)
    got = gpu.read(yd, m * n + 64)
    assert np.all(got[m * n:] == 12345.5), "wrote past the last token"
    got = got[:m * n].reshape(m, n)
    for t in range(m):
        assert peak_err(got[t], orc.matvec_kq(w, Q6_K, n, k, xf[t])) <= 2e-5, t
    if m > 1:
        # a token's logits do not depend on the batch: the last token alone (the one-token kernel) agrees
        # to the last ulps (the few-token kernel folds the -32 offset into signed codes)
        y1 = gpu.alloc(n)
        gpu.mm(gpu.upload_bytes(xb.reshape(m, k)[m - 1].copy()), lin, y1, 1, x_dtype=pkg.X_BF16, act_mode=pkg.ACT_Q8K)
        assert peak_err(gpu.read(y1, n), got[m - 1]) <= 2e-6


@pytest.mark.parametrize("n,k", [(14336, 4096), (4096, 14336)])
@pytest.mark.parametrize("m", [128, 512, 2048])
def test_prefill_in_the_cpu_arithmetic_at_full_size(gpu, orc, pkg, n, k, m):
    """The same shapes under OJH_ACT_Q8K — activations quantized per 256, integer dots on the int8 matrix cores —
    against `matvec_kq`, the CPU reference itself, token by token on sampled weight rows (tile borders included):
    the prefill path that meets the parity bar of the CPU reference.  A token's outputs do not depend on its
    position in the batch (bit for bit)."""
    w = pkg.synth.q4k_weights(n, k, "full", "gemm", n, k)
    xb = pkg.synth.to_bf16_bits(pkg.synth.normal_f32(m * k, "full", "q8k-x", m, k))
    xf = pkg.synth.bf16_bits_to_f32(xb).reshape(m, k)
    lin = gpu.lin(Q4_K, n, k, w)
    yd = gpu.upload(np.full(m * n + 64, 12345.5, np.float32))
    gpu.mm(gpu.upload_bytes(xb), lin, yd, m, x_dtype=pkg.X_BF16, act_mode=pkg.ACT_Q8K)
    got = gpu.read(yd, m * n + 64)
    assert np.all(got[m * n:] == 12345.5), "wrote past row M"
    got = got[:m * n].reshape(m, n)
    g = pkg.synth.rng("full", "q8k-rows", n, k, m)
    rows = np.unique(np.concatenate([[0, 15, 16, 63, 64, n - 17, n - 1], g.integers(0, n, 25)]))
    wsub = _rows(w, Q4_K, pkg, k, rows)
    # every token up to 512; of 2048 (sixteen token tiles in grid.y) the borders of every 128-token tile and every 11th
    tokens = range(m) if m <= 512 else np.unique(np.concatenate([np.arange(0, m, 128), np.arange(127, m, 128), np.arange(0, m, 11)]))
    for t in tokens:
        want = orc.matvec_kq(wsub, Q4_K, len(rows), k, xf[t], threads=1 if len(rows) < 64 else 8)
        assert peak_err(got[t, rows], want) <= 2e-5, t
    perm = np.roll(np.arange(m), 37)
    y2 = gpu.alloc(m * n)
    gpu.mm(gpu.upload_bytes(xb.reshape(m, k)[perm].copy()), lin, y2, m, x_dtype=pkg.X_BF16, act_mode=pkg.ACT_Q8K)
    assert np.array_equal(gpu.read(y2, m * n).reshape(m, n), got[perm])


@pytest.mark.parametrize("ty", [Q6_K, Q5_K])
@pytest.mark.parametrize("n,k", [(14336, 4096), (4096, 14336)])
@pytest.mark.parametrize("m", [64, 512])
def test_q6k_q5k_prefill_in_the_cpu_arithmetic_at_full_size(gpu, orc, pkg, ty, n, k, m):
    """Q6_K and Q5_K rows under OJH_ACT_Q8K at the sizes the benchmark times (`gemm_q8k_{q6k,q5k}_gs`, whole and over K
    slices as the library picks them): sampled weight rows (tile borders included) against `matvec_kq`, every token up
    to 64, every seventh of 512 and the borders of the 128-token tiles; a token's outputs do not depend on its
    position in the batch (bit for bit)."""
    gen = {Q6_K: pkg.synth.q6k_weights, Q5_K: pkg.synth.q5k_weights}[ty]
    w = gen(n, k, "full", "gs", n, k)
    xf = pkg.synth.normal_f32(m * k, "full", "gs-x", m, k).reshape(m, k)
    lin = gpu.lin(ty, n, k, w)
    yd = gpu.upload(np.full(m * n + 64, 12345.5, np.float32))
    gpu.mm(gpu.upload(xf), lin, yd, m, act_mode=pkg.ACT_Q8K)
    got = gpu.read(yd, m * n + 64)
    assert np.all(got[m * n:] == 12345.5), "wrote past row M"
    got = got[:m * n].reshape(m, n)
    g = pkg.synth.rng("full", "gs-rows", n, k, m)
    rows = np.unique(np.concatenate([[0, 31, 32, 63, 64, n - 33, n - 1], g.integers(0, n, 25)]))
    wsub = _rows(w, ty, pkg, k, rows)
    tokens = range(m) if m <= 64 else np.unique(np.concatenate([np.arange(0, m, 128), np.arange(127, m, 128), np.arange(0, m, 7)]))
    for t in tokens:
        want = orc.matvec_kq(wsub, ty, len(rows), k, xf[t], threads=1)
        assert peak_err(got[t, rows], want) <= 2e-5, t
    perm = np.roll(np.arange(m), 37)
    y2 = gpu.alloc(m * n)
    gpu.mm(gpu.upload(xf[perm].copy()), lin, y2, m, act_mode=pkg.ACT_Q8K)
    assert np.array_equal(gpu.read(y2, m * n).reshape(m, n), got[perm])
    lin.free()


@pytest.mark.parametrize("n,k", [(14336, 4096), (4096, 14336)])
@pytest.mark.parametrize("m", [512, 2048])
def test_prefill_gemm_at_full_size(gpu, orc, pkg, n, k, m):
    """Q4_K gate/up and down shapes, bf16 activations: 48 sampled weight rows against every token
    (the oracle holds the tile's specified f16 weights), the batch rolled by 37 positions, and the
    first 128 tokens launched alone against their rows in the big launch."""
    w = pkg.synth.q4k_weights(n, k, "full", "gemm", n, k)
    xb = pkg.synth.to_bf16_bits(pkg.synth.normal_f32(m * k, "full", "gemm-x", m, k))
    xf = pkg.synth.bf16_bits_to_f32(xb).reshape(m, k)
    lin = gpu.lin(Q4_K, n, k, w)
    yd = gpu.upload(np.full(m * n + 64, 12345.5, np.float32))
    xd = gpu.upload_bytes(xb)
    gpu.mm(xd, lin, yd, m, x_dtype=pkg.X_BF16, act_mode=pkg.ACT_FLOAT)
    got = gpu.read(yd, m * n + 64)
    assert np.all(got[m * n:] == 12345.5), "wrote past row M"
    got = got[:m * n].reshape(m, n)
    assert np.all(np.isfinite(got))
    g = pkg.synth.rng("full", "gemm-rows", n, k, m)
    rows = np.unique(np.concatenate([[0, 255, 256, n - 1], g.integers(0, n, 44)]))
    wsub = _rows(w, Q4_K, pkg, k, rows)
    want = orc.matmul_ref(wsub, Q4_K, len(rows), k, xf, wmode=2, xmode=1)
    e = rms_errs(got[:, rows], want)
    assert e[0] < 5e-4 and e[1] < 5e-5, e
    # the same tokens in other positions of the batch: the same bits, moved
    perm = np.roll(np.arange(m), 37)
    y2 = gpu.alloc(m * n)
    gpu.mm(gpu.upload_bytes(xb.reshape(m, k)[perm].copy()), lin, y2, m, x_dtype=pkg.X_BF16, act_mode=pkg.ACT_FLOAT)
    got2 = gpu.read(y2, m * n).reshape(m, n)
    e = rms_errs(got2, got[perm])
    assert e[0] < 2e-6, e          # three or more K slices meet in f32 atomics, in no fixed order
    gpu.ensure_family("gemm_xl")
    tall = gpu.launch_shape("gemm_mm_q4kl_sk", k, n, m)[0][2]
    half = gpu.launch_shape("gemm_mm_q4kl_bd_sk", k, n, m)[0][2]
    if max(tall, half) <= 2:       # one or two slices: a + b = b + a, so bit for bit
        assert np.array_equal(got2, got[perm])
    # the first 128 tokens alone: another tile height and K split, so sums associate differently
    y3 = gpu.alloc(128 * n)
    gpu.mm(gpu.upload_bytes(xb[:128 * k].copy()), lin, y3, 128, x_dtype=pkg.X_BF16, act_mode=pkg.ACT_FLOAT)
    got3 = gpu.read(y3, 128 * n).reshape(128, n)
    e = rms_errs(got3, got[:128])
    assert e[0] < 5e-5 and e[1] < 5e-6, e
    # ... and against the oracle itself, like the big launch
    e = rms_errs(got3[:, rows], want[:128])
    assert e[0] < 5e-4 and e[1] < 5e-5, e
