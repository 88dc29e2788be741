"""Decode-step matvecs on the GPU against the CPU oracle.

Two contracts, each against its own oracle:
  * int8-activation kernels (gemv_q8k_*)  vs  matvec_kq, the CPU reference's arithmetic
    (crates/ojas-cpu/src/cpu_math.rs:1145-1189): max|d| / max|ref| <= 1e-3 required, ~1e-6 seen;
  * f32-activation kernels (gemv_nat_*)   vs  dequant-in-double dot, the reference's GPU-test
    oracle (crates/ojas-cuda/tests/conformance.rs:798-823): its bound 2e-3, ours 1e-4.
"""
import numpy as np
import pytest

from conftest import peak_err

pytestmark = pytest.mark.gpu
Q8_0, Q4_K, Q5_K, Q6_K, IQ4_NL, IQ4_XS = 8, 12, 13, 14, 20, 23
Q4_0, Q4_1, Q5_0, Q5_1 = 2, 3, 6, 7
Q2_K, Q3_K = 10, 11
TAG = {Q8_0: "q80", Q4_K: "q4k", Q5_K: "q5k", Q6_K: "q6k"}
TOL_Q8K = 1e-3     # the parity bar against the CPU reference
TOL_Q8K_SEEN = 2e-5
TOL_FLOAT = 1e-4   # reference bound is 2e-3


def _inputs(pkg, ty, n, k, tag):
    return pkg.synth.weights(ty, n, k, "gemv", tag, ty, n, k), pkg.synth.normal_f32(k, "gemv", tag, "x", k)


def test_quantize_q8k_is_bit_exact(gpu, orc, pkg):
    for k, m in [(4096, 1), (14336, 3), (300, 2), (256, 1)]:
        x = pkg.synth.normal_f32(m * k, "q8k", k, m).reshape(m, k)
        x[0, :7] = [0.5, -0.5, 1.5, -2.5, 0.0, 1e-30, -1e-30]
        if k >= 512:
            x[-1, 256:512] = 0.0
        if k >= 4096:     # non-finite inputs: NaN -> code 0 and outside the maximum; an infinity zeroes its segment's codes
            x[0, 1000], x[0, 2000], x[0, 2001] = np.nan, np.inf, -np.inf
        nsb = (k + 255) // 256
        xd = gpu.upload(x)
        q, s = gpu.alloc_bytes(m * nsb * 256), gpu.alloc(m * nsb)
        gpu.quant_q8k(xd, m, k, q, s)
        gq = gpu.read(q, m * nsb * 256, np.int8).reshape(m, -1)
        gs = gpu.read(s, m * nsb).reshape(m, -1)
        for t in range(m):
            ws, wq, _ = orc.quant_q8k(x[t])
            assert np.array_equal(gs[t], ws), (k, t)
            assert np.array_equal(gq[t], wq), (k, t)


@pytest.mark.parametrize("k,m,off,dt", [(768, 400, 0, "f32"), (300, 700, 0, "f32"), (4096, 70, 1, "f32"), (1024, 300, 0, "bf16"),
                                        (300, 600, 1, "bf16")])
def test_quantize_q8k_batches_a_segment_per_wave(gpu, orc, pkg, k, m, off, dt):
    """From 1024 segments `ojh_quant_q8k` launches `quantize_q8k{,_bf16}_w` (a segment per wave): sampled tokens bit for
    bit, a ragged last segment zero-padded, an input that starts off the vector alignment, nothing past the outputs; and
    by name the same bits as the workgroup-per-segment entry."""
    nsb = (k + 255) // 256
    assert nsb * m >= 1024
    x = pkg.synth.normal_f32(m * k + off, "q8kw", k, m)
    if dt == "bf16":
        bits = pkg.synth.to_bf16_bits(x)
        xd, esz, xf = gpu.upload_bytes(bits), 2, pkg.synth.bf16_bits_to_f32(bits)
    else:
        xd, esz, xf = gpu.upload(x), 4, x
    xf = xf[off:].reshape(m, k)
    q, s = gpu.alloc_bytes(m * nsb * 256 + 16), gpu.alloc(m * nsb + 1)
    gpu.memset0(q)
    gpu.quant_q8k(xd, m, k, q, s, x_dtype=pkg.X_BF16 if dt == "bf16" else pkg.X_F32, x_off=off * esz)
    gq = gpu.read(q, m * nsb * 256 + 16, np.int8)
    assert not gq[m * nsb * 256:].any()
    gq, gs = gq[:m * nsb * 256].reshape(m, -1), gpu.read(s, m * nsb).reshape(m, -1)
    for t in sorted({0, 1, m // 2, m - 1}):
        ws, wq, _ = orc.quant_q8k(xf[t])
        assert np.array_equal(gs[t], ws) and np.array_equal(gq[t], wq), t
    gpu.ensure_family("gemv_q8k")
    name = "quantize_q8k_bf16" if dt == "bf16" else "quantize_q8k"
    q2, s2 = gpu.alloc_bytes(m * nsb * 256), gpu.alloc(m * nsb)
    gpu.dispatch(gpu.begin(), name, [(xd, off * esz), (q2, 0), (s2, 0)], [k, m], [nsb, m, 1], [256, 1, 1])
    assert np.array_equal(gpu.read(q2, m * nsb * 256, np.int8).reshape(m, -1), gq)
    assert np.array_equal(gpu.read(s2, m * nsb).view(np.uint32).reshape(m, -1), gs.view(np.uint32))
    with pytest.raises(pkg.OjasHipError, match="grid must be"):
        gpu.dispatch(gpu.begin(), name + "_w", [(xd, off * esz), (q2, 0), (s2, 0)], [k, m], [nsb, m, 1], [256, 1, 1])


def test_quantize_q8k_bf16_input(gpu, orc, pkg):
    k, m = 4096, 2
    xb = pkg.synth.to_bf16_bits(pkg.synth.normal_f32(m * k, "q8kb"))
    xd = gpu.upload_bytes(xb)
    q, s = gpu.alloc_bytes(m * 16 * 256), gpu.alloc(m * 16)
    gpu.quant_q8k(xd, m, k, q, s, x_dtype=pkg.X_BF16)
    xf = pkg.synth.bf16_bits_to_f32(xb).reshape(m, k)
    gq = gpu.read(q, m * k, np.int8).reshape(m, k)
    for t in range(m):
        ws, wq, _ = orc.quant_q8k(xf[t])
        assert np.array_equal(gq[t], wq)


@pytest.mark.parametrize("ty", [Q4_K, Q5_K, Q6_K])
@pytest.mark.parametrize("n,k", [(13, 256), (64, 512), (1024, 4096), (333, 2560), (96, 14336), (4099, 4096)])
def test_q8k_matvec_matches_cpu_reference(gpu, orc, pkg, ty, n, k):
    w, x = _inputs(pkg, ty, n, k, "a")
    lin = gpu.lin(ty, n, k, w)
    xd, yd = gpu.upload(x), gpu.upload(np.full(n + 2, 12345.0, np.float32))
    gpu.mm(xd, lin, yd, 1, False, act_mode=pkg.ACT_Q8K, y_off=4)
    got = gpu.read(yd, n + 2)
    assert got[0] == 12345.0 and got[-1] == 12345.0, "wrote outside y"
    want = orc.matvec_kq(w, ty, n, k, x)
    err = peak_err(got[1:-1], want)
    assert err <= TOL_Q8K_SEEN <= TOL_Q8K, err


@pytest.mark.parametrize("ty", [Q8_0, Q4_K, Q5_K, Q6_K, IQ4_NL, IQ4_XS, Q4_0, Q4_1, Q5_0, Q5_1, Q2_K, Q3_K])
@pytest.mark.parametrize("n,k", [(13, 2560), (1024, 4096), (96, 14336), (4099, 4096), (33001, 2816)])
def test_float_matvec_matches_dequant_dot(gpu, orc, pkg, ty, n, k):
    w, x = _inputs(pkg, ty, n, k, "b")
    lin = gpu.lin(ty, n, k, w)
    xd, yd = gpu.upload(x), gpu.upload(np.full(n + 2, 12345.0, np.float32))
    gpu.mm(xd, lin, yd, 1, False, act_mode=pkg.ACT_FLOAT, y_off=4)
    got = gpu.read(yd, n + 2)
    assert got[0] == 12345.0 and got[-1] == 12345.0
    want = orc.matmul_ref(w, ty, n, k, x)[0]
    assert peak_err(got[1:-1], want) <= TOL_FLOAT
    # the reference's own oracle rounds each weight to f16 first; its bound is 2e-3
    want16 = orc.matmul_ref(w, ty, n, k, x, wmode=1)[0]
    assert peak_err(got[1:-1], want16) <= 2e-3


def test_q80_matvec_matches_dot_q80(gpu, orc, pkg):
    """Config 0: Q8_0 4096x4096 against the CPU path `dot_q80` (f32 activations)."""
    n = k = 4096
    w, x = _inputs(pkg, Q8_0, n, k, "c0")
    lin = gpu.lin(Q8_0, n, k, w)
    xd, yd = gpu.upload(x), gpu.alloc(n)
    gpu.mm(xd, lin, yd, 1)
    want = orc.matvec_kq(w, Q8_0, n, k, x)
    assert peak_err(gpu.read(yd, n), want) <= 1e-5


@pytest.mark.parametrize("ty,tag", [(Q4_K, "q4k"), (Q6_K, "q6k"), (Q2_K, "q2k"), (Q3_K, "q3k"), (Q5_K, "q5k")])
@pytest.mark.parametrize("n,k", [(33000, 256), (40001, 2560), (32768, 4096)])
def test_float_head_form_keeps_activations_in_registers(gpu, orc, pkg, ty, tag, n, k):
    """From 32768 rows a float-activation matvec runs grid-stride with the wave's f32 activations in
    registers: the lane arithmetic and order of the row-per-wave kernels, so the same bits (checked by
    name against `_r2`), and the dequantized dot in f64; partly filled steps (K = 256, 2560), odd rows."""
    w, x = _inputs(pkg, ty, n, k, "fpx")
    gpu.ensure_family("gemv")
    wd, xd = gpu.upload_bytes(w), gpu.upload(x)
    outs = []
    for name in (f"gemv_nat_{tag}_px", f"gemv_nat_{tag}_r2"):
        grid, block = gpu.launch_shape(name, k, n, 1)
        yd = gpu.upload(np.full(n + 2, 12345.0, np.float32))
        gpu.dispatch(gpu.begin(), name, [(xd, 0), (wd, 0), (yd, 4)], [k, n], grid, block)
        got = gpu.read(yd, n + 2)
        assert got[0] == 12345.0 and got[-1] == 12345.0, "wrote outside y"
        outs.append(got[1:-1].copy())
    assert np.array_equal(outs[0], outs[1])
    assert peak_err(outs[0], orc.matmul_ref(w, ty, n, k, x)[0]) <= TOL_FLOAT
    # the router takes it for a plain store
    lin = gpu.lin(ty, n, k, w)
    yr = gpu.alloc(n)
    gpu.mm(xd, lin, yr, 1, act_mode=pkg.ACT_FLOAT)
    assert np.array_equal(gpu.read(yr, n), outs[0])
    with pytest.raises(pkg.OjasHipError, match="registers"):
        gpu.dispatch(gpu.begin(), f"gemv_nat_{tag}_px", [(xd, 0), (wd, 0), (yr, 0)], [4352, n, ], [8, 1, 1], [256, 1, 1])


@pytest.mark.parametrize("ty", [IQ4_NL, IQ4_XS])
@pytest.mark.parametrize("n,k,m", [(4096, 4096, 1), (37, 256, 1), (130, 2816, 4), (1000, 1024, 2), (33001, 2816, 1),
                                   (40000, 4096, 1), (32768, 256, 1)])
def test_iq4_rows_match_the_cpu_dots(gpu, orc, pkg, ty, n, k, m):
    """IQ4_NL / IQ4_XS rows against `matvec_kq`, which sends these types to dot_iq4nl / dot_iq4xs on
    f32 activations (crates/ojas-cpu/src/cpu_math.rs:1179); the int8-activation contract is refused."""
    w = pkg.synth.weights(ty, n, k, "iq4", ty, n, k)
    x = pkg.synth.normal_f32(m * k, "iq4", "x", ty, m, k).reshape(m, k)
    lin = gpu.lin(ty, n, k, w)
    yd = gpu.upload(np.full(m * n + 2, 12345.0, np.float32))
    gpu.mm(gpu.upload(x), lin, yd, m, y_off=4)
    got = gpu.read(yd, m * n + 2)
    assert got[0] == 12345.0 and got[-1] == 12345.0, "wrote outside y"
    for t in range(m):
        assert peak_err(got[1 + t * n:1 + (t + 1) * n], orc.matvec_kq(w, ty, n, k, x[t])) <= 1e-5, t
    with pytest.raises(pkg.OjasHipError, match="f32 activations"):
        gpu.mm(gpu.upload(x), lin, yd, m, act_mode=pkg.ACT_Q8K)


def test_q80_closed_form_rows_with_guards(gpu, pkg):
    """crates/ojas-metal/tests/dispatch.rs:357-429: K=2560, N=13, output between sentinels,
    absolute tolerance 2e-4 against an f64 loop over the same bytes."""
    n, k = 13, 2560
    w, x = pkg.synth.q80_rows_closed_form(n, k)
    blocks = w.reshape(n, k // 32, 34)
    d = blocks[:, :, 0:2].copy().view(np.float16).astype(np.float64)[:, :, 0]
    q = blocks[:, :, 2:].view(np.int8).astype(np.float64)
    want = np.einsum("rb,rbj,bj->r", d, q, x.astype(np.float64).reshape(-1, 32))
    lin = gpu.lin(Q8_0, n, k, w)
    yd = gpu.upload(np.full(n + 4, 12345.0, np.float32))
    gpu.mm(gpu.upload(x), lin, yd, 1, y_off=8)
    got = gpu.read(yd, n + 4)
    assert np.all(got[:2] == 12345.0) and np.all(got[-2:] == 12345.0)
    assert np.max(np.abs(got[2:-2] - want)) < 2e-4


IQ2_XXS, IQ2_XS, IQ3_XXS, IQ1_S, IQ3_S, IQ2_S, IQ1_M = 16, 17, 18, 19, 21, 22, 29


@pytest.mark.parametrize("ty", [Q8_0, Q4_K, Q5_K, Q6_K, IQ4_NL, IQ4_XS, Q4_0, Q4_1, Q5_0, Q5_1, Q2_K, Q3_K,
                                IQ2_XXS, IQ2_XS, IQ3_XXS, IQ1_S, IQ3_S, IQ2_S, IQ1_M, 139])
@pytest.mark.parametrize("mode", ["float", "q8k"])
def test_bias_accum_and_batched_variants(gpu, orc, pkg, ty, mode):
    """The five checks of crates/ojas-models/examples/nat_gemv_gate.rs:36-163: plain, bias
    (1000 + i), accumulate onto a seeded y, batched M=3 with different rows, batched accumulate."""
    if ty in (Q8_0, IQ4_NL, IQ4_XS, Q4_0, Q4_1, Q5_0, Q5_1, Q2_K, Q3_K, IQ2_XS, IQ1_S, IQ3_S, IQ2_S, IQ1_M, 139) and mode == "q8k":
        pytest.skip("this format keeps f32 activations in the CPU reference")
    n, k, m = 200, 1024, 3
    w = pkg.synth.weights(ty, n, k, "var", ty)
    xs = pkg.synth.normal_f32(m * k, "var", "x").reshape(m, k)
    act = pkg.ACT_FLOAT if mode == "float" else pkg.ACT_Q8K
    if mode == "float":
        ref = orc.matmul_ref(w, ty, n, k, xs).astype(np.float32)
        tol = TOL_FLOAT
    else:
        ref = np.stack([orc.matvec_kq(w, ty, n, k, xs[t]) for t in range(m)])
        tol = TOL_Q8K_SEEN
    lin = gpu.lin(ty, n, k, w)
    xd = gpu.upload(xs)
    peak = np.max(np.abs(ref))
    # bias
    bias = (1000.0 + np.arange(n)).astype(np.float32)
    yd = gpu.alloc(n)
    gpu.mm(xd, lin, yd, 1, act_mode=act, bias=gpu.upload(bias))
    assert np.max(np.abs(gpu.read(yd, n) - (ref[0] + bias))) <= tol * peak + 1e-3
    # accumulate
    y0 = pkg.synth.normal_f32(n, "var", "y0")
    yd = gpu.upload(y0)
    gpu.mm(xd, lin, yd, 1, True, act_mode=act)
    assert np.max(np.abs(gpu.read(yd, n) - (ref[0] + y0))) <= tol * peak + 1e-5
    # batched, then batched accumulate; nothing written past row M
    for accum in (False, True):
        y0 = pkg.synth.normal_f32(m * n, "var", "ym").reshape(m, n) if accum else np.zeros((m, n), np.float32)
        init = np.concatenate([y0.ravel(), np.full(n, 12345.5, np.float32)])
        yd = gpu.upload(init)
        gpu.mm(xd, lin, yd, m, accum, act_mode=act)
        got = gpu.read(yd, m * n + n)
        assert np.all(got[m * n:] == 12345.5), "wrote past row M"
        assert np.max(np.abs(got[:m * n].reshape(m, n) - (ref + y0))) <= tol * peak + 1e-5


@pytest.mark.parametrize("m", [1, 2, 4, 5, 8, 16])
def test_small_m_verify_shapes(gpu, orc, pkg, m):
    """Speculative-verify widths on a Q6_K head slice with bf16 activations."""
    n, k = 777, 4096
    w = pkg.synth.q6k_weights(n, k, "verify", "w")
    xb = pkg.synth.to_bf16_bits(pkg.synth.normal_f32(m * k, "verify", "x", m))
    xf = pkg.synth.bf16_bits_to_f32(xb).reshape(m, k)
    lin = gpu.lin(Q6_K, n, k, w)
    yd = gpu.alloc(m * n)
    gpu.mm(gpu.upload_bytes(xb), lin, yd, m, x_dtype=pkg.X_BF16, act_mode=pkg.ACT_Q8K)
    got = gpu.read(yd, m * n).reshape(m, n)
    want = np.stack([orc.matvec_kq(w, Q6_K, n, k, xf[t]) for t in range(m)])
    assert peak_err(got, want) <= TOL_Q8K_SEEN


def test_kernel_seam_dispatch_by_name(gpu, orc, pkg):
    """gemv_nat_q4k through ensure_family / has_kernel / launch_shape / dispatch / submit."""
    gpu.ensure_family("gemv")
    n, k = 130, 2048
    w, x = _inputs(pkg, Q4_K, n, k, "seam")
    wd, xd, yd = gpu.upload_bytes(w), gpu.upload(x), gpu.alloc(n)
    for name in ("gemv_nat_q4k", "gemv_nat_q4k_r1", "gemv_nat_q4k_r2"):
        assert gpu.has_kernel(name)
        grid, block = gpu.launch_shape(name, k, n)
        enc = gpu.begin()
        gpu.memset0(yd)
        gpu.dispatch(enc, name, [(xd, 0), (wd, 0), (yd, 0)], [k, n], grid, block)
        gpu.submit(enc)
        assert peak_err(gpu.read(yd, n), orc.matmul_ref(w, Q4_K, n, k, x)[0]) <= TOL_FLOAT


def test_errors_are_reported_not_launched(gpu, pkg):
    gpu.ensure_family("gemv")
    n, k = 64, 512
    wd = gpu.alloc_bytes(n * pkg.row_bytes(Q4_K, k))
    xd, yd = gpu.alloc(k), gpu.alloc(n)
    grid, block = gpu.launch_shape("gemv_nat_q4k", k, n)
    enc = gpu.begin()
    with pytest.raises(pkg.OjasHipError, match="not loaded"):
        gpu.dispatch(enc, "gemv_nat_q9k", [(xd, 0), (wd, 0), (yd, 0)], [k, n], grid, block)
    with pytest.raises(pkg.OjasHipError, match="needs"):   # y too small for N
        gpu.dispatch(enc, "gemv_nat_q4k", [(xd, 0), (wd, 0), (yd, 0)], [k, n + 1], [grid[0] + 1, 1, 1], block)
    with pytest.raises(pkg.OjasHipError, match="multiple of 256"):
        gpu.dispatch(enc, "gemv_nat_q4k", [(xd, 0), (wd, 0), (yd, 0)], [k - 32, n], grid, block)
    with pytest.raises(pkg.OjasHipError, match="covers"):
        gpu.dispatch(enc, "gemv_nat_q4k", [(xd, 0), (wd, 0), (yd, 0)], [k, n], [1, 1, 1], block)
    with pytest.raises(pkg.OjasHipError, match="takes 3 buffers"):
        gpu.dispatch(enc, "gemv_nat_q4k", [(xd, 0), (wd, 0)], [k, n], grid, block)
    with pytest.raises((pkg.OjasHipError, ValueError)):
        gpu.lin(Q4_K, 4, 100, np.zeros(4, np.uint8))
    with pytest.raises(pkg.OjasHipError, match="unknown kernel family"):
        gpu.ensure_family("attn")
    gpu.submit(enc)


@pytest.mark.parametrize("n,k", [(1024, 4096), (4099, 4096), (96, 14336), (13, 256), (40000, 512)])
def test_fused_quantizer_is_bit_identical_to_the_two_launch_form(gpu, orc, pkg, n, k):
    """gemv_fq8k_q4k_* (one launch, x quantized in-kernel) == ojh_quant_q8k + ojh_mm_q8k, bit for bit."""
    w, x = _inputs(pkg, Q4_K, n, k, "fq")
    x[:5] = [0.5, -2.5, 0.0, 1e-30, 3.0]
    lin = gpu.lin(Q4_K, n, k, w)
    wd = gpu.upload_bytes(w)
    xd, y1, y2 = gpu.upload(x), gpu.alloc(n), gpu.alloc(n)
    xq, xs = gpu.alloc_bytes(k), gpu.alloc(k // 256)
    gpu.ensure_family("gemv_q8k")
    nrb = 24 if n > 100 else 8
    gpu.dispatch(gpu.begin(), "gemv_fq8k_q4k_r2", [(xd, 0), (wd, 0), (y1, 0)], [k, n, nrb], [(n + nrb - 1) // nrb, 1, 1],
                 [256, 1, 1])
    gpu.quant_q8k(xd, 1, k, xq, xs)
    gpu.mm_q8k(xq, xs, lin, y2)
    a, b = gpu.read(y1, n), gpu.read(y2, n)
    assert np.array_equal(a, b)
    assert peak_err(a, orc.matvec_kq(w, Q4_K, n, k, x)) <= TOL_Q8K_SEEN


@pytest.mark.parametrize("ns,k", [((4096, 1024, 1024), 4096), ((14336, 14336), 4096), ((13, 1, 7, 2), 512),
                                  ((5, 300), 2560), ((33,), 256)])
def test_grouped_projections_equal_separate_launches(gpu, orc, pkg, ns, k):
    """ojh_mm_q8k_multi: q/k/v (or gate/up) as separate tensors in one launch; every output must equal
    the single-tensor launch bit for bit, sit within the parity bar of matvec_kq, and no output may
    be written past its N rows (odd row counts make a wave straddle two tensors)."""
    x = pkg.synth.normal_f32(k, "multi", "x", k)
    ws = [pkg.synth.q4k_weights(n, k, "multi", i, n, k) for i, n in enumerate(ns)]
    lins = [gpu.lin(Q4_K, n, k, w) for n, w in zip(ns, ws)]
    xq, xs = gpu.alloc_bytes(k), gpu.alloc(k // 256)
    gpu.quant_q8k(gpu.upload(x), 1, k, xq, xs)
    guard = np.float32(-7.25)
    ys = [gpu.upload(np.full(n + 4, guard, np.float32)) for n in ns]
    gpu.mm_q8k_multi(xq, xs, lins, ys)
    for n, w, lin, y in zip(ns, ws, lins, ys):
        got = gpu.read(y, n + 4)
        assert np.all(got[n:] == guard)
        y1 = gpu.alloc(n)
        gpu.mm_q8k(xq, xs, lin, y1)
        assert np.array_equal(got[:n], gpu.read(y1, n))
        assert peak_err(got[:n], orc.matvec_kq(w, Q4_K, n, k, x)) <= TOL_Q8K_SEEN


@pytest.mark.parametrize("ns,k", [((4096, 1024, 1024), 4096), ((14336, 14336), 4096), ((13, 1, 7, 2), 512),
                                  ((5, 300), 2560), ((33,), 256), ((40,), 14336), ((4096,), 8192)])
@pytest.mark.parametrize("accum", [False, True])
def test_stage_launch_with_the_quantizer_inside(gpu, orc, pkg, ns, k, accum):
    """ojh_mm_multi: f32 activations in, one launch per stage (quantizer folded in for small Q4_K stages, a quantizer
    launch plus the grouped launch otherwise) — every output bit-equal to quantizer + single-tensor launches, within
    the parity bar of matvec_kq, nothing written past a tensor's rows; also with the single launch forced at every
    size and workgroup shape."""
    import os
    x = pkg.synth.normal_f32(k, "stage", "x", k)
    ws = [pkg.synth.q4k_weights(n, k, "stage", i, n, k) for i, n in enumerate(ns)]
    y0s = [pkg.synth.normal_f32(n, "stage", "y0", i) for i, n in enumerate(ns)]
    guard = np.float32(-7.25)
    xd = gpu.upload(x)
    xq, xs = gpu.alloc_bytes(k), gpu.alloc(k // 256)
    gpu.quant_q8k(xd, 1, k, xq, xs)
    lins = [gpu.lin(Q4_K, n, k, w) for n, w in zip(ns, ws)]
    want = []
    for n, lin, y0 in zip(ns, lins, y0s):
        y1 = gpu.upload(y0)
        gpu.mm_q8k(xq, xs, lin, y1, accum=accum)
        want.append(gpu.read(y1, n))
    for env in ({}, {"OJAS_HIP_FQ_MULTI": "2"}, {"OJAS_HIP_FQ_MULTI": "2", "OJAS_HIP_FQ_THREADS": "256", "OJAS_HIP_FQ_MULTI_BLOCKS": "8", "OJAS_HIP_FQ_ROWS": "1"},
                {"OJAS_HIP_FQ_MULTI": "2", "OJAS_HIP_FQ_THREADS": "512", "OJAS_HIP_FQ_MULTI_BLOCKS": "3"}):
        old = {k_: os.environ.get(k_) for k_ in env}
        os.environ.update(env)
        g2 = pkg.HipGpu(0) if env else gpu            # the settings are read when a device is opened
        try:
            l2 = lins if not env else [g2.lin(Q4_K, n, k, w) for n, w in zip(ns, ws)]
            ys = [g2.upload(np.concatenate([y0, np.full(4, guard, np.float32)])) for y0 in y0s]
            g2.mm_multi(g2.upload(x), l2, ys, accum=accum)
            for n, w, y, wnt, y0 in zip(ns, ws, ys, want, y0s):
                got = g2.read(y, n + 4)
                assert np.all(got[n:] == guard), env
                assert np.array_equal(got[:n].view(np.uint32), wnt.view(np.uint32)), env
                assert peak_err(got[:n] - (y0 if accum else 0), orc.matvec_kq(w, Q4_K, n, k, x)) <= TOL_Q8K_SEEN
        finally:
            for k_, v_ in old.items():
                if v_ is None:
                    os.environ.pop(k_, None)
                else:
                    os.environ[k_] = v_
            if env:
                g2.close()


def test_grouped_projections_other_formats_and_errors(gpu, orc, pkg):
    k = 512
    x = pkg.synth.normal_f32(k, "multi", "x6", k)
    w4, w6 = pkg.synth.q4k_weights(40, k, "multi", "a"), pkg.synth.q6k_weights(24, k, "multi", "b")
    l4, l6 = gpu.lin(Q4_K, 40, k, w4), gpu.lin(Q6_K, 24, k, w6)
    xq, xs = gpu.alloc_bytes(k), gpu.alloc(k // 256)
    gpu.quant_q8k(gpu.upload(x), 1, k, xq, xs)
    y4, y6 = gpu.alloc(40), gpu.alloc(24)
    gpu.mm_q8k_multi(xq, xs, [l4, l6], [y4, y6])      # mixed formats: one launch each
    assert peak_err(gpu.read(y4, 40), orc.matvec_kq(w4, Q4_K, 40, k, x)) <= TOL_Q8K_SEEN
    assert peak_err(gpu.read(y6, 24), orc.matvec_kq(w6, Q6_K, 24, k, x)) <= TOL_Q8K_SEEN
    other = gpu.lin(Q4_K, 8, 256, pkg.synth.q4k_weights(8, 256, "multi", "c"))
    with pytest.raises(pkg.OjasHipError, match="has K="):
        gpu.mm_q8k_multi(xq, xs, [l4, other], [y4, y6])
    with pytest.raises(pkg.OjasHipError, match="1 to 4"):
        gpu.mm_q8k_multi(xq, xs, [l4] * 5, [y4] * 5)
    with pytest.raises(pkg.OjasHipError, match="needs"):
        gpu.mm_q8k_multi(xq, xs, [l4, l4], [y4, y6])
    # the stage entry over mixed formats: a quantizer launch, then one launch per format
    xd = gpu.upload(x)
    gpu.memset0(y4)
    gpu.memset0(y6)
    gpu.mm_multi(xd, [l4, l6], [y4, y6])
    assert peak_err(gpu.read(y4, 40), orc.matvec_kq(w4, Q4_K, 40, k, x)) <= TOL_Q8K_SEEN
    assert peak_err(gpu.read(y6, 24), orc.matvec_kq(w6, Q6_K, 24, k, x)) <= TOL_Q8K_SEEN
    q80 = gpu.lin(8, 8, k, pkg.synth.q80_weights(8, k, "multi", "q80"))
    with pytest.raises(pkg.OjasHipError, match="need no quantizer"):
        gpu.mm_multi(xd, [q80], [y4])


@pytest.mark.parametrize("m,n,k,accum", [(3, 50, 256, False), (4, 130, 14336, True), (16, 301, 4096, False),
                                         (9, 64, 2560, True), (17, 40, 4096, False), (5, 33, 16384, False)])
def test_q6k_few_tokens_staged_and_streamed_forms_agree(gpu, orc, pkg, m, n, k, accum):
    """Q6_K rows against a few tokens: the router's choice (activations staged in LDS when they fit,
    the streamed `_m` entry otherwise) within the parity bar of matvec_kq, ragged super-block
    counts and accumulate included; where both forms apply they must agree bit for bit in the
    integer part, i.e. to the last-ulp association of the f32 sums."""
    w = pkg.synth.q6k_weights(n, k, "mx", n, k)
    x = pkg.synth.normal_f32(m * k, "mx", "x", m, k).reshape(m, k)
    lin = gpu.lin(Q6_K, n, k, w)
    y0 = pkg.synth.normal_f32(m * n, "mx", "y0").reshape(m, n) if accum else np.zeros((m, n), np.float32)
    yd = gpu.upload(np.concatenate([y0.ravel(), np.full(8, 4242.5, np.float32)]))
    gpu.mm(gpu.upload(x), lin, yd, m, accum, act_mode=pkg.ACT_Q8K)
    got = gpu.read(yd, m * n + 8)
    assert np.all(got[m * n:] == 4242.5)
    want = np.stack([orc.matvec_kq(w, Q6_K, n, k, x[t]) for t in range(m)])
    assert peak_err(got[:m * n].reshape(m, n) - y0, want) <= TOL_Q8K_SEEN
    # the streamed entry by name on the same quantized activations
    gpu.ensure_family("gemv_q8k")
    nsb = k // 256
    xq, xs = gpu.alloc_bytes(m * k), gpu.alloc(m * nsb)
    gpu.quant_q8k(gpu.upload(x), m, k, xq, xs)
    y2 = gpu.upload(y0)
    gpu.dispatch(gpu.begin(), "gemv_q8k_q6k_m", [(xq, 0), (xs, 0), (gpu.upload_bytes(w), 0), (y2, 0)],
                 [k, n, m, int(accum)], [(n + 3) // 4, 1, 1], [256, 1, 1])
    assert peak_err(gpu.read(y2, m * n).reshape(m, n) - y0, got[:m * n].reshape(m, n) - y0) <= 2e-6
    if m > 16:
        with pytest.raises(pkg.OjasHipError, match="do not fit"):
            gpu.dispatch(gpu.begin(), "gemv_q8k_q6k_mx", [(xq, 0), (xs, 0), (gpu.upload_bytes(w), 0), (y2, 0)],
                         [k, n, m, 0], [8, 1, 1], [256, 1, 1])


def test_q5k_takes_the_int8_path_below_the_tile_crossover(gpu, orc, pkg):
    """Q5_K defaults to dot_q5k's arithmetic (crates/ojas-cpu/src/cpu_math.rs:638-670): AUTO resolves to it below the
    crossover to the f16 tile (for Q5_K 65 tokens: its int8 tile is the faster one up to 64), OJH_ACT_Q8K at every token
    count; a floating-point contract runs the f32-activation matvecs below 32 tokens and the f16 tile from there (the
    dequantized dot in f64 is the judge; the tile rounds the activations to f16); the wide-row form (N >= 32768) agrees
    with the oracle too."""
    n, k = 300, 1024
    w = pkg.synth.weights(Q5_K, n, k, "q5k", "any-m")
    lin = gpu.lin(Q5_K, n, k, w)
    for m, act in ((1, pkg.ACT_AUTO), (9, pkg.ACT_AUTO), (24, pkg.ACT_AUTO), (40, pkg.ACT_AUTO), (64, pkg.ACT_AUTO), (200, pkg.ACT_Q8K)):
        xs = pkg.synth.normal_f32(m * k, "q5k", "x", m).reshape(m, k)
        yd = gpu.alloc(m * n)
        gpu.mm(gpu.upload(xs), lin, yd, m, act_mode=act)
        want = np.stack([orc.matvec_kq(w, Q5_K, n, k, xs[t]) for t in range(m)])
        assert peak_err(gpu.read(yd, m * n).reshape(m, n), want) <= TOL_Q8K_SEEN
    for m in (24, 40, 80):
        xs = pkg.synth.normal_f32(m * k, "q5k", "x", m).reshape(m, k)
        yd = gpu.alloc(m * n)
        for act in (pkg.ACT_FLOAT, pkg.ACT_FLOAT_EXACT) + ((pkg.ACT_AUTO,) if m >= 65 else ()):
            gpu.mm(gpu.upload(xs), lin, yd, m, act_mode=act)
            got = gpu.read(yd, m * n).reshape(m, n)
            assert peak_err(got, orc.matmul_ref(w, Q5_K, n, k, xs)) <= (2e-3 if m >= 32 else TOL_FLOAT)
            if m >= 32:     # the tile's own error: against f16-rounded activations and dequant_to_f16 weights
                assert peak_err(got, orc.matmul_ref(w, Q5_K, n, k, xs, wmode=1, xmode=1)) <= 2e-5
    n, k = 33000, 256
    w, x = _inputs(pkg, Q5_K, n, k, "wide")
    yd = gpu.alloc(n)
    gpu.mm(gpu.upload(x), gpu.lin(Q5_K, n, k, w), yd, 1, act_mode=pkg.ACT_Q8K)
    assert peak_err(gpu.read(yd, n), orc.matvec_kq(w, Q5_K, n, k, x)) <= TOL_Q8K_SEEN


@pytest.mark.parametrize("n,k", [(4096, 4096), (4099, 4096), (2049, 8192), (2050, 14336), (3000, 2560), (5, 256),
                                 (1, 4096), (7, 14336), (70000, 256)])
def test_q80_rows_staged_through_lds(pkg, orc, monkeypatch, n, k):
    """The Q8_0 matvec that keeps activations in registers and has rows copied into LDS: one, two
    and four K chunks, partly filled chunks (K = 2560, 14336), row counts that leave surplus waves
    and surplus steps, bias and accumulate — against dot_q80 and against the streaming kernel."""
    w, x = _inputs(pkg, Q8_0, n, k, "lds")
    bias = (1000.0 + np.arange(n)).astype(np.float32)
    y0 = pkg.synth.normal_f32(n, "lds", "y0", n)
    want = orc.matvec_kq(w, Q8_0, n, k, x)
    outs = {}
    for lds in ("1", "0"):
        monkeypatch.setenv("OJAS_HIP_Q80_LDS", lds)
        monkeypatch.setenv("OJAS_HIP_Q80_LDS_MIN_N", "1")
        g = pkg.HipGpu(0)
        try:
            lin, xd = g.lin(Q8_0, n, k, w), g.upload(x)
            yd = g.upload(np.full(n + 2, 12345.0, np.float32))
            g.mm(xd, lin, yd, 1, y_off=4)
            got = g.read(yd, n + 2)
            assert got[0] == 12345.0 and got[-1] == 12345.0, "wrote outside y"
            yb, ya = g.alloc(n), g.upload(y0)
            g.mm(xd, lin, yb, 1, bias=g.upload(bias))
            g.mm(xd, lin, ya, 1, True)
            outs[lds] = (got[1:-1].copy(), g.read(yb, n), g.read(ya, n))
        finally:
            g.close()
    peak = np.max(np.abs(want))
    for lds in ("1", "0"):
        plain, with_bias, onto = outs[lds]
        assert peak_err(plain, want) <= 1e-5, lds
        assert np.max(np.abs(with_bias - (want + bias))) <= 1e-5 * peak + 1e-3, lds
        assert np.max(np.abs(onto - (want + y0))) <= 1e-5 * peak + 1e-5, lds
    assert peak_err(outs["1"][0], outs["0"][0]) <= 2e-6


@pytest.mark.parametrize("m,n,k,accum", [(4, 50, 256, False), (8, 130, 4096, True), (9, 301, 4096, False),
                                         (16, 1000, 4096, False), (16, 17, 512, True), (12, 4099, 2560, False),
                                         (6, 64, 7168, False), (40, 300, 4096, True), (64, 33, 1024, False),
                                         (150, 40, 512, False)])
def test_q6k_tokens_on_the_int8_matrix_cores(gpu, orc, pkg, m, n, k, accum):
    """5 to 16 tokens against Q6_K rows: `gemv_q8k_q6k_mf` by name and through the router, against
    matvec_kq per token and against the LDS-staged integer-dot entry on the same quantized
    activations (same integer sums; the f32 sums associate differently)."""
    w = pkg.synth.q6k_weights(n, k, "mf", n, k)
    x = pkg.synth.normal_f32(m * k, "mf", "x", m, k).reshape(m, k)
    x[0, :256] = 0.0
    y0 = pkg.synth.normal_f32(m * n, "mf", "y0").reshape(m, n) if accum else np.zeros((m, n), np.float32)
    want = np.stack([orc.matvec_kq(w, Q6_K, n, k, x[t]) for t in range(m)])
    lin = gpu.lin(Q6_K, n, k, w)
    yd = gpu.upload(np.concatenate([y0.ravel(), np.full(8, 4242.5, np.float32)]))
    gpu.mm(gpu.upload(x), lin, yd, m, accum, act_mode=pkg.ACT_Q8K)
    got = gpu.read(yd, m * n + 8)
    assert np.all(got[m * n:] == 4242.5), "wrote past the last token"
    assert peak_err(got[:m * n].reshape(m, n) - y0, want) <= TOL_Q8K_SEEN
    if m > 16:
        return          # the router ran it as launches of 16 tokens; the entries themselves take at most 16
    gpu.ensure_family("gemv_q8k")
    nsb = k // 256
    xq, xs = gpu.alloc_bytes(m * k), gpu.alloc(m * nsb)
    gpu.quant_q8k(gpu.upload(x), m, k, xq, xs)
    wd = gpu.upload_bytes(w)
    outs = []
    for name in ("gemv_q8k_q6k_mf", "gemv_q8k_q6k_mx"):
        grid, block = gpu.launch_shape(name, k, n, m)
        y2 = gpu.upload(y0)
        gpu.dispatch(gpu.begin(), name, [(xq, 0), (xs, 0), (wd, 0), (y2, 0)], [k, n, m, int(accum)], grid, block)
        outs.append(gpu.read(y2, m * n).reshape(m, n) - y0)
    assert peak_err(outs[0], want) <= TOL_Q8K_SEEN
    assert peak_err(outs[0], outs[1]) <= 2e-6
    with pytest.raises(pkg.OjasHipError, match="do not fit"):
        gpu.dispatch(gpu.begin(), "gemv_q8k_q6k_mf", [(xq, 0), (xs, 0), (wd, 0), (y2, 0)], [k, n, 17, 0], [8, 1, 1], [256, 1, 1])


@pytest.mark.parametrize("m,n,k,accum,grid_x", [(4, 50, 256, False, None), (8, 130, 4096, True, 3), (9, 301, 4096, False, 2),
                                                (16, 1000, 4096, False, 7), (16, 17, 512, True, None),
                                                (3, 4099, 2560, False, None), (8, 77, 7168, True, 1), (12, 333, 5632, False, 1)])
def test_q6k_tokens_with_rows_copied_through_lds(gpu, orc, pkg, m, n, k, accum, grid_x):
    """`gemv_q8k_q6k_ml`: the matrix-core tile with each wave's rows copied global -> LDS a
    super-block at a time.  Against matvec_kq per token and, bit for bit, the direct-load entry on
    the same quantized activations (the same arithmetic on the same bytes).  Small grids make a
    wave walk many tiles, so its copy ring wraps and runs ahead across tile borders.  The copies
    move whole aligned 16-byte pieces: the buffer must reach the next multiple of 16 past the last
    row (poisoned here), and a shorter one is refused."""
    w = pkg.synth.q6k_weights(n, k, "ml", n, k)
    x = pkg.synth.normal_f32(m * k, "ml", "x", m, k).reshape(m, k)
    y0 = pkg.synth.normal_f32(m * n, "ml", "y0").reshape(m, n) if accum else np.zeros((m, n), np.float32)
    want = np.stack([orc.matvec_kq(w, Q6_K, n, k, x[t]) for t in range(m)])
    gpu.ensure_family("gemv_q8k")
    nsb = k // 256
    xq, xs = gpu.alloc_bytes(m * k), gpu.alloc(m * nsb)
    gpu.quant_q8k(gpu.upload(x), m, k, xq, xs)
    wd = gpu.upload_bytes(np.concatenate([w, np.full(-w.size % 16, 0xA5, np.uint8)]))
    outs = {}
    mf_fits = (8 if m <= 8 else 16) * (k + 32) + k // 4 + 256 <= 69632
    if w.size % 16:
        with pytest.raises(pkg.OjasHipError):
            gpu.dispatch(gpu.begin(), "gemv_q8k_q6k_ml", [(xq, 0), (xs, 0), (gpu.upload_bytes(w), 0), (gpu.alloc(m * n), 0)],
                         [k, n, m, 0], [8, 1, 1], [512, 1, 1])
    for name in ("gemv_q8k_q6k_ml", "gemv_q8k_q6k_mf") if mf_fits else ("gemv_q8k_q6k_ml",):
        grid, block = gpu.launch_shape(name, k, n, m)
        if grid_x and name.endswith("ml"):
            grid = [grid_x, 1, 1]
        yd = gpu.upload(np.concatenate([y0.ravel(), np.full(8, 4242.5, np.float32)]))
        gpu.dispatch(gpu.begin(), name, [(xq, 0), (xs, 0), (wd, 0), (yd, 0)], [k, n, m, int(accum)], grid, block)
        got = gpu.read(yd, m * n + 8)
        assert np.all(got[m * n:] == 4242.5), "wrote past the last token"
        outs[name] = got[:m * n].reshape(m, n) - y0
    assert peak_err(outs["gemv_q8k_q6k_ml"], want) <= TOL_Q8K_SEEN
    if mf_fits:
        assert np.array_equal(outs["gemv_q8k_q6k_ml"], outs["gemv_q8k_q6k_mf"])
    with pytest.raises(pkg.OjasHipError, match="do not fit"):
        gpu.dispatch(gpu.begin(), "gemv_q8k_q6k_ml", [(xq, 0), (xs, 0), (wd, 0), (yd, 0)], [k, n, 17, 0], [8, 1, 1], [512, 1, 1])


@pytest.mark.parametrize("m,n,k,accum,grid_x", [(4, 50, 256, False, None), (8, 130, 4096, True, 3), (9, 301, 4096, False, None),
                                                (16, 100, 8192, False, 2), (8, 33, 14336, True, None), (3, 4099, 2560, False, None)])
def test_q6k_tokens_with_k_split_over_the_waves(gpu, orc, pkg, m, n, k, accum, grid_x):
    """`gemv_q8k_q6k_mk`: a workgroup per 16-row tile, super-blocks dealt to its eight waves, partial
    sums added in wave order.  Against matvec_kq per token; the router takes it for few rows."""
    w = pkg.synth.q6k_weights(n, k, "mk", n, k)
    x = pkg.synth.normal_f32(m * k, "mk", "x", m, k).reshape(m, k)
    y0 = pkg.synth.normal_f32(m * n, "mk", "y0").reshape(m, n) if accum else np.zeros((m, n), np.float32)
    want = np.stack([orc.matvec_kq(w, Q6_K, n, k, x[t]) for t in range(m)])
    gpu.ensure_family("gemv_q8k")
    nsb = k // 256
    xq, xs = gpu.alloc_bytes(m * k), gpu.alloc(m * nsb)
    gpu.quant_q8k(gpu.upload(x), m, k, xq, xs)
    wd = gpu.upload_bytes(w)
    grid, block = gpu.launch_shape("gemv_q8k_q6k_mk", k, n, m)
    if grid_x:
        grid = [grid_x, 1, 1]
    yd = gpu.upload(np.concatenate([y0.ravel(), np.full(8, 4242.5, np.float32)]))
    gpu.dispatch(gpu.begin(), "gemv_q8k_q6k_mk", [(xq, 0), (xs, 0), (wd, 0), (yd, 0)], [k, n, m, int(accum)], grid, block)
    got = gpu.read(yd, m * n + 8)
    assert np.all(got[m * n:] == 4242.5), "wrote past the last token"
    assert peak_err(got[:m * n].reshape(m, n) - y0, want) <= TOL_Q8K_SEEN
    # through the router (few rows: this entry from 5 tokens, or 3 of a long K), in chunks where 16 tokens do not fit
    lin = gpu.lin(Q6_K, n, k, w)
    for mm in (m, 2 * m + 1):
        xx = np.concatenate([x, x[::-1], x[:1]])[:mm]
        yr = gpu.alloc(mm * n)
        gpu.mm(gpu.upload(xx), lin, yr, mm, act_mode=pkg.ACT_Q8K)
        wantr = np.stack([orc.matvec_kq(w, Q6_K, n, k, xx[t]) for t in range(mm)])
        assert peak_err(gpu.read(yr, mm * n).reshape(mm, n), wantr) <= TOL_Q8K_SEEN, mm
    with pytest.raises(pkg.OjasHipError, match="do not fit"):
        gpu.dispatch(gpu.begin(), "gemv_q8k_q6k_mk", [(xq, 0), (xs, 0), (wd, 0), (yd, 0)], [k, n, 17, 0], [8, 1, 1], [512, 1, 1])


@pytest.mark.parametrize("n,k", [(33000, 256), (40001, 2560), (32768, 8192)])
def test_q6k_head_form_keeps_activations_in_registers(gpu, orc, pkg, n, k):
    """From 32768 rows a Q6_K matvec runs grid-stride with the activations in registers: the lane
    arithmetic of the row-per-wave kernel, so the same bits, checked by name against `_r2`, and the
    oracle's values; partly filled steps (K = 256, 2560), two steps (K = 8192), odd row counts."""
    w, x = _inputs(pkg, Q6_K, n, k, "px")
    lin = gpu.lin(Q6_K, n, k, w)
    yd = gpu.upload(np.full(n + 2, 12345.0, np.float32))
    gpu.mm(gpu.upload(x), lin, yd, 1, act_mode=pkg.ACT_Q8K, y_off=4)
    got = gpu.read(yd, n + 2)
    assert got[0] == 12345.0 and got[-1] == 12345.0, "wrote outside y"
    assert peak_err(got[1:-1], orc.matvec_kq(w, Q6_K, n, k, x)) <= TOL_Q8K_SEEN
    gpu.ensure_family("gemv_q8k")
    xq, xs = gpu.alloc_bytes(k), gpu.alloc(k // 256)
    gpu.quant_q8k(gpu.upload(x), 1, k, xq, xs)
    wd = gpu.upload_bytes(w)
    outs = []
    for name in ("gemv_q8k_q6k_px", "gemv_q8k_q6k_r2"):
        grid, block = gpu.launch_shape(name, k, n, 1)
        y2 = gpu.alloc(n)
        gpu.dispatch(gpu.begin(), name, [(xq, 0), (xs, 0), (wd, 0), (y2, 0)], [k, n], grid, block)
        outs.append(gpu.read(y2, n))
    assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[0], got[1:-1])
    with pytest.raises(pkg.OjasHipError, match="8192"):
        gpu.dispatch(gpu.begin(), "gemv_q8k_q6k_px", [(xq, 0), (xs, 0), (wd, 0), (y2, 0)], [16384, n, 0][:2], [8, 1, 1], [256, 1, 1])
