"""Q8_0 blocks against activations quantized per 32 values: the reference GPU decode path's kernels by their own
names (crates/ojas-cuda/src/kernels/gemv_q8.rs:152-260, gemv.rs:33-52), checked the way its conformance tests check
them (crates/ojas-cuda/tests/conformance.rs:563-760: K = 1024, N = 128, the vector peak as the scale, bound 1e-2
against the dequantized dot) and, much tighter, against the CPU restatement of the same integer arithmetic."""
import numpy as np
import pytest

from conftest import peak_err

pytestmark = pytest.mark.gpu
Q8_0 = 8
TOL = 2e-6          # against the restatement: a few f32 roundings of the row sum
REF_BOUND = 1e-2    # the reference's own bound against the reader's values


def _quantize(gpu, xd, k):
    q8, d8, d8s = gpu.alloc_bytes(k), gpu.alloc(k // 32), gpu.alloc(k // 32)
    grid, block = gpu.launch_shape("quantize_q8_1", k, 0, 0)
    gpu.dispatch(gpu.begin(), "quantize_q8_1", [(xd, 0), (q8, 0), (d8, 0), (d8s, 0)], [k], grid, block)
    return q8, d8, d8s


@pytest.mark.parametrize("k", [32, 1024, 4096, 4128, 14336])
def test_quantize_q8_1_bit_for_bit(gpu, orc, pkg, k):
    gpu.ensure_family("q80_dp4a")
    x = pkg.synth.normal_f32(k, "q81", "x", k)
    x[:7] = [0.5, -0.5, 1.5, -2.5, 0.0, 1e-30, -1e-30]
    if k >= 1024:
        x[64:96] = 0.0                       # a block of zeros: scale 0, codes 0
        x[200], x[300] = np.nan, np.inf      # a NaN is code 0 and outside the maximum; an infinity zeroes its block's codes
    q8, d8, d8s = _quantize(gpu, gpu.upload(x), k)
    wq, wd, ws = orc.quantize_q8_1(x)
    assert np.array_equal(gpu.read(q8, k, np.int8), wq)
    assert np.array_equal(gpu.read(d8, k // 32), wd)
    assert np.array_equal(gpu.read(d8s, k // 32), ws, equal_nan=True)     # (the infinite block's sum is inf * 0)


def test_reference_case_and_variants(gpu, orc, pkg):
    """K = 1024, N = 128, x = tvec(K, 81): plain, bias, accumulate, fused q/k/v (GQA shaped, with bias) and fused
    gate/up, each against the reader's dot as the reference judges it and against the integer restatement."""
    gpu.ensure_family("q80_dp4a")
    k, n = 1024, 128
    x = pkg.synth.tvec(k, 81)
    w, plain = pkg.synth.q80_rows_mod5(n, k, 82)
    dot = (plain.astype(np.float64) * x.astype(np.float64)).sum(1)
    wd, xd = gpu.upload_bytes(w), gpu.upload(x)
    q8, d8, _ = _quantize(gpu, xd, k)
    hq, hd, _ = orc.quantize_q8_1(x)
    want = orc.gemv_q80_dp4a(w, hq, hd, n, k)
    grid, block = gpu.launch_shape("gemv_q80_dp4a", k, n, 1)
    assert grid == [n // 8, 1, 1] and block == [256, 1, 1]
    yd = gpu.upload(np.full(n + 2, 777.0, np.float32))
    gpu.dispatch(gpu.begin(), "gemv_q80_dp4a", [(wd, 0), (q8, 0), (d8, 0), (yd, 4)], [k, n], grid, block)
    got = gpu.read(yd, n + 2)
    assert got[0] == 777.0 and got[-1] == 777.0, "wrote outside y"
    assert peak_err(got[1:-1], want) <= TOL
    assert peak_err(got[1:-1], dot) < REF_BOUND
    # bias
    bias = pkg.synth.tvec(n, 83)
    yb = gpu.alloc(n)
    gpu.dispatch(gpu.begin(), "gemv_q80_dp4a_bias", [(wd, 0), (q8, 0), (d8, 0), (yb, 0), (gpu.upload(bias), 0)], [k, n], grid, block)
    assert peak_err(gpu.read(yb, n), want + bias) <= TOL
    assert peak_err(gpu.read(yb, n), dot + bias) < REF_BOUND
    # accumulate: the prior contents plus the dot
    seed_y = pkg.synth.tvec(n, 84)
    ya = gpu.upload(seed_y)
    gpu.dispatch(gpu.begin(), "gemv_q80_dp4a_accum", [(wd, 0), (q8, 0), (d8, 0), (ya, 0)], [k, n], grid, block)
    assert peak_err(gpu.read(ya, n), seed_y + want) <= TOL
    assert peak_err(gpu.read(ya, n), seed_y + dot) < REF_BOUND
    # fused q/k/v
    nq, nkv = 128, 32
    kb, kplain = pkg.synth.q80_rows_mod5(nkv, k, 85)
    vb, vplain = pkg.synth.q80_rows_mod5(nkv, k, 86)
    qkv_bias = pkg.synth.tvec(nq + 2 * nkv, 87)
    qo, ko, vo = gpu.alloc(nq), gpu.alloc(nkv), gpu.alloc(nkv)
    g3, b3 = gpu.launch_shape("qkv_q80_dp4a", k, nq + 2 * nkv, 1)
    gpu.dispatch(gpu.begin(), "qkv_q80_dp4a",
                 [(wd, 0), (gpu.upload_bytes(kb), 0), (gpu.upload_bytes(vb), 0), (q8, 0), (d8, 0), (qo, 0), (ko, 0), (vo, 0),
                  (gpu.upload(qkv_bias), 0)], [k, nq, nkv], g3, b3)
    for buf, raw, vals, rows, boff in ((qo, w, plain, nq, 0), (ko, kb, kplain, nkv, nq), (vo, vb, vplain, nkv, nq + nkv)):
        got = gpu.read(buf, rows)
        assert peak_err(got, orc.gemv_q80_dp4a(raw, hq, hd, rows, k) + qkv_bias[boff:boff + rows]) <= TOL
        assert peak_err(got, (vals.astype(np.float64) * x).sum(1) + qkv_bias[boff:boff + rows]) < REF_BOUND
    # fused gate/up, both activation functions
    ub, uplain = pkg.synth.q80_rows_mod5(n, k, 88)
    ud, out = gpu.upload_bytes(ub), gpu.alloc(n)
    g5, b5 = gpu.launch_shape("ffn_gu_q80_dp4a", k, n, 1)
    assert g5 == [n // 4, 1, 1]
    up_want = orc.gemv_q80_dp4a(ub, hq, hd, n, k).astype(np.float64)
    up_dot = (uplain.astype(np.float64) * x).sum(1)
    for act in (0, 1):
        def f(g):
            if act == 0:
                return g / (1.0 + np.exp(-g))
            return 0.5 * g * (1.0 + np.tanh(np.clip(0.7978845608 * (g + 0.044715 * g ** 3), -30.0, 30.0)))
        gpu.dispatch(gpu.begin(), "ffn_gu_q80_dp4a", [(wd, 0), (ud, 0), (q8, 0), (d8, 0), (out, 0)], [k, n, act], g5, b5)
        got = gpu.read(out, n)
        assert peak_err(got, f(want.astype(np.float64)) * up_want) <= 5e-6, act
        assert peak_err(got, f(dot) * up_dot) < REF_BOUND, act


@pytest.mark.parametrize("n,k", [(1, 32), (13, 2560), (4096, 4096), (777, 14336), (4099, 4096), (9, 96)])
def test_rows_of_any_shape(gpu, orc, pkg, n, k):
    """Odd row counts (a wave's second row past the end), K that leaves steps partly filled, long rows."""
    gpu.ensure_family("q80_dp4a")
    w = pkg.synth.q80_weights(n, k, "q81", n, k)
    x = pkg.synth.normal_f32(k, "q81", "x2", n, k)
    wd, xd = gpu.upload_bytes(w), gpu.upload(x)
    q8, d8, _ = _quantize(gpu, xd, k)
    hq, hd, _ = orc.quantize_q8_1(x)
    want = orc.gemv_q80_dp4a(w, hq, hd, n, k)
    grid, block = gpu.launch_shape("gemv_q80_dp4a", k, n, 1)
    yd = gpu.upload(np.full(n + 2, 777.0, np.float32))
    gpu.dispatch(gpu.begin(), "gemv_q80_dp4a", [(wd, 0), (q8, 0), (d8, 0), (yd, 4)], [k, n], grid, block)
    got = gpu.read(yd, n + 2)
    assert got[0] == 777.0 and got[-1] == 777.0, "wrote outside y"
    assert peak_err(got[1:-1], want) <= TOL
    # the quantized dot stays within the reference's bound of the CPU path's dot_q80 on f32 activations
    assert peak_err(got[1:-1], orc.matvec_kq(w, Q8_0, n, k, x)) < REF_BOUND
    # fused q/k/v with borders inside a wave's pair of rows
    if n >= 9:
        nq, nkv = n - 6, 3
        rb = (k // 32) * 34
        qo, ko, vo = gpu.alloc(nq), gpu.alloc(nkv), gpu.alloc(nkv)
        zeros = gpu.upload(np.zeros(n, np.float32))
        g3, b3 = gpu.launch_shape("qkv_q80_dp4a", k, n, 1)
        gpu.dispatch(gpu.begin(), "qkv_q80_dp4a",
                     [(wd, 0), (wd, nq * rb), (wd, (nq + nkv) * rb), (q8, 0), (d8, 0), (qo, 0), (ko, 0), (vo, 0), (zeros, 0)],
                     [k, nq, nkv], g3, b3)
        both = np.concatenate([gpu.read(qo, nq), gpu.read(ko, nkv), gpu.read(vo, nkv)])
        assert np.array_equal(both, got[1:-1])


def test_op_level_route_and_refusals(gpu, orc, pkg):
    """`mm` under ACT_Q8_1: quantize_q8_1 + gemv_q80_dp4a per token, with bias or accumulation; other formats refused."""
    n, k, m = 300, 2048, 3
    w = pkg.synth.q80_weights(n, k, "q81", "op")
    x = pkg.synth.normal_f32(m * k, "q81", "opx").reshape(m, k)
    lin = gpu.lin(Q8_0, n, k, w)
    yd = gpu.alloc(m * n)
    gpu.mm(gpu.upload(x), lin, yd, m, act_mode=pkg.ACT_Q8_1)
    got = gpu.read(yd, m * n).reshape(m, n)
    for t in range(m):
        hq, hd, _ = orc.quantize_q8_1(x[t])
        assert peak_err(got[t], orc.gemv_q80_dp4a(w, hq, hd, n, k)) <= TOL, t
    gpu.mm(gpu.upload(x), lin, yd, m, True, act_mode=pkg.ACT_Q8_1)
    assert peak_err(gpu.read(yd, m * n).reshape(m, n), 2.0 * got) <= TOL
    lin4 = gpu.lin(12, 8, 256, pkg.synth.q4k_weights(8, 256, "q81", "q4k"))
    with pytest.raises(pkg.OjasHipError, match="Q8_0"):
        gpu.mm(gpu.upload(x[0, :256].copy()), lin4, gpu.alloc(8), 1, act_mode=pkg.ACT_Q8_1)
    gpu.ensure_family("q80_dp4a")
    with pytest.raises(pkg.OjasHipError, match="multiple of 32"):
        gpu.dispatch(gpu.begin(), "gemv_q80_dp4a", [(yd, 0), (yd, 0), (yd, 0), (yd, 0)], [48, 4], [1, 1, 1], [256, 1, 1])
    with pytest.raises(pkg.OjasHipError, match="does not cover"):
        gpu.dispatch(gpu.begin(), "gemv_q80_dp4a", [(yd, 0), (yd, 0), (yd, 0), (yd, 0)], [64, 17], [2, 1, 1], [256, 1, 1])
