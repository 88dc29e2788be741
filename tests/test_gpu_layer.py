"""Decode-layer epilogues fused around the matvec: RMS norm + activation quantizer, and gate/up
with the activation function (the reference's GPU path fuses the same steps:
crates/ojas-cuda/src/kernels/gemv.rs:37-53, gemv_q8.rs:246-260).  Oracles: `rmsnorm`
(crates/ojas-cpu/src/cpu_math.rs:456-460), `quant_q8k` (:539-563), `silu` / `gelu` (:486, :497-501)
over `matvec_kq`.
"""
import numpy as np
import pytest

from conftest import peak_err

pytestmark = pytest.mark.gpu
Q4_K = 12
TOL = 1e-3
TOL_SEEN = 5e-5


@pytest.mark.parametrize("m,k", [(1, 4096), (3, 2560), (2, 300), (1, 14336), (5, 256)])
def test_rmsnorm_quantizer(gpu, orc, pkg, m, k):
    x = (pkg.synth.normal_f32(m * k, "layer", "x", m, k) * 3.0).reshape(m, k)
    gamma = 1.0 + 0.1 * pkg.synth.normal_f32(k, "layer", "g", k)
    eps = 1e-6
    nsb = (k + 255) // 256
    q, s, xn = gpu.alloc_bytes(m * nsb * 256), gpu.alloc(m * nsb), gpu.alloc(m * k)
    gpu.rmsnorm_quant_q8k(gpu.upload(x), gpu.upload(gamma), eps, m, k, q, s, xn)
    gxn = gpu.read(xn, m * k).reshape(m, k)
    gq = gpu.read(q, m * nsb * 256, np.int8).reshape(m, -1)
    gs = gpu.read(s, m * nsb).reshape(m, -1)
    for t in range(m):
        want = orc.rmsnorm(x[t], gamma, eps)
        # the normalized row: the reference's f32 running sum of k squares carries ~k * 2^-25 of relative
        # error, the kernel sums in f64 — every element moves by the same few ulps through 1/sqrt
        assert np.max(np.abs(gxn[t] - want)) <= 2e-6 * np.max(np.abs(want))
        # the quantizer half is exact: quant_q8k of the row the GPU produced gives the GPU's codes
        ws, wq, _ = orc.quant_q8k(gxn[t])
        assert np.array_equal(gs[t], ws) and np.array_equal(gq[t, :wq.size], wq)
        assert np.all(gq[t, k:] == 0)
    # without the f32 copy
    q2, s2 = gpu.alloc_bytes(m * nsb * 256), gpu.alloc(m * nsb)
    gpu.rmsnorm_quant_q8k(gpu.upload(x), gpu.upload(gamma), eps, m, k, q2, s2)
    assert np.array_equal(gpu.read(q2, m * nsb * 256, np.int8).reshape(m, -1), gq)
    assert np.array_equal(gpu.read(s2, m * nsb).reshape(m, -1), gs)


@pytest.mark.parametrize("act", [0, 1])
@pytest.mark.parametrize("n,k", [(50, 256), (1000, 4096), (333, 2560)])
def test_gate_up_with_activation(gpu, orc, pkg, n, k, act):
    wg = pkg.synth.q4k_weights(n, k, "layer", "wg", n, k)
    wu = pkg.synth.q4k_weights(n, k, "layer", "wu", n, k)
    x = pkg.synth.normal_f32(k, "layer", "gx", k)
    xq, xs = gpu.alloc_bytes(k), gpu.alloc(k // 256)
    gpu.quant_q8k(gpu.upload(x), 1, k, xq, xs)
    out = gpu.upload(np.full(n + 4, 55.5, np.float32))
    gpu.ffn_gu_q8k(xq, xs, gpu.lin(Q4_K, n, k, wg), gpu.lin(Q4_K, n, k, wu), out, act)
    got = gpu.read(out, n + 4)
    assert np.all(got[n:] == 55.5)
    want = orc.ffn_act(orc.matvec_kq(wg, Q4_K, n, k, x), act) * orc.matvec_kq(wu, Q4_K, n, k, x)
    assert peak_err(got[:n], want) <= TOL_SEEN


def test_ffn_block_against_the_cpu_path(gpu, orc, pkg):
    """norm -> gate/up + SiLU -> down accumulated onto the residual: four launches against the
    composition of the CPU path's functions."""
    d, nff = 1024, 2816 - 2816 % 256
    wg = pkg.synth.q4k_weights(nff, d, "blk", "g")
    wu = pkg.synth.q4k_weights(nff, d, "blk", "u")
    wd = pkg.synth.q4k_weights(d, nff, "blk", "d")
    x = pkg.synth.normal_f32(d, "blk", "x")
    gamma = 1.0 + 0.1 * pkg.synth.normal_f32(d, "blk", "gm")
    xq, xs = gpu.alloc_bytes(d), gpu.alloc(d // 256)
    gpu.rmsnorm_quant_q8k(gpu.upload(x), gpu.upload(gamma), 1e-5, 1, d, xq, xs)
    act = gpu.alloc(nff)
    gpu.ffn_gu_q8k(xq, xs, gpu.lin(Q4_K, nff, d, wg), gpu.lin(Q4_K, nff, d, wu), act)
    y = gpu.upload(x)   # the residual stream
    gpu.mm(act, gpu.lin(Q4_K, d, nff, wd), y, 1, True, act_mode=pkg.ACT_Q8K)
    xn = orc.rmsnorm(x, gamma, 1e-5)
    a = orc.ffn_act(orc.matvec_kq(wg, Q4_K, nff, d, xn)) * orc.matvec_kq(wu, Q4_K, nff, d, xn)
    want = orc.matvec_kq(wd, Q4_K, d, nff, a)
    assert peak_err(gpu.read(y, d) - x, want) <= 3e-4 <= TOL


def test_errors(gpu, pkg):
    k = 256
    x, g = gpu.alloc(k), gpu.alloc(k)
    q, s = gpu.alloc_bytes(k), gpu.alloc(1)
    with pytest.raises(pkg.OjasHipError, match="out of range"):
        gpu.rmsnorm_quant_q8k(x, g, 1e-6, 1, 20000, q, s)
    with pytest.raises(pkg.OjasHipError, match="needs"):
        gpu.rmsnorm_quant_q8k(x, g, 1e-6, 2, k, q, s)
    a = gpu.lin(Q4_K, 8, 256, pkg.synth.q4k_weights(8, 256, "e", 1))
    b = gpu.lin(Q4_K, 4, 256, pkg.synth.q4k_weights(4, 256, "e", 2))
    with pytest.raises(pkg.OjasHipError, match="gate is"):
        gpu.ffn_gu_q8k(q, s, a, b, gpu.alloc(8))
    with pytest.raises(pkg.OjasHipError, match="act="):
        gpu.ffn_gu_q8k(q, s, a, a, gpu.alloc(8), act=3)


Q5_K, Q6_K = 13, 14


def _kq_weights(pkg, ty, n, k, *tag):
    gen = {Q4_K: pkg.synth.q4k_weights, Q5_K: pkg.synth.q5k_weights, Q6_K: pkg.synth.q6k_weights}[ty]
    return gen(n, k, "layer-kq", *tag)


@pytest.mark.parametrize("act", [0, 1])
@pytest.mark.parametrize("tg,tu", [(Q6_K, Q6_K), (Q5_K, Q5_K), (Q4_K, Q6_K), (Q5_K, Q4_K)])
@pytest.mark.parametrize("n,k", [(50, 256), (1001, 4096), (333, 2560)])
def test_gate_up_with_activation_in_the_other_k_quants(gpu, orc, pkg, n, k, tg, tu, act):
    """`ojh_ffn_gu_q8k` over Q5_K / Q6_K / mixed tensors (the reference fuses gate/up for every format it decodes
    with, crates/ojas-cuda/src/kernels/gemv_q8.rs:105-143): the CPU path's dots, and bit for bit the product of the
    two single-tensor matvecs."""
    wg, wu = _kq_weights(pkg, tg, n, k, "wg", n, k, tg), _kq_weights(pkg, tu, n, k, "wu", n, k, tu)
    x = pkg.synth.normal_f32(k, "layer-kq", "gx", k)
    xq, xs = gpu.alloc_bytes(k), gpu.alloc(k // 256)
    gpu.quant_q8k(gpu.upload(x), 1, k, xq, xs)
    lg, lu = gpu.lin(tg, n, k, wg), gpu.lin(tu, n, k, wu)
    out = gpu.upload(np.full(n + 4, 55.5, np.float32))
    gpu.ffn_gu_q8k(xq, xs, lg, lu, out, act)
    got = gpu.read(out, n + 4)
    assert np.all(got[n:] == 55.5)
    want = orc.ffn_act(orc.matvec_kq(wg, tg, n, k, x), act) * orc.matvec_kq(wu, tu, n, k, x)
    assert peak_err(got[:n], want) <= TOL_SEEN
    yg, yu = gpu.alloc(n), gpu.alloc(n)
    gpu.mm_q8k(xq, xs, lg, yg)
    gpu.mm_q8k(xq, xs, lu, yu)
    sep = (orc.ffn_act(gpu.read(yg, n), act) * gpu.read(yu, n)).astype(np.float32)
    assert peak_err(got[:n], sep) <= 1e-6          # the activation function itself runs on the GPU in one, on the host in the other


@pytest.mark.parametrize("types", [(Q4_K, Q4_K, Q6_K), (Q6_K, Q5_K), (Q5_K, Q6_K, Q4_K, Q6_K), (Q6_K, Q6_K)])
@pytest.mark.parametrize("k", [256, 4096, 2304])
def test_mixed_k_quant_stage_is_one_launch_with_each_formats_bits(gpu, orc, pkg, types, k):
    """q/k/v (or any group) of one quantized vector with Q4_K, Q5_K and Q6_K tensors side by side —
    `ojh_mm_q8k_multi` / `ojh_mm_multi`: every output bit for bit what `ojh_mm_q8k` gives for that tensor alone, and
    the CPU path's `matvec_kq` within 2e-5."""
    ns = [300, 129, 64, 1000][:len(types)]
    hs = [_kq_weights(pkg, t, n, k, "mix", i, n, k) for i, (t, n) in enumerate(zip(types, ns))]
    lins = [gpu.lin(t, n, k, h) for t, n, h in zip(types, ns, hs)]
    x = pkg.synth.normal_f32(k, "layer-kq", "mixx", k)
    xd = gpu.upload(x)
    xq, xs = gpu.alloc_bytes(k), gpu.alloc(k // 256)
    gpu.quant_q8k(xd, 1, k, xq, xs)
    ys = [gpu.upload(np.full(n + 2, 9.25, np.float32)) for n in ns]
    gpu.mm_q8k_multi(xq, xs, lins, ys)
    ym = [gpu.upload(np.full(n + 2, 9.25, np.float32)) for n in ns]
    gpu.mm_multi(xd, lins, ym)
    for t, n, h, l, y, y2 in zip(types, ns, hs, lins, ys, ym):
        got = gpu.read(y, n + 2)
        assert np.all(got[n:] == 9.25)
        one = gpu.alloc(n)
        gpu.mm_q8k(xq, xs, l, one)
        assert np.array_equal(got[:n].view(np.uint32), gpu.read(one, n).view(np.uint32)), (t, n)
        assert np.array_equal(gpu.read(y2, n + 2).view(np.uint32), got.view(np.uint32))
        assert peak_err(got[:n], orc.matvec_kq(h, t, n, k, x)) <= 2e-5
