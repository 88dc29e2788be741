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
