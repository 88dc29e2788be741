"""`ojh_mm_noalloc` — the matmul entry that allocates nothing — against `ojh_mm(..., OJH_ACT_Q8K)`, bit for bit,
on calls in a row that share the static scratch array (the later ones with smaller inputs), and against the
CPU oracle."""
import numpy as np
import pytest

from conftest import peak_err

pytestmark = pytest.mark.gpu
Q4_K, Q5_K, Q6_K, Q8_0 = 12, 13, 14, 8


def _weights(pkg, ty, n, k, tag):
    gen = {Q4_K: pkg.synth.q4k_weights, Q6_K: pkg.synth.q6k_weights}[ty]
    return gen(n, k, "noalloc", tag)


def _both(gpu, pkg, orc, ty, n, k, m, tag, x_dtype=0, accum=False):
    """One call through each entry on the same inputs; returns the no-alloc result after comparing."""
    w = _weights(pkg, ty, n, k, tag)
    lin = gpu.lin(ty, n, k, w)
    x = pkg.synth.normal_f32(m * k, "noalloc", "x" + tag).reshape(m, k)
    if x_dtype == 1:
        bits = pkg.synth.to_bf16_bits(x)
        xd = gpu.upload_bytes(bits)
        x = pkg.synth.bf16_bits_to_f32(bits).reshape(m, k)
    else:
        xd = gpu.upload(x)
    y0 = pkg.synth.normal_f32(m * n, "noalloc", "y" + tag)
    ya, yb = gpu.upload(y0), gpu.upload(y0)
    gpu.mm(xd, lin, ya, m, accum, x_dtype=x_dtype, act_mode=pkg.ACT_Q8K)
    gpu.mm_noalloc(xd, lin, yb, m, accum, x_dtype=x_dtype)
    want_gpu = gpu.read(ya, m * n)
    got = gpu.read(yb, m * n)
    assert np.array_equal(got.view(np.uint32), want_gpu.view(np.uint32)), (ty, n, k, m)
    ref = np.stack([orc.matvec_kq(w, ty, n, k, x[t]) for t in range(m)]).ravel()
    if accum:
        ref = ref + y0
    assert peak_err(got, ref) <= 2e-5, (ty, n, k, m)
    lin.free()
    return got


def test_no_alloc_matches_mm_on_consecutive_calls(gpu, pkg, orc):
    gpu.ensure_family("gemv_q8k")
    gpu.ensure_family("gemm_q8k")
    assert gpu._L.ojh_noalloc_scratch_bytes() == (1 << 20) + (1 << 14)
    # large first, then smaller inputs over the same scratch: stale bytes of the earlier call must not show
    _both(gpu, pkg, orc, Q4_K, 512, 4096, 16, "a")           # int8 matrix-core form
    _both(gpu, pkg, orc, Q4_K, 300, 1024, 1, "b")            # one-token matvec, ragged N
    _both(gpu, pkg, orc, Q4_K, 300, 512, 3, "c")             # per-token loop of the dot kernel
    _both(gpu, pkg, orc, Q6_K, 256, 2048, 4, "d", x_dtype=1)  # bf16 activations, Q6_K few-token form
    _both(gpu, pkg, orc, Q6_K, 130, 256, 1, "e", accum=True)


def test_no_alloc_takes_the_unsliced_prefill_tile(gpu, pkg, orc):
    """Q6_K rows against 40 tokens: `ojh_mm` runs the 128-token tile over K slices that meet in library scratch, the entry
    that allocates nothing runs the same tile whole — the same integer sums, the super-blocks' f32 terms added in one
    pass instead of per slice: equal to rounding, and each within the bar of matvec_kq."""
    gpu.ensure_family("gemv_q8k")
    gpu.ensure_family("gemm_q8k")
    n, k, m = 256, 2048, 40
    w = _weights(pkg, Q6_K, n, k, "tile")
    lin = gpu.lin(Q6_K, n, k, w)
    x = pkg.synth.normal_f32(m * k, "noalloc", "xtile").reshape(m, k)
    xd, ya, yb = gpu.upload(x), gpu.alloc(m * n), gpu.alloc(m * n)
    gpu.mm(xd, lin, ya, m, act_mode=pkg.ACT_Q8K)
    gpu.mm_noalloc(xd, lin, yb, m)
    a, b = gpu.read(ya, m * n), gpu.read(yb, m * n)
    ref = np.stack([orc.matvec_kq(w, Q6_K, n, k, x[t]) for t in range(m)]).ravel()
    assert peak_err(a, ref) <= 2e-5 and peak_err(b, ref) <= 2e-5 and peak_err(a, b) <= 2e-6
    lin.free()


def test_no_alloc_limits_and_errors(gpu, pkg):
    n, k = 64, 4096
    lin = gpu.lin(Q4_K, n, k, _weights(pkg, Q4_K, n, k, "lim"))
    m_max = (1 << 20) // k
    xd, yd = gpu.alloc((m_max + 1) * k), gpu.alloc((m_max + 1) * n)
    gpu.memset0(xd)
    gpu.ensure_family("gemv_q8k")
    gpu.ensure_family("gemm_q8k")
    gpu.mm_noalloc(xd, lin, yd, m_max)                       # exactly the maximum fits
    gpu.submit()
    assert not gpu.read(yd, m_max * n).any()                 # zero activations quantize to zeros
    with pytest.raises(pkg.OjasHipError, match="static scratch holds") as e:
        gpu.mm_noalloc(xd, lin, yd, m_max + 1)
    assert e.value.code == -5
    q80 = gpu.lin(Q8_0, 32, 64, pkg.synth.q80_weights(32, 64, "noalloc", "q80"))
    with pytest.raises(pkg.OjasHipError, match="ojh_mm") as e:
        gpu.mm_noalloc(xd, q80, yd, 1)
    assert e.value.code == -4
    # a handle whose families are not resident is told to load them first instead of loading (= allocating)
    other = pkg.HipGpu(0)
    try:
        lin2 = other.lin(Q4_K, n, k, _weights(pkg, Q4_K, n, k, "lim"))
        x2, y2 = other.alloc(k), other.alloc(n)
        with pytest.raises(pkg.OjasHipError, match="ensure_family") as e:
            other.mm_noalloc(x2, lin2, y2, 1)
        assert e.value.code == -3
        lin2.free()
    finally:
        other.close()


def test_no_alloc_records_where_every_allocation_is_refused(pkg):
    """While a chain of launches is being recorded the library refuses to allocate (scratch that would have to grow,
    code objects that would have to load: OJH_ERR_ARG).  `ojh_mm_noalloc` must go through there on a handle whose
    scratch no earlier call has sized (a handle of its own: the other tests' calls cannot have grown it), `ojh_mm` on
    the same shapes must be refused, and the replay must give the bits of an eager `ojh_mm`."""
    gpu = pkg.HipGpu(0)
    try:
        gpu.ensure_family("gemv_q8k")
        gpu.ensure_family("gemm_q8k")
        n, k, m = 768, 8192, 96
        lin = gpu.lin(Q4_K, n, k, _weights(pkg, Q4_K, n, k, "rec"))
        xd = gpu.upload(pkg.synth.normal_f32(m * k, "noalloc", "xrec"))
        ya, yb = gpu.alloc(m * n), gpu.alloc(m * n)
        gpu.capture_begin()
        try:
            with pytest.raises(pkg.OjasHipError):
                gpu.mm(xd, lin, ya, m, act_mode=pkg.ACT_Q8K)       # would have to allocate the library's scratch
            gpu.mm_noalloc(xd, lin, yb, m)
        finally:
            graph = gpu.capture_end()
        graph.launch()
        gpu.submit()
        gpu.mm(xd, lin, ya, m, act_mode=pkg.ACT_Q8K)
        assert np.array_equal(gpu.read(yb, m * n).view(np.uint32), gpu.read(ya, m * n).view(np.uint32))
    finally:
        gpu.close()
