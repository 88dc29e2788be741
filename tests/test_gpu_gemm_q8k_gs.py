"""Q6_K and Q5_K rows against batches of 5 to hundreds of tokens in the CPU path's arithmetic (`gemm_q8k_{q6k,q5k}_gs{,_sr}`):
every token against matvec_kq (crates/ojas-cpu/src/cpu_math.rs:638-722, :1145-1189), the bar of the few-token kernels."""
import numpy as np
import pytest

from conftest import peak_err

pytestmark = pytest.mark.gpu
Q5_K, Q6_K = 13, 14
TOL_SEEN = 2e-5
FMT = {Q6_K: "q6k", Q5_K: "q5k"}


def _case(pkg, ty, m, n, k, tag):
    gen = {Q6_K: pkg.synth.q6k_weights, Q5_K: pkg.synth.q5k_weights}[ty]
    w = gen(n, k, "gs", tag, n, k)
    x = pkg.synth.normal_f32(m * k, "gs", tag, "x", m, k).reshape(m, k)
    x[0, :256] = 0.0                      # an all-zero segment: scale 1
    x[m - 1, -256:] *= 40.0               # and one whose sub-block sums reach far
    return w, x


@pytest.mark.parametrize("ty", [Q6_K, Q5_K])
@pytest.mark.parametrize("m,n,k", [(17, 100, 512), (128, 64, 256), (130, 77, 2048), (300, 1000, 1024), (33, 130, 768)])
def test_tiles_by_name(gpu, orc, pkg, ty, m, n, k):
    """Ragged tokens and rows, plain store and accumulate, nothing written past row M; K slices: one slice gives the
    unsliced bits, more give the same bits on every launch and leave the tile counters at zero."""
    w, x = _case(pkg, ty, m, n, k, "name")
    gpu.ensure_family("gemm_q8k")
    gpu.ensure_family("gemv_q8k")
    nsb = k // 256
    xq, xs = gpu.alloc_bytes(m * k), gpu.alloc(m * nsb)
    gpu.quant_q8k(gpu.upload(x), m, k, xq, xs)
    wd = gpu.upload_bytes(w)
    want = np.stack([orc.matvec_kq(w, ty, n, k, x[t]) for t in range(m)])
    name = f"gemm_q8k_{FMT[ty]}_gs"
    grid = [(n + 127) // 128, (m + 63) // 64, 1]
    plain = None
    for acc in (0, 1):
        y0 = pkg.synth.normal_f32(m * n, "gs", "y0", acc).reshape(m, n)
        yd = gpu.upload(np.concatenate([y0.ravel(), np.full(n, 4242.5, np.float32)]))
        gpu.dispatch(gpu.begin(), name, [(xq, 0), (xs, 0), (wd, 0), (yd, 0)], [k, n, m, acc], grid, [256, 1, 1])
        got = gpu.read(yd, m * n + n)
        assert np.all(got[m * n:] == 4242.5), "wrote past the last token"
        got = got[:m * n].reshape(m, n)
        if acc:
            assert peak_err(got - y0, want) <= TOL_SEEN
        else:
            assert peak_err(got, want) <= TOL_SEEN
            plain = got.view(np.uint32).copy()
    tiles = grid[0] * grid[1]
    cnt = gpu.alloc_bytes(tiles * 4)
    gpu.memset0(cnt)
    for nsplit in sorted({min(s, nsb) for s in (1, 2, 3, nsb)}):
        per = (nsb + nsplit - 1) // nsplit
        slices = (nsb + per - 1) // per
        part = gpu.alloc(tiles * slices * 8192)
        seen = []
        for acc in (0, 1, 0):
            y0 = pkg.synth.normal_f32(m * n, "gs", "y0", acc).reshape(m, n)
            yd = gpu.upload(np.concatenate([y0.ravel(), np.full(n, 4242.5, np.float32)]))
            gpu.dispatch(gpu.begin(), name + "_sr", [(xq, 0), (xs, 0), (wd, 0), (yd, 0), (part, 0), (cnt, 0)],
                         [k, n, m, acc, nsplit], [grid[0], grid[1], slices], [256, 1, 1])
            got = gpu.read(yd, m * n + n)
            assert np.all(got[m * n:] == 4242.5), "wrote past the last token"
            assert not gpu.read(cnt, tiles, np.uint32).any()
            got = got[:m * n].reshape(m, n)
            if acc:
                assert peak_err(got - y0, want) <= TOL_SEEN
            else:
                assert peak_err(got, want) <= TOL_SEEN
                seen.append(got.view(np.uint32).copy())
        assert np.array_equal(seen[0], seen[1]), nsplit
        if slices == 1:
            assert np.array_equal(seen[0], plain)
    with pytest.raises(pkg.OjasHipError, match="grid must be"):
        gpu.dispatch(gpu.begin(), name, [(xq, 0), (xs, 0), (wd, 0), (gpu.alloc(m * n), 0)], [k, n, m, 0],
                     [grid[0] + 1, grid[1], 1], [256, 1, 1])


@pytest.mark.parametrize("ty", [Q6_K, Q5_K])
@pytest.mark.parametrize("m,n,k,accum", [(17, 333, 2560, False), (40, 64, 14336, True), (129, 300, 512, False),
                                         (64, 4096, 4096, False), (300, 40, 4096, True)])
def test_router_path_matches_the_cpu_reference(gpu, orc, pkg, ty, m, n, k, accum):
    """Through `ojh_mm(..., OJH_ACT_Q8K)`: whole tiles and K slices as the library picks them, f32 and bf16 tokens."""
    w, x = _case(pkg, ty, m, n, k, "route")
    lin = gpu.lin(ty, n, k, w)
    y0 = pkg.synth.normal_f32(m * n, "gs", "y0r", m, n).reshape(m, n) if accum else np.zeros((m, n), np.float32)
    yd = gpu.upload(np.concatenate([y0.ravel(), np.full(n, 4242.5, np.float32)]))
    gpu.mm(gpu.upload(x), lin, yd, m, accum, act_mode=pkg.ACT_Q8K)
    got = gpu.read(yd, m * n + n)
    assert np.all(got[m * n:] == 4242.5), "wrote past the last token"
    want = np.stack([orc.matvec_kq(w, ty, n, k, x[t]) for t in range(m)])
    assert peak_err(got[:m * n].reshape(m, n) - y0, want) <= TOL_SEEN
    # a token's result does not depend on its batch: the same rows, one token at a time
    one = gpu.alloc(n)
    for t in (0, m - 1):
        gpu.mm(gpu.upload(x[t]), lin, one, 1, act_mode=pkg.ACT_Q8K)
        assert peak_err(gpu.read(one, n), got[t * n:(t + 1) * n] - y0[t]) <= TOL_SEEN
    lin.free()
