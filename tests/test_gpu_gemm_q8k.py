"""Q4_K rows against batches of tokens on the int8 matrix cores (`gemm_q8k_q4k_mf`): the CPU
reference's arithmetic at verify and prefill sizes — every token against matvec_kq
(crates/ojas-cpu/src/cpu_math.rs:1145-1189), the same bar as the one-token kernels."""
import numpy as np
import pytest

from conftest import peak_err

pytestmark = pytest.mark.gpu
Q4_K = 12
TOL_SEEN = 2e-5


def _case(pkg, m, n, k, tag):
    w = pkg.synth.q4k_weights(n, k, "gq", tag, n, k)
    x = pkg.synth.normal_f32(m * k, "gq", tag, "x", m, k).reshape(m, k)
    x[0, :256] = 0.0                      # an all-zero segment: scale 1
    return w, x


@pytest.mark.parametrize("m,n,k,accum", [(2, 50, 256, False), (16, 130, 4096, True), (17, 333, 2560, False),
                                         (40, 64, 14336, True), (128, 100, 1024, False), (129, 300, 512, False),
                                         (300, 40, 4096, True), (8, 4099, 4096, False), (64, 17, 8192, False),
                                         (130, 6200, 512, True),
                                         # the 128-token tile in K slices below 128 tokens: from 17 tokens where K >= 2 N, from 33 otherwise
                                         (20, 1030, 4096, True), (33, 2100, 2048, False), (64, 4096, 4096, False)])
def test_router_path_matches_the_cpu_reference(gpu, orc, pkg, m, n, k, accum):
    w, x = _case(pkg, m, n, k, "a")
    lin = gpu.lin(Q4_K, n, k, w)
    y0 = pkg.synth.normal_f32(m * n, "gq", "y0", m, n).reshape(m, n) if accum else np.zeros((m, n), np.float32)
    yd = gpu.upload(np.concatenate([y0.ravel(), np.full(n, 4242.5, np.float32)]))
    gpu.mm(gpu.upload(x), lin, yd, m, accum, act_mode=pkg.ACT_Q8K)
    got = gpu.read(yd, m * n + n)
    assert np.all(got[m * n:] == 4242.5), "wrote past the last token"
    want = np.stack([orc.matvec_kq(w, Q4_K, n, k, x[t]) for t in range(m)])
    assert peak_err(got[:m * n].reshape(m, n) - y0, want) <= TOL_SEEN


@pytest.mark.parametrize("m,n,k", [(5, 70, 4096), (33, 200, 2048), (100, 48, 14336), (128, 64, 512)])
def test_every_row_tiling_and_the_integer_dot_kernel_agree(gpu, orc, pkg, m, n, k):
    """By name: RW = 1, 2, 4 row tiles per workgroup (4, 2, 1 waves on K) where the tokens' chunk
    allows it, and `gemv_q8k_q4k_m` on the same quantized activations.  Integer sums are exact in
    all of them; the f32 sums over super-blocks associate differently."""
    w, x = _case(pkg, m, n, k, "b")
    gpu.ensure_family("gemm_q8k")
    gpu.ensure_family("gemv_q8k")
    nsb = k // 256
    xq, xs = gpu.alloc_bytes(m * k), gpu.alloc(m * nsb)
    gpu.quant_q8k(gpu.upload(x), m, k, xq, xs)
    wd = gpu.upload_bytes(w)
    want = np.stack([orc.matvec_kq(w, Q4_K, n, k, x[t]) for t in range(m)])
    y = gpu.alloc(m * n)
    gpu.dispatch(gpu.begin(), "gemv_q8k_q4k_m", [(xq, 0), (xs, 0), (wd, 0), (y, 0)], [k, n, m, 0],
                 [(n + 3) // 4, 1, 1], [256, 1, 1])
    dots = gpu.read(y, m * n).reshape(m, n)
    ran = 0
    for rw in (1, 2, 4):
        grid = [(n + 16 * rw - 1) // (16 * rw), (m + 63) // 64, 1]
        y = gpu.upload(np.full(m * n, 7.0, np.float32))
        try:
            gpu.dispatch(gpu.begin(), "gemm_q8k_q4k_mf", [(xq, 0), (xs, 0), (wd, 0), (y, 0)], [k, n, m, 0, rw, 1], grid,
                         [256, 1, 1])
        except pkg.OjasHipError as e:
            assert "super-blocks" in str(e)            # the chunk is too short for that many waves on K
            continue
        got = gpu.read(y, m * n).reshape(m, n)
        assert peak_err(got, want) <= TOL_SEEN, rw
        assert peak_err(got, dots) <= 2e-6, rw
        ran += 1
    assert ran >= 1
    with pytest.raises(pkg.OjasHipError, match="RT"):
        gpu.dispatch(gpu.begin(), "gemm_q8k_q4k_mf", [(xq, 0), (xs, 0), (wd, 0), (y, 0)], [k, n, m, 0, 4, 4],
                     [(n + 255) // 256, (m + 63) // 64, 1], [256, 1, 1])
    with pytest.raises(pkg.OjasHipError, match="RW"):
        gpu.dispatch(gpu.begin(), "gemm_q8k_q4k_mf", [(xq, 0), (xs, 0), (wd, 0), (y, 0)], [k, n, m, 0, 3, 1],
                     [(n + 47) // 48, (m + 63) // 64, 1], [256, 1, 1])
    with pytest.raises(pkg.OjasHipError, match="grid"):
        gpu.dispatch(gpu.begin(), "gemm_q8k_q4k_mf", [(xq, 0), (xs, 0), (wd, 0), (y, 0)], [k, n, m, 0, 4, 1], [100000, 1, 1],
                     [256, 1, 1])


@pytest.mark.parametrize("m,n,k,accum,grid_x,block_x", [(2, 50, 256, False, None, 512), (16, 130, 4096, True, 3, 512),
                                                        (9, 301, 4096, False, 2, 256), (16, 1000, 5120, False, 7, 512),
                                                        (1, 17, 512, True, None, 64), (5, 4099, 2560, False, None, 512),
                                                        (8, 77, 1024, True, 1, 128)])
def test_rows_copied_through_lds_by_name(gpu, orc, pkg, m, n, k, accum, grid_x, block_x):
    """`gemm_q8k_q4k_ml`, up to 16 tokens: against matvec_kq per token and, bit for bit, against
    `gemm_q8k_q4k_mf` with four row tiles per workgroup (no wave splits K there either, so the same
    sums in the same order).  Small grids make a wave walk many tiles: its copy ring wraps and runs
    ahead across tile borders; the last row ends exactly at the end of the weight buffer."""
    w, x = _case(pkg, m, n, k, "ml")
    y0 = pkg.synth.normal_f32(m * n, "gq", "ml-y0", m, n).reshape(m, n) if accum else np.zeros((m, n), np.float32)
    want = np.stack([orc.matvec_kq(w, Q4_K, n, k, x[t]) for t in range(m)])
    gpu.ensure_family("gemm_q8k")
    nsb = k // 256
    xq, xs = gpu.alloc_bytes(m * k), gpu.alloc(m * nsb)
    gpu.quant_q8k(gpu.upload(x), m, k, xq, xs)
    wd = gpu.upload_bytes(w)
    grid, block = gpu.launch_shape("gemm_q8k_q4k_ml", k, n, m)
    assert block == [512, 1, 1]
    grid, block = [grid_x or grid[0], 1, 1], [block_x, 1, 1]
    yd = gpu.upload(np.concatenate([y0.ravel(), np.full(8, 4242.5, np.float32)]))
    gpu.dispatch(gpu.begin(), "gemm_q8k_q4k_ml", [(xq, 0), (xs, 0), (wd, 0), (yd, 0)], [k, n, m, int(accum)], grid, block)
    got = gpu.read(yd, m * n + 8)
    assert np.all(got[m * n:] == 4242.5), "wrote past the last token"
    got = got[:m * n].reshape(m, n) - y0
    assert peak_err(got, want) <= TOL_SEEN
    y2 = gpu.upload(y0)
    gpu.dispatch(gpu.begin(), "gemm_q8k_q4k_mf", [(xq, 0), (xs, 0), (wd, 0), (y2, 0)], [k, n, m, int(accum), 4, 1],
                 [(n + 63) // 64, 1, 1], [256, 1, 1])
    assert np.array_equal(got, gpu.read(y2, m * n).reshape(m, n) - y0)
    for consts, what in (([k, n, 17, 0], "do not fit"), ([8192, n, 4, 0], "do not fit")):
        with pytest.raises(pkg.OjasHipError, match=what):
            gpu.dispatch(gpu.begin(), "gemm_q8k_q4k_ml", [(xq, 0), (xs, 0), (wd, 0), (yd, 0)], consts, [8, 1, 1], [512, 1, 1])


@pytest.mark.parametrize("m,n,k,accum,grid_x", [(2, 50, 256, False, None), (16, 130, 4096, True, 3), (9, 301, 14336, False, None),
                                                (16, 100, 8192, False, 2), (5, 4099, 2560, True, None)])
def test_k_split_over_the_waves_by_name(gpu, orc, pkg, m, n, k, accum, grid_x):
    """`gemm_q8k_q4k_mk`: a workgroup per 16-row tile, super-blocks dealt to its eight waves, partial
    sums added in wave order; token rows past M are a shared block of zeros."""
    w, x = _case(pkg, m, n, k, "mk")
    y0 = pkg.synth.normal_f32(m * n, "gq", "mk-y0", m, n).reshape(m, n) if accum else np.zeros((m, n), np.float32)
    want = np.stack([orc.matvec_kq(w, Q4_K, n, k, x[t]) for t in range(m)])
    gpu.ensure_family("gemm_q8k")
    nsb = k // 256
    xq, xs = gpu.alloc_bytes(m * k), gpu.alloc(m * nsb)
    gpu.quant_q8k(gpu.upload(x), m, k, xq, xs)
    wd = gpu.upload_bytes(w)
    grid, block = gpu.launch_shape("gemm_q8k_q4k_mk", k, n, m)
    grid = [grid_x or grid[0], 1, 1]
    yd = gpu.upload(np.concatenate([y0.ravel(), np.full(8, 4242.5, np.float32)]))
    gpu.dispatch(gpu.begin(), "gemm_q8k_q4k_mk", [(xq, 0), (xs, 0), (wd, 0), (yd, 0)], [k, n, m, int(accum)], grid, block)
    got = gpu.read(yd, m * n + 8)
    assert np.all(got[m * n:] == 4242.5), "wrote past the last token"
    assert peak_err(got[:m * n].reshape(m, n) - y0, want) <= TOL_SEEN
    with pytest.raises(pkg.OjasHipError, match="do not fit"):
        gpu.dispatch(gpu.begin(), "gemm_q8k_q4k_mk", [(xq, 0), (xs, 0), (wd, 0), (yd, 0)], [14336, n, 12, 0], [8, 1, 1], [512, 1, 1])
    with pytest.raises(pkg.OjasHipError, match="block"):
        gpu.dispatch(gpu.begin(), "gemm_q8k_q4k_mk", [(xq, 0), (xs, 0), (wd, 0), (yd, 0)], [k, n, m, 0], [8, 1, 1], [256, 1, 1])


def test_a_token_does_not_depend_on_its_batch(gpu, pkg):
    """The same tokens rolled by 37 positions: every output bit for bit, moved."""
    m, n, k = 200, 512, 4096
    w, x = _case(pkg, m, n, k, "c")
    lin = gpu.lin(Q4_K, n, k, w)
    y1, y2 = gpu.alloc(m * n), gpu.alloc(m * n)
    gpu.mm(gpu.upload(x), lin, y1, m, act_mode=pkg.ACT_Q8K)
    perm = np.roll(np.arange(m), 37)
    gpu.mm(gpu.upload(x[perm].copy()), lin, y2, m, act_mode=pkg.ACT_Q8K)
    assert np.array_equal(gpu.read(y2, m * n).reshape(m, n), gpu.read(y1, m * n).reshape(m, n)[perm])


@pytest.mark.parametrize("m,n,k", [(130, 200, 512), (128, 128, 256), (300, 77, 2048), (97, 1000, 4096)])
def test_prefill_tiles_by_name(gpu, orc, pkg, m, n, k):
    """`q8k_token_sides` + `gemm_q8k_q4k_xt` / `_xt64` by name: ragged tokens and rows, plain store and accumulate,
    nothing written past row M — against matvec_kq and (a few ulp: the min term is associated per 32-position run
    there, per super-block here) against `gemm_q8k_q4k_mf`; the two tile heights give the same bits."""
    w, x = _case(pkg, m, n, k, "xt")
    gpu.ensure_family("gemm_q8k")
    gpu.ensure_family("gemv_q8k")
    nsb, mp = k // 256, (m + 127) // 128 * 128
    xq, xs = gpu.alloc_bytes(m * k), gpu.alloc(m * nsb)
    gpu.quant_q8k(gpu.upload(x), m, k, xq, xs)
    wd = gpu.upload_bytes(w)
    xst, sums = gpu.alloc(nsb * mp), gpu.alloc(nsb * mp * 8)
    gpu.dispatch(gpu.begin(), "q8k_token_sides", [(xq, 0), (xs, 0), (xst, 0), (sums, 0)], [k, m, mp], [nsb, (mp + 255) // 256, 1], [256, 1, 1])
    # the side arrays: scales transposed; scale x the sum of every 32-position run, runs in the order 0 4 1 5 2 6 3 7;
    # zeros past row M
    q = gpu.read(xq, m * k, np.int8).reshape(m, nsb, 8, 32).astype(np.int32).sum(3)
    st = gpu.read(xst, nsb * mp).reshape(nsb, mp)
    assert np.array_equal(st[:, :m], gpu.read(xs, m * nsb).reshape(m, nsb).T) and not st[:, m:].any()
    sd = gpu.read(sums, nsb * mp * 8).reshape(nsb, mp, 8)
    scaled = st[:, :m, None] * q.transpose(1, 0, 2)[:, :, [0, 4, 1, 5, 2, 6, 3, 7]].astype(np.float32)
    assert np.array_equal(sd[:, :m].view(np.uint32), scaled.astype(np.float32).view(np.uint32)) and not sd[:, m:].any()
    # the quantizer that leaves the side arrays as well: the same bytes in all four outputs, from f32 and from bf16 tokens
    xb = (x.view(np.uint32) >> 16).astype(np.uint16)
    for name, src in (("quantize_q8k_sides", gpu.upload(x)), ("quantize_q8k_bf16_sides", gpu.upload_bytes(xb))):
        q2, s2 = gpu.alloc_bytes(m * k), gpu.alloc(m * nsb)
        xst2 = gpu.upload(np.full(nsb * mp, 7.5, np.float32))
        sums2 = gpu.upload(np.full(nsb * mp * 8, 7.5, np.float32))
        gpu.dispatch(gpu.begin(), name, [(src, 0), (q2, 0), (s2, 0), (xst2, 0), (sums2, 0)], [k, m, mp], [nsb * mp // 4, 1, 1], [256, 1, 1])
        if "bf16" in name:
            q1, s1 = gpu.alloc_bytes(m * k), gpu.alloc(m * nsb)
            gpu.quant_q8k(gpu.upload((xb.astype(np.uint32) << 16).view(np.float32)), m, k, q1, s1)
            xst1, sums1 = gpu.alloc(nsb * mp), gpu.alloc(nsb * mp * 8)
            gpu.dispatch(gpu.begin(), "q8k_token_sides", [(q1, 0), (s1, 0), (xst1, 0), (sums1, 0)], [k, m, mp], [nsb, (mp + 255) // 256, 1], [256, 1, 1])
        else:
            q1, s1, xst1, sums1 = xq, xs, xst, sums
        assert np.array_equal(gpu.read(q2, m * k, np.int8), gpu.read(q1, m * k, np.int8)), name
        assert np.array_equal(gpu.read(s2, m * nsb).view(np.uint32), gpu.read(s1, m * nsb).view(np.uint32)), name
        assert np.array_equal(gpu.read(xst2, nsb * mp).view(np.uint32), gpu.read(xst1, nsb * mp).view(np.uint32)), name
        assert np.array_equal(gpu.read(sums2, nsb * mp * 8).view(np.uint32), gpu.read(sums1, nsb * mp * 8).view(np.uint32)), name
    with pytest.raises(pkg.OjasHipError, match="rounded up to 128"):
        gpu.dispatch(gpu.begin(), "quantize_q8k_sides", [(gpu.upload(x), 0), (xq, 0), (xs, 0), (xst, 0), (sums, 0)], [k, m, mp + 128],
                     [nsb * (mp + 128) // 4, 1, 1], [256, 1, 1])
    want = np.stack([orc.matvec_kq(w, Q4_K, n, k, x[t]) for t in range(m)])
    ymf = gpu.alloc(m * n)
    gpu.dispatch(gpu.begin(), "gemm_q8k_q4k_mf", [(xq, 0), (xs, 0), (wd, 0), (ymf, 0)], [k, n, m, 0, 4, 1],
                 [(n + 63) // 64, (m + 63) // 64, 1], [256, 1, 1])
    ref, bits = gpu.read(ymf, m * n).reshape(m, n), {}
    for name, br in (("gemm_q8k_q4k_xt", 128), ("gemm_q8k_q4k_xt64", 64)):
        for acc in (0, 1):
            y0 = pkg.synth.normal_f32(m * n, "gq", "xt-y0", acc).reshape(m, n)
            yd = gpu.upload(np.concatenate([y0.ravel(), np.full(n, 4242.5, np.float32)]))
            gpu.dispatch(gpu.begin(), name, [(xq, 0), (xst, 0), (sums, 0), (wd, 0), (yd, 0)], [k, n, m, acc, mp],
                         [(n + br - 1) // br, mp // 128, 1], [512, 1, 1])
            got = gpu.read(yd, m * n + n)
            assert np.all(got[m * n:] == 4242.5), "wrote past the last token"
            got = got[:m * n].reshape(m, n)
            if acc:
                assert peak_err(got - y0, want) <= TOL_SEEN
            else:
                assert peak_err(got, want) <= TOL_SEEN and peak_err(got, ref) <= 2e-6
                bits[name] = got.view(np.uint32).copy()
    assert np.array_equal(bits["gemm_q8k_q4k_xt"], bits["gemm_q8k_q4k_xt64"])
    # the 64-row tile over K slices: one slice gives the unsliced bits; more give the slice sums added in slice order
    # (the same bits on every launch, whoever finishes last), and every launch leaves the tile counters at zero
    tiles = (n + 63) // 64 * (mp // 128)
    cnt = gpu.alloc_bytes(tiles * 4)
    gpu.memset0(cnt)
    for nsplit in sorted({min(s, nsb) for s in (1, 2, 3, nsb)}):
        per = (nsb + nsplit - 1) // nsplit
        slices = (nsb + per - 1) // per
        part = gpu.alloc(tiles * slices * 8192)
        seen = []
        for acc in (0, 1, 0):
            y0 = pkg.synth.normal_f32(m * n, "gq", "xt-y0", acc).reshape(m, n)
            yd = gpu.upload(np.concatenate([y0.ravel(), np.full(n, 4242.5, np.float32)]))
            gpu.dispatch(gpu.begin(), "gemm_q8k_q4k_xt64_sr", [(xq, 0), (xst, 0), (sums, 0), (wd, 0), (yd, 0), (part, 0), (cnt, 0)],
                         [k, n, m, acc, mp, nsplit], [(n + 63) // 64, mp // 128, slices], [512, 1, 1])
            got = gpu.read(yd, m * n + n)
            assert np.all(got[m * n:] == 4242.5), "wrote past the last token"
            assert not gpu.read(cnt, tiles, np.uint32).any()
            got = got[:m * n].reshape(m, n)
            if acc:
                assert peak_err(got - y0, want) <= TOL_SEEN
            else:
                assert peak_err(got, want) <= TOL_SEEN and peak_err(got, ref) <= 2e-6
                seen.append(got.view(np.uint32).copy())
        assert np.array_equal(seen[0], seen[1]), nsplit
        if slices == 1:
            assert np.array_equal(seen[0], bits["gemm_q8k_q4k_xt64"])
    with pytest.raises(pkg.OjasHipError, match="grid must be"):
        gpu.dispatch(gpu.begin(), "gemm_q8k_q4k_xt64_sr", [(xq, 0), (xst, 0), (sums, 0), (wd, 0), (ymf, 0), (part, 0), (cnt, 0)],
                     [k, n, m, 0, mp, 1], [(n + 63) // 64, mp // 128, 2], [512, 1, 1])
    with pytest.raises(pkg.OjasHipError, match="rounded up to 128"):
        gpu.dispatch(gpu.begin(), "gemm_q8k_q4k_xt", [(xq, 0), (xst, 0), (sums, 0), (wd, 0), (ymf, 0)], [k, n, m, 0, mp + 128],
                     [(n + 127) // 128, mp // 128, 1], [512, 1, 1])
