"""A seeded sweep over what `ojh_mm` can be asked: formats, row counts on both sides of every routing
threshold (tiles per CU, output heads), K from one super-block to 14336, 1 to 40 tokens, plain and
accumulating stores.  Whatever entry the router picks, every token must match the CPU reference's
`matvec_kq` (int8-activation contract; f32 activations for Q8_0, the IQ4 types and the legacy blocks), nothing may be
written past the last token, and a token's result must not depend on the batch it came in."""
import numpy as np
import pytest

from conftest import peak_err

pytestmark = pytest.mark.gpu
Q8_0, Q4_K, Q5_K, Q6_K, IQ4_NL, IQ4_XS = 8, 12, 13, 14, 20, 23
Q4_0, Q4_1, Q5_0, Q5_1 = 2, 3, 6, 7
Q2_K, Q3_K = 10, 11
IQ2_XXS, IQ2_XS, IQ3_XXS, IQ1_S, IQ3_S, IQ2_S, IQ1_M = 16, 17, 18, 19, 21, 22, 29
MXFP4 = 139
FLOAT_ROWS = (Q8_0, IQ4_NL, IQ4_XS, Q4_0, Q4_1, Q5_0, Q5_1, Q2_K, Q3_K, IQ3_S, IQ2_S, IQ2_XS, IQ1_S, IQ1_M, MXFP4)
LEGACY = (Q4_0, Q4_1, Q5_0, Q5_1, Q2_K, Q3_K, IQ2_XS, IQ1_S, IQ1_M, MXFP4)   # no dot in the CPU path: GPU-path formats


def _cases():
    g = np.random.default_rng(20240611)
    rows = [17, 130, 1000, 4099, 6144, 8200, 14336, 24576, 33000, 40001]
    ks = [256, 512, 1024, 2560, 4096, 5120, 7168, 14336]
    out = []
    for ty in (Q4_K, Q6_K, Q5_K, Q8_0, IQ4_NL, IQ4_XS, Q4_0, Q4_1, Q5_0, Q5_1, Q2_K, Q3_K,
               IQ2_XXS, IQ3_XXS, IQ3_S, IQ2_S, IQ2_XS, IQ1_S, IQ1_M, MXFP4):     # (new formats go last: the draws before them stay)
        for _ in range(7 if ty not in LEGACY and ty not in (IQ3_S, IQ2_S) else 3):
            n, k = int(g.choice(rows)), int(g.choice(ks))
            m = int(g.choice([1, 2, 3, 4, 5, 7, 8, 9, 16, 17, 33, 40]))
            while n * k * m > 6.0e9 or n * k > 2.4e8:      # keep the oracle side to a second or so
                n, m = max(17, n // 2), max(1, m // 2)
            out.append((ty, n, k, m, bool(g.integers(0, 2))))
    return out


@pytest.mark.parametrize("ty,n,k,m,accum", _cases())
def test_router_sweep(gpu, orc, pkg, ty, n, k, m, accum):
    w = pkg.synth.weights(ty, n, k, "sweep", ty, n, k)
    x = pkg.synth.normal_f32(m * k, "sweep", "x", ty, n, k, m).reshape(m, k)
    y0 = pkg.synth.normal_f32(m * n, "sweep", "y0", n, m).reshape(m, n) if accum else np.zeros((m, n), np.float32)
    lin = gpu.lin(ty, n, k, w)
    yd = gpu.upload(np.concatenate([y0.ravel(), np.full(16, 4242.5, np.float32)]))
    gpu.mm(gpu.upload(x), lin, yd, m, accum, act_mode=pkg.ACT_AUTO if m < 32 else
           (pkg.ACT_FLOAT if ty in FLOAT_ROWS else pkg.ACT_Q8K))
    got = gpu.read(yd, m * n + 16)
    assert np.all(got[m * n:] == 4242.5), "wrote past the last token"
    got = got[:m * n].reshape(m, n) - y0
    tol = 1e-5 if ty in FLOAT_ROWS else 2e-5
    # Q8_0 under OJH_ACT_AUTO from 4 tokens (6 on matrices below 32 Mi weights): the f16 MFMA tile, activations rounded
    # to f16 (its own contract, the one the reference's GPU path switches to from 8 rows)
    tile = ty == Q8_0 and m >= (4 if n * k >= (32 << 20) else 6)
    # formats with matvecs only: from 5 tokens (9 on matrices below 32 Mi weights) decoded into scratch and run on the
    # f16 tile (IQ2_XXS / IQ3_XXS keep the int8 kernels where OJH_ACT_Q8K is asked for: here from 32 tokens)
    # (IQ4_NL / IQ4_XS, Q4_0 .. Q5_1, MXFP4, Q2_K and Q3_K rows, which the tile reads through loaders of its own, from 5 tokens on
    # every shape)
    own = ty in (20, 23, 2, 3, 6, 7, 139, 10, 11) and (ty not in (23, 10, 11) or k % 256 == 0) and (ty != 11 or m <= 128)
    if ty not in (Q8_0, Q4_K, Q5_K, Q6_K) and k % 64 == 0 and m >= (5 if own or n * k >= (32 << 20) else 9) and (m < 32 or ty in FLOAT_ROWS):
        tile = True
    if tile:
        tol = 2e-3
    scale = 1.0 + (float(np.max(np.abs(y0))) if accum else 0.0)   # accumulating onto y0 rounds at y0's magnitude
    for t in sorted({0, m // 2, m - 1}):
        # (the CPU path has no dot for the legacy blocks: the reference runs them on its GPU path, f32
        # activations against the dequantized weights, which is what the f64 reference evaluates)
        want = orc.matmul_ref(w, ty, n, k, x[t])[0] if ty in LEGACY or (tile and ty != Q8_0) else orc.matvec_kq(w, ty, n, k, x[t])
        assert peak_err(got[t], want) <= tol * max(1.0, scale * 4.0 / max(1e-30, float(np.max(np.abs(want))))), (t,)
    if m > 1 and not accum and not tile:
        # the middle token alone: the one-token kernels associate their f32 sums differently (last ulps)
        y1 = gpu.alloc(n)
        gpu.mm(gpu.upload(x[m // 2].copy()), lin, y1, 1)
        assert peak_err(gpu.read(y1, n), got[m // 2]) <= 4e-6
