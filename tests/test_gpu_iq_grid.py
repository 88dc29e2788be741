"""The grid-codebook GGUF formats on the GPU (family "iq_grid"): decoders bit for bit against the reference's digests
and the oracle, the f32-activation matvecs by name and through `mm`, the int8-activation matvecs of IQ2_XXS / IQ3_XXS
against `matvec_kq` — the CPU path's routing of these types (crates/ojas-cpu/src/cpu_math.rs:1174-1181)."""
import json
import os

import numpy as np
import pytest

from conftest import peak_err

pytestmark = pytest.mark.gpu
IQ2_XXS, IQ2_XS, IQ3_XXS, IQ1_S, IQ3_S, IQ2_S, IQ1_M = 16, 17, 18, 19, 21, 22, 29
GRID = [IQ2_XXS, IQ2_XS, IQ3_XXS, IQ1_S, IQ3_S, IQ2_S, IQ1_M]
TAG = {IQ2_XXS: "iq2xxs", IQ2_XS: "iq2xs", IQ3_XXS: "iq3xxs", IQ1_S: "iq1s", IQ3_S: "iq3s", IQ2_S: "iq2s", IQ1_M: "iq1m"}
with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "quant_format_digests.json")) as _f:
    DIGESTS = {int(ty): int(row["digest"], 16) for ty, row in json.load(_f)["digests"].items()}


def _dequant(gpu, ty, raw, n):
    out = gpu.alloc_bytes(n * 2)
    gpu.dequant_f16(ty, gpu.upload_bytes(raw), n, out)
    return gpu.read(out, n, np.uint16)


@pytest.mark.parametrize("ty", GRID)
def test_reference_digests_on_device(gpu, orc, ty):
    """crates/ojas-formats/tests/quant_formats.rs:41-44,46-47,49 over what the GPU decoded."""
    bits = _dequant(gpu, ty, orc.synth_blocks(ty, 40), 40 * 256)
    assert orc.digest_f16(bits) == DIGESTS[ty]


@pytest.mark.parametrize("ty", GRID)
def test_decoder_bit_exact_with_every_scale_shape(gpu, orc, pkg, ty):
    """Random blocks (every byte uniform: all indices, signs and sub-scales) under subnormal, tiny, huge and negative
    block scales; a ragged block count; an offset into the buffer."""
    bb = pkg.synth.BLOCK_SHAPE[ty][0]
    scales = np.array([0x0001, 0x0200, 0x03FF, 0x0400, 0x7BFF, 0x8001, 0xBC00, 0x3555, 0x0000, 0x1234], np.uint16)
    nb = 333
    raw = pkg.synth.grid_weights(ty, nb, 256, "extreme", ty).reshape(nb, bb).copy()
    for i in range(0, nb, 3):
        d = int(scales[(i // 3) % scales.size])
        if ty == IQ1_M:
            for w in range(4):
                raw[i, 49 + 2 * w] = (int(raw[i, 49 + 2 * w]) & 0x0F) | (((d >> (4 * w)) & 0xF) << 4)
        else:
            raw[i, 0], raw[i, 1] = d & 0xFF, d >> 8
    raw = raw.reshape(-1)
    want = orc.dequant_to_f16(raw, ty, nb * 256)
    got = _dequant(gpu, ty, raw, nb * 256)
    same = (got == want) | (np.isnan(got.view(np.float16)) & np.isnan(want.view(np.float16)))
    assert np.all(same), np.flatnonzero(~same)[:8]
    # a window of the buffer (blocks 5 .. 16) decodes to the same bits
    rb, out = gpu.upload_bytes(raw), gpu.alloc_bytes(12 * 256 * 2)
    gpu.dequant_f16(ty, rb, 12 * 256, out, raw_off=5 * bb)
    assert np.array_equal(gpu.read(out, 12 * 256, np.uint16), got[5 * 256:17 * 256])


@pytest.mark.parametrize("ty", GRID)
@pytest.mark.parametrize("n,k", [(1, 256), (13, 2560), (1000, 4096), (96, 14336), (4099, 4096), (33001, 2816)])
def test_float_matvec_matches_the_exact_dot(gpu, orc, pkg, ty, n, k):
    """`mm` under OJH_ACT_FLOAT (gemv_nat_<fmt>, from 32768 rows the register-resident form) against the exactly
    decoded weights in double: 1e-5 of peak (the reference's bound for its GPU kernels is 2e-3)."""
    w = pkg.synth.weights(ty, n, k, "gridf", n, k)
    x = pkg.synth.normal_f32(k, "gridf", "x", ty, n, k)
    lin = gpu.lin(ty, n, k, w)
    yd = gpu.upload(np.full(n + 2, 12345.0, np.float32))
    gpu.mm(gpu.upload(x), lin, yd, 1, False, act_mode=pkg.ACT_FLOAT, y_off=4)
    got = gpu.read(yd, n + 2)
    assert got[0] == 12345.0 and got[-1] == 12345.0, "wrote outside y"
    assert peak_err(got[1:-1], orc.matmul_ref(w, ty, n, k, x)[0]) <= 1e-5


@pytest.mark.parametrize("ty", GRID)
def test_entries_by_name(gpu, orc, pkg, ty):
    """gemv_nat_<fmt>{,_r1,_r2,_accum,_bias,_m,_px} dispatched as a reference caller would: same sums whatever the rows
    per wave (bit for bit between _r1, _r2, the 4-row entry and — where it keeps the group-per-lane map — _px; the head
    form of IQ2_XXS / IQ2_S / IQ3_XXS / IQ3_S sums a sub-block per lane: the same terms in another order), bias and
    accumulation in the store, three tokens."""
    gpu.ensure_family("iq_grid")
    n, k, m = 203, 1024, 3
    tag = TAG[ty]
    w = pkg.synth.weights(ty, n, k, "gridn", ty)
    xs = pkg.synth.normal_f32(m * k, "gridn", "x", ty).reshape(m, k)
    ref = orc.matmul_ref(w, ty, n, k, xs).astype(np.float32)
    wd, xd = gpu.upload_bytes(w), gpu.upload(xs)
    outs = {}
    for name in (f"gemv_nat_{tag}", f"gemv_nat_{tag}_r1", f"gemv_nat_{tag}_r2", f"gemv_nat_{tag}_px"):
        grid, block = gpu.launch_shape(name, k, n, 1)
        yd = gpu.upload(np.full(n + 2, 777.0, np.float32))
        gpu.dispatch(gpu.begin(), name, [(xd, 0), (wd, 0), (yd, 4)], [k, n], grid, block)
        got = gpu.read(yd, n + 2)
        assert got[0] == 777.0 and got[-1] == 777.0, name
        outs[name] = got[1:-1].copy()
        assert peak_err(outs[name], ref[0]) <= 1e-5, name
    first = outs[f"gemv_nat_{tag}"]
    sub32 = tag in ("iq2xxs", "iq2s", "iq3xxs", "iq3s")
    assert all(np.array_equal(first, o) for nm, o in outs.items() if not (sub32 and nm.endswith("_px")))
    assert peak_err(outs[f"gemv_nat_{tag}_px"], first) <= 1e-6
    grid, block = gpu.launch_shape(f"gemv_nat_{tag}_bias", k, n, 1)
    bias = (1000.0 + np.arange(n)).astype(np.float32)
    yb = gpu.alloc(n)
    gpu.dispatch(gpu.begin(), f"gemv_nat_{tag}_bias", [(xd, 0), (wd, 0), (yb, 0), (gpu.upload(bias), 0)], [k, n], grid, block)
    assert np.array_equal(gpu.read(yb, n), first + bias)
    y0 = pkg.synth.normal_f32(n, "gridn", "y0")
    ya = gpu.upload(y0)
    gpu.dispatch(gpu.begin(), f"gemv_nat_{tag}_accum", [(xd, 0), (wd, 0), (ya, 0)], [k, n], grid, block)
    assert np.array_equal(gpu.read(ya, n), y0 + first)
    grid, block = gpu.launch_shape(f"gemv_nat_{tag}_m", k, n, m)
    ym = gpu.upload(np.full(m * n + 2, 777.0, np.float32))
    gpu.dispatch(gpu.begin(), f"gemv_nat_{tag}_m", [(xd, 0), (wd, 0), (ym, 4)], [k, n, m, 0], grid, block)
    got = gpu.read(ym, m * n + 2)
    assert got[0] == 777.0 and got[-1] == 777.0
    assert peak_err(got[1:-1].reshape(m, n), ref) <= 1e-5
    gpu.dispatch(gpu.begin(), f"gemv_nat_{tag}_m", [(xd, 0), (wd, 0), (ym, 4)], [k, n, m, 1], grid, block)
    assert peak_err(gpu.read(ym, m * n + 2)[1:-1].reshape(m, n), 2.0 * ref) <= 1e-5


@pytest.mark.parametrize("ty", [IQ3_S, IQ2_S])
@pytest.mark.parametrize("n,k,m", [(4096, 4096, 1), (37, 256, 1), (130, 2816, 5), (33001, 2816, 1), (8201, 768, 1)])
def test_f32_rows_match_the_cpu_dots(gpu, orc, pkg, ty, n, k, m):
    """IQ3_S / IQ2_S: `matvec_kq` sends them to dot_iq3s / dot_iq2s on f32 activations; int8 activations are refused."""
    w = pkg.synth.weights(ty, n, k, "grids", n, k)
    x = pkg.synth.normal_f32(m * k, "grids", "x", ty, m, k).reshape(m, k)
    lin = gpu.lin(ty, n, k, w)
    yd = gpu.upload(np.full(m * n + 2, 12345.0, np.float32))
    gpu.mm(gpu.upload(x), lin, yd, m, y_off=4)
    got = gpu.read(yd, m * n + 2)
    assert got[0] == 12345.0 and got[-1] == 12345.0, "wrote outside y"
    for t in range(m):
        assert peak_err(got[1 + t * n:1 + (t + 1) * n], orc.matvec_kq(w, ty, n, k, x[t])) <= 1e-5, t
    with pytest.raises(pkg.OjasHipError, match="f32 activations"):
        gpu.mm(gpu.upload(x), lin, yd, m, act_mode=pkg.ACT_Q8K)


@pytest.mark.parametrize("ty", [IQ2_XXS, IQ3_XXS])
@pytest.mark.parametrize("n,k,m", [(4096, 4096, 1), (37, 256, 1), (130, 2816, 5), (33001, 2816, 1), (777, 14336, 2), (64, 1024, 40)])
def test_int8_rows_match_the_cpu_dots(gpu, orc, pkg, ty, n, k, m):
    """IQ2_XXS / IQ3_XXS: `matvec_kq` quantizes the activations per 256 and runs dot_iq2xxs_q8k / dot_iq3xxs_q8k —
    what `mm` does for a few tokens unless f32 activations are asked for, which give dot_iq2xxs / dot_iq3xxs (dot_iq);
    from 8 tokens OJH_ACT_AUTO decodes the rows for the f16 tile, and the int8 kernels answer to OJH_ACT_Q8K."""
    w = pkg.synth.weights(ty, n, k, "gridq", n, k)
    x = pkg.synth.normal_f32(m * k, "gridq", "x", ty, m, k).reshape(m, k)
    lin = gpu.lin(ty, n, k, w)
    yd = gpu.upload(np.full(m * n + 2, 12345.0, np.float32))
    gpu.mm(gpu.upload(x), lin, yd, m, y_off=4, act_mode=pkg.ACT_Q8K if m >= 8 else pkg.ACT_AUTO)
    got = gpu.read(yd, m * n + 2)
    assert got[0] == 12345.0 and got[-1] == 12345.0, "wrote outside y"
    for t in sorted({0, m // 2, m - 1}):
        assert peak_err(got[1 + t * n:1 + (t + 1) * n], orc.matvec_kq(w, ty, n, k, x[t])) <= 2e-5, t
    if n <= 4096 and m <= 5:
        yf = gpu.alloc(m * n)
        gpu.mm(gpu.upload(x), lin, yf, m, act_mode=pkg.ACT_FLOAT)
        gf = gpu.read(yf, m * n).reshape(m, n)
        for t in range(m):
            assert peak_err(gf[t], orc.matvec_iq_f32(w, ty, n, k, x[t])) <= 1e-5, t


@pytest.mark.parametrize("ty", [IQ2_XXS, IQ3_XXS])
def test_int8_entries_by_name(gpu, orc, pkg, ty):
    """gemv_q8k_<fmt>{,_r1,_r2,_wide,_accum,_bias,_m} over activations quantized by the library's own quantize_q8k."""
    gpu.ensure_family("iq_grid")
    gpu.ensure_family("gemv_q8k")
    n, k, m = 203, 1280, 3
    tag = TAG[ty]
    w = pkg.synth.weights(ty, n, k, "gridqn", ty)
    xs = pkg.synth.normal_f32(m * k, "gridqn", "x", ty).reshape(m, k)
    ref = np.stack([orc.matvec_kq(w, ty, n, k, xs[t]) for t in range(m)])
    wd = gpu.upload_bytes(w)
    nsb = k // 256
    q, s = gpu.alloc_bytes(m * nsb * 256), gpu.alloc(m * nsb)
    gpu.quant_q8k(gpu.upload(xs), m, k, q, s)
    outs = []
    for suffix in ("", "_r1", "_r2", "_wide"):
        name = f"gemv_q8k_{tag}{suffix}"
        grid, block = gpu.launch_shape(name, k, n, 1)
        yd = gpu.upload(np.full(n + 2, 777.0, np.float32))
        gpu.dispatch(gpu.begin(), name, [(q, 0), (s, 0), (wd, 0), (yd, 4)], [k, n], grid, block)
        got = gpu.read(yd, n + 2)
        assert got[0] == 777.0 and got[-1] == 777.0, name
        assert peak_err(got[1:-1], ref[0]) <= 2e-5, name
        outs.append(got[1:-1].copy())
    assert all(np.array_equal(outs[0], o) for o in outs)
    grid, block = gpu.launch_shape(f"gemv_q8k_{tag}_bias", k, n, 1)
    bias = (1000.0 + np.arange(n)).astype(np.float32)
    yb = gpu.alloc(n)
    gpu.dispatch(gpu.begin(), f"gemv_q8k_{tag}_bias", [(q, 0), (s, 0), (wd, 0), (yb, 0), (gpu.upload(bias), 0)], [k, n], grid, block)
    assert np.array_equal(gpu.read(yb, n), outs[0] + bias)
    y0 = pkg.synth.normal_f32(n, "gridqn", "y0")
    ya = gpu.upload(y0)
    gpu.dispatch(gpu.begin(), f"gemv_q8k_{tag}_accum", [(q, 0), (s, 0), (wd, 0), (ya, 0)], [k, n], grid, block)
    assert np.array_equal(gpu.read(ya, n), y0 + outs[0])
    grid, block = gpu.launch_shape(f"gemv_q8k_{tag}_m", k, n, m)
    ym = gpu.upload(np.full(m * n + 2, 777.0, np.float32))
    gpu.dispatch(gpu.begin(), f"gemv_q8k_{tag}_m", [(q, 0), (s, 0), (wd, 0), (ym, 4)], [k, n, m, 0], grid, block)
    got = gpu.read(ym, m * n + 2)
    assert got[0] == 777.0 and got[-1] == 777.0
    assert peak_err(got[1:-1].reshape(m, n), ref) <= 2e-5


@pytest.mark.parametrize("ty", [IQ2_XS, IQ1_S, IQ1_M])
def test_gpu_path_formats_take_f32_activations_only(gpu, pkg, ty):
    n, k = 64, 512
    lin = gpu.lin(ty, n, k, pkg.synth.weights(ty, n, k, "gridr", ty))
    x, y = gpu.upload(pkg.synth.normal_f32(k, "gridr", "x")), gpu.alloc(n)
    with pytest.raises(pkg.OjasHipError, match="f32 activations"):
        gpu.mm(x, lin, y, 1, act_mode=pkg.ACT_Q8K)


def _route(gpu, lg, ksel):
    T, E = lg.shape
    idx_d, wgt_d = gpu.alloc_bytes(T * ksel * 4), gpu.alloc(T * ksel)
    gpu.moe_route(gpu.upload(lg), T, E, ksel, idx_d, wgt_d)
    return gpu.read(idx_d, T * ksel, np.uint32).reshape(T, ksel), gpu.read(wgt_d, T * ksel).reshape(T, ksel), idx_d, wgt_d


def test_iq3s_gate_up_reference_procedure(gpu, orc, pkg):
    """`moe_gu_iq3s` and `moe_gu_iq3s_slots` of family "moe_iq" as the reference checks them
    (crates/ojas-cuda/tests/conformance.rs:827-910): E = 4, K = 512, N = 16, two slots with experts (3 j + 1) mod 4,
    x = tvec(K, 31), gate and up both synth::blocks(21, ..), against products of the values dequant_to_f16 decodes
    within 5e-3 of the peak; the offset-addressed form (byte offsets that do not follow the slot order) bit for bit."""
    k, n, experts, ksel = 512, 16, 4, 2
    nblk = k // 256
    ebytes = n * nblk * 110
    x = pkg.synth.tvec(k, 31)
    gb = orc.synth_blocks(IQ3_S, experts * n * nblk)
    ub = orc.synth_blocks(IQ3_S, experts * n * nblk)
    w16 = orc.dequant_to_f16(gb, IQ3_S, experts * n * k).view(np.float16).astype(np.float64).reshape(experts * n, k)
    ids = np.array([(j * 3 + 1) % experts for j in range(ksel)], np.uint32)
    want = []
    for e in ids:
        gt = w16[e * n:(e + 1) * n] @ x.astype(np.float64)
        want.append(gt / (1.0 + np.exp(-gt)) * gt)          # gate and up hold the same bytes
    want = np.concatenate(want)
    assert np.any(np.abs(want) > 1e-4)
    gpu.ensure_family("moe_iq")
    xd, gd, ud, idxd = gpu.upload(x), gpu.upload_bytes(gb), gpu.upload_bytes(ub), gpu.upload_bytes(ids)
    act = gpu.alloc(ksel * n)
    grid, block = gpu.launch_shape("moe_gu_iq3s", k, n, ksel)
    assert grid == [-(-n // 8), ksel, 1] and block == [256, 1, 1]
    gpu.dispatch(gpu.begin(), "moe_gu_iq3s", [(xd, 0), (gd, 0), (ud, 0), (act, 0), (idxd, 0)], [k, n], grid, block)
    got = gpu.read(act, ksel * n)
    assert peak_err(got, want) < 5e-3
    wx = orc.dequant_to_f64(gb, IQ3_S, experts * n * k).reshape(experts * n, k)
    exact = np.concatenate([(lambda g: g / (1.0 + np.exp(-g)) * g)(wx[e * n:(e + 1) * n] @ x.astype(np.float64)) for e in ids])
    assert peak_err(got, exact) <= 1e-5
    offs = gpu.upload_bytes((ids.astype(np.uint64) * ebytes).astype(np.uint32))
    act2 = gpu.alloc(ksel * n)
    gpu.dispatch(gpu.begin(), "moe_gu_iq3s_slots", [(xd, 0), (gd, 0), (ud, 0), (act2, 0), (offs, 0), (offs, 0)], [k, n], grid, block)
    assert np.array_equal(gpu.read(act2, ksel * n), got)
    # an expert index past the tensors contributes zeros; an offset past the arena is clamped into it
    bad = gpu.upload_bytes(np.array([1, 9], np.uint32))
    gpu.dispatch(gpu.begin(), "moe_gu_iq3s", [(xd, 0), (gd, 0), (ud, 0), (act, 0), (bad, 0)], [k, n], grid, block)
    again = gpu.read(act, ksel * n)
    assert np.array_equal(again[:n], got[:n]) and np.all(again[n:] == 0.0)
    wild = gpu.upload_bytes(np.array([0xFFFFFFF0, ebytes + 1], np.uint32))
    gpu.dispatch(gpu.begin(), "moe_gu_iq3s_slots", [(xd, 0), (gd, 0), (ud, 0), (act2, 0), (wild, 0), (wild, 0)], [k, n], grid, block)
    assert np.all(np.isfinite(gpu.read(act2, ksel * n)))


@pytest.mark.parametrize("tg,td", [(IQ3_S, 20), (IQ2_XXS, IQ2_XXS), (IQ2_S, IQ3_XXS), (IQ3_S, IQ3_XXS), (23, IQ2_XXS)])
@pytest.mark.parametrize("T,E,ksel,d,nff,accum", [(1, 8, 2, 256, 256, False), (6, 16, 4, 512, 768, True), (33, 4, 3, 1024, 256, False)])
def test_grid_experts_through_the_ffn_entry(gpu, orc, pkg, tg, td, T, E, ksel, d, nff, accum):
    """The grid-codebook rows of the reference's expert table (crates/ojas-core/src/quant_src.rs:180-190) under
    `ojh_moe_ffn`, mixed with the IQ4 rows: f32 activations against the exact block values, as the reference's GPU
    expert kernels compute (IQ3_S gate/up + IQ4_NL down is the combination its streamed models ship in)."""
    gate = pkg.synth.weights(tg, E * nff, d, "moegrid", "gate", tg, E, d, nff)
    up = pkg.synth.weights(tg, E * nff, d, "moegrid", "up", tg, E, d, nff)
    down = pkg.synth.weights(td, E * d, nff, "moegrid", "down", td, E, d, nff)
    x = pkg.synth.normal_f32(T * d, "moegrid", "x", T, d).reshape(T, d)
    lg = pkg.synth.normal_f32(T * E, "moegrid", "lg", T, E).reshape(T, E)
    gi, gw, idx_d, wgt_d = _route(gpu, lg, ksel)
    want = orc.moe_ffn(x, gi, gw, gate, up, tg, down, td, E, nff, mode=1)
    peak = float(np.max(np.abs(want)))
    y0 = np.float32(peak) * pkg.synth.normal_f32(T * d, "moegrid", "y0").reshape(T, d) if accum else np.zeros((T, d), np.float32)
    yd = gpu.upload(np.concatenate([y0.ravel() if accum else np.full(T * d, 777.0, np.float32), np.full(d, 12345.5, np.float32)]))
    lg_, lu_, ld_ = gpu.lin(tg, E * nff, d, gate), gpu.lin(tg, E * nff, d, up), gpu.lin(td, E * d, nff, down)
    gpu.moe_ffn(gpu.upload(x), T, d, nff, E, ksel, idx_d, wgt_d, lg_, lu_, ld_, yd, accum=accum)
    got = gpu.read(yd, T * d + d)
    assert np.all(got[T * d:] == 12345.5), "wrote past the last token"
    # from 8 assignments per expert a batch is decoded into f16 and grouped on the f16 matrix tile (activations
    # rounded to f16 on the way in); OJH_ACT_FLOAT keeps the per-assignment kernels at every size
    tiled = T * ksel >= 8 * E and d % 64 == 0 and nff % 64 == 0
    assert peak_err(got[:T * d].reshape(T, d) - y0, want) <= (1e-3 if tiled else 2e-5)
    if tiled:
        gpu.write_bytes(yd, 0, np.concatenate([y0.ravel() if accum else np.full(T * d, 777.0, np.float32), np.full(d, 12345.5, np.float32)]))
        gpu.moe_ffn(gpu.upload(x), T, d, nff, E, ksel, idx_d, wgt_d, lg_, lu_, ld_, yd, accum=accum, act_mode=pkg.ACT_FLOAT)
        assert peak_err(gpu.read(yd, T * d).reshape(T, d) - y0, want) <= 2e-5
