"""MoE router and grouped expert FFN on the GPU against the CPU oracle.

Router: indices must match exactly and weights within 1e-5, the reference's own bounds
(crates/ojas-cuda/tests/conformance.rs:380-408).  Expert FFN: against the composition of the CPU
path's matvecs (crates/ojas-cpu/src/cpu_glm.rs:551-582 over matvec_kq), peak-normalised error
<= 1e-3 required.  The activation of every assignment is re-quantized to int8 before the down
projection, so a last-ulp difference upstream can flip one int8 code; 3e-4 is what that costs at
most in these cases.
"""
import numpy as np
import pytest

from conftest import peak_err

pytestmark = pytest.mark.gpu
Q4_K = 12
Q8_0 = 8
IQ4_NL, IQ4_XS = 20, 23
TOL = 1e-3
TOL_SEEN = 3e-4


def _route(gpu, logits, ksel):
    T, E = logits.shape
    ld = gpu.upload(logits)
    idx, wgt = gpu.alloc_bytes(T * ksel * 4), gpu.alloc(T * ksel)
    gpu.moe_route(ld, T, E, ksel, idx, wgt)
    return gpu.read(idx, T * ksel, np.uint32).reshape(T, ksel), gpu.read(wgt, T * ksel).reshape(T, ksel), idx, wgt


def test_router_reference_case(gpu, orc, pkg):
    """E=64, KSEL=8, logits = tvec(64, 51): the reference's known-answer procedure."""
    lg = pkg.synth.tvec(64, 51)[None, :]
    gi, gw, _, _ = _route(gpu, lg, 8)
    wi, ww = orc.moe_topk(lg, 8)
    assert np.array_equal(gi, wi)
    assert np.max(np.abs(gw - ww)) < 1e-5
    # through the kernel seam, single-token entry
    gpu.ensure_family("moe")
    ld, idx, wgt = gpu.upload(lg), gpu.alloc_bytes(32), gpu.alloc(8)
    grid, block = gpu.launch_shape("moe_topk", 0, 0, 1)
    gpu.dispatch(gpu.begin(), "moe_topk", [(ld, 0), (idx, 0), (wgt, 0)], [64, 8], grid, block)
    assert np.array_equal(gpu.read(idx, 8, np.uint32), wi[0])


@pytest.mark.parametrize("T,E,ksel", [(1, 128, 8), (16, 128, 8), (256, 128, 8), (5, 1000, 6), (3, 7, 7)])
def test_router_matches_oracle(gpu, orc, pkg, T, E, ksel):
    lg = pkg.synth.normal_f32(T * E, "moe", "logits", T, E).reshape(T, E)
    gi, gw, _, _ = _route(gpu, lg, ksel)
    wi, ww = orc.moe_topk(lg, ksel)
    assert np.array_equal(gi, wi)
    assert np.max(np.abs(gw - ww)) < 1e-5
    assert np.allclose(gw.sum(1), 1.0, atol=1e-5)


def test_router_ties_take_the_lowest_index(gpu):
    lg = np.zeros((2, 128), np.float32)
    lg[1, 70] = lg[1, 3] = lg[1, 127] = 1.0
    gi, _, _, _ = _route(gpu, lg, 4)
    assert list(gi[0]) == [0, 1, 2, 3]
    assert list(gi[1]) == [3, 70, 127, 0]


@pytest.mark.parametrize("T,E,ksel", [(1, 64, 6), (9, 160, 6), (4, 256, 8), (3, 1000, 5), (2, 7, 7)])
def test_other_routers_by_their_reference_names(gpu, orc, pkg, T, E, ksel):
    """moe_topk_nonorm (raw softmax probabilities) and moe_topk_v3 (sigmoid scores, bias-corrected choice, renormalised
    and scaled weights): crates/ojas-metal/src/kernels/moe.rs:130-150, :531-551."""
    gpu.ensure_family("moe")
    lg = pkg.synth.normal_f32(T * E, "moe", "logits2", T, E).reshape(T, E)
    bias = (0.3 * pkg.synth.normal_f32(E, "moe", "bias", E)).astype(np.float32)
    ld, bd = gpu.upload(lg), gpu.upload(bias)
    idx, wgt = gpu.alloc_bytes(T * ksel * 4), gpu.alloc(T * ksel)
    grid, block = gpu.launch_shape("moe_topk_nonorm", 0, 0, T)
    assert grid == [T, 1, 1] and block == [64, 1, 1]
    gpu.dispatch(gpu.begin(), "moe_topk_nonorm", [(ld, 0), (idx, 0), (wgt, 0)], [E, ksel], grid, block)
    wi, ww = orc.moe_topk_nonorm(lg, ksel)
    assert np.array_equal(gpu.read(idx, T * ksel, np.uint32).reshape(T, ksel), wi)
    assert np.max(np.abs(gpu.read(wgt, T * ksel).reshape(T, ksel) - ww)) < 1e-6
    for norm, rs in ((1, 1.0), (1, 2.5), (0, 1.0)):
        rbits = int(np.float32(rs).view(np.uint32))
        gpu.dispatch(gpu.begin(), "moe_topk_v3", [(ld, 0), (bd, 0), (idx, 0), (wgt, 0)], [E, ksel, rbits, norm], grid, block)
        wi, ww = orc.moe_topk_v3(lg, bias, ksel, rs, bool(norm))
        assert np.array_equal(gpu.read(idx, T * ksel, np.uint32).reshape(T, ksel), wi)
        assert np.max(np.abs(gpu.read(wgt, T * ksel).reshape(T, ksel) - ww)) < 2e-6 * rs
    # ties take the lowest index; an out-of-range request is refused before any launch
    z = gpu.upload(np.zeros((1, E), np.float32))
    gpu.dispatch(gpu.begin(), "moe_topk_v3", [(z, 0), (z, 0), (idx, 0), (wgt, 0)], [E, ksel, int(np.float32(1).view(np.uint32)), 0],
                 [1, 1, 1], block)
    assert list(gpu.read(idx, ksel, np.uint32)) == list(range(ksel))
    assert np.all(gpu.read(wgt, ksel) == 0.5)
    with pytest.raises(Exception):
        gpu.dispatch(gpu.begin(), "moe_topk_nonorm", [(ld, 0), (idx, 0), (wgt, 0)], [E, E + 1], grid, block)


@pytest.mark.parametrize("T,E,ksel,d", [(16, 128, 8, 2048), (3, 7, 2, 768), (40, 1000, 5, 256)])
def test_quantizer_and_grouping_in_one_launch(gpu, orc, pkg, T, E, ksel, d):
    """`moe_quant_group` against the two launches it stands for: the quantizer's bytes bit for bit (and the CPU
    oracle's), and a grouping that holds every assignment once under its expert."""
    gpu.ensure_family("moe")
    gpu.ensure_family("gemv_q8k")
    x = pkg.synth.normal_f32(T * d, "moe", "qg-x", T, d).reshape(T, d)
    idx_h = pkg.synth.rng("moe", "qg-idx", T, E).integers(0, E, T * ksel).astype(np.uint32)
    NA, nsb = T * ksel, d // 256
    xd, idx = gpu.upload(x), gpu.upload_bytes(idx_h.view(np.uint8))
    xq, xs = gpu.alloc_bytes(T * d), gpu.alloc(T * nsb)
    counts, offsets, lst = gpu.alloc_bytes(E * 4), gpu.alloc_bytes((E + 1) * 4), gpu.alloc_bytes(NA * 4)
    grid, block = gpu.launch_shape("moe_quant_group", d, 0, T)
    assert grid == [T + 1, 1, 1]
    gpu.dispatch(gpu.begin(), "moe_quant_group", [(xd, 0), (xq, 0), (xs, 0), (idx, 0), (counts, 0), (offsets, 0), (lst, 0)],
                 [d, T, NA, E], grid, block)
    q2, s2 = gpu.alloc_bytes(T * d), gpu.alloc(T * nsb)
    gpu.quant_q8k(xd, T, d, q2, s2)
    assert np.array_equal(gpu.read(xq, T * d, np.int8), gpu.read(q2, T * d, np.int8))
    assert np.array_equal(gpu.read(xs, T * nsb), gpu.read(s2, T * nsb))
    ws, wq, _ = orc.quant_q8k(x[T - 1])
    assert np.array_equal(gpu.read(xq, T * d, np.int8).reshape(T, d)[T - 1], wq)
    cnt, off, ls = gpu.read(counts, E, np.uint32), gpu.read(offsets, E + 1, np.uint32), gpu.read(lst, NA, np.uint32)
    assert np.array_equal(cnt, np.bincount(idx_h, minlength=E))
    assert np.array_equal(off, np.concatenate([[0], np.cumsum(cnt)]))
    assert sorted(ls) == list(range(NA))
    for e in range(E):
        assert np.all(idx_h[ls[off[e]:off[e + 1]]] == e)


def _experts(pkg, E, d, nff, tag):
    gate = pkg.synth.q4k_weights(E * nff, d, "moe", tag, "gate")
    up = pkg.synth.q4k_weights(E * nff, d, "moe", tag, "up")
    down = pkg.synth.q4k_weights(E * d, nff, "moe", tag, "down")
    return gate, up, down


@pytest.mark.parametrize("T,E,ksel,d,nff,accum", [(1, 8, 2, 256, 256, False), (7, 16, 4, 512, 256, True),
                                                   (33, 8, 8, 1024, 768, False), (4, 4, 1, 2304, 512, False)])
def test_expert_ffn_matches_cpu_path(gpu, orc, pkg, T, E, ksel, d, nff, accum):
    gate, up, down = _experts(pkg, E, d, nff, (E, d, nff))
    x = pkg.synth.normal_f32(T * d, "moe", "x", T, d).reshape(T, d)
    lg = pkg.synth.normal_f32(T * E, "moe", "lg", T, E).reshape(T, E)
    gi, gw, idx_d, wgt_d = _route(gpu, lg, ksel)
    y0 = pkg.synth.normal_f32(T * d, "moe", "y0").reshape(T, d) if accum else np.zeros((T, d), np.float32)
    yd = gpu.upload(np.concatenate([y0.ravel(), np.full(d, 12345.5, np.float32)]))
    lg_, lu_, ld_ = gpu.lin(Q4_K, E * nff, d, gate), gpu.lin(Q4_K, E * nff, d, up), gpu.lin(Q4_K, E * d, nff, down)
    gpu.moe_ffn(gpu.upload(x), T, d, nff, E, ksel, idx_d, wgt_d, lg_, lu_, ld_, yd, accum=accum, act_mode=pkg.ACT_Q8K)
    got = gpu.read(yd, T * d + d)
    assert np.all(got[T * d:] == 12345.5), "wrote past the last token"
    want = orc.moe_ffn(x, gi, gw, gate, up, Q4_K, down, Q4_K, E, nff, mode=0, y0=y0)
    err = peak_err(got[:T * d].reshape(T, d) - y0, want - y0)
    assert err <= TOL_SEEN <= TOL, err


def test_expert_ffn_at_the_benchmark_shape(gpu, orc, pkg):
    """128 experts, top-8, hidden 2048, expert FFN 768: T = 1 and 16 against the CPU path in full,
    T = 256 against the CPU path on sampled tokens, against a second T = 256 batch holding the
    same tokens in other positions (a token's result cannot depend on who else is in the batch:
    bit for bit), and against the T = 1 launches of the same tokens (the small-batch form of the
    expert products rounds its f32 sums in another order: last ulps)."""
    E, ksel, d, nff = 128, 8, 2048, 768
    gate, up, down = _experts(pkg, E, d, nff, "bench")
    lg_, lu_, ld_ = gpu.lin(Q4_K, E * nff, d, gate), gpu.lin(Q4_K, E * nff, d, up), gpu.lin(Q4_K, E * d, nff, down)
    for T in (1, 16, 256):
        x = pkg.synth.normal_f32(T * d, "moe", "bx", T).reshape(T, d)
        lg = pkg.synth.normal_f32(T * E, "moe", "blg", T).reshape(T, E)
        gi, gw, idx_d, wgt_d = _route(gpu, lg, ksel)
        yd = gpu.alloc(T * d)
        gpu.moe_ffn(gpu.upload(x), T, d, nff, E, ksel, idx_d, wgt_d, lg_, lu_, ld_, yd)
        got = gpu.read(yd, T * d).reshape(T, d)
        sample = range(T) if T <= 16 else [0, 17, 100, 255]
        for t in sample:
            want = orc.moe_ffn(x[t:t + 1], gi[t:t + 1], gw[t:t + 1], gate, up, Q4_K, down, Q4_K, E, nff, mode=0)
            assert peak_err(got[t], want[0]) <= TOL_SEEN, (T, t)
        if T == 256:
            for t in (3, 200):
                y1 = gpu.alloc(d)
                i1, w1 = gpu.upload_bytes(gi[t]), gpu.upload(gw[t])
                gpu.moe_ffn(gpu.upload(x[t]), 1, d, nff, E, ksel, i1, w1, lg_, lu_, ld_, y1)
                assert peak_err(gpu.read(y1, d), got[t]) <= TOL   # an int8 code of `act` may flip between the forms
            perm = np.roll(np.arange(T), 37)
            y2 = gpu.alloc(T * d)
            gpu.moe_ffn(gpu.upload(x[perm]), T, d, nff, E, ksel, gpu.upload_bytes(gi[perm]), gpu.upload(gw[perm]),
                        lg_, lu_, ld_, y2)
            assert np.array_equal(gpu.read(y2, T * d).reshape(T, d), got[perm])


@pytest.mark.parametrize("T,E,ksel,d,nff", [(200, 8, 2, 512, 768), (130, 4, 3, 256, 1280), (64, 2, 2, 384 * 2, 256)])
@pytest.mark.parametrize("dty", [13, 14])
def test_q5k_q6k_down_tensors_on_the_int8_matrix_tile(gpu, orc, pkg, T, E, ksel, d, nff, dty):
    """From a handful of assignments per expert `ojh_moe_ffn` sends Q5_K / Q6_K down tensors to
    `moe_down_{q5k,q6k}_gs` (experts with one, two and three token tiles, ragged last tiles): sampled tokens against the
    CPU arithmetic, every token against the integer-dot form, and — by name — one token tile per expert in the grid
    (the workgroup walks the others) against one workgroup per tile, bit for bit."""
    gate = pkg.synth.q4k_weights(E * nff, d, "moe5g", "gate", E, d, nff)
    up = pkg.synth.q4k_weights(E * nff, d, "moe5g", "up", E, d, nff)
    down = pkg.synth.weights(dty, E * d, nff, "moe5g", "down", E, d, nff, dty)
    x = pkg.synth.normal_f32(T * d, "moe5g", "x", T, d).reshape(T, d)
    lg = pkg.synth.normal_f32(T * E, "moe5g", "lg", T, E).reshape(T, E)
    lg[:, 0] += 1.0                                      # a popular expert: more than one tile of assignments
    outs = {}
    for gs in ("1", "0"):
        monkey = pytest.MonkeyPatch()
        monkey.setenv("OJAS_HIP_MOE_DOWN_GS", gs)
        g = pkg.HipGpu(0)
        try:
            gi, gw, idx_d, wgt_d = _route(g, lg, ksel)
            lg_, lu_, ld_ = g.lin(Q4_K, E * nff, d, gate), g.lin(Q4_K, E * nff, d, up), g.lin(dty, E * d, nff, down)
            yd = g.upload(np.full(T * d + d, 12345.5, np.float32))
            g.moe_ffn(g.upload(x), T, d, nff, E, ksel, idx_d, wgt_d, lg_, lu_, ld_, yd)
            got = g.read(yd, T * d + d)
            assert np.all(got[T * d:] == 12345.5), "wrote past the last token"
            outs[gs] = got[:T * d].reshape(T, d)
            if gs == "1":
                assert g.has_kernel("moe_down_%s_gs" % {13: "q5k", 14: "q6k"}[dty]), "the tile was not taken"
        finally:
            g.close()
            monkey.undo()
    for t in (0, T // 2, T - 1):
        want = orc.moe_ffn(x[t:t + 1], gi[t:t + 1], gw[t:t + 1], gate, up, Q4_K, down, dty, E, nff, mode=0)
        assert peak_err(outs["1"][t], want[0]) <= TOL, t
    assert peak_err(outs["1"], outs["0"]) <= TOL


@pytest.mark.parametrize("dty", [13, 14])
def test_grouped_int8_tile_by_name(gpu, orc, pkg, dty):
    """`moe_down_{q5k,q6k}_gs(aq, as, wd, dv, offsets, list, K, N, NA)`: every assignment's row against matvec_kq of its
    expert; an empty expert; any number of token tiles in the grid gives the same bits."""
    tag = {13: "q5k", 14: "q6k"}[dty]
    E, n, k = 3, 200, 512
    counts = [150, 0, 37]
    na = sum(counts)
    w = pkg.synth.weights(dty, E * n, k, "moegs", "w", dty)
    act = pkg.synth.normal_f32(na * k, "moegs", "act", dty).reshape(na, k)
    perm = pkg.synth.rng("moegs", "perm").permutation(na).astype(np.uint32)
    offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.uint32)
    gpu.ensure_family("gemm_q8k")
    gpu.ensure_family("gemv_q8k")
    nsb = k // 256
    aq, as_ = gpu.alloc_bytes(na * k), gpu.alloc(na * nsb)
    gpu.quant_q8k(gpu.upload(act), na, k, aq, as_)
    wd, od, ld = gpu.upload_bytes(w), gpu.upload_bytes(offsets), gpu.upload_bytes(perm)
    rb = len(w) // (E * n)
    seen = []
    for tiles in (1, 2, 3, 7):
        dv = gpu.upload(np.full(na * n + n, 777.25, np.float32))
        gpu.dispatch(gpu.begin(), "moe_down_%s_gs" % tag, [(aq, 0), (as_, 0), (wd, 0), (dv, 0), (od, 0), (ld, 0)], [k, n, na],
                     [(n + 127) // 128, tiles, E], [256, 1, 1])
        got = gpu.read(dv, na * n + n)
        assert np.all(got[na * n:] == np.float32(777.25))
        seen.append(got[:na * n].reshape(na, n).view(np.uint32).copy())
    for other in seen[1:]:
        assert np.array_equal(seen[0], other)
    got = seen[0].view(np.float32)
    for e in range(E):
        we = w[e * n * rb:(e + 1) * n * rb]
        for i in list(range(offsets[e], offsets[e + 1]))[::9]:
            a = int(perm[i])
            assert peak_err(got[a], orc.matvec_kq(we, dty, n, k, act[a])) <= 2e-5, (e, a)
    with pytest.raises(pkg.OjasHipError, match="grid must be"):
        gpu.dispatch(gpu.begin(), "moe_down_%s_gs" % tag, [(aq, 0), (as_, 0), (wd, 0), (gpu.alloc(na * n), 0), (od, 0), (ld, 0)],
                     [k, n, na], [(n + 127) // 128 + 1, 1, E], [256, 1, 1])


@pytest.mark.parametrize("T,E,ksel,d,nff,accum", [(1, 128, 8, 2048, 768, False), (3, 16, 5, 2304, 512, True),
                                                   (4, 8, 8, 768, 256, False), (2, 70, 64, 256, 256, False)])
def test_decode_form_is_bit_identical_to_the_grouped_integer_dots(gpu, pkg, monkeypatch, T, E, ksel, d, nff, accum):
    """Few tokens run as two launches addressed by assignment (activations quantized in registers,
    weighted sum inside the down launch); the same arithmetic step for step as quantize -> group ->
    gate/up -> quantize -> down -> combine, so the same bits, including accumulate onto y."""
    gate, up, down = _experts(pkg, E, d, nff, ("dec", E, d, nff))
    x = pkg.synth.normal_f32(T * d, "moe", "dx", T, d).reshape(T, d)
    x[0, :256] = 0.0                                    # an all-zero segment: scale 1
    lg = pkg.synth.normal_f32(T * E, "moe", "dlg", T, E).reshape(T, E)
    gi, gw, _, _ = _route(gpu, lg, ksel)
    y0 = pkg.synth.normal_f32(T * d, "moe", "dy0").reshape(T, d)
    outs = []
    for mode in ("3", "2"):
        monkeypatch.setenv("OJAS_HIP_MOE", mode)
        g = pkg.HipGpu(0)
        try:
            lg_, lu_, ld_ = g.lin(Q4_K, E * nff, d, gate), g.lin(Q4_K, E * nff, d, up), g.lin(Q4_K, E * d, nff, down)
            yd = g.upload(np.concatenate([y0.ravel(), np.full(d, 12345.5, np.float32)]))
            g.moe_ffn(g.upload(x), T, d, nff, E, ksel, g.upload_bytes(gi), g.upload(gw), lg_, lu_, ld_, yd, accum=accum)
            got = g.read(yd, T * d + d)
            assert np.all(got[T * d:] == 12345.5), "wrote past the last token"
            outs.append(got[:T * d].copy())
        finally:
            g.close()
    assert np.array_equal(outs[0], outs[1])
    assert np.all(np.isfinite(outs[0])) and np.any(outs[0] != (y0.ravel() if accum else 0.0))


@pytest.mark.parametrize("T,E,ksel,d,nff,accum,dty", [(1, 128, 8, 2048, 768, False, Q4_K), (3, 16, 5, 2304, 512, True, Q4_K),
                                                       (8, 8, 8, 768, 256, False, 13), (2, 70, 64, 256, 256, False, 14),
                                                       (5, 300, 6, 512, 256, True, Q4_K), (33, 16, 4, 512, 512, False, Q4_K)])
def test_router_inside_the_decode_form(gpu, orc, pkg, T, E, ksel, d, nff, accum, dty):
    """`ojh_moe_ffn_routed`: for a few tokens the router runs inside the gate/up launch (`moe_gu_q4k_decr`) — the idx and
    wgt it writes are the bits of `moe_route`, the output the bits of route + `moe_ffn`; more tokens (33) take the two
    calls as they are."""
    gate = pkg.synth.q4k_weights(E * nff, d, "moer", "g", E, d, nff)
    up = pkg.synth.q4k_weights(E * nff, d, "moer", "u", E, d, nff)
    down = pkg.synth.weights(dty, E * d, nff, "moer", "d", dty, E, d, nff)
    x = pkg.synth.normal_f32(T * d, "moer", "x", T, d).reshape(T, d)
    lg = pkg.synth.normal_f32(T * E, "moer", "lg", T, E).reshape(T, E)
    lg[0, :4] = lg[0, 4]                                  # ties: the lowest index wins
    gi, gw, idx_d, wgt_d = _route(gpu, lg, ksel)
    lg_, lu_, ld_ = gpu.lin(Q4_K, E * nff, d, gate), gpu.lin(Q4_K, E * nff, d, up), gpu.lin(dty, E * d, nff, down)
    y0 = pkg.synth.normal_f32(T * d, "moer", "y0").reshape(T, d)
    ya = gpu.upload(np.concatenate([y0.ravel(), np.full(d, 12345.5, np.float32)]))
    gpu.moe_ffn(gpu.upload(x), T, d, nff, E, ksel, idx_d, wgt_d, lg_, lu_, ld_, ya, accum=accum)
    want = gpu.read(ya, T * d + d)
    yb = gpu.upload(np.concatenate([y0.ravel(), np.full(d, 12345.5, np.float32)]))
    idx2, wgt2 = gpu.upload_bytes(np.full(T * ksel + 2, 0xFFFFFFFF, np.uint32)), gpu.upload(np.full(T * ksel + 2, 777.0, np.float32))
    gpu.moe_ffn_routed(gpu.upload(x), T, d, nff, E, ksel, gpu.upload(lg), idx2, wgt2, lg_, lu_, ld_, yb, accum=accum)
    assert np.array_equal(gpu.read(idx2, T * ksel + 2, np.uint32), np.concatenate([gi.ravel(), [0xFFFFFFFF, 0xFFFFFFFF]]))
    assert np.array_equal(gpu.read(wgt2, T * ksel + 2), np.concatenate([gw.ravel(), [777.0, 777.0]]))
    assert np.array_equal(gpu.read(yb, T * d + d), want)
    assert peak_err(want[:T * d].reshape(T, d) - (y0 if accum else 0.0), orc.moe_ffn(x, gi, gw, gate, up, Q4_K, down, dty, E, nff)) <= 2e-5


@pytest.mark.parametrize("T,E,ksel,d,nff,accum", [(40, 4, 2, 512, 768, False), (9, 16, 3, 2304, 256, True),
                                                   (130, 6, 5, 1024, 1280, False), (64, 128, 8, 2048, 768, False)])
def test_matrix_core_forms_agree(gpu, orc, pkg, monkeypatch, T, E, ksel, d, nff, accum):
    """The two matrix-core forms of the grouped products (a wave per row tile with the expert's tokens
    staged in LDS; a workgroup per tile with K split over its waves) and the grouped integer dots:
    integer sums are exact in all three and the f32 sums over super-blocks associate differently, so
    an int8 code of the intermediate activation may flip between forms.  Experts with no, few, 16 and
    more than 16 assignments (several passes), sampled tokens against the CPU path."""
    gate, up, down = _experts(pkg, E, d, nff, ("mt", E, d, nff))
    x = pkg.synth.normal_f32(T * d, "moe", "mtx", T, d).reshape(T, d)
    lg = pkg.synth.normal_f32(T * E, "moe", "mtlg", T, E).reshape(T, E)
    lg[:, 1] -= 50.0                                    # expert 1 is never chosen
    lg[: T // 2, 0] += 50.0                             # expert 0 takes half the tokens
    gi, gw, _, _ = _route(gpu, lg, ksel)
    y0 = pkg.synth.normal_f32(T * d, "moe", "mty0").reshape(T, d) if accum else np.zeros((T, d), np.float32)
    outs = {}
    for mode in ("1", "4", "2"):
        monkeypatch.setenv("OJAS_HIP_MOE", mode)
        g = pkg.HipGpu(0)
        try:
            lg_, lu_, ld_ = g.lin(Q4_K, E * nff, d, gate), g.lin(Q4_K, E * nff, d, up), g.lin(Q4_K, E * d, nff, down)
            yd = g.upload(np.concatenate([y0.ravel(), np.full(d, 12345.5, np.float32)]))
            g.moe_ffn(g.upload(x), T, d, nff, E, ksel, g.upload_bytes(gi), g.upload(gw), lg_, lu_, ld_, yd, accum=accum)
            got = g.read(yd, T * d + d)
            assert np.all(got[T * d:] == 12345.5), "wrote past the last token"
            outs[mode] = got[:T * d].reshape(T, d) - y0
        finally:
            g.close()
    for t in (0, T // 2, T - 1):
        want = orc.moe_ffn(x[t:t + 1], gi[t:t + 1], gw[t:t + 1], gate, up, Q4_K, down, Q4_K, E, nff, mode=0)
        assert peak_err(outs["1"][t], want[0]) <= TOL_SEEN, t
    assert peak_err(outs["1"], outs["4"]) <= TOL
    assert peak_err(outs["1"], outs["2"]) <= TOL


@pytest.mark.parametrize("T,E,ksel,d,nff", [(1, 16, 4, 512, 768), (3, 8, 8, 2304, 256), (20, 8, 3, 512, 768),
                                             (70, 4, 2, 256, 2304), (5, 8, 2, 300 * 256 // 100, 1280)])
@pytest.mark.parametrize("dty", [13, 14])
def test_expert_ffn_with_q5k_down_tensors(gpu, orc, pkg, T, E, ksel, d, nff, dty):
    """Expert `down` tensors in Q5_K or Q6_K (dot_q5k / dot_q6k, crates/ojas-cpu/src/cpu_math.rs:638-722)
    beside Q4_K gate / up: the decode form, the grouped integer dots (short rows of 1 to 3 super-blocks,
    up to 8, and longer), and a batch large enough that gate / up run on the matrix cores while down stays
    on integer dots."""
    gate = pkg.synth.q4k_weights(E * nff, d, "moe5", "gate", E, d, nff)
    up = pkg.synth.q4k_weights(E * nff, d, "moe5", "up", E, d, nff)
    down = pkg.synth.weights(dty, E * d, nff, "moe5", "down", E, d, nff, dty)
    x = pkg.synth.normal_f32(T * d, "moe5", "x", T, d).reshape(T, d)
    lg = pkg.synth.normal_f32(T * E, "moe5", "lg", T, E).reshape(T, E)
    gi, gw, idx_d, wgt_d = _route(gpu, lg, ksel)
    lg_, lu_, ld_ = gpu.lin(Q4_K, E * nff, d, gate), gpu.lin(Q4_K, E * nff, d, up), gpu.lin(dty, E * d, nff, down)
    yd = gpu.upload(np.full(T * d + d, 12345.5, np.float32))
    gpu.moe_ffn(gpu.upload(x), T, d, nff, E, ksel, idx_d, wgt_d, lg_, lu_, ld_, yd)
    got = gpu.read(yd, T * d + d)
    assert np.all(got[T * d:] == 12345.5), "wrote past the last token"
    want = orc.moe_ffn(x, gi, gw, gate, up, Q4_K, down, dty, E, nff, mode=0)
    assert peak_err(got[:T * d].reshape(T, d), want) <= TOL


@pytest.mark.parametrize("T,E,ksel,d,nff,accum", [(1, 128, 8, 2048, 768, False), (3, 16, 5, 2304, 512, True),
                                                   (9, 6, 2, 256, 256, False)])
def test_streamed_experts_by_slot_offsets(gpu, pkg, T, E, ksel, d, nff, accum):
    """Experts scattered over an arena in cache-slot order, addressed by one byte offset per
    assignment (crates/ojas-cuda/src/kernels/moe.rs:133-174): the same bits as the resident,
    index-addressed decode form on the same experts; an offset past the arena is clamped, not read."""
    gate, up, down = _experts(pkg, E, d, nff, ("slots", E, d, nff))
    x = pkg.synth.normal_f32(T * d, "moe", "sx", T, d).reshape(T, d)
    lg = pkg.synth.normal_f32(T * E, "moe", "slg", T, E).reshape(T, E)
    gi, gw, idx_d, wgt_d = _route(gpu, lg, ksel)
    y0 = pkg.synth.normal_f32(T * d, "moe", "sy0").reshape(T, d)
    monkey = pytest.MonkeyPatch()
    monkey.setenv("OJAS_HIP_MOE", "3")
    g = pkg.HipGpu(0)
    try:
        lg_, lu_, ld_ = g.lin(Q4_K, E * nff, d, gate), g.lin(Q4_K, E * nff, d, up), g.lin(Q4_K, E * d, nff, down)
        yr = g.upload(y0)
        g.moe_ffn(g.upload(x), T, d, nff, E, ksel, g.upload_bytes(gi), g.upload(gw), lg_, lu_, ld_, yr, accum=accum)
        want = g.read(yr, T * d)
    finally:
        g.close()
        monkey.undo()
    # an arena per tensor: the experts in a shuffled slot order, 4 KiB of padding in front
    eb_gu, eb_d = nff * (d // 256) * 144, d * (nff // 256) * 144
    perm = pkg.synth.rng("slots", E).permutation(E)
    slot_of = np.empty(E, np.int64)
    slot_of[perm] = np.arange(E)
    pad = 4096

    def arena(raw, eb):
        a = np.zeros(pad + E * eb, np.uint8)
        for s_, e in enumerate(perm):
            a[pad + s_ * eb:pad + (s_ + 1) * eb] = raw[e * eb:(e + 1) * eb]
        return a
    ag, au, ad = gpu.upload_bytes(arena(gate, eb_gu)), gpu.upload_bytes(arena(up, eb_gu)), gpu.upload_bytes(arena(down, eb_d))
    sel = np.asarray(gi, np.int64).reshape(-1)
    og = (pad + slot_of[sel] * eb_gu).astype(np.uint64)
    od = (pad + slot_of[sel] * eb_d).astype(np.uint64)
    yd = gpu.upload(np.concatenate([y0.ravel(), np.full(d, 12345.5, np.float32)]))
    gpu.moe_ffn_slots(gpu.upload(x), T, d, nff, ksel, ag, gpu.upload_bytes(og), au, gpu.upload_bytes(og), ad,
                      gpu.upload_bytes(od), wgt_d, yd, accum=accum)
    got = gpu.read(yd, T * d + d)
    assert np.all(got[T * d:] == 12345.5), "wrote past the last token"
    assert np.array_equal(got[:T * d], want)
    # offsets far outside the arenas: clamped to the last slot, the launch completes
    bad = np.full(T * ksel, 1 << 40, np.uint64)
    gpu.moe_ffn_slots(gpu.upload(x), T, d, nff, ksel, ag, gpu.upload_bytes(bad), au, gpu.upload_bytes(bad), ad,
                      gpu.upload_bytes(bad), wgt_d, yd)
    assert np.all(np.isfinite(gpu.read(yd, T * d)))
    with pytest.raises(pkg.OjasHipError, match="needs"):
        gpu.moe_ffn_slots(gpu.upload(x), T, d, nff, ksel, ag, gpu.upload_bytes(og[:-1]), au, gpu.upload_bytes(og), ad,
                          gpu.upload_bytes(od), wgt_d, yd)


def _rel_err(got, want):
    """The reference's per-element measure (crates/ojas-cuda/tests/conformance.rs:215-220)."""
    return float(np.max(np.abs(got - want) / np.maximum(np.abs(want), 1e-6)))


def test_q80_experts_reference_procedure(gpu, pkg):
    """Q8_0 experts through `moe_gu_q80` and `moe_down_q80` with the reference's own arguments and
    launch geometry (crates/ojas-cuda/tests/conformance.rs:412-457): E=8, K=256, N=64, experts {3, 6}
    weighted {0.7, 0.3}, against the plain products of the decoded values, bound 2e-3 per element."""
    k, n, experts, ksel = 256, 64, 8, 2
    x = pkg.synth.tvec(k, 61)
    gbytes, gplain = pkg.synth.q80_rows_lcg(experts * n, k, 62)
    ubytes, uplain = pkg.synth.q80_rows_lcg(experts * n, k, 63)
    dbytes, dplain = pkg.synth.q80_rows_lcg(experts * k, n, 64)
    idx, wgt = np.array([3, 6], np.uint32), np.array([0.7, 0.3], np.float32)
    want = np.zeros(k, np.float64)
    x64 = x.astype(np.float64)
    for j, e in enumerate(idx):
        gv = gplain[e * n:(e + 1) * n].astype(np.float64) @ x64
        uv = uplain[e * n:(e + 1) * n].astype(np.float64) @ x64
        act = gv / (1.0 + np.exp(-gv)) * uv
        want += float(wgt[j]) * (dplain[e * k:(e + 1) * k].astype(np.float64) @ act)
    gpu.ensure_family("moe")
    xd, gd, ud, dd = gpu.upload(x), gpu.upload_bytes(gbytes), gpu.upload_bytes(ubytes), gpu.upload_bytes(dbytes)
    idxd, wgtd = gpu.upload_bytes(idx), gpu.upload(wgt)
    actd, outd = gpu.alloc(ksel * n), gpu.upload(np.zeros(k, np.float32))
    enc = gpu.begin()
    gpu.dispatch(enc, "moe_gu_q80", [(xd, 0), (gd, 0), (ud, 0), (actd, 0), (idxd, 0)], [k, n], [-(-n // 8), ksel, 1], [256, 1, 1])
    gpu.dispatch(enc, "moe_down_q80", [(actd, 0), (dd, 0), (outd, 0), (idxd, 0), (wgtd, 0)], [n, k, ksel],
                 [-(-k // 32), 1, 1], [256, 1, 1])
    gpu.submit(enc)
    got = gpu.read(outd, k)
    assert _rel_err(got, want.astype(np.float32)) < 2e-3
    assert peak_err(got, want) <= 2e-6
    # the geometry the library itself names gives the same bits, and the down launch accumulates
    g2, b2 = gpu.launch_shape("moe_down_q80", n, k, 1)
    assert g2 == [-(-k // 4), 1, 1] and b2 == [256, 1, 1]
    out2 = gpu.upload(np.ones(k, np.float32))
    gpu.dispatch(gpu.begin(), "moe_down_q80", [(actd, 0), (dd, 0), (out2, 0), (idxd, 0), (wgtd, 0)], [n, k, ksel], g2, b2)
    assert np.array_equal(gpu.read(out2, k), np.float32(1.0) + got)
    # an index past the tensors multiplies nothing: the same as that slot with weight zero
    bad = gpu.upload_bytes(np.array([3, experts], np.uint32))
    act3, out3, out4 = gpu.alloc(ksel * n), gpu.upload(np.zeros(k, np.float32)), gpu.upload(np.zeros(k, np.float32))
    gpu.dispatch(gpu.begin(), "moe_gu_q80", [(xd, 0), (gd, 0), (ud, 0), (act3, 0), (bad, 0)], [k, n], [-(-n // 8), ksel, 1], [256, 1, 1])
    gpu.dispatch(gpu.begin(), "moe_down_q80", [(act3, 0), (dd, 0), (out3, 0), (bad, 0), (wgtd, 0)], [n, k, ksel], g2, b2)
    assert np.all(gpu.read(act3, ksel * n)[n:] == 0.0)
    w0 = gpu.upload(np.array([0.7, 0.0], np.float32))
    gpu.dispatch(gpu.begin(), "moe_down_q80", [(actd, 0), (dd, 0), (out4, 0), (idxd, 0), (w0, 0)], [n, k, ksel], g2, b2)
    assert np.array_equal(gpu.read(out3, k), gpu.read(out4, k))
    with pytest.raises(pkg.OjasHipError, match="needs"):
        gpu.dispatch(gpu.begin(), "moe_down_q80", [(actd, 0), (dd, len(dbytes) - 34), (out3, 0), (idxd, 0), (wgtd, 0)],
                     [n, k, ksel], g2, b2)


@pytest.mark.parametrize("T,E,ksel,d,nff,accum", [(1, 8, 2, 256, 64, False), (5, 16, 4, 512, 352, True),
                                                   (40, 8, 8, 1024, 768, False), (3, 4, 1, 2080, 96, True)])
def test_q80_experts_through_the_ffn_entry(gpu, orc, pkg, T, E, ksel, d, nff, accum):
    """The same kernels under `ojh_moe_ffn`, many tokens in one launch, against the CPU path's f32
    products over Q8_0 rows (crates/ojas-cpu/src/cpu_math.rs:971-981 under cpu_glm.rs:551-582)."""
    gate = pkg.synth.q80_weights(E * nff, d, "moe8", "gate", E, d, nff)
    up = pkg.synth.q80_weights(E * nff, d, "moe8", "up", E, d, nff)
    down = pkg.synth.q80_weights(E * d, nff, "moe8", "down", E, d, nff)
    x = pkg.synth.normal_f32(T * d, "moe8", "x", T, d).reshape(T, d)
    lg = pkg.synth.normal_f32(T * E, "moe8", "lg", T, E).reshape(T, E)
    gi, gw, idx_d, wgt_d = _route(gpu, lg, ksel)
    # the running output is given the products' own magnitude, so its f32 rounding does not mask theirs
    y0 = np.float32(0.01) * pkg.synth.normal_f32(T * d, "moe8", "y0").reshape(T, d) if accum else np.zeros((T, d), np.float32)
    init = np.concatenate([y0.ravel() if accum else np.full(T * d, 777.0, np.float32), np.full(d, 12345.5, np.float32)])
    yd = gpu.alloc(T * d + d)
    lg_, lu_, ld_ = gpu.lin(Q8_0, E * nff, d, gate), gpu.lin(Q8_0, E * nff, d, up), gpu.lin(Q8_0, E * d, nff, down)
    want = orc.moe_ffn(x, gi, gw, gate, up, Q8_0, down, Q8_0, E, nff, mode=0, y0=y0)
    for mode in (pkg.ACT_AUTO, pkg.ACT_FLOAT):
        gpu.write_bytes(yd, 0, init)
        gpu.moe_ffn(gpu.upload(x), T, d, nff, E, ksel, idx_d, wgt_d, lg_, lu_, ld_, yd, accum=accum, act_mode=mode)
        got = gpu.read(yd, T * d + d)
        assert np.all(got[T * d:] == 12345.5), "wrote past the last token"
        # a batch under ACT_AUTO runs grouped on the f16 matrix tile: activations rounded to f16 on the way in
        tiled = mode == pkg.ACT_AUTO and T * ksel >= 4 * E and d % 64 == 0 and nff % 64 == 0
        assert peak_err(got[:T * d].reshape(T, d) - y0, want - y0) <= (1e-3 if tiled else 2e-5)
    with pytest.raises(pkg.OjasHipError, match="f32 activations"):
        gpu.moe_ffn(gpu.upload(x), T, d, nff, E, ksel, idx_d, wgt_d, lg_, lu_, ld_, yd, act_mode=pkg.ACT_Q8K)


@pytest.mark.parametrize("T,E,ksel,d,nff,accum", [(300, 4, 2, 512, 320, False), (130, 16, 3, 256, 768, True)])
def test_q80_experts_in_batches_on_the_grouped_matrix_tile(gpu, orc, pkg, T, E, ksel, d, nff, accum):
    """From 4 assignments per expert `ojh_moe_ffn(..., OJH_ACT_AUTO)` groups Q8_0 experts' products on the f16 matrix
    tile (experts with one and several 128-token tiles, ragged last tiles, N no multiple of 128): sampled tokens
    against the f32 products of the CPU path, every token against the per-assignment kernels (OJH_ACT_FLOAT)."""
    gate = pkg.synth.q80_weights(E * nff, d, "moe8t", "gate", E, d, nff)
    up = pkg.synth.q80_weights(E * nff, d, "moe8t", "up", E, d, nff)
    down = pkg.synth.q80_weights(E * d, nff, "moe8t", "down", E, d, nff)
    x = pkg.synth.normal_f32(T * d, "moe8t", "x", T, d).reshape(T, d)
    lg = pkg.synth.normal_f32(T * E, "moe8t", "lg", T, E).reshape(T, E)
    lg[:, 1] += 1.5                                     # a popular expert
    gi, gw, idx_d, wgt_d = _route(gpu, lg, ksel)
    y0 = np.float32(0.01) * pkg.synth.normal_f32(T * d, "moe8t", "y0").reshape(T, d) if accum else np.zeros((T, d), np.float32)
    lg_, lu_, ld_ = gpu.lin(Q8_0, E * nff, d, gate), gpu.lin(Q8_0, E * nff, d, up), gpu.lin(Q8_0, E * d, nff, down)
    outs = {}
    for mode in (pkg.ACT_AUTO, pkg.ACT_FLOAT):
        yd = gpu.upload(np.concatenate([y0.ravel() if accum else np.full(T * d, 777.0, np.float32), np.full(d, 12345.5, np.float32)]))
        gpu.moe_ffn(gpu.upload(x), T, d, nff, E, ksel, idx_d, wgt_d, lg_, lu_, ld_, yd, accum=accum, act_mode=mode)
        got = gpu.read(yd, T * d + d)
        assert np.all(got[T * d:] == 12345.5), "wrote past the last token"
        outs[mode] = got[:T * d].reshape(T, d) - y0
    assert gpu.has_kernel("moe_mm_q8_0"), "the tile was not taken"
    assert peak_err(outs[pkg.ACT_AUTO], outs[pkg.ACT_FLOAT]) <= 1e-3
    for t in (0, T // 2, T - 1):
        want = orc.moe_ffn(x[t:t + 1], gi[t:t + 1], gw[t:t + 1], gate, up, Q8_0, down, Q8_0, E, nff, mode=0)
        assert peak_err(outs[pkg.ACT_AUTO][t], want[0]) <= 1e-3, t
        assert peak_err(outs[pkg.ACT_FLOAT][t], want[0]) <= 2e-5, t


@pytest.mark.parametrize("fmt,tile", [(Q8_0, "moe_mm_q8_0"), (IQ4_NL, "moe_mm_iq4nl"), (IQ4_XS, "moe_mm_iq4xs"),
                                      (Q8_0, "moe_few_q8_0"), (IQ4_NL, "moe_few_iq4nl"), (IQ4_XS, "moe_few_iq4xs")])
def test_grouped_f16_tile_by_name(gpu, orc, pkg, fmt, tile):
    """`moe_mm_<fmt>(xh, w0, w1, y0, y1, offsets, list, K, N, NA, E, DIV)`: a pair of tensors in one launch (gate and up:
    assignment a reads token a / DIV) and a single tensor (down: DIV = 1, NULL second tensor); an empty expert; any
    number of token tiles in the grid gives the same bits; every row against the f64 product of the exact block values
    with the f16-rounded activations."""
    E, n, k, div = 3, 200, 256, 2
    bn = 64 if tile.startswith("moe_few") else 128      # rows per workgroup (the few-token form: 32 assignments per pass)
    counts = [150, 0, 38]
    na = sum(counts)
    tokens = na // div
    w0, w1 = pkg.synth.weights(fmt, E * n, k, "moemm", "w0"), pkg.synth.weights(fmt, E * n, k, "moemm", "w1")
    x = pkg.synth.normal_f32(tokens * k, "moemm", "x").reshape(tokens, k)
    xh = x.astype(np.float16)
    perm = pkg.synth.rng("moemm", "perm").permutation(na).astype(np.uint32)
    offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.uint32)
    gpu.ensure_family("gemm")
    xd, od, ld = gpu.upload_bytes(xh.view(np.uint8)), gpu.upload_bytes(offsets), gpu.upload_bytes(perm)
    w0d, w1d = gpu.upload_bytes(w0), gpu.upload_bytes(w1)
    rb = len(w0) // (E * n)
    seen = []
    for tiles in (1, 2, 5):
        y0d, y1d = (gpu.upload(np.full(na * n + n, 777.25, np.float32)) for _ in range(2))
        gpu.dispatch(gpu.begin(), tile, [(xd, 0), (w0d, 0), (w1d, 0), (y0d, 0), (y1d, 0), (od, 0), (ld, 0)],
                     [k, n, na, E, div], [(n + bn - 1) // bn, tiles, 2 * E], [256, 1, 1])
        g0, g1 = gpu.read(y0d, na * n + n), gpu.read(y1d, na * n + n)
        assert np.all(g0[na * n:] == np.float32(777.25)) and np.all(g1[na * n:] == np.float32(777.25))
        seen.append(np.stack([g0[:na * n], g1[:na * n]]).reshape(2, na, n).view(np.uint32).copy())
    for other in seen[1:]:
        assert np.array_equal(seen[0], other)
    got = seen[0].view(np.float32)
    for e in range(E):
        for i in list(range(offsets[e], offsets[e + 1]))[::7]:
            a = int(perm[i])
            for which, w in enumerate((w0, w1)):
                want = orc.matmul_ref(w[e * n * rb:(e + 1) * n * rb], fmt, n, k, xh[a // div].astype(np.float32)[None, :], wmode=1)[0]
                assert peak_err(got[which, a], want) <= 1e-5, (e, a, which)
    # a single tensor: per-assignment activation rows (DIV = 1), the second tensor and output NULL
    xa = pkg.synth.normal_f32(na * k, "moemm", "xa").reshape(na, k).astype(np.float16)
    yd = gpu.upload(np.full(na * n + n, 777.25, np.float32))
    gpu.dispatch(gpu.begin(), tile, [(gpu.upload_bytes(xa.view(np.uint8)), 0), (w0d, 0), (None, 0), (yd, 0), (None, 0), (od, 0), (ld, 0)],
                 [k, n, na, E, 1], [(n + bn - 1) // bn, 2, E], [256, 1, 1])
    g = gpu.read(yd, na * n + n)
    assert np.all(g[na * n:] == np.float32(777.25))
    g = g[:na * n].reshape(na, n)
    for e in (0, 2):
        for i in list(range(offsets[e], offsets[e + 1]))[::11]:
            a = int(perm[i])
            want = orc.matmul_ref(w0[e * n * rb:(e + 1) * n * rb], fmt, n, k, xa[a].astype(np.float32)[None, :], wmode=1)[0]
            assert peak_err(g[a], want) <= 1e-5, (e, a)
    with pytest.raises(pkg.OjasHipError, match="grid must be"):
        gpu.dispatch(gpu.begin(), tile, [(xd, 0), (w0d, 0), (w1d, 0), (gpu.alloc(na * n), 0), (gpu.alloc(na * n), 0), (od, 0), (ld, 0)],
                     [k, n, na, E, div], [(n + bn - 1) // bn, 1, E + 1], [256, 1, 1])


@pytest.mark.parametrize("T,E,ksel,k,n", [(1, 8, 2, 256, 64), (3, 6, 4, 512, 224)])
def test_q80_streamed_experts_by_byte_offsets(gpu, pkg, T, E, ksel, k, n):
    """`moe_gu_q80_slots` / `moe_down_q80_slots` (crates/ojas-cuda/src/kernels/moe.rs:133-174): experts at shuffled
    slots of an arena, one u32 byte offset per selected expert — the same bits as the index-addressed kernels
    on the same experts; an offset past the arena is clamped, never read."""
    gate = pkg.synth.q80_weights(E * n, k, "slots8", "gate", E, k, n)
    up = pkg.synth.q80_weights(E * n, k, "slots8", "up", E, k, n)
    down = pkg.synth.q80_weights(E * k, n, "slots8", "down", E, k, n)
    x = pkg.synth.normal_f32(T * k, "slots8", "x", T, k)
    g = pkg.synth.rng("slots8", T, E)
    idx = np.stack([g.permutation(E)[:ksel] for _ in range(T)]).astype(np.uint32)
    wgt = g.random((T, ksel)).astype(np.float32)
    gpu.ensure_family("moe")
    xd, idxd, wgtd = gpu.upload(x), gpu.upload_bytes(idx), gpu.upload(wgt)
    act1, y1 = gpu.alloc(T * ksel * n), gpu.upload(np.ones(T * k, np.float32))
    gd, ud, dd = gpu.upload_bytes(gate), gpu.upload_bytes(up), gpu.upload_bytes(down)
    gpu.dispatch(gpu.begin(), "moe_gu_q80", [(xd, 0), (gd, 0), (ud, 0), (act1, 0), (idxd, 0)], [k, n], [-(-n // 8), ksel, T], [256, 1, 1])
    gpu.dispatch(gpu.begin(), "moe_down_q80", [(act1, 0), (dd, 0), (y1, 0), (idxd, 0), (wgtd, 0)], [n, k, ksel], [-(-k // 16), T, 1], [256, 1, 1])
    # arenas: the experts in a shuffled order behind 70 bytes of padding (block alignment is two bytes)
    eb_gu, eb_d, pad = n * (k // 32) * 34, k * (n // 32) * 34, 70
    perm = g.permutation(E)
    slot_of = np.empty(E, np.int64)
    slot_of[perm] = np.arange(E)
    arena = lambda w, eb: np.concatenate([np.full(pad, 0xEE, np.uint8), w.reshape(E, eb)[perm].reshape(-1)])
    ag, au, ad = gpu.upload_bytes(arena(gate, eb_gu)), gpu.upload_bytes(arena(up, eb_gu)), gpu.upload_bytes(arena(down, eb_d))
    og = (pad + slot_of[idx] * eb_gu).astype(np.uint32)
    od = (pad + slot_of[idx] * eb_d).astype(np.uint32)
    act2, y2 = gpu.alloc(T * ksel * n), gpu.upload(np.ones(T * k, np.float32))
    ogd, odd = gpu.upload_bytes(og), gpu.upload_bytes(od)
    gpu.dispatch(gpu.begin(), "moe_gu_q80_slots", [(xd, 0), (ag, 0), (au, 0), (act2, 0), (ogd, 0), (ogd, 0)], [k, n], [-(-n // 8), ksel, T], [256, 1, 1])
    gpu.dispatch(gpu.begin(), "moe_down_q80_slots", [(act2, 0), (ad, 0), (y2, 0), (odd, 0), (wgtd, 0)], [n, k, ksel], [-(-k // 8), T, 1], [256, 1, 1])
    assert np.array_equal(gpu.read(act1, T * ksel * n), gpu.read(act2, T * ksel * n))
    assert np.array_equal(gpu.read(y1, T * k), gpu.read(y2, T * k))
    # offsets far past the arena: clamped to the last whole expert, finite output, no fault
    wild = gpu.upload_bytes(np.full((T, ksel), 0xFFFFFFF0, np.uint32))
    y3 = gpu.upload(np.zeros(T * k, np.float32))
    gpu.dispatch(gpu.begin(), "moe_gu_q80_slots", [(xd, 0), (ag, 0), (au, 0), (act2, 0), (wild, 0), (wild, 0)], [k, n], [-(-n // 8), ksel, T], [256, 1, 1])
    gpu.dispatch(gpu.begin(), "moe_down_q80_slots", [(act2, 0), (ad, 0), (y3, 0), (wild, 0), (wgtd, 0)], [n, k, ksel], [-(-k // 8), T, 1], [256, 1, 1])
    assert np.all(np.isfinite(gpu.read(y3, T * k)))
    with pytest.raises(pkg.OjasHipError, match="needs"):
        gpu.dispatch(gpu.begin(), "moe_down_q80_slots", [(act2, 0), (ad, pad + (E - 1) * eb_d + 2), (y3, 0), (odd, 0), (wgtd, 0)],
                     [n, k, ksel], [-(-k // 8), T, 1], [256, 1, 1])


def test_iq4_experts_reference_procedure(gpu, orc, pkg):
    """IQ4_XS gate/up and IQ4_NL down through `moe_gu_iq4xs` / `moe_down_iq4nl` of family "moe_iq" with the
    reference's arguments and launch geometry (crates/ojas-cuda/tests/conformance.rs:505-560): E=8, K=512,
    N=256, experts {1, 5} weighted {0.6, 0.4}, against the products of the values `dequant_to_f16` decodes,
    largest deviation over the peak below 5e-3 as there (the f16 rounding of the decoded weights is most of it)."""
    k, n, experts, ksel = 512, 256, 8, 2
    x = pkg.synth.tvec(k, 71)
    gbytes = pkg.synth.iq4_rows_lcg(IQ4_XS, experts * n, k, 72)
    ubytes = pkg.synth.iq4_rows_lcg(IQ4_XS, experts * n, k, 73)
    dbytes = pkg.synth.iq4_rows_lcg(IQ4_NL, experts * k, n, 74)
    plain = lambda b, ty, rows, cols: orc.dequant_to_f16(b, ty, rows * cols).view(np.float16).astype(np.float64).reshape(rows, cols)
    gplain, uplain, dplain = plain(gbytes, IQ4_XS, experts * n, k), plain(ubytes, IQ4_XS, experts * n, k), plain(dbytes, IQ4_NL, experts * k, n)
    idx, wgt = np.array([1, 5], np.uint32), np.array([0.6, 0.4], np.float32)
    want = np.zeros(k, np.float64)
    silu = lambda v: v / (1.0 + np.exp(np.minimum(-v, 700.0)))      # random sub-scales make some gates very negative
    for j, e in enumerate(idx):
        gv, uv = gplain[e * n:(e + 1) * n] @ x.astype(np.float64), uplain[e * n:(e + 1) * n] @ x.astype(np.float64)
        want += float(wgt[j]) * (dplain[e * k:(e + 1) * k] @ (silu(gv) * uv))
    gpu.ensure_family("moe_iq")
    xd, gd, ud, dd = gpu.upload(x), gpu.upload_bytes(gbytes), gpu.upload_bytes(ubytes), gpu.upload_bytes(dbytes)
    idxd, wgtd = gpu.upload_bytes(idx), gpu.upload(wgt)
    actd, outd = gpu.alloc(ksel * n), gpu.upload(np.zeros(k, np.float32))
    enc = gpu.begin()
    gpu.dispatch(enc, "moe_gu_iq4xs", [(xd, 0), (gd, 0), (ud, 0), (actd, 0), (idxd, 0)], [k, n], [-(-n // 8), ksel, 1], [256, 1, 1])
    gpu.dispatch(enc, "moe_down_iq4nl", [(actd, 0), (dd, 0), (outd, 0), (idxd, 0), (wgtd, 0)], [n, k, ksel], [-(-k // 8), 1, 1], [256, 1, 1])
    gpu.submit(enc)
    got = gpu.read(outd, k)
    assert peak_err(got, want) < 5e-3
    # against the exact values of the same blocks the kernels are much closer
    exact = lambda b, ty, rows, cols: orc.dequant_to_f64(b, ty, rows * cols).reshape(rows, cols)
    ge, ue, de = exact(gbytes, IQ4_XS, experts * n, k), exact(ubytes, IQ4_XS, experts * n, k), exact(dbytes, IQ4_NL, experts * k, n)
    want2 = np.zeros(k, np.float64)
    for j, e in enumerate(idx):
        gv, uv = ge[e * n:(e + 1) * n] @ x.astype(np.float64), ue[e * n:(e + 1) * n] @ x.astype(np.float64)
        want2 += float(wgt[j]) * (de[e * k:(e + 1) * k] @ (silu(gv) * uv))
    assert peak_err(got, want2) <= 1e-5


@pytest.mark.parametrize("tg,td", [(IQ4_XS, IQ4_NL), (IQ4_NL, IQ4_XS), (IQ4_XS, Q8_0), (Q8_0, IQ4_NL)])
@pytest.mark.parametrize("T,E,ksel,d,nff,accum", [(1, 8, 2, 256, 256, False), (6, 16, 4, 512, 768, True), (33, 4, 3, 1024, 256, False)])
def test_iq4_experts_through_the_ffn_entry(gpu, orc, pkg, tg, td, T, E, ksel, d, nff, accum):
    """Any mix of the f32-activation expert formats under `ojh_moe_ffn`, against the CPU path's dots
    (dot_iq4xs / dot_iq4nl / dot_q80 under crates/ojas-cpu/src/cpu_glm.rs:551-582)."""
    gate = pkg.synth.weights(tg, E * nff, d, "moeiq", "gate", tg, E, d, nff)
    up = pkg.synth.weights(tg, E * nff, d, "moeiq", "up", tg, E, d, nff)
    down = pkg.synth.weights(td, E * d, nff, "moeiq", "down", td, E, d, nff)
    x = pkg.synth.normal_f32(T * d, "moeiq", "x", T, d).reshape(T, d)
    lg = pkg.synth.normal_f32(T * E, "moeiq", "lg", T, E).reshape(T, E)
    gi, gw, idx_d, wgt_d = _route(gpu, lg, ksel)
    want0 = orc.moe_ffn(x, gi, gw, gate, up, tg, down, td, E, nff, mode=0)
    peak = float(np.max(np.abs(want0)))
    y0 = np.float32(peak) * pkg.synth.normal_f32(T * d, "moeiq", "y0").reshape(T, d) if accum else np.zeros((T, d), np.float32)
    yd = gpu.upload(np.concatenate([y0.ravel() if accum else np.full(T * d, 777.0, np.float32), np.full(d, 12345.5, np.float32)]))
    lg_, lu_, ld_ = gpu.lin(tg, E * nff, d, gate), gpu.lin(tg, E * nff, d, up), gpu.lin(td, E * d, nff, down)
    gpu.moe_ffn(gpu.upload(x), T, d, nff, E, ksel, idx_d, wgt_d, lg_, lu_, ld_, yd, accum=accum)
    got = gpu.read(yd, T * d + d)
    assert np.all(got[T * d:] == 12345.5), "wrote past the last token"
    # from 4 assignments per expert a batch is grouped on the f16 matrix tile (activations rounded to f16 on the way
    # in); OJH_ACT_FLOAT keeps the per-assignment kernels at every size
    tiled = T * ksel >= 4 * E and d % 64 == 0 and nff % 64 == 0      # (Q8_0 and IQ4 rows: read by the tile's own loaders)
    assert peak_err(got[:T * d].reshape(T, d) - y0, want0) <= (1e-3 if tiled else 2e-5)
    if tiled:
        gpu.write_bytes(yd, 0, np.concatenate([y0.ravel() if accum else np.full(T * d, 777.0, np.float32), np.full(d, 12345.5, np.float32)]))
        gpu.moe_ffn(gpu.upload(x), T, d, nff, E, ksel, idx_d, wgt_d, lg_, lu_, ld_, yd, accum=accum, act_mode=pkg.ACT_FLOAT)
        assert peak_err(gpu.read(yd, T * d).reshape(T, d) - y0, want0) <= 2e-5
    with pytest.raises(pkg.OjasHipError, match="f32 activations"):
        gpu.moe_ffn(gpu.upload(x), T, d, nff, E, ksel, idx_d, wgt_d, lg_, lu_, ld_, yd, act_mode=pkg.ACT_Q8K)


@pytest.mark.parametrize("td", [12, 13, 14])
def test_kquant_experts_on_f32_activations_by_their_reference_names(gpu, orc, pkg, td):
    """`moe_gu_q4k` and `moe_down_{q5k,q6k}` (and this library's `moe_down_q4k`) — the reference's expert table
    (crates/ojas-core/src/quant_src.rs:174-179) — dispatched by name with the Q8_0 pair's argument lists and the
    reference's grids, against products of the exact block values in double (the float contract: f32 activations meet
    the dequantized weights, crates/ojas-metal/src/kernels/moe.rs:497-527, :722-815); then through `ojh_moe_ffn` with
    OJH_ACT_FLOAT."""
    tag = {12: "q4k", 13: "q5k", 14: "q6k"}[td]
    k, n, E, ksel, T = 512, 256, 8, 3, 2
    x = pkg.synth.normal_f32(T * k, "moekq", "x").reshape(T, k)
    gbytes, ubytes = pkg.synth.q4k_weights(E * n, k, "moekq", "g"), pkg.synth.q4k_weights(E * n, k, "moekq", "u")
    dbytes = pkg.synth.weights(td, E * k, n, "moekq", "d", td)
    idx = np.array([[1, 5, 2], [7, 0, 5]], np.uint32)
    wgt = np.array([[0.5, 0.3, 0.2], [0.6, 0.25, 0.15]], np.float32)
    want = orc.moe_ffn(x, idx, wgt, gbytes, ubytes, Q4_K, dbytes, td, E, n, mode=1)
    gpu.ensure_family("moe")
    xd, gd, ud, dd = gpu.upload(x), gpu.upload_bytes(gbytes), gpu.upload_bytes(ubytes), gpu.upload_bytes(dbytes)
    idxd, wgtd = gpu.upload_bytes(idx), gpu.upload(wgt)
    actd, outd = gpu.alloc(T * ksel * n), gpu.upload(np.zeros(T * k, np.float32))
    enc = gpu.begin()
    gpu.dispatch(enc, "moe_gu_q4k", [(xd, 0), (gd, 0), (ud, 0), (actd, 0), (idxd, 0)], [k, n], [-(-n // 8), ksel, T], [256, 1, 1])
    gpu.dispatch(enc, "moe_down_" + tag, [(actd, 0), (dd, 0), (outd, 0), (idxd, 0), (wgtd, 0)], [n, k, ksel], [-(-k // 8), T, 1], [256, 1, 1])
    gpu.submit(enc)
    got = gpu.read(outd, T * k).reshape(T, k)
    assert peak_err(got, want) <= 1e-5
    # the op seam under the float contract, accumulating onto y
    lg_, lu_, ld_ = gpu.lin(Q4_K, E * n, k, gbytes), gpu.lin(Q4_K, E * n, k, ubytes), gpu.lin(td, E * k, n, dbytes)
    y0 = pkg.synth.normal_f32(T * k, "moekq", "y0").reshape(T, k)
    yd = gpu.upload(y0)
    gpu.moe_ffn(xd, T, k, n, E, ksel, idxd, wgtd, lg_, lu_, ld_, yd, accum=True, act_mode=pkg.ACT_FLOAT)
    assert peak_err(gpu.read(yd, T * k).reshape(T, k) - y0, want) <= 1e-5
    # an index past the tensors multiplies nothing
    bad = gpu.upload_bytes(np.array([[1, 99, 2], [7, 0, 5]], np.uint32))
    gpu.memset0(outd)
    gpu.dispatch(enc, "moe_gu_q4k", [(xd, 0), (gd, 0), (ud, 0), (actd, 0), (bad, 0)], [k, n], [-(-n // 8), ksel, T], [256, 1, 1])
    gpu.dispatch(enc, "moe_down_" + tag, [(actd, 0), (dd, 0), (outd, 0), (bad, 0), (wgtd, 0)], [n, k, ksel], [-(-k // 8), T, 1], [256, 1, 1])
    idx2, wgt2 = np.array([[1, 2], [7, 0]], np.uint32), np.array([[0.5, 0.2], [0.6, 0.25]], np.float32)
    want2 = orc.moe_ffn(x[:1], idx2[:1], wgt2[:1], gbytes, ubytes, Q4_K, dbytes, td, E, n, mode=1)
    assert peak_err(gpu.read(outd, k), want2[0]) <= 1e-5


def test_expert_ffn_rejects_what_it_cannot_run(gpu, pkg):
    E, d, nff = 4, 256, 256
    gate, up, down = _experts(pkg, E, d, nff, "err")
    lg_, lu_, ld_ = gpu.lin(Q4_K, E * nff, d, gate), gpu.lin(Q4_K, E * nff, d, up), gpu.lin(Q4_K, E * d, nff, down)
    x, y = gpu.alloc(d), gpu.alloc(d)
    idx, wgt = gpu.upload_bytes(np.array([1, 2], np.uint32)), gpu.upload(np.array([0.5, 0.5], np.float32))
    with pytest.raises(pkg.OjasHipError, match="shapes do not match"):
        gpu.moe_ffn(x, 1, d, nff, E + 1, 2, idx, wgt, lg_, lu_, ld_, y)
    with pytest.raises(pkg.OjasHipError, match="needs"):
        gpu.moe_ffn(x, 2, d, nff, E, 2, idx, wgt, lg_, lu_, ld_, y)
