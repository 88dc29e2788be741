"""The single-launch decode chain (`ojh_decode_chain`): dependent Q4_K stages in one launch, each stage reading what
an earlier one wrote.  Checked three ways: bit for bit against the same stages as separate launches (`ojh_mm_multi`,
`ojh_ffn_gu_q8k`, `ojh_rmsnorm_quant_q8k` + `ojh_mm_q8k_multi`); stage by stage against the CPU oracle's `matvec_kq`
(crates/ojas-cpu/src/cpu_math.rs:1145-1189) on the inputs the GPU actually produced, <= 2e-5 of peak; and against the
oracle applied in sequence from the first input, within the 1e-3 the path is held to.  The bounded wait is made to give
up from the host (limit 0): the call must come back with an error and every kernel must have exited.
"""
import numpy as np
import pytest

from conftest import peak_err

pytestmark = pytest.mark.gpu
Q4_K = 12
TOL = 1e-3          # the bar of the path against the CPU reference
TOL_STAGE = 2e-5    # one stage against matvec_kq on identical inputs


def _bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def _lin(gpu, pkg, n, k, *tag):
    w = pkg.synth.q4k_weights(n, k, "chain", *tag)
    return w, gpu.lin(Q4_K, n, k, w)


def _oracle_stage(orc, x, ws, shapes):
    return [orc.matvec_kq(w, Q4_K, n, k, x) for w, (n, k) in zip(ws, shapes)]


# (hidden, kv rows, feed-forward rows, head rows): a small model, one with ragged tails (odd row counts, a K that is
# not a multiple of 2048), one with a feed-forward width that needs all four input segments per wave
@pytest.mark.parametrize("d,nkv,nff,nhead", [(1024, 256, 1536, 5000), (2304, 131, 2560, 7001), (512, 64, 14336, 1031)])
def test_dependent_chain_is_the_separate_launches_bit_for_bit(gpu, orc, pkg, d, nkv, nff, nhead):
    R = pkg.runtime
    shapes = dict(q=(d, d), k=(nkv, d), v=(nkv, d), o=(d, d), gate=(nff, d), up=(nff, d), down=(d, nff), head=(nhead, d))
    host, lin = {}, {}
    for name, (n, k) in shapes.items():
        host[name], lin[name] = _lin(gpu, pkg, n, k, name, n, k)
    x0h = pkg.synth.normal_f32(d, "chain", "x0", d)
    gammah = (1.0 + 0.1 * pkg.synth.normal_f32(d, "chain", "gamma", d)).astype(np.float32)
    x0, gamma = gpu.upload(x0h), gpu.upload(gammah)
    eps = 1e-5

    def fresh():
        return {n: gpu.upload(np.full(shapes[n][0] + 3, 77.0, np.float32)) for n in shapes}

    # ---- separate launches: x0 -> q,k,v; q -> o; rmsnorm(o) -> gate,up; silu(gate)*up -> down; rmsnorm(down) -> head
    ya = fresh()
    gpu.mm_multi(x0, [lin["q"], lin["k"], lin["v"]], [ya["q"], ya["k"], ya["v"]])
    gpu.mm_multi(ya["q"], [lin["o"]], [ya["o"]])
    xq, xs = gpu.alloc_bytes(d), gpu.alloc(d // 256)
    gpu.rmsnorm_quant_q8k(ya["o"], gamma, eps, 1, d, xq, xs)
    gpu.mm_q8k_multi(xq, xs, [lin["gate"], lin["up"]], [ya["gate"], ya["up"]])
    act = gpu.alloc(nff)
    gpu.ffn_gu_q8k(xq, xs, lin["gate"], lin["up"], act)
    gpu.mm_multi(act, [lin["down"]], [ya["down"]])
    gpu.rmsnorm_quant_q8k(ya["down"], gamma, eps, 1, d, xq, xs)
    gpu.mm_q8k_multi(xq, xs, [lin["head"]], [ya["head"]])
    gpu.submit()
    sep = {n: gpu.read(ya[n], shapes[n][0] + 3) for n in shapes}

    # ---- the same as one launch, twice (the second launch finds the first one's handed-on values in place and must
    # not take them for its own) with a different first input in between
    yb = fresh()
    chain = [dict(x=x0, ws=[lin["q"], lin["k"], lin["v"]], ys=[yb["q"], yb["k"], yb["v"]]),
             dict(x=yb["q"], ws=[lin["o"]], ys=[yb["o"]]),
             dict(x=yb["o"], x2=gamma, prologue=R.CHAIN_X_RMSNORM, eps=eps, ws=[lin["gate"], lin["up"]], ys=[yb["gate"], yb["up"]]),
             dict(x=yb["gate"], x2=yb["up"], prologue=R.CHAIN_X_SILU_MUL, ws=[lin["down"]], ys=[yb["down"]]),
             dict(x=yb["down"], x2=gamma, prologue=R.CHAIN_X_RMSNORM, eps=eps, ws=[lin["head"]], ys=[yb["head"]])]
    other = gpu.upload(-x0h[::-1].copy())
    for attempt in range(2):
        if attempt:
            wrong = [dict(c) for c in chain]
            wrong[0]["x"] = other
            gpu.decode_chain(wrong)
        gpu.decode_chain(chain)
        gpu.submit()
        got = {n: gpu.read(yb[n], shapes[n][0] + 3) for n in shapes}
        for n in shapes:
            assert np.all(got[n][shapes[n][0]:] == 77.0), f"{n}: wrote past its rows"
            assert np.array_equal(_bits(got[n]), _bits(sep[n])), f"{n} differs from the separate launches (attempt {attempt})"

    # ---- each stage against the CPU arithmetic on the inputs the GPU produced, and the whole chain from x0
    g = {n: got[n][:shapes[n][0]] for n in shapes}
    stage_in = dict(q=x0h, k=x0h, v=x0h, o=g["q"], gate=orc.rmsnorm(g["o"], gammah, eps), up=orc.rmsnorm(g["o"], gammah, eps),
                    down=(orc.ffn_act(g["gate"]) * g["up"]).astype(np.float32), head=orc.rmsnorm(g["down"], gammah, eps))
    for n, (rows, k) in shapes.items():
        want = orc.matvec_kq(host[n], Q4_K, rows, k, np.ascontiguousarray(stage_in[n], np.float32))
        assert peak_err(g[n], want) <= TOL_STAGE, n
    c = {n: orc.matvec_kq(host[n], Q4_K, *shapes[n], x0h) for n in ("q", "k", "v")}
    c["o"] = orc.matvec_kq(host["o"], Q4_K, *shapes["o"], c["q"])
    xn = orc.rmsnorm(c["o"], gammah, eps)
    c["gate"], c["up"] = (orc.matvec_kq(host[n], Q4_K, *shapes[n], xn) for n in ("gate", "up"))
    c["down"] = orc.matvec_kq(host["down"], Q4_K, *shapes["down"], (orc.ffn_act(c["gate"]) * c["up"]).astype(np.float32))
    c["head"] = orc.matvec_kq(host["head"], Q4_K, *shapes["head"], orc.rmsnorm(c["down"], gammah, eps))
    for n in shapes:
        assert peak_err(g[n], c[n]) <= TOL, n


def test_accumulating_stages_and_a_part_of_an_output_as_input(gpu, orc, pkg):
    """A feed-forward block as one launch: rmsnorm(resid) -> gate/up, GELU(gate)*up -> down accumulated onto the
    residual, then a second down-sized projection that reads the second half of a stacked output."""
    R = pkg.runtime
    d, nff = 768, 2048
    hg, lg = _lin(gpu, pkg, nff, d, "acc_g")
    hu, lu = _lin(gpu, pkg, nff, d, "acc_u")
    hd, ld = _lin(gpu, pkg, d, nff, "acc_d")
    hp, lp = _lin(gpu, pkg, 300, 1024, "acc_p")
    residh = pkg.synth.normal_f32(d, "chain", "resid")
    gammah = (1.0 + 0.1 * pkg.synth.normal_f32(d, "chain", "acc_gamma")).astype(np.float32)
    gamma = gpu.upload(gammah)
    eps = 1e-6
    # separate launches
    ra = gpu.upload(residh)
    xq, xs = gpu.alloc_bytes(d), gpu.alloc(d // 256)
    gpu.rmsnorm_quant_q8k(ra, gamma, eps, 1, d, xq, xs)
    gu_a = gpu.alloc(2 * nff)                      # gate and up stacked in one buffer
    gpu.mm_q8k_multi(xq, xs, [lg, lu], [gu_a, gu_a], y_offs=[0, nff * 4])
    act = gpu.alloc(nff)
    gpu.ffn_gu_q8k(xq, xs, lg, lu, act, 1)
    gpu.mm_multi(act, [ld], [ra], accum=True)
    pa = gpu.alloc(300)
    gpu.mm_multi(gu_a, [lp], [pa], x_off=(nff + 512) * 4)      # 1024 values out of the up half
    gpu.submit()
    # one launch
    rb, gu_b, pb = gpu.upload(residh), gpu.alloc(2 * nff), gpu.alloc(300)
    gpu.decode_chain([
        dict(x=rb, x2=gamma, prologue=R.CHAIN_X_RMSNORM, eps=eps, ws=[lg, lu], ys=[gu_b, gu_b], y_offs=[0, nff * 4]),
        dict(x=gu_b, x2=gu_b, x2_off=nff * 4, prologue=R.CHAIN_X_GELU_MUL, ws=[ld], ys=[rb], accum=True),
        dict(x=gu_b, x_off=(nff + 512) * 4, ws=[lp], ys=[pb]),
    ])
    gpu.submit()
    for a, b_, n in ((ra, rb, d), (gu_a, gu_b, 2 * nff), (pa, pb, 300)):
        assert np.array_equal(_bits(gpu.read(a, n)), _bits(gpu.read(b_, n)))
    xn = orc.rmsnorm(residh, gammah, eps)
    gv, uv = orc.matvec_kq(hg, Q4_K, nff, d, xn), orc.matvec_kq(hu, Q4_K, nff, d, xn)
    want = residh + orc.matvec_kq(hd, Q4_K, d, nff, (orc.ffn_act(gv, 1) * uv).astype(np.float32))
    assert peak_err(gpu.read(rb, d), want) <= 3e-4 <= TOL
    assert peak_err(gpu.read(pb, 300), orc.matvec_kq(hp, Q4_K, 300, 1024, gpu.read(gu_b, 2 * nff)[nff + 512:nff + 1536])) <= TOL_STAGE


def test_one_stage_and_eight_stages(gpu, orc, pkg):
    k = 1024
    h, l = _lin(gpu, pkg, k, k, "sq")
    xh = pkg.synth.normal_f32(k, "chain", "sqx")
    x = gpu.upload(xh)
    ys = [gpu.alloc(k) for _ in range(8)]
    gpu.decode_chain([dict(x=x, ws=[l], ys=[ys[0]])])
    assert peak_err(gpu.read(ys[0], k), orc.matvec_kq(h, Q4_K, k, k, xh)) <= TOL_STAGE
    gammah = np.ones(k, np.float32)
    gamma = gpu.upload(gammah)
    chain = [dict(x=x, ws=[l], ys=[ys[0]])]
    for s in range(1, 8):   # the norm keeps the magnitudes where they are
        chain.append(dict(x=ys[s - 1], x2=gamma, prologue=pkg.runtime.CHAIN_X_RMSNORM, eps=1e-6, ws=[l], ys=[ys[s]]))
    gpu.decode_chain(chain)
    cur = xh
    for s in range(8):
        got = gpu.read(ys[s], k)
        assert peak_err(got, orc.matvec_kq(h, Q4_K, k, k, cur if s == 0 else orc.rmsnorm(cur, gammah, 1e-6))) <= TOL_STAGE, s
        cur = got
    with pytest.raises(pkg.OjasHipError):
        gpu.decode_chain(chain + [dict(x=ys[7], ws=[l], ys=[ys[0]])])      # nine stages


def test_what_the_chain_refuses(gpu, pkg):
    k = 512
    _, l = _lin(gpu, pkg, k, k, "ref")
    x, y, y2 = gpu.alloc(k), gpu.alloc(k), gpu.alloc(k)
    bad = [
        [dict(x=x, ws=[l], ys=[x])],                                     # output over its own input
        [dict(x=x, ws=[l, l], ys=[y, y])],                               # two outputs over each other
        [dict(x=x, ws=[l], ys=[y]), dict(x=y, x_off=256 * 4, ws=[l], ys=[y2])],   # input straddles the end of an output
        [dict(x=x, prologue=pkg.runtime.CHAIN_X_SILU_MUL, ws=[l], ys=[y])],        # product without its second operand
        [dict(x=x, x_off=4, ws=[l], ys=[y])],                            # misaligned input
    ]
    for stages in bad:
        with pytest.raises(pkg.OjasHipError):
            gpu.decode_chain(stages)
    w6 = pkg.synth.q6k_weights(64, k, "chain", "ref6")
    with pytest.raises(pkg.OjasHipError):
        gpu.decode_chain([dict(x=x, ws=[gpu.lin(pkg.Q6_K, 64, k, w6)], ys=[y])])
    gpu.submit()   # nothing was launched, nothing is pending


def test_a_wait_that_gives_up_reports_and_every_kernel_exits(gpu, orc, pkg):
    """Limit 0: the first wait for a handed-on input gives up at once.  The launch must end by itself, the next
    synchronisation must report it, and with the limit restored the same chain must run and give the right result."""
    k = 1024
    h, l = _lin(gpu, pkg, k, k, "gu")
    xh = pkg.synth.normal_f32(k, "chain", "gux")
    x, y1, y2 = gpu.upload(xh), gpu.alloc(k), gpu.alloc(k)
    chain = [dict(x=x, ws=[l], ys=[y1]), dict(x=y1, ws=[l], ys=[y2])]
    gpu.decode_chain(chain)
    gpu.submit()
    good = gpu.read(y2, k)
    gpu.chain_spin_limit(0)
    try:
        gpu.decode_chain(chain)
        with pytest.raises(pkg.OjasHipError) as err:
            gpu.submit()
        assert err.value.code == -2 and "gave up" in str(err.value)       # OJH_ERR_HIP
        gpu.submit()                                                        # reported once; the device is usable
    finally:
        gpu.chain_spin_limit(1 << 22)
    gpu.decode_chain(chain)
    gpu.submit()
    assert np.array_equal(_bits(gpu.read(y2, k)), _bits(good))
    assert peak_err(gpu.read(y1, k), orc.matvec_kq(h, Q4_K, k, k, xh)) <= TOL_STAGE


def test_recorded_chain_replays(gpu, pkg):
    k = 1024
    _, l = _lin(gpu, pkg, k, k, "rec")
    xh = pkg.synth.normal_f32(k, "chain", "recx")
    x, y1, y2 = gpu.upload(xh), gpu.alloc(k), gpu.alloc(k)
    chain = [dict(x=x, ws=[l], ys=[y1]), dict(x=y1, ws=[l], ys=[y2])]
    gpu.decode_chain(chain)
    gpu.submit()
    want = gpu.read(y2, k)
    gpu.capture_begin()
    gpu.decode_chain(chain)
    graph = gpu.capture_end()
    for rep in range(3):
        gpu.memset0(y2)
        gpu.write_bytes(x, 0, xh * (rep + 2))       # y1 and y2 scale with x only through the quantizer: compare per replay
        graph.launch()
        gpu.submit()
        gpu.write_bytes(x, 0, xh)
        gpu.memset0(y2)
        graph.launch()
        gpu.submit()
        assert np.array_equal(_bits(gpu.read(y2, k)), _bits(want)), rep
