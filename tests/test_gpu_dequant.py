"""Device decoders against the CPU oracle: dequantized weights must be bit-exact."""
import json
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
Q8_0, Q4_K, Q5_K, Q6_K, IQ4_NL, IQ4_XS = 8, 12, 13, 14, 20, 23
Q4_0, Q4_1, Q5_0, Q5_1 = 2, 3, 6, 7
Q2_K, Q3_K = 10, 11
# the reference's own regression digests, kept as a fixture (tests/golden/quant_format_digests.json)
with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "quant_format_digests.json")) as _f:
    _GOLDEN = json.load(_f)["digests"]
DIGESTS = {int(ty): int(row["digest"], 16) for ty, row in _GOLDEN.items()}
COUNTS = {int(ty): row["values"] for ty, row in _GOLDEN.items()}


def _dequant(gpu, ty, raw, n):
    rb = gpu.upload_bytes(raw)
    out = gpu.alloc_bytes(n * 2)
    gpu.dequant_f16(ty, rb, n, out)
    return gpu.read(out, n, np.uint16)


@pytest.mark.parametrize("ty", [Q2_K, Q3_K, Q4_K, Q5_K, Q6_K, IQ4_NL, IQ4_XS])
def test_reference_digests_on_device(gpu, orc, pkg, ty):
    """The reference's own regression digests (crates/ojas-formats/tests/quant_formats.rs:38-48),
    computed over what the GPU decoded."""
    raw = orc.synth_blocks(ty, 40)
    bits = _dequant(gpu, ty, raw, 40 * pkg.synth.BLOCK_SHAPE[ty][1])
    assert orc.digest_f16(bits) == DIGESTS[ty]


@pytest.mark.parametrize("ty,n,k", [(Q8_0, 37, 4096), (Q4_K, 129, 4096), (Q6_K, 65, 4096), (Q5_K, 16, 1024),
                                    (IQ4_NL, 33, 2080), (IQ4_XS, 21, 4096), (Q4_0, 33, 2080), (Q4_1, 9, 4096),
                                    (Q5_0, 33, 2080), (Q5_1, 9, 4096), (Q2_K, 21, 2304), (Q3_K, 33, 4096)])
def test_bit_exact_on_benchmark_distributions(gpu, orc, pkg, ty, n, k):
    raw = orc.synth_blocks(ty, n * k // pkg.synth.BLOCK_SHAPE[ty][1]) if ty == Q5_K else \
        pkg.synth.weights(ty, n, k, "dq", ty)
    got = _dequant(gpu, ty, raw, n * k)
    assert np.array_equal(got, orc.dequant_to_f16(raw, ty, n * k))


@pytest.mark.parametrize("ty", [Q8_0, Q4_K, Q5_K, Q6_K, IQ4_NL, IQ4_XS, Q4_0, Q4_1, Q5_0, Q5_1, Q2_K, Q3_K])
def test_bit_exact_with_extreme_scales(gpu, orc, pkg, ty):
    """Subnormal, tiny, huge and negative f16 scales: every rounding path of the decoder."""
    bb, wpb = pkg.synth.BLOCK_SHAPE[ty]
    scales = np.array([0x0001, 0x0200, 0x03FF, 0x0400, 0x7BFF, 0x8001, 0xBC00, 0x3555, 0x0000, 0x1234], np.uint16)
    nb = scales.size * 3
    raw = orc.synth_blocks(ty, nb).reshape(nb, bb).copy()
    off = {Q6_K: 208, Q2_K: 80, Q3_K: 108}.get(ty, 0)
    for i in range(nb):
        raw[i, off:off + 2] = np.array([scales[i % scales.size]], np.uint16).view(np.uint8)
        if ty in (Q4_K, Q5_K, Q4_1, Q5_1, Q2_K):
            at = 82 if ty == Q2_K else 2
            raw[i, at:at + 2] = np.array([scales[(i * 7 + 3) % scales.size]], np.uint16).view(np.uint8)
    raw = raw.reshape(-1)
    got = _dequant(gpu, ty, raw, nb * wpb)
    want = orc.dequant_to_f16(raw, ty, nb * wpb)
    assert np.array_equal(got, want)


def test_dequant_through_the_kernel_seam(gpu, orc):
    """Same decoder reached by name through dispatch, with an offset into a larger buffer."""
    gpu.ensure_family("dequant")
    assert gpu.has_kernel("dequant_q4k_f16") and not gpu.has_kernel("dequant_q4k_f32")
    raw = orc.synth_blocks(Q4_K, 24)
    pad = 144 * 2
    rb = gpu.upload_bytes(np.concatenate([np.full(pad, 0xEE, np.uint8), raw]))
    out = gpu.upload_bytes(np.full(24 * 256 + 16, 0x7777, np.uint16))
    grid, block = gpu.launch_shape("dequant_q4k_f16", 0, 24)
    enc = gpu.begin()
    gpu.dispatch(enc, "dequant_q4k_f16", [(rb, pad), (out, 16)], [24], grid, block)
    gpu.submit(enc)
    bits = gpu.read(out, 24 * 256 + 16, np.uint16)
    assert np.all(bits[:8] == 0x7777) and np.all(bits[-8:] == 0x7777)
    assert np.array_equal(bits[8:-8], orc.dequant_to_f16(raw, Q4_K, 24 * 256))


def test_relayout_q4k_q4l_is_bit_exact(gpu, orc, pkg):
    """crates/ojas-formats/src/quant.rs:192-222 on the device: nibble pairs, qa, qb all equal to the
    CPU restatement (which the oracle tests pin against the decoder), including extreme scales."""
    n, k = 37, 1024
    raw = orc.synth_blocks(12, n * k // 256).reshape(-1, 144).copy()
    probes = np.array([0x0001, 0x03FF, 0x0400, 0x8001, 0xBC00, 0x3555, 0x7BFF, 0x0000], np.uint16)
    for i in range(raw.shape[0]):
        raw[i, 0:2] = probes[i % 8:i % 8 + 1].view(np.uint8)
        raw[i, 2:4] = probes[(3 * i + 1) % 8:(3 * i + 1) % 8 + 1].view(np.uint8)
    raw = raw.reshape(-1)
    nib, qa, qb = gpu.alloc_bytes(n * k // 2), gpu.alloc_bytes(n * k // 16), gpu.alloc_bytes(n * k // 16)
    gpu.relayout_q4k_q4l(gpu.upload_bytes(raw), n, k, nib, qa, qb)
    wn, wa, wb = orc.relayout_q4k_q4l(raw, k, n)
    assert np.array_equal(gpu.read(nib, n * k // 2, np.uint8), wn)
    assert np.array_equal(gpu.read(qa, n * k // 32, np.uint16), wa)
    assert np.array_equal(gpu.read(qb, n * k // 32, np.uint16), wb)


def test_embed_q80_matches_reader(gpu, orc, pkg):
    """`embed_q80` / `embed_q80_g` gather a row out of Q8_0 storage (crates/ojas-cuda/tests/conformance.rs:738-764:
    vocab 64, d 512, tokens 0, 7, 63, the reference's grid [8] x 128 threads): rounding the output to f16
    reproduces `dequant_to_f16` exactly, and the f32 values are the exact products d * q."""
    vocab, d = 64, 512
    raw = pkg.synth.q80_weights_lcg(vocab, d, 90)
    vals16 = orc.dequant_to_f16(raw, Q8_0, vocab * d).reshape(vocab, d)
    blocks = raw.reshape(vocab, d // 32, 34)
    exact = (blocks[:, :, :2].copy().view(np.float16).astype(np.float32) * blocks[:, :, 2:].view(np.int8).astype(np.float32)).reshape(vocab, d)
    gpu.ensure_family("dequant")
    pad = 34 * 3
    td = gpu.upload_bytes(np.concatenate([np.full(pad, 0xEE, np.uint8), raw]))
    od = gpu.alloc(d + 2)
    ctl = gpu.alloc_bytes(4)
    for token in (0, 7, 63):
        for name in ("embed_q80", "embed_q80_g"):
            gpu.write_bytes(od, 0, np.full(d + 2, 777.0, np.float32))
            if name == "embed_q80":
                gpu.dispatch(gpu.begin(), name, [(td, pad), (od, 4)], [token, d], [8, 1, 1], [128, 1, 1])
            else:
                gpu.write_bytes(ctl, 0, np.array([token], np.uint32))
                gpu.dispatch(gpu.begin(), name, [(td, pad), (od, 4), (ctl, 0)], [d], [8, 1, 1], [128, 1, 1])
            got = gpu.read(od, d + 2)
            assert got[0] == 777.0 and got[-1] == 777.0, "wrote outside the row"
            assert np.array_equal(got[1:-1], exact[token]), (name, token)
            assert np.array_equal(got[1:-1].astype(np.float16).view(np.uint16), vals16[token]), (name, token)
    # the library's own geometry, and an id past the table: zeros, nothing read
    grid, block = gpu.launch_shape("embed_q80", d, 0)
    gpu.dispatch(gpu.begin(), "embed_q80", [(td, pad), (od, 4)], [63, d], grid, block)
    assert np.array_equal(gpu.read(od, d + 2)[1:-1], exact[63])
    gpu.dispatch(gpu.begin(), "embed_q80", [(td, pad), (od, 4)], [64, d], grid, block)
    assert np.all(gpu.read(od, d + 2)[1:-1] == 0.0)
    with pytest.raises(pkg.OjasHipError, match="multiple of 32"):
        gpu.dispatch(gpu.begin(), "embed_q80", [(td, pad), (od, 4)], [0, 48], grid, block)


@pytest.mark.parametrize("ty", [Q8_0, Q4_K, Q5_K, Q6_K, IQ4_NL, IQ4_XS, Q4_0, Q5_1, Q2_K, Q3_K])
@pytest.mark.parametrize("out_off", [2, 8, 14])
def test_output_that_is_not_16_byte_aligned(gpu, orc, pkg, ty, out_off):
    """A thread writes its eight values as one 16-byte store where the output is 16-byte aligned; an output that starts
    2, 8 or 14 bytes past such a boundary gets the same bits, nothing before or after them."""
    bb, wpb = pkg.synth.BLOCK_SHAPE[ty]
    nb = 48
    raw = orc.synth_blocks(ty, nb)
    n = nb * wpb
    want = _dequant(gpu, ty, raw, n)
    assert np.array_equal(want, orc.dequant_to_f16(raw, ty, n))
    out = gpu.upload_bytes(np.full(n * 2 + 64, 0xA5, np.uint8))
    gpu.dequant_f16(ty, gpu.upload_bytes(raw), n, out, out_off=out_off)
    got = gpu.read(out, n * 2 + 64, np.uint8)
    assert np.all(got[:out_off] == 0xA5) and np.all(got[out_off + n * 2:] == 0xA5)
    assert np.array_equal(got[out_off:out_off + n * 2].view(np.uint16), want)
