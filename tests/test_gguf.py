"""The GGUF reader (host logic, no GPU) and the tensor loader (GPU), against files the tests
write themselves.  Behaviour follows crates/ojas-formats/src/gguf.rs:100-206 (parse, limits),
:440-452 / :551-556 (read_tensor_raw, tensor_meta) and `Lin::load`
(crates/ojas-cuda/src/qwen35.rs:174-201)."""
import numpy as np
import pytest

import gguf_writer as gw
from conftest import peak_err

Q8_0, Q4_K, Q6_K, IQ4_NL, IQ4_XS = 8, 12, 14, 20, 23


def _model(pkg, tmp_path, alignment=None, version=3):
    k = 512
    t = {
        "blk.0.attn_q.weight": (pkg.synth.q4k_weights(64, k, "gguf", "q"), [k, 64], Q4_K),
        "blk.0.attn_k.weight": (pkg.synth.q4k_weights(16, k, "gguf", "k"), [k, 16], Q4_K),
        "blk.0.attn_v.weight": (pkg.synth.q4k_weights(16, k, "gguf", "v"), [k, 16], Q4_K),
        "output.weight": (pkg.synth.q6k_weights(40, k, "gguf", "o"), [k, 40], Q6_K),
        "tok.weight": (pkg.synth.q80_weights(24, 64, "gguf", "e"), [64, 24], Q8_0),
        "blk.0.ffn_up.weight": (pkg.synth.iq4xs_weights(48, k, "gguf", "u"), [k, 48], IQ4_XS),
        "blk.0.ffn_gate.weight": (pkg.synth.iq4xs_weights(48, k, "gguf", "g"), [k, 48], IQ4_XS),
        "blk.0.ffn_down.weight": (pkg.synth.iq4nl_weights(40, 96, "gguf", "d"), [96, 40], IQ4_NL),
        "blk.0.exp_gate.weight": (pkg.synth.grid_weights(21, 24, k, "gguf", "eg"), [k, 24], 21),     # IQ3_S
        "blk.0.exp_up.weight": (pkg.synth.grid_weights(21, 24, k, "gguf", "eu"), [k, 24], 21),
        "blk.0.exp_down.weight": (pkg.synth.grid_weights(16, 8, k, "gguf", "ed"), [k, 8], 16),       # IQ2_XXS
        "norm.weight": (pkg.synth.normal_f32(k, "gguf", "n"), [k], 0),
    }
    meta = [("general.architecture", gw.STR, "llama"), ("llama.block_count", gw.U32, 1),
            ("tokenizer.ggml.tokens", gw.ARR, (gw.STR, ["a", "bc", "def"])),
            ("tokenizer.ggml.scores", gw.ARR, (gw.F32, [0.5, -1.0, 2.0])),
            ("some.i64", gw.I64, 77), ("some.bool", gw.BOOL, 1), ("some.f64", gw.F64, 2.5)]
    path = str(tmp_path / "m.gguf")
    offs = gw.write_gguf(path, meta, [(n, d, ty, b) for n, (b, d, ty) in t.items()], version=version, alignment=alignment)
    return path, t, offs


@pytest.mark.parametrize("alignment,version", [(None, 3), (64, 3), (32, 2)])
def test_reader_index_metadata_and_bytes(pkg, tmp_path, alignment, version):
    path, t, offs = _model(pkg, tmp_path, alignment, version)
    g = pkg.Gguf(path)
    assert sorted(g.tensor_names()) == sorted(t)
    assert g.meta_str("general.architecture") == "llama"
    assert g.meta_u64("llama.block_count") == 1 and g.meta_u64("some.i64") == 77 and g.meta_u64("some.bool") == 1
    for name, (data, dims, ty) in t.items():
        gdims, gty, off, nb = g.tensor_meta(name)
        raw = np.ascontiguousarray(data).view(np.uint8)
        assert (gdims, gty, off, nb) == (dims, ty, offs[name], raw.size)
        assert off % (alignment or 32) == 0
        rdims, rty, rb = g.read_tensor_raw(name)
        assert rdims == dims and rty == ty and np.array_equal(rb, raw)
    with pytest.raises(pkg.OjasHipError, match="not found"):
        g.tensor_meta("nope")
    with pytest.raises(pkg.OjasHipError, match="not a string"):
        g.meta_str("llama.block_count")
    g.close()


def test_reader_refuses_what_the_reference_refuses(pkg, tmp_path):
    p = str(tmp_path / "bad.gguf")
    open(p, "wb").write(b"GGML" + b"\0" * 64)
    with pytest.raises(pkg.OjasHipError, match="not a GGUF file"):
        pkg.Gguf(p)
    gw.write_gguf(p, [], [], version=1)
    with pytest.raises(pkg.OjasHipError, match="unsupported GGUF version 1"):
        pkg.Gguf(p)
    w = pkg.synth.q4k_weights(4, 256, "gguf", "x")
    gw.write_gguf(p, [], [("a", [256, 4], Q4_K, w), ("a", [256, 4], Q4_K, w)])
    with pytest.raises(pkg.OjasHipError, match="duplicate GGUF tensor a"):
        pkg.Gguf(p)
    gw.write_gguf(p, [], [("a", [256, 4, 1, 1, 1], Q4_K, w)])
    with pytest.raises(pkg.OjasHipError, match="invalid GGUF tensor rank 5"):
        pkg.Gguf(p)
    gw.write_gguf(p, [], [("a", [256, 0], Q4_K, w)])
    with pytest.raises(pkg.OjasHipError, match="invalid or overflowing"):
        pkg.Gguf(p)
    gw.write_gguf(p, [], [("a", [256, 4], Q4_K, w)], alignment=48)
    with pytest.raises(pkg.OjasHipError, match="invalid GGUF alignment 48"):
        pkg.Gguf(p)
    full = gw.write_gguf(p, [], [("a", [256, 4], Q4_K, w)])
    gw.write_gguf(p, [], [("a", [256, 4], Q4_K, w)], truncate=full["a"] + 100)
    with pytest.raises(pkg.OjasHipError, match="extends past the end"):
        pkg.Gguf(p)
    gw.write_gguf(p, [], [("a", [256, 4], Q4_K, w)], truncate=full["a"])
    with pytest.raises(pkg.OjasHipError, match="starts outside file"):
        pkg.Gguf(p)
    gw.write_gguf(p, [("k", gw.ARR, (gw.ARR, []))], [])
    with pytest.raises(pkg.OjasHipError, match="nested GGUF array"):
        pkg.Gguf(p)
    gw.write_gguf(p, [("split.count", gw.U32, 2)], [("a", [256, 4], Q4_K, w)])
    with pytest.raises(pkg.OjasHipError, match="split"):
        pkg.Gguf(p)
    gw.write_gguf(p, [], [("a", [256, 4], Q4_K, w)], truncate=20)
    with pytest.raises(pkg.OjasHipError):
        pkg.Gguf(p)


@pytest.mark.gpu
def test_lin_load_stacks_tensors_and_keeps_the_files_bytes(gpu, orc, pkg, tmp_path):
    path, t, _ = _model(pkg, tmp_path)
    g = pkg.Gguf(path)
    names = ["blk.0.attn_q.weight", "blk.0.attn_k.weight", "blk.0.attn_v.weight"]
    qkv = gpu.lin_load(g, names)
    k, n = 512, 96
    assert (qkv.n, qkv.k, qkv.ty) == (n, k, Q4_K)
    x = pkg.synth.normal_f32(k, "gguf", "x")
    y = gpu.alloc(n)
    gpu.mm(gpu.upload(x), qkv, y, 1, act_mode=pkg.ACT_Q8K)
    stacked = np.concatenate([t[nm][0] for nm in names])
    assert peak_err(gpu.read(y, n), orc.matvec_kq(stacked, Q4_K, n, k, x)) <= 2e-5
    out = gpu.lin_load(g, ["output.weight"])
    y2 = gpu.alloc(40)
    gpu.mm(gpu.upload(x), out, y2, 1, act_mode=pkg.ACT_Q8K)
    assert peak_err(gpu.read(y2, 40), orc.matvec_kq(t["output.weight"][0], Q6_K, 40, k, x)) <= 2e-5
    emb = gpu.lin_load(g, ["tok.weight"])
    x64 = pkg.synth.normal_f32(64, "gguf", "x64")
    y3 = gpu.alloc(24)
    gpu.mm(gpu.upload(x64), emb, y3, 1)
    assert peak_err(gpu.read(y3, 24), orc.matvec_kq(t["tok.weight"][0], Q8_0, 24, 64, x64)) <= 1e-5
    # IQ4 tensors stay in their block bytes too and stack like the others (f32 activations)
    gu = gpu.lin_load(g, ["blk.0.ffn_gate.weight", "blk.0.ffn_up.weight"])
    assert (gu.n, gu.k, gu.ty) == (96, k, IQ4_XS)
    y4 = gpu.alloc(96)
    gpu.mm(gpu.upload(x), gu, y4, 1)
    both = np.concatenate([t["blk.0.ffn_gate.weight"][0], t["blk.0.ffn_up.weight"][0]])
    assert peak_err(gpu.read(y4, 96), orc.matvec_kq(both, IQ4_XS, 96, k, x)) <= 1e-5
    dn = gpu.lin_load(g, ["blk.0.ffn_down.weight"])
    x96 = pkg.synth.normal_f32(96, "gguf", "x96")
    y5 = gpu.alloc(40)
    gpu.mm(gpu.upload(x96), dn, y5, 1)
    assert peak_err(gpu.read(y5, 40), orc.matvec_kq(t["blk.0.ffn_down.weight"][0], IQ4_NL, 40, 96, x96)) <= 1e-5
    # grid-codebook tensors: IQ3_S stacked (f32 activations, dot_iq3s), IQ2_XXS on int8 activations (dot_iq2xxs_q8k)
    eg = gpu.lin_load(g, ["blk.0.exp_gate.weight", "blk.0.exp_up.weight"])
    assert (eg.n, eg.k, eg.ty) == (48, k, 21)
    y6 = gpu.alloc(48)
    gpu.mm(gpu.upload(x), eg, y6, 1)
    both = np.concatenate([t["blk.0.exp_gate.weight"][0], t["blk.0.exp_up.weight"][0]])
    assert peak_err(gpu.read(y6, 48), orc.matvec_kq(both, 21, 48, k, x)) <= 1e-5
    ed = gpu.lin_load(g, ["blk.0.exp_down.weight"])
    y7 = gpu.alloc(8)
    gpu.mm(gpu.upload(x), ed, y7, 1)
    assert peak_err(gpu.read(y7, 8), orc.matvec_kq(t["blk.0.exp_down.weight"][0], 16, 8, k, x)) <= 2e-5
    with pytest.raises(pkg.OjasHipError, match="type differs"):
        gpu.lin_load(g, ["blk.0.attn_q.weight", "output.weight"])
    with pytest.raises(pkg.OjasHipError, match="K 64 differs"):
        gpu.lin_load(g, ["output.weight", "tok.weight"])
    with pytest.raises(pkg.OjasHipError, match="missing tensor"):
        gpu.lin_load(g, ["blk.9.attn_q.weight"])
    with pytest.raises(pkg.OjasHipError, match="not kept in place"):
        gpu.lin_load(g, ["norm.weight"])
