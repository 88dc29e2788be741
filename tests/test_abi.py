"""Host-only checks of the C-ABI library: it loads, exports every symbol the header declares, and
its manifest obeys the reference's structural rules (crates/ojas-cuda/tests/conformance.rs:85-202):
every name defined exactly once, in exactly one family, pointers before scalars."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "ojas_hip.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ojh_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(pkg):
    lib = pkg.load_library()
    names = declared_symbols()
    assert len(names) >= 30
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in include/ojas_hip.h but not exported"
    # and the binding covers them all
    assert set(names) <= set(lib._ojh_signatures), set(names) - set(lib._ojh_signatures)
    assert lib.ojh_abi_version() == 1


def test_manifest_names_are_unique_and_resolve_to_one_family(pkg):
    m = pkg.manifest()
    names = [e[0] for e in m]
    assert len(names) == len(set(names))
    lib = pkg.load_library()
    for name, family, nb, nc in m:
        assert lib.ojh_kernel_family(name.encode()).decode() == family
        if name == "decode_chain_q4k":      # takes one argument block, launched by ojh_decode_chain only
            assert (nb, nc) == (0, 0)
            continue
        assert 1 <= nb <= 13 and 0 <= nc <= 8 and nb + nc <= 16      # qkv_q8 takes 13 buffers and 3 constants: the launch limit
    assert lib.ojh_kernel_family(b"no_such_kernel") is None


def test_canonical_names_are_present(pkg):
    names = {e[0] for e in pkg.manifest()}
    for fmt in ("q80", "q4k", "q6k"):
        for suffix in ("", "_accum", "_bias", "_m"):
            assert f"gemv_nat_{fmt}{suffix}" in names   # crates/ojas-cuda/src/kernels/nat.rs:57-66
    for fmt in ("q4k", "q5k", "q6k"):
        for suffix in ("", "_accum", "_bias", "_m"):
            assert f"gemv_q8k_{fmt}{suffix}" in names
    assert "quantize_q8k" in names


def _hsaco_kernel_symbols(path):
    """Kernel descriptors (`<name>.kd`) named in the code object's string table."""
    data = open(path, "rb").read()
    return set(m.decode() for m in re.findall(rb"([A-Za-z_][A-Za-z0-9_]*)\.kd\x00", data))


def test_every_manifest_entry_is_defined_in_its_code_object(pkg):
    hs = os.path.join(ROOT, "ojas-engine_amd", "hsaco")
    defined = {}
    for f in os.listdir(hs):
        if f.endswith(".hsaco"):
            defined[f[:-6]] = _hsaco_kernel_symbols(os.path.join(hs, f))
    for name, family, _, _ in pkg.manifest():
        assert family in defined, f"family {family} has no code object"
        assert name in defined[family], f"{name} is not defined in {family}.hsaco"
        others = [fam for fam, syms in defined.items() if fam != family and name in syms]
        assert not others, f"{name} is also defined in {others}"


def test_kernel_sources_put_pointers_before_scalars():
    """A pointer after a scalar lands in a constant's argument slot when `dispatch` appends
    buffers then constants (crates/ojas-cuda/tests/conformance.rs:77-109)."""
    kdir = os.path.join(ROOT, "ojas-engine_amd", "csrc", "kernels")
    n = 0
    for f in os.listdir(kdir):
        if not f.endswith(".hip"):
            continue
        src = open(os.path.join(kdir, f)).read()
        for m in re.finditer(r'extern "C" __global__ void[^(]*?(\w+)\s*\(([^)]*)\)', src, flags=re.S):
            args = [a.strip() for a in m.group(2).replace("\\", " ").split(",") if a.strip()]
            seen_scalar = False
            for a in args:
                is_ptr = "*" in a
                assert not (is_ptr and seen_scalar), f"{f}:{m.group(1)}: pointer after scalar in ({m.group(2)})"
                seen_scalar |= not is_ptr
            n += 1
    assert n >= 10


def test_row_bytes(pkg):
    lib = pkg.load_library()
    assert lib.ojh_row_bytes(12, 4096) == 2304
    assert lib.ojh_row_bytes(14, 4096) == 3360
    assert lib.ojh_row_bytes(8, 4096) == 4352
    assert lib.ojh_row_bytes(12, 100) == 0 and lib.ojh_row_bytes(99, 256) == 0


def test_open_without_a_gpu_fails_loudly(pkg):
    import torch
    if os.path.exists("/dev/kfd") or torch.cuda.is_available():
        pytest.skip("a GPU is present")
    with pytest.raises(pkg.OjasHipError) as e:
        pkg.HipGpu(0)
    assert "no CPU fallback" in str(e.value) or "device" in str(e.value).lower()
