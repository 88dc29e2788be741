"""Host-side mirror of the reference's kernel and op seams over the C ABI of libojas_hip.so.

`HipGpu` has the shape of the reference's `Device` + `KernelRuntime` traits
(crates/ojas-core/src/lib.rs:26-40, crates/ojas-core/src/kernel.rs:67-81; CUDA implementation
crates/ojas-cuda/src/device.rs:418-537): `ensure_family`, `has_kernel`, `caps`, `begin`,
`dispatch(enc, name, bufs, consts, grid, block)`, `submit`, `alloc`, `upload`, `read`.
`Lin` / `HipGpu.mm` mirror `Lin::load` / `CudaSsm::mm` (crates/ojas-cuda/src/qwen35.rs:174-201,
:644-702).

Everything here binds the shared library with ctypes; there is no CPU implementation behind it.
If the library or a GPU is missing the calls raise.
"""
from __future__ import annotations

import ctypes as C
import os
from dataclasses import dataclass

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libojas_hip.so")

Q8_0, Q4_K, Q5_K, Q6_K, IQ4_NL, IQ4_XS = 8, 12, 13, 14, 20, 23
Q4_0, Q4_1, Q5_0, Q5_1 = 2, 3, 6, 7
Q2_K, Q3_K = 10, 11
IQ2_XXS, IQ2_XS, IQ3_XXS, IQ1_S, IQ3_S, IQ2_S, IQ1_M = 16, 17, 18, 19, 21, 22, 29
GRID_TYPES = (IQ2_XXS, IQ2_XS, IQ3_XXS, IQ1_S, IQ3_S, IQ2_S, IQ1_M)
MXFP4 = 139     # the reference's synthetic id for its 17-byte MXFP4 blocks (a safetensors format, not a GGUF type)
X_F32, X_BF16, X_F16 = 0, 1, 2
ACT_AUTO, ACT_Q8K, ACT_FLOAT, ACT_FLOAT_EXACT, ACT_Q8_1 = 0, 1, 2, 3, 4

BLOCK_SHAPE = {Q8_0: (34, 32), Q4_K: (144, 256), Q5_K: (176, 256), Q6_K: (210, 256), IQ4_NL: (18, 32), IQ4_XS: (136, 256),
               Q4_0: (18, 32), Q4_1: (20, 32), Q5_0: (22, 32), Q5_1: (24, 32), Q2_K: (84, 256), Q3_K: (110, 256),
               IQ2_XXS: (66, 256), IQ2_XS: (74, 256), IQ3_XXS: (98, 256), IQ1_S: (50, 256), IQ3_S: (110, 256), IQ2_S: (82, 256),
               IQ1_M: (56, 256), MXFP4: (17, 32)}


class OjasHipError(RuntimeError):
    def __init__(self, code: int, msg: str):
        super().__init__(f"[{code}] {msg}")
        self.code = code


class _Caps(C.Structure):
    _fields_ = [("tier", C.c_int32), ("f16_compute", C.c_int32), ("simd_width", C.c_uint32),
                ("unified_memory", C.c_int32), ("max_buffer", C.c_uint64), ("compute_units", C.c_uint32),
                ("clock_mhz", C.c_uint32), ("total_memory", C.c_uint64), ("arch", C.c_char * 32),
                ("features", C.c_char_p)]


@dataclass
class Caps:
    """Mirrors `Caps` (crates/ojas-core/src/kernel.rs:26-41)."""
    tier: str
    f16_compute: bool
    simd_width: int
    unified_memory: bool
    max_buffer: int
    compute_units: int
    clock_mhz: int
    arch: str
    features: tuple

    def has(self, feature: str) -> bool:
        return feature in self.features


_lib = None
# int load(void *user, uint32_t id, void *dst, size_t bytes)
EXPERT_LOAD_FN = C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_uint32, C.c_void_p, C.c_size_t)


class _ChainStage(C.Structure):
    """`ojh_chain_stage` of include/ojas_hip.h."""
    _fields_ = [("x", C.c_void_p), ("x_off", C.c_size_t), ("x2", C.c_void_p), ("x2_off", C.c_size_t),
                ("prologue", C.c_int), ("eps", C.c_float), ("count", C.c_int), ("ws", C.c_void_p * 4),
                ("ys", C.c_void_p * 4), ("y_offs", C.c_size_t * 4), ("accum", C.c_int)]


CHAIN_X_PLAIN, CHAIN_X_SILU_MUL, CHAIN_X_GELU_MUL, CHAIN_X_RMSNORM = 0, 1, 2, 3
CHAIN_MAX_STAGES = 8


class _GatherStats(C.Structure):
    _fields_ = [("hits", C.c_uint64), ("misses", C.c_uint64), ("bytes_streamed", C.c_uint64), ("evictions", C.c_uint64)]


def load_library(path: str | None = None) -> C.CDLL:
    """Load libojas_hip.so (built offline by build.py) and declare its signatures."""
    global _lib
    if _lib is not None and path is None:
        return _lib
    p = path or LIB_PATH
    if not os.path.exists(p):
        raise FileNotFoundError(f"{p} is missing: build it with `python ojas-engine_amd/build.py`")
    L = C.CDLL(p)
    vp, sz, u32, i32, u64 = C.c_void_p, C.c_size_t, C.c_uint32, C.c_int, C.c_uint64
    pp = C.POINTER(vp)
    sig = {
        "ojh_open": (i32, [i32, pp]),
        "ojh_close": (i32, [vp]),
        "ojh_name": (C.c_char_p, [vp]),
        "ojh_caps_get": (i32, [vp, C.POINTER(_Caps)]),
        "ojh_last_error": (C.c_char_p, []),
        "ojh_abi_version": (i32, []),
        "ojh_alloc": (i32, [vp, sz, pp]),
        "ojh_free": (i32, [vp, vp]),
        "ojh_wrap": (i32, [vp, vp, sz, pp]),
        "ojh_buf_bytes": (sz, [vp]),
        "ojh_buf_ptr": (vp, [vp]),
        "ojh_upload": (i32, [vp, vp, sz, vp, sz]),
        "ojh_download": (i32, [vp, vp, sz, vp, sz]),
        "ojh_memset0": (i32, [vp, vp, sz, sz]),
        "ojh_ensure_family": (i32, [vp, C.c_char_p]),
        "ojh_has_kernel": (i32, [vp, C.c_char_p]),
        "ojh_kernel_family": (C.c_char_p, [C.c_char_p]),
        "ojh_manifest": (i32, [i32, C.POINTER(C.c_char_p), C.POINTER(C.c_char_p), C.POINTER(i32), C.POINTER(i32)]),
        "ojh_launch_shape": (i32, [vp, C.c_char_p, u32, u32, u32, C.POINTER(u32), C.POINTER(u32)]),
        "ojh_dispatch": (i32, [vp, C.c_char_p, i32, pp, C.POINTER(u64), i32, C.POINTER(u32), C.POINTER(u32),
                               C.POINTER(u32)]),
        "ojh_submit": (i32, [vp]),
        "ojh_timer_start": (i32, [vp]),
        "ojh_timer_stop": (i32, [vp, C.POINTER(C.c_float)]),
        "ojh_lin_create": (i32, [vp, u32, u32, u32, vp, pp]),
        "ojh_lin_wrap": (i32, [vp, u32, u32, u32, vp, sz, pp]),
        "ojh_lin_free": (i32, [vp, vp]),
        "ojh_row_bytes": (sz, [u32, u32]),
        "ojh_mm": (i32, [vp, vp, sz, i32, vp, vp, sz, vp, u32, i32, i32]),
        "ojh_mm_noalloc": (i32, [vp, vp, sz, i32, vp, vp, sz, vp, u32, i32]),
        "ojh_noalloc_scratch_bytes": (sz, []),
        "ojh_mm_q8k": (i32, [vp, vp, vp, vp, vp, sz, vp, u32, i32]),
        "ojh_mm_q8k_multi": (i32, [vp, vp, vp, i32, vp, vp, vp]),
        "ojh_mm_multi": (i32, [vp, vp, sz, i32, vp, vp, vp, i32]),
        "ojh_decode_chain": (i32, [vp, C.POINTER(_ChainStage), i32]),
        "ojh_chain_spin_limit": (i32, [vp, u32]),
        "ojh_chain_trace": (i32, [vp, vp]),
        "ojh_gguf_open": (i32, [C.c_char_p, vp]),
        "ojh_gguf_close": (i32, [vp]),
        "ojh_gguf_tensor_count": (i32, [vp]),
        "ojh_gguf_tensor_name": (C.c_char_p, [vp, i32]),
        "ojh_gguf_tensor_meta": (i32, [vp, C.c_char_p, vp, vp, vp, vp, vp]),
        "ojh_gguf_meta_u64": (i32, [vp, C.c_char_p, vp]),
        "ojh_gguf_meta_str": (i32, [vp, C.c_char_p, vp, sz]),
        "ojh_gguf_read_raw": (i32, [vp, C.c_char_p, vp, C.c_uint64]),
        "ojh_lin_load": (i32, [vp, vp, vp, i32, vp]),
        "ojh_rmsnorm_quant_q8k": (i32, [vp, vp, sz, vp, C.c_float, u32, u32, vp, vp, vp]),
        "ojh_ffn_gu_q8k": (i32, [vp, vp, vp, vp, vp, vp, sz, i32]),
        "ojh_relayout_q4k_q4l": (i32, [vp, vp, sz, u32, u32, vp, vp, vp]),
        "ojh_q8rows_from_f16": (i32, [vp, vp, sz, u32, u32, vp, vp]),
        "ojh_matmul_q8": (i32, [vp, vp, sz, vp, vp, vp, vp, sz, u32, u32, u32]),
        "ojh_capture_begin": (i32, [vp]),
        "ojh_capture_end": (i32, [vp, pp]),
        "ojh_graph_launch": (i32, [vp, vp]),
        "ojh_graph_free": (i32, [vp, vp]),
        "ojh_mark": (i32, [vp, i32]),
        "ojh_mark_elapsed": (i32, [vp, i32, i32, C.POINTER(C.c_float)]),
        "ojh_dequant_f16": (i32, [vp, u32, vp, sz, sz, vp, sz]),
        "ojh_quant_q8k": (i32, [vp, vp, sz, i32, u32, u32, vp, vp]),
        "ojh_moe_route": (i32, [vp, vp, u32, u32, u32, vp, vp]),
        "ojh_moe_ffn": (i32, [vp, vp, u32, u32, u32, u32, u32, vp, vp, vp, vp, vp, vp, i32, i32]),
        "ojh_moe_ffn_routed": (i32, [vp, vp, u32, u32, u32, u32, u32, vp, vp, vp, vp, vp, vp, vp, i32, i32]),
        "ojh_moe_ffn_slots": (i32, [vp, vp, u32, u32, u32, u32, vp, vp, vp, vp, vp, vp, vp, vp, i32]),
        "ojh_expert_cache_create": (i32, [vp, sz, sz, C.POINTER(vp)]),
        "ojh_expert_cache_destroy": (i32, [vp]),
        "ojh_expert_cache_slots": (u32, [vp]),
        "ojh_expert_cache_resident_bytes": (sz, [vp]),
        "ojh_expert_cache_arena": (vp, [vp]),
        "ojh_expert_cache_gather": (i32, [vp, vp, sz, EXPERT_LOAD_FN, vp, vp]),
        "ojh_expert_cache_stats": (i32, [vp, vp]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(L, name)
        fn.restype = res
        fn.argtypes = args
    L._ojh_signatures = sig
    if path is None:
        _lib = L
    return L


class ExpertCache:
    """Device arena of expert slots with LRU eviction (`ExpertCache`, crates/ojas-cuda/src/expert_cache.rs:34-152).
    `gather(ids, load)` returns one u64 byte offset into `arena` per id; `load(id) -> bytes-like of expert_bytes`
    supplies a missing expert.  With `gpu=None` only the bookkeeping runs (hit rates of a routing trace)."""

    def __init__(self, gpu: "HipGpu | None", budget_bytes: int, expert_bytes: int):
        self._L = gpu._L if gpu is not None else load_library()
        self.gpu, self.expert_bytes = gpu, expert_bytes
        h = C.c_void_p()
        rc = self._L.ojh_expert_cache_create(gpu._dev if gpu is not None else None, budget_bytes, expert_bytes, C.byref(h))
        if rc:
            raise OjasHipError(rc, (self._L.ojh_last_error() or b"").decode())
        self._h = h
        self.arena = None
        if gpu is not None:
            self.arena = Buf(gpu, self._L.ojh_expert_cache_arena(h), self.resident_bytes)
            self.arena.free = lambda: None      # the cache owns it

    @property
    def slots(self) -> int:
        return self._L.ojh_expert_cache_slots(self._h)

    @property
    def resident_bytes(self) -> int:
        return self._L.ojh_expert_cache_resident_bytes(self._h)

    @property
    def stats(self) -> dict:
        st = _GatherStats()
        rc = self._L.ojh_expert_cache_stats(self._h, C.byref(st))
        if rc:
            raise OjasHipError(rc, (self._L.ojh_last_error() or b"").decode())
        return {k: int(getattr(st, k)) for k, _ in _GatherStats._fields_}

    @property
    def hit_rate(self) -> float:
        st = self.stats
        total = st["hits"] + st["misses"]
        return st["hits"] / total if total else 0.0

    def gather(self, ids, load=None) -> np.ndarray:
        ids = np.ascontiguousarray(ids, np.uint32).ravel()
        offs = np.empty(ids.size, np.uint64)
        failure = []

        def _cb(_user, eid, dst, nbytes):
            try:
                src = np.frombuffer(load(int(eid)), np.uint8)
                if src.size != nbytes:
                    raise ValueError(f"expert {eid}: load returned {src.size} bytes, the slot holds {nbytes}")
                C.memmove(dst, src.ctypes.data, nbytes)
                return 0
            except Exception as e:      # an exception must not unwind through the C frame
                failure.append(e)
                return 1

        cb = EXPERT_LOAD_FN(_cb) if load is not None else C.cast(None, EXPERT_LOAD_FN)
        rc = self._L.ojh_expert_cache_gather(self._h, C.c_void_p(ids.ctypes.data), ids.size, cb, None,
                                             C.c_void_p(offs.ctypes.data))
        if failure:
            raise failure[0]
        if rc:
            raise OjasHipError(rc, (self._L.ojh_last_error() or b"").decode())
        return offs

    def close(self) -> None:
        # a cache belongs to its device and is destroyed before it; one that outlived a closed device is dropped
        # unreleased rather than handed a freed device (the arena then lives until the process ends)
        if self._h and (self.gpu is None or self.gpu._dev):
            self._L.ojh_expert_cache_destroy(self._h)
        self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Gguf:
    """An open GGUF file (metadata + tensor index), the shape of the reference's `Gguf`
    (crates/ojas-formats/src/gguf.rs:297-339, 440-452, 551-556).  Needs no GPU."""

    def __init__(self, path: str):
        self._L = load_library()
        h = C.c_void_p()
        rc = self._L.ojh_gguf_open(os.fsencode(path), C.byref(h))
        if rc:
            raise OjasHipError(rc, self._L.ojh_last_error().decode())
        self.handle = h

    def _check(self, rc: int) -> None:
        if rc:
            raise OjasHipError(rc, self._L.ojh_last_error().decode())

    def close(self) -> None:
        if self.handle:
            self._L.ojh_gguf_close(self.handle)
        self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def tensor_names(self) -> list[str]:
        return [self._L.ojh_gguf_tensor_name(self.handle, i).decode() for i in range(self._L.ojh_gguf_tensor_count(self.handle))]

    def tensor_meta(self, name: str):
        """(dims, ggml_type, absolute file offset, raw byte length)."""
        ty, nd, off, nb = C.c_uint32(), C.c_uint32(), C.c_uint64(), C.c_uint64()
        dims = (C.c_uint64 * 4)()
        self._check(self._L.ojh_gguf_tensor_meta(self.handle, name.encode(), C.byref(ty), C.byref(nd), dims, C.byref(off), C.byref(nb)))
        return list(dims[:nd.value]), ty.value, off.value, nb.value

    def meta_u64(self, key: str) -> int:
        v = C.c_uint64()
        self._check(self._L.ojh_gguf_meta_u64(self.handle, key.encode(), C.byref(v)))
        return v.value

    def meta_str(self, key: str) -> str:
        buf = C.create_string_buffer(4096)
        self._check(self._L.ojh_gguf_meta_str(self.handle, key.encode(), buf, 4096))
        return buf.value.decode()

    def read_tensor_raw(self, name: str):
        """(dims, ggml_type, bytes) — `read_tensor_raw`."""
        dims, ty, _, nb = self.tensor_meta(name)
        if nb == 0:
            raise OjasHipError(4, f"read_tensor_raw: unsupported GGUF type {ty}")
        out = np.empty(nb, np.uint8)
        self._check(self._L.ojh_gguf_read_raw(self.handle, name.encode(), C.c_void_p(out.ctypes.data), nb))
        return dims, ty, out


def manifest() -> list[tuple[str, str, int, int]]:
    """(name, family, n_bufs, n_consts) of every kernel the library claims. Needs no GPU."""
    L = load_library()
    n = L.ojh_manifest(-1, None, None, None, None)
    out = []
    for i in range(n):
        name, fam = C.c_char_p(), C.c_char_p()
        nb, nc = C.c_int(), C.c_int()
        L.ojh_manifest(i, C.byref(name), C.byref(fam), C.byref(nb), C.byref(nc))
        out.append((name.value.decode(), fam.value.decode(), nb.value, nc.value))
    return out


def row_bytes(ty: int, k: int) -> int:
    bb, wpb = BLOCK_SHAPE[ty]
    if k % wpb:
        raise ValueError(f"K={k} is not a multiple of {wpb}")
    return k // wpb * bb


class Buf:
    """Device buffer. Dropping it frees the memory, as the reference's `CuBuf` does
    (crates/ojas-cuda/src/device.rs:20-23)."""

    def __init__(self, gpu: "HipGpu", handle: int, nbytes: int):
        self.gpu, self.handle, self.nbytes = gpu, handle, nbytes

    @property
    def ptr(self) -> int:
        return self.gpu._L.ojh_buf_ptr(self.handle) or 0

    def free(self) -> None:
        if self.handle and self.gpu._dev:
            self.gpu._check(self.gpu._L.ojh_free(self.gpu._dev, self.handle))
        self.handle = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Enc:
    """Stand-in for the reference's encoder: this backend has one stream per device, so an
    encoder is only a marker that ties `dispatch` calls to the `submit` that waits for them."""

    def __init__(self, gpu: "HipGpu"):
        self.gpu = gpu


class Lin:
    """A weight matrix W[N,K] kept in its GGUF block bytes (crates/ojas-cuda/src/qwen35.rs:146-201)."""

    def __init__(self, gpu: "HipGpu", handle: int, ty: int, n: int, k: int, keep=None):
        self.gpu, self.handle, self.ty, self.n, self.k = gpu, handle, ty, n, k
        self._keep = keep  # a wrapped Buf must outlive the handle

    @property
    def nbytes(self) -> int:
        return self.n * row_bytes(self.ty, self.k)

    def free(self) -> None:
        if self.handle and self.gpu._dev:
            self.gpu._check(self.gpu._L.ojh_lin_free(self.gpu._dev, self.handle))
        self.handle = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Graph:
    """A recorded chain of dispatches; `launch()` replays it with one host call."""

    def __init__(self, gpu: "HipGpu", handle):
        self.gpu, self.handle = gpu, handle

    def launch(self) -> None:
        self.gpu._check(self.gpu._L.ojh_graph_launch(self.gpu._dev, self.handle))

    def free(self) -> None:
        if self.handle and self.gpu._dev:
            self.gpu._L.ojh_graph_free(self.gpu._dev, self.handle)
        self.handle = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class HipGpu:
    """`Device + KernelRuntime` over the C ABI."""

    def __init__(self, ordinal: int = 0):
        self._L = load_library()
        self._dev = None
        dev = C.c_void_p()
        self._check(self._L.ojh_open(ordinal, C.byref(dev)))
        self._dev = dev

    # -- plumbing
    def _check(self, rc: int) -> None:
        if rc != 0:
            raise OjasHipError(rc, (self._L.ojh_last_error() or b"").decode())

    def close(self) -> None:
        if self._dev:
            self._L.ojh_close(self._dev)
            self._dev = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # -- Device
    def name(self) -> str:
        return self._L.ojh_name(self._dev).decode()

    def alloc_bytes(self, nbytes: int) -> Buf:
        h = C.c_void_p()
        self._check(self._L.ojh_alloc(self._dev, nbytes, C.byref(h)))
        return Buf(self, h, nbytes)

    def alloc(self, len_f32: int) -> Buf:
        return self.alloc_bytes(len_f32 * 4)

    def wrap(self, device_ptr: int, nbytes: int) -> Buf:
        """Borrow device memory owned elsewhere (e.g. a torch tensor's storage)."""
        h = C.c_void_p()
        self._check(self._L.ojh_wrap(self._dev, C.c_void_p(device_ptr), nbytes, C.byref(h)))
        return Buf(self, h, nbytes)

    def upload_bytes(self, data) -> Buf:
        a = np.ascontiguousarray(data)
        b = self.alloc_bytes(a.nbytes)
        self.write_bytes(b, 0, a)
        return b

    def upload(self, data) -> Buf:
        return self.upload_bytes(np.ascontiguousarray(data, np.float32))

    def write_bytes(self, buf: Buf, off: int, data) -> None:
        a = np.ascontiguousarray(data)
        self._check(self._L.ojh_upload(self._dev, buf.handle, off, C.c_void_p(a.ctypes.data), a.nbytes))

    def read_bytes(self, buf: Buf, off: int, out: np.ndarray) -> np.ndarray:
        assert out.flags["C_CONTIGUOUS"]
        self._check(self._L.ojh_download(self._dev, buf.handle, off, C.c_void_p(out.ctypes.data), out.nbytes))
        return out

    def read(self, buf: Buf, n: int, dtype=np.float32, off: int = 0) -> np.ndarray:
        return self.read_bytes(buf, off, np.empty(n, dtype))

    def memset0(self, buf: Buf, off: int = 0, nbytes: int | None = None) -> None:
        self._check(self._L.ojh_memset0(self._dev, buf.handle, off, buf.nbytes - off if nbytes is None else nbytes))

    # -- KernelRuntime
    def ensure_family(self, family: str) -> None:
        self._check(self._L.ojh_ensure_family(self._dev, family.encode()))

    def has_kernel(self, name: str) -> bool:
        return bool(self._L.ojh_has_kernel(self._dev, name.encode()))

    def caps(self) -> Caps:
        c = _Caps()
        self._check(self._L.ojh_caps_get(self._dev, C.byref(c)))
        return Caps(tier="CBA"[c.tier], f16_compute=bool(c.f16_compute), simd_width=c.simd_width,
                    unified_memory=bool(c.unified_memory), max_buffer=c.max_buffer,
                    compute_units=c.compute_units, clock_mhz=c.clock_mhz, arch=c.arch.decode(),
                    features=tuple((c.features or b"").decode().split(",")))

    def begin(self) -> Enc:
        return Enc(self)

    def launch_shape(self, name: str, K: int, N: int, M: int = 1):
        g, b = (C.c_uint32 * 3)(), (C.c_uint32 * 3)()
        self._check(self._L.ojh_launch_shape(self._dev, name.encode(), K, N, M, g, b))
        return list(g), list(b)

    def dispatch(self, enc: Enc, name: str, bufs, consts, grid, block) -> None:
        """`bufs` is a list of (Buf, byte_offset); buffers first, then u32 constants.  A Buf of None is passed as NULL,
        for the few kernels that take an optional buffer (the biases of `qkv_q8`)."""
        n = len(bufs)
        hs = (C.c_void_p * max(n, 1))(*[b.handle if b is not None else None for b, _ in bufs])
        offs = (C.c_uint64 * max(n, 1))(*[o for _, o in bufs])
        cs = (C.c_uint32 * max(len(consts), 1))(*consts)
        g, b = (C.c_uint32 * 3)(*grid), (C.c_uint32 * 3)(*block)
        self._check(self._L.ojh_dispatch(self._dev, name.encode(), n, hs, offs, len(consts), cs, g, b))

    def submit(self, enc: Enc | None = None) -> None:
        self._check(self._L.ojh_submit(self._dev))

    def timer_start(self) -> None:
        self._check(self._L.ojh_timer_start(self._dev))

    def timer_stop(self) -> float:
        ms = C.c_float()
        self._check(self._L.ojh_timer_stop(self._dev, C.byref(ms)))
        return ms.value

    # -- op seam
    def lin(self, ty: int, n: int, k: int, raw) -> Lin:
        a = np.ascontiguousarray(raw, np.uint8)
        if a.size != n * row_bytes(ty, k):
            raise ValueError(f"Lin {n}x{k} of type {ty} needs {n * row_bytes(ty, k)} bytes, got {a.size}")
        h = C.c_void_p()
        self._check(self._L.ojh_lin_create(self._dev, ty, n, k, C.c_void_p(a.ctypes.data), C.byref(h)))
        return Lin(self, h, ty, n, k)

    def lin_wrap(self, ty: int, n: int, k: int, raw: Buf, off: int = 0) -> Lin:
        h = C.c_void_p()
        self._check(self._L.ojh_lin_wrap(self._dev, ty, n, k, raw.handle, off, C.byref(h)))
        return Lin(self, h, ty, n, k, keep=raw)

    def lin_load(self, g: Gguf, names: list[str]) -> Lin:
        """`Lin::load`: the named tensors stacked along N, kept in the file's block bytes."""
        arr = (C.c_char_p * len(names))(*[n.encode() for n in names])
        h = C.c_void_p()
        self._check(self._L.ojh_lin_load(self._dev, g.handle, arr, len(names), C.byref(h)))
        n = sum((g.tensor_meta(nm)[0] + [1])[1] for nm in names)
        dims, ty, _, _ = g.tensor_meta(names[0])
        return Lin(self, h, ty, n, dims[0])

    def mm(self, x: Buf, w: Lin, y: Buf, m: int = 1, accum: bool = False, *, x_dtype: int = X_F32,
           act_mode: int = ACT_AUTO, bias: Buf | None = None, x_off: int = 0, y_off: int = 0) -> None:
        self._check(self._L.ojh_mm(self._dev, x.handle, x_off, x_dtype, w.handle, y.handle, y_off,
                                   bias.handle if bias else None, m, int(accum), act_mode))

    def mm_noalloc(self, x: Buf, w: Lin, y: Buf, m: int = 1, accum: bool = False, *, x_dtype: int = X_F32,
                   bias: Buf | None = None, x_off: int = 0, y_off: int = 0) -> None:
        """`mm` with ACT_Q8K through the entry that allocates nothing (activations staged in a static device array)."""
        self._check(self._L.ojh_mm_noalloc(self._dev, x.handle, x_off, x_dtype, w.handle, y.handle, y_off,
                                           bias.handle if bias else None, m, int(accum)))

    def mm_q8k(self, xq: Buf, xscales: Buf, w: Lin, y: Buf, m: int = 1, accum: bool = False, *,
               bias: Buf | None = None, y_off: int = 0) -> None:
        """Matmul from activations already quantized by `quant_q8k` (shared by several projections)."""
        self._check(self._L.ojh_mm_q8k(self._dev, xq.handle, xscales.handle, w.handle, y.handle, y_off,
                                       bias.handle if bias else None, m, int(accum)))

    def mm_q8k_multi(self, xq: Buf, xscales: Buf, ws: list, ys: list, y_offs: list | None = None) -> None:
        """Up to four projections of one quantized vector in one launch (fused q/k/v, gate/up)."""
        n = len(ws)
        if n != len(ys) or (y_offs is not None and len(y_offs) != n):
            raise ValueError("mm_q8k_multi: ws, ys and y_offs must have the same length")
        wa = (C.c_void_p * n)(*[w.handle for w in ws])
        ya = (C.c_void_p * n)(*[y.handle for y in ys])
        oa = (C.c_size_t * n)(*y_offs) if y_offs is not None else None
        self._check(self._L.ojh_mm_q8k_multi(self._dev, xq.handle, xscales.handle, n, wa, ya, oa))

    def mm_multi(self, x: Buf, ws: list, ys: list, y_offs: list | None = None, accum: bool = False, x_off: int = 0) -> None:
        """One decode stage in one launch: up to four projections of one f32 vector, quantized inside the launch."""
        n = len(ws)
        if n != len(ys) or (y_offs is not None and len(y_offs) != n):
            raise ValueError("mm_multi: ws, ys and y_offs must have the same length")
        wa = (C.c_void_p * n)(*[w.handle for w in ws])
        ya = (C.c_void_p * n)(*[y.handle for y in ys])
        oa = (C.c_size_t * n)(*y_offs) if y_offs is not None else None
        self._check(self._L.ojh_mm_multi(self._dev, x.handle, x_off, n, wa, ya, oa, int(accum)))

    def decode_chain(self, stages: list) -> None:
        """Dependent decode stages in ONE launch.  Each stage is a dict: x (Buf), ws (list of Lin), ys (list of Buf)
        and optionally x_off, x2, x2_off, prologue (CHAIN_X_*), eps, y_offs, accum."""
        n = len(stages)
        arr = (_ChainStage * max(n, 1))()
        for st, d in zip(arr, stages):
            ws, ys = d["ws"], d["ys"]
            if len(ws) != len(ys) or not 1 <= len(ws) <= 4:
                raise ValueError("decode_chain: a stage takes 1 to 4 projections and as many outputs")
            st.x, st.x_off = d["x"].handle, d.get("x_off", 0)
            x2 = d.get("x2")
            st.x2, st.x2_off = (x2.handle if x2 is not None else None), d.get("x2_off", 0)
            st.prologue, st.eps, st.count = d.get("prologue", CHAIN_X_PLAIN), d.get("eps", 0.0), len(ws)
            offs = d.get("y_offs") or [0] * len(ws)
            for i, (w, y) in enumerate(zip(ws, ys)):
                st.ws[i], st.ys[i], st.y_offs[i] = w.handle, y.handle, offs[i]
            st.accum = int(bool(d.get("accum", False)))
        self._check(self._L.ojh_decode_chain(self._dev, arr, n))

    def chain_trace(self, buf: "Buf | None") -> None:
        """Timestamps of the following chain launches go to `buf` (u64 [compute units][8 stages][6 events]); None: off."""
        self._check(self._L.ojh_chain_trace(self._dev, buf.handle if buf is not None else None))

    def chain_spin_limit(self, polls: int) -> None:
        """Polls a chain's device-wide waits may take (0: every wait gives up at once)."""
        self._check(self._L.ojh_chain_spin_limit(self._dev, polls))

    def rmsnorm_quant_q8k(self, x: Buf, gamma: Buf, eps: float, m: int, k: int, q: Buf, scales: Buf,
                          xn: Buf | None = None, x_off: int = 0) -> None:
        """RMS norm + quant_q8k in one launch (xn optional f32 copy of the normalized rows)."""
        self._check(self._L.ojh_rmsnorm_quant_q8k(self._dev, x.handle, x_off, gamma.handle, eps, m, k, q.handle,
                                                  scales.handle, xn.handle if xn else None))

    def ffn_gu_q8k(self, xq: Buf, xscales: Buf, gate: Lin, up: Lin, out: Buf, act: int = 0, out_off: int = 0) -> None:
        """out = act(gate . x) * (up . x) in one launch (act 0 SiLU, 1 GELU)."""
        self._check(self._L.ojh_ffn_gu_q8k(self._dev, xq.handle, xscales.handle, gate.handle, up.handle, out.handle,
                                           out_off, act))

    def relayout_q4k_q4l(self, raw: Buf, n: int, k: int, nib: Buf, qa: Buf, qb: Buf, raw_off: int = 0) -> None:
        """Q4_K blocks -> the Q4L arrays (nibble pairs, f16 qa / qb per 32 weights)."""
        self._check(self._L.ojh_relayout_q4k_q4l(self._dev, raw.handle, raw_off, n, k, nib.handle, qa.handle, qb.handle))

    def q8rows_from_f16(self, w16: Buf, n: int, k: int, q: Buf, scale: Buf, w_off: int = 0) -> None:
        """Load-time requantization of f16 weights [n][k] to int8 rows + per-row f32 scales."""
        self._check(self._L.ojh_q8rows_from_f16(self._dev, w16.handle, w_off, n, k, q.handle, scale.handle))

    def matmul_q8(self, x: Buf, wq: Buf, wscale: Buf, y: Buf, n: int, k: int, m: int = 1, *,
                  bias: Buf | None = None, x_off: int = 0, y_off: int = 0) -> None:
        """The CPU models' row-int8 matmul: y[m][n] = bias + (qx . qw) * sw * sx."""
        self._check(self._L.ojh_matmul_q8(self._dev, x.handle, x_off, wq.handle, wscale.handle,
                                          bias.handle if bias else None, y.handle, y_off, n, k, m))

    def capture_begin(self) -> None:
        """Start recording dispatches on the device's stream instead of running them."""
        self._check(self._L.ojh_capture_begin(self._dev))

    def capture_end(self) -> "Graph":
        h = C.c_void_p()
        self._check(self._L.ojh_capture_end(self._dev, C.byref(h)))
        return Graph(self, h)

    def mark(self, slot: int) -> None:
        self._check(self._L.ojh_mark(self._dev, slot))

    def mark_elapsed(self, a: int, b: int) -> float:
        ms = C.c_float()
        self._check(self._L.ojh_mark_elapsed(self._dev, a, b, C.byref(ms)))
        return ms.value

    def dequant_f16(self, ty: int, raw: Buf, n_weights: int, out: Buf, raw_off: int = 0, out_off: int = 0) -> None:
        self._check(self._L.ojh_dequant_f16(self._dev, ty, raw.handle, raw_off, n_weights, out.handle, out_off))

    def quant_q8k(self, x: Buf, m: int, k: int, q: Buf, scales: Buf, x_dtype: int = X_F32, x_off: int = 0) -> None:
        self._check(self._L.ojh_quant_q8k(self._dev, x.handle, x_off, x_dtype, m, k, q.handle, scales.handle))

    def moe_route(self, logits: Buf, n_tokens: int, n_expert: int, ksel: int, idx: Buf, wgt: Buf) -> None:
        self._check(self._L.ojh_moe_route(self._dev, logits.handle, n_tokens, n_expert, ksel, idx.handle, wgt.handle))

    def moe_ffn_slots(self, x: Buf, n_tokens: int, d: int, n_ff: int, ksel: int, arena_gate: Buf, off_gate: Buf,
                      arena_up: Buf, off_up: Buf, arena_down: Buf, off_down: Buf, wgt: Buf, y: Buf,
                      accum: bool = False) -> None:
        """Expert FFN over streamed experts: u64 byte offsets per (token, slot) into three arenas."""
        self._check(self._L.ojh_moe_ffn_slots(self._dev, x.handle, n_tokens, d, n_ff, ksel, arena_gate.handle,
                                              off_gate.handle, arena_up.handle, off_up.handle, arena_down.handle,
                                              off_down.handle, wgt.handle, y.handle, int(accum)))

    def moe_ffn_routed(self, x: Buf, n_tokens: int, d: int, n_ff: int, n_expert: int, ksel: int, logits: Buf, idx: Buf,
                       wgt: Buf, gate: Lin, up: Lin, down: Lin, y: Buf, accum: bool = False, act_mode: int = ACT_AUTO) -> None:
        """Router + expert FFN; idx and wgt are written.  A few tokens: the router runs inside the gate/up launch."""
        self._check(self._L.ojh_moe_ffn_routed(self._dev, x.handle, n_tokens, d, n_ff, n_expert, ksel, logits.handle,
                                               idx.handle, wgt.handle, gate.handle, up.handle, down.handle, y.handle,
                                               int(accum), act_mode))

    def moe_ffn(self, x: Buf, n_tokens: int, d: int, n_ff: int, n_expert: int, ksel: int, idx: Buf, wgt: Buf,
                gate: Lin, up: Lin, down: Lin, y: Buf, accum: bool = False, act_mode: int = ACT_AUTO) -> None:
        self._check(self._L.ojh_moe_ffn(self._dev, x.handle, n_tokens, d, n_ff, n_expert, ksel, idx.handle,
                                        wgt.handle, gate.handle, up.handle, down.handle, y.handle, int(accum),
                                        act_mode))
