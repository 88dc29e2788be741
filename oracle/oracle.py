"""TEST INFRASTRUCTURE — ctypes binding of the CPU oracle (libojas_oracle.so).

The oracle restates the reference's CPU arithmetic for the quantized-matmul path and is what the
HIP kernels are checked against.  Only the test-suite, the smoke check and the CPU-baseline leg of
the benchmark may import this module; the product path never does.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libojas_oracle.so")

Q8_0, Q4_K, Q5_K, Q6_K, IQ4_NL, IQ4_XS = 8, 12, 13, 14, 20, 23
IQ2_XXS, IQ2_XS, IQ3_XXS, IQ1_S, IQ3_S, IQ2_S, IQ1_M = 16, 17, 18, 19, 21, 22, 29
MXFP4 = 139
Q4_0, Q4_1, Q5_0, Q5_1 = 2, 3, 6, 7
Q2_K, Q3_K = 10, 11


def build(force: bool = False) -> str:
    """Compile the oracle with the Makefile beside this file."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.check_call(["make", "-s", "-C", _HERE])
    return _LIB_PATH


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = C.CDLL(_LIB_PATH)
        vp, sz, u32, i32 = C.c_void_p, C.c_size_t, C.c_uint32, C.c_int
        L.ojo_f16_to_f32.restype = C.c_float
        L.ojo_f16_to_f32.argtypes = [C.c_uint16]
        L.ojo_f32_to_f16.restype = C.c_uint16
        L.ojo_f32_to_f16.argtypes = [C.c_float]
        L.ojo_f32_to_bf16.restype = C.c_uint16
        L.ojo_f32_to_bf16.argtypes = [C.c_float]
        L.ojo_block_shape.argtypes = [u32, C.POINTER(u32), C.POINTER(u32)]
        L.ojo_synth_blocks.argtypes = [u32, sz, vp]
        L.ojo_dequant_to_f16.argtypes = [vp, u32, sz, vp]
        L.ojo_dequant_to_f64.argtypes = [vp, u32, sz, vp]
        L.ojo_digest_f16.restype = C.c_uint64
        L.ojo_digest_f16.argtypes = [vp, sz]
        L.ojo_quant_q8k.restype = None
        L.ojo_quant_q8k.argtypes = [vp, sz, vp, vp, vp]
        for name in ("ojo_dot_q80", "ojo_dot_iq4nl", "ojo_dot_iq4xs"):
            f = getattr(L, name)
            f.restype = C.c_float
            f.argtypes = [vp, vp, sz]
        L.ojo_dot_iq_grid.restype = C.c_float
        L.ojo_dot_iq_grid.argtypes = [u32, vp, vp, sz]
        for name in ("ojo_dot_iq2xxs_q8k", "ojo_dot_iq3xxs_q8k"):
            f = getattr(L, name)
            f.restype = C.c_float
            f.argtypes = [vp, sz, vp, vp]
        L.ojo_iq_grid_bytes.restype = sz
        L.ojo_iq_grid_bytes.argtypes = [i32, vp]
        for name in ("ojo_dot_q4k", "ojo_dot_q5k", "ojo_dot_q6k"):
            f = getattr(L, name)
            f.restype = C.c_float
            f.argtypes = [vp, sz, vp, vp, vp]
        L.ojo_matvec_kq.argtypes = [vp, u32, sz, sz, vp, i32, vp]
        L.ojo_quant_row_i8.restype = C.c_float
        L.ojo_quant_row_i8.argtypes = [vp, sz, vp]
        L.ojo_quantize_q8_1.restype = None
        L.ojo_quantize_q8_1.argtypes = [vp, sz, vp, vp, vp]
        L.ojo_gemv_q80_dp4a.restype = None
        L.ojo_gemv_q80_dp4a.argtypes = [vp, vp, vp, sz, sz, vp]
        L.ojo_gemv_q8_rows.argtypes = [vp, vp, vp, sz, sz, vp]
        L.ojo_gemv_q8_rows.restype = None
        L.ojo_quantize_q8_pertoken.argtypes = [vp, sz, sz, vp, vp]
        L.ojo_quantize_q8_pertoken.restype = None
        L.ojo_q8_rows_from_f16.restype = None
        L.ojo_q8_rows_from_f16.argtypes = [vp, sz, sz, vp, vp]
        L.ojo_matmul_q8.restype = None
        L.ojo_matmul_q8.argtypes = [vp, vp, sz, sz, vp, sz, vp, i32, vp]
        L.ojo_relayout_q4k_q4l.restype = None
        L.ojo_relayout_q4k_q4l.argtypes = [vp, sz, sz, vp, vp, vp]
        L.ojo_q4l_weights_f16.restype = None
        L.ojo_q4l_weights_f16.argtypes = [vp, sz, sz, vp]
        L.ojo_matmul_ref.argtypes = [vp, u32, sz, sz, vp, sz, i32, i32, i32, vp]
        L.ojo_rmsnorm.restype = None
        L.ojo_rmsnorm.argtypes = [vp, vp, sz, C.c_float, vp]
        L.ojo_ffn_act.restype = C.c_float
        L.ojo_ffn_act.argtypes = [C.c_float, i32]
        L.ojo_moe_topk.restype = None
        L.ojo_moe_topk.argtypes = [vp, i32, i32, vp, vp]
        L.ojo_moe_topk_nonorm.restype = None
        L.ojo_moe_topk_nonorm.argtypes = [vp, i32, i32, vp, vp]
        L.ojo_moe_topk_v3.restype = None
        L.ojo_moe_topk_v3.argtypes = [vp, vp, i32, i32, C.c_float, i32, vp, vp]
        L.ojo_moe_ffn.argtypes = [vp, sz, sz, sz, i32, i32, vp, vp, vp, vp, u32, vp, u32, i32, i32, vp]
        _lib = L
    return _lib


def _p(a: np.ndarray) -> C.c_void_p:
    assert a.flags["C_CONTIGUOUS"]
    return C.c_void_p(a.ctypes.data)


def block_shape(ty: int) -> tuple[int, int]:
    b, w = C.c_uint32(), C.c_uint32()
    if not lib().ojo_block_shape(ty, C.byref(b), C.byref(w)):
        raise ValueError(f"unknown GGUF type {ty}")
    return b.value, w.value


def row_bytes(ty: int, k: int) -> int:
    bb, wpb = block_shape(ty)
    assert k % wpb == 0
    return k // wpb * bb


def synth_blocks(ty: int, nb: int) -> np.ndarray:
    bb, _ = block_shape(ty)
    out = np.empty(nb * bb, np.uint8)
    assert lib().ojo_synth_blocks(ty, nb, _p(out)) == 0
    return out


def dequant_to_f16(raw: np.ndarray, ty: int, n: int) -> np.ndarray:
    """Bit patterns (uint16) of the dequantized weights."""
    raw = np.ascontiguousarray(raw, np.uint8)
    out = np.empty(n, np.uint16)
    assert lib().ojo_dequant_to_f16(_p(raw), ty, n, _p(out)) == 0
    return out


def dequant_to_f64(raw: np.ndarray, ty: int, n: int) -> np.ndarray:
    raw = np.ascontiguousarray(raw, np.uint8)
    out = np.empty(n, np.float64)
    assert lib().ojo_dequant_to_f64(_p(raw), ty, n, _p(out)) == 0
    return out


def digest_f16(bits: np.ndarray) -> int:
    bits = np.ascontiguousarray(bits, np.uint16)
    return int(lib().ojo_digest_f16(_p(bits), bits.size))


def quant_q8k(x: np.ndarray):
    x = np.ascontiguousarray(x, np.float32)
    nsb = (x.size + 255) // 256
    scales = np.empty(nsb, np.float32)
    q = np.empty(nsb * 256, np.int8)
    bsums = np.empty(nsb * 8, np.int32)
    lib().ojo_quant_q8k(_p(x), x.size, _p(scales), _p(q), _p(bsums))
    return scales, q, bsums


def dot_q80(row: np.ndarray, x: np.ndarray) -> float:
    row = np.ascontiguousarray(row, np.uint8)
    x = np.ascontiguousarray(x, np.float32)
    return float(lib().ojo_dot_q80(_p(row), _p(x), x.size))


def dot_iq(ty: int, row: np.ndarray, x: np.ndarray) -> float:
    """dot_iq4nl / dot_iq4xs / dot_iq2xxs / dot_iq3xxs / dot_iq2s / dot_iq3s: raw row against f32 activations."""
    row = np.ascontiguousarray(row, np.uint8)
    x = np.ascontiguousarray(x, np.float32)
    if ty in (IQ2_XXS, IQ3_XXS, IQ3_S, IQ2_S):
        return float(lib().ojo_dot_iq_grid(ty, _p(row), _p(x), x.size))
    fn = {IQ4_NL: lib().ojo_dot_iq4nl, IQ4_XS: lib().ojo_dot_iq4xs}[ty]
    return float(fn(_p(row), _p(x), x.size))


def dot_iq_q8k(ty: int, row: np.ndarray, k: int, act) -> float:
    """dot_iq2xxs_q8k / dot_iq3xxs_q8k: raw row against quant_q8k activations."""
    fn = {IQ2_XXS: lib().ojo_dot_iq2xxs_q8k, IQ3_XXS: lib().ojo_dot_iq3xxs_q8k}[ty]
    row = np.ascontiguousarray(row, np.uint8)
    s, q, _ = act
    return float(fn(_p(row), k, _p(s), _p(q)))


def matvec_iq_f32(raw: np.ndarray, ty: int, n: int, k: int, x: np.ndarray) -> np.ndarray:
    """Rows of an IQ format against f32 activations (dot_iq, cpu_math.rs:1131-1141), row by row."""
    rb = row_bytes(ty, k)
    raw = np.ascontiguousarray(raw, np.uint8)
    return np.array([dot_iq(ty, raw[r * rb:(r + 1) * rb], x) for r in range(n)], np.float32)


def iq_grid_bytes(which: int) -> np.ndarray:
    """A published codebook (0 iq2xxs, 1 iq2xs, 2 iq2s, 3 iq3xxs, 4 iq3s, 5 iq1s) expanded from its packed form."""
    out = np.empty(lib().ojo_iq_grid_bytes(which, None), np.uint8)
    lib().ojo_iq_grid_bytes(which, _p(out))
    return out


def dot_kq(ty: int, row: np.ndarray, k: int, act) -> float:
    fn = {Q4_K: lib().ojo_dot_q4k, Q5_K: lib().ojo_dot_q5k, Q6_K: lib().ojo_dot_q6k}[ty]
    row = np.ascontiguousarray(row, np.uint8)
    s, q, b = act
    return float(fn(_p(row), k, _p(s), _p(q), _p(b)))


def matvec_kq(raw: np.ndarray, ty: int, n: int, k: int, x: np.ndarray, threads: int = 8) -> np.ndarray:
    raw = np.ascontiguousarray(raw, np.uint8)
    x = np.ascontiguousarray(x, np.float32)
    assert raw.size == n * row_bytes(ty, k) and x.size == k
    y = np.empty(n, np.float32)
    assert lib().ojo_matvec_kq(_p(raw), ty, n, k, _p(x), threads, _p(y)) == 0
    return y


def quant_row_i8(row: np.ndarray):
    row = np.ascontiguousarray(row, np.float32)
    q = np.empty(row.size, np.int8)
    s = lib().ojo_quant_row_i8(_p(row), row.size, _p(q))
    return q, float(s)


def quantize_q8_1(x: np.ndarray):
    x = np.ascontiguousarray(x, np.float32)
    q8, d8, d8sum = np.empty(x.size, np.int8), np.empty(x.size // 32, np.float32), np.empty(x.size // 32, np.float32)
    lib().ojo_quantize_q8_1(_p(x), x.size, _p(q8), _p(d8), _p(d8sum))
    return q8, d8, d8sum


def gemv_q80_dp4a(raw: np.ndarray, q8: np.ndarray, d8: np.ndarray, n: int, k: int) -> np.ndarray:
    raw, q8, d8 = np.ascontiguousarray(raw, np.uint8), np.ascontiguousarray(q8, np.int8), np.ascontiguousarray(d8, np.float32)
    assert raw.size == n * (k // 32) * 34 and q8.size == k and d8.size == k // 32
    y = np.empty(n, np.float32)
    lib().ojo_gemv_q80_dp4a(_p(raw), _p(q8), _p(d8), k, n, _p(y))
    return y


def gemv_q8_rows(w: np.ndarray, scale: np.ndarray, x: np.ndarray) -> np.ndarray:
    """y[n] = scale[n] * sum_k w[n][k] x[k] for row-int8 weights w [N][K] (the reference GPU decoder's `gemv_q8`)."""
    w, scale, x = np.ascontiguousarray(w, np.int8), np.ascontiguousarray(scale, np.float32), np.ascontiguousarray(x, np.float32)
    n, k = w.shape
    assert scale.size == n and x.size == k
    y = np.empty(n, np.float32)
    lib().ojo_gemv_q8_rows(_p(w), _p(scale), _p(x), k, n, _p(y))
    return y


def quantize_q8_pertoken(x: np.ndarray):
    x = np.ascontiguousarray(x, np.float32)
    m, k = x.shape
    q8, d8 = np.empty((m, k), np.int8), np.empty(m, np.float32)
    lib().ojo_quantize_q8_pertoken(_p(x), m, k, _p(q8), _p(d8))
    return q8, d8


def q8_rows_from_f16(w16: np.ndarray, n: int, k: int):
    w16 = np.ascontiguousarray(w16, np.uint16)
    q = np.empty(n * k, np.int8)
    s = np.empty(n, np.float32)
    lib().ojo_q8_rows_from_f16(_p(w16), n, k, _p(q), _p(s))
    return q, s


def matmul_q8(wq, wscale, n, k, xs, bias=None, threads: int = 8) -> np.ndarray:
    wq = np.ascontiguousarray(wq, np.int8)
    wscale = np.ascontiguousarray(wscale, np.float32)
    xs = np.ascontiguousarray(xs, np.float32).reshape(-1, k)
    m = xs.shape[0]
    ys = np.empty((m, n), np.float32)
    bp = None
    if bias is not None:
        bias = np.ascontiguousarray(bias, np.float32)
        bp = _p(bias)
    lib().ojo_matmul_q8(_p(wq), _p(wscale), n, k, _p(xs), m, bp, threads, _p(ys))
    return ys


def relayout_q4k_q4l(w: np.ndarray, k: int, n: int):
    w = np.ascontiguousarray(w, np.uint8)
    nib = np.empty(n * k // 2, np.uint8)
    qa = np.empty(n * k // 32, np.uint16)
    qb = np.empty(n * k // 32, np.uint16)
    lib().ojo_relayout_q4k_q4l(_p(w), k, n, _p(nib), _p(qa), _p(qb))
    return nib, qa, qb


def q4l_weights_f16(w: np.ndarray, k: int, n: int) -> np.ndarray:
    """binary16 bit patterns [n*k] of fma(qa, q, qb): the Q4L GPU kernel's in-tile weights."""
    w = np.ascontiguousarray(w, np.uint8)
    assert w.size == n * k // 256 * 144
    out = np.empty(n * k, np.uint16)
    lib().ojo_q4l_weights_f16(_p(w), k, n, _p(out))
    return out


def matmul_ref(raw, ty, n, k, x, wmode: int = 0, xmode: int = 0, threads: int = 8) -> np.ndarray:
    """y[m][n] in float64; wmode 0 exact / 1 f16-rounded weights / 2 Q4L kernel weights; xmode 0 / 1 f16 / 2 bf16."""
    raw = np.ascontiguousarray(raw, np.uint8)
    x = np.ascontiguousarray(x, np.float32).reshape(-1, k)
    m = x.shape[0]
    assert raw.size == n * row_bytes(ty, k)
    y = np.empty((m, n), np.float64)
    assert lib().ojo_matmul_ref(_p(raw), ty, n, k, _p(x), m, wmode, xmode, threads, _p(y)) == 0
    return y


def rmsnorm(x: np.ndarray, w: np.ndarray, eps: float) -> np.ndarray:
    x = np.ascontiguousarray(x, np.float32)
    w = np.ascontiguousarray(w, np.float32)
    y = np.empty_like(x)
    lib().ojo_rmsnorm(_p(x), _p(w), x.size, eps, _p(y))
    return y


def ffn_act(g: np.ndarray, act: int = 0) -> np.ndarray:
    g = np.ascontiguousarray(g, np.float32)
    return np.array([lib().ojo_ffn_act(float(v), act) for v in g.ravel()], np.float32).reshape(g.shape)


def moe_topk(logits: np.ndarray, ksel: int):
    logits = np.ascontiguousarray(logits, np.float32)
    T, E = logits.reshape(-1, logits.shape[-1]).shape
    idx = np.empty((T, ksel), np.uint32)
    wgt = np.empty((T, ksel), np.float32)
    lg = logits.reshape(T, E)
    for t in range(T):
        lib().ojo_moe_topk(C.c_void_p(lg[t].ctypes.data), E, ksel,
                           C.c_void_p(idx[t].ctypes.data), C.c_void_p(wgt[t].ctypes.data))
    return idx, wgt


def moe_topk_nonorm(logits: np.ndarray, ksel: int):
    lg = np.ascontiguousarray(logits, np.float32).reshape(-1, logits.shape[-1])
    T, E = lg.shape
    idx, wgt = np.empty((T, ksel), np.uint32), np.empty((T, ksel), np.float32)
    for t in range(T):
        lib().ojo_moe_topk_nonorm(C.c_void_p(lg[t].ctypes.data), E, ksel, C.c_void_p(idx[t].ctypes.data), C.c_void_p(wgt[t].ctypes.data))
    return idx, wgt


def moe_topk_v3(logits: np.ndarray, bias: np.ndarray, ksel: int, rscale: float = 1.0, norm: bool = True):
    lg = np.ascontiguousarray(logits, np.float32).reshape(-1, logits.shape[-1])
    b = np.ascontiguousarray(bias, np.float32)
    T, E = lg.shape
    idx, wgt = np.empty((T, ksel), np.uint32), np.empty((T, ksel), np.float32)
    for t in range(T):
        lib().ojo_moe_topk_v3(C.c_void_p(lg[t].ctypes.data), C.c_void_p(b.ctypes.data), E, ksel, C.c_float(rscale), int(norm),
                              C.c_void_p(idx[t].ctypes.data), C.c_void_p(wgt[t].ctypes.data))
    return idx, wgt


def moe_ffn(x, idx, wgt, gate, up, ty_gu, down, ty_d, n_expert, n_ff, mode: int = 0,
            threads: int = 8, y0=None) -> np.ndarray:
    x = np.ascontiguousarray(x, np.float32)
    T, d = x.shape
    idx = np.ascontiguousarray(idx, np.uint32).reshape(T, -1)
    wgt = np.ascontiguousarray(wgt, np.float32).reshape(T, -1)
    ksel = idx.shape[1]
    gate = np.ascontiguousarray(gate, np.uint8)
    up = np.ascontiguousarray(up, np.uint8)
    down = np.ascontiguousarray(down, np.uint8)
    y = np.zeros((T, d), np.float32) if y0 is None else np.array(y0, np.float32, copy=True).reshape(T, d)
    rc = lib().ojo_moe_ffn(_p(x), T, d, n_ff, n_expert, ksel, _p(idx), _p(wgt), _p(gate), _p(up),
                           ty_gu, _p(down), ty_d, mode, threads, _p(y))
    assert rc == 0, rc
    return y
