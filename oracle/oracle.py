"""ctypes binding of the CPU oracle (oracle/libnvfp4_oracle.so).  TEST INFRASTRUCTURE ONLY.

Only tests, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` import this
module; the product package never does.  ``build()`` compiles the C restatement with the
Makefile beside this file; ``lib()`` loads what is built (and builds it if nothing is).
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libnvfp4_oracle.so")
_lib = None

u8p = np.ctypeslib.ndpointer(np.uint8, flags="C_CONTIGUOUS")
f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
f64p = np.ctypeslib.ndpointer(np.float64, flags="C_CONTIGUOUS")
i32p = np.ctypeslib.ndpointer(np.int32, flags="C_CONTIGUOUS")


def build() -> None:
    subprocess.run(["make", "-C", _HERE, "-B", "libnvfp4_oracle.so"], check=True, capture_output=True)


def lib():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_SO):
        build()
    L = C.CDLL(_SO)
    sz, f, i = C.c_size_t, C.c_float, C.c_int
    L.orc_e2m1.restype = f
    L.orc_e2m1.argtypes = [C.c_uint32]
    L.orc_ue4m3.restype = f
    L.orc_ue4m3.argtypes = [C.c_uint32]
    L.orc_scale_rule.restype = C.c_uint8
    L.orc_scale_rule.argtypes = [C.c_uint8]
    L.orc_scale_lut.argtypes = [f, f32p]
    L.orc_dequant_raw.argtypes = [u8p, sz, f, f32p]
    L.orc_dequant.argtypes = [u8p, sz, f, f32p]
    L.orc_byte_len.restype = sz
    L.orc_byte_len.argtypes = [sz, sz]
    L.orc_encode_ue4m3_ceil.restype = C.c_uint32
    L.orc_encode_ue4m3_ceil.argtypes = [f]
    L.orc_quantize_ceil.restype = f
    L.orc_quantize_ceil.argtypes = [f32p, sz, u8p]
    L.orc_gemv.restype = i
    L.orc_gemv.argtypes = [u8p, sz, sz, f, f32p, sz, f32p, i, i]
    L.orc_expert_ffn.restype = i
    L.orc_expert_ffn.argtypes = [u8p, f, u8p, f, u8p, f, sz, sz, f32p, sz, f32p, i, i]
    L.orc_ffn_clamped.restype = i
    L.orc_ffn_clamped.argtypes = [u8p, f, u8p, f, u8p, f, sz, sz, f, f32p, sz, f32p, i, i]
    L.orc_gemv_f64.argtypes = [u8p, sz, sz, f, f32p, sz, i, f64p, f64p]
    L.orc_gamma.restype = C.c_double
    L.orc_gamma.argtypes = [sz]
    L.orc_silu_mul.restype = f
    L.orc_silu_mul.argtypes = [f, f]
    L.orc_silu_mul_combo.argtypes = [f32p, sz, sz, f32p]
    L.orc_acc_combo.argtypes = [f32p, f32p, sz, sz, sz, f32p]
    L.orc_router_topk.argtypes = [f32p, sz, sz, sz, i32p, f32p]
    L.orc_argmax_ref.restype = C.c_int32
    L.orc_argmax_ref.argtypes = [f32p, sz]
    L.orc_moe_layer.restype = i
    L.orc_moe_layer.argtypes = [u8p, f, u8p, f, sz, sz, sz, f32p, f32p, sz, sz, i32p, f32p, f32p, i, i]
    L.orc_f32_to_bf16.restype = C.c_uint16
    L.orc_f32_to_bf16.argtypes = [f]
    _lib = L
    return L


def _u8(a):
    return np.ascontiguousarray(a, dtype=np.uint8).reshape(-1)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def byte_len(rows: int, cols: int) -> int:
    return rows * (cols // 64) * 36


def e2m1(n: int) -> float:
    return lib().orc_e2m1(n)


def ue4m3(b: int) -> float:
    return lib().orc_ue4m3(b)


def scale_lut(gs: float) -> np.ndarray:
    out = np.zeros(256, np.float32)
    lib().orc_scale_lut(gs, out)
    return out


def dequant(blocks, gs: float, rule: bool = True) -> np.ndarray:
    b = _u8(blocks)
    assert b.size % 36 == 0
    out = np.empty(b.size // 36 * 64, np.float32)
    (lib().orc_dequant if rule else lib().orc_dequant_raw)(b, b.size // 36, gs, out)
    return out


def quantize_ceil(values) -> tuple[np.ndarray, float]:
    v = _f32(values).reshape(-1)
    assert v.size % 64 == 0
    out = np.empty(v.size // 64 * 36, np.uint8)
    gs = lib().orc_quantize_ceil(v, v.size, out)
    return out, float(np.float32(gs))


def gemv(w, rows: int, cols: int, gs: float, x, threads: int = 1, path: int = 1) -> np.ndarray:
    wb = _u8(w)
    if cols == 0 or cols % 64 != 0:
        raise ValueError(f"cpu_nvfp4: {cols} columns are not whole 64-value NVFP4 blocks")
    if wb.size != byte_len(rows, cols):
        raise ValueError(f"cpu_nvfp4: [{rows}, {cols}] needs {byte_len(rows, cols)} B, got {wb.size}")
    xv = _f32(x).reshape(-1, cols)
    y = np.empty((xv.shape[0], rows), np.float32)
    rc = lib().orc_gemv(wb, rows, cols, gs, xv, xv.shape[0], y, threads, path)
    assert rc == 0
    return y


def gemv_f64(w, rows: int, cols: int, gs: float, x, rule: bool = True):
    wb = _u8(w)
    xv = _f32(x).reshape(-1, cols)
    y = np.empty((xv.shape[0], rows), np.float64)
    a = np.empty((xv.shape[0], rows), np.float64)
    lib().orc_gemv_f64(wb, rows, cols, gs, xv, xv.shape[0], int(rule), y, a)
    return y, a


def gamma(cols: int) -> float:
    return lib().orc_gamma(cols)


def ffn(gate, gs_g, up, gs_u, down, gs_d, hidden, inter, x, limit: float = 0.0, threads: int = 1, path: int = 1):
    xv = _f32(x).reshape(-1, hidden)
    y = np.empty_like(xv)
    rc = lib().orc_ffn_clamped(_u8(gate), gs_g, _u8(up), gs_u, _u8(down), gs_d, hidden, inter, limit, xv,
                               xv.shape[0], y, threads, path)
    assert rc == 0
    return y


def silu_mul(g, u) -> np.ndarray:
    g, u = _f32(g), _f32(u)
    L = lib()
    return np.array([L.orc_silu_mul(float(a), float(b)) for a, b in zip(g.reshape(-1), u.reshape(-1))],
                    np.float32).reshape(g.shape)


def silu_mul_combo(h1, inter: int) -> np.ndarray:
    h = _f32(h1).reshape(-1, 2 * inter)
    out = np.empty((h.shape[0], inter), np.float32)
    lib().orc_silu_mul_combo(h, h.shape[0], inter, out)
    return out


def acc_combo(x, rw, tokens: int, topk: int, hidden: int, y0=None) -> np.ndarray:
    y = np.zeros((tokens, hidden), np.float32) if y0 is None else _f32(y0).copy()
    lib().orc_acc_combo(_f32(x), _f32(rw), tokens, topk, hidden, y)
    return y


def router_topk(logits, topk: int):
    l = _f32(logits)
    t, e = l.shape
    assert e & (e - 1) == 0, "the reference's tree reductions need a power-of-two expert count"
    ids = np.empty((t, topk), np.int32)
    w = np.empty((t, topk), np.float32)
    lib().orc_router_topk(l, t, e, topk, ids, w)
    return ids, w


def argmax_ref(logits) -> int:
    l = _f32(logits).reshape(-1)
    return int(lib().orc_argmax_ref(l, l.size))


def moe_layer(gate_up, gs_gu, down, gs_dn, experts, hidden, inter, x, logits, topk, threads: int = 1, path: int = 1):
    xv = _f32(x).reshape(-1, hidden)
    t = xv.shape[0]
    ids = np.empty((t, topk), np.int32)
    w = np.empty((t, topk), np.float32)
    y = np.empty((t, hidden), np.float32)
    rc = lib().orc_moe_layer(_u8(gate_up), gs_gu, _u8(down), gs_dn, experts, hidden, inter, xv, _f32(logits), t, topk,
                             ids, w, y, threads, path)
    assert rc == 0
    return ids, w, y


def f32_to_bf16_bits(v) -> np.ndarray:
    x = _f32(v).view(np.uint32).astype(np.uint64)
    return (((x + 0x7FFF + ((x >> 16) & 1)) >> 16) & 0xFFFF).astype(np.uint16)


def bf16_bits_to_f32(b) -> np.ndarray:
    return (np.asarray(b, np.uint16).astype(np.uint32) << 16).view(np.float32)


def gemv_bf16(w_bits, rows: int, cols: int, x) -> np.ndarray:
    """BF16-keep GEMV of the reference (engine/src/kernels.rs:1130-1157): y[t][r] = sum_k bf16(w[r][k]) * x[t][k].  The product
    is defined by the real-number sum; this restatement evaluates it in f64 (every bf16 * f32 product is exact in f64, the
    sum of K <= 2^20 of them carries a relative error below 2^-32) and rounds once to f32.  Device results are held to
    that value within the f32 dot-product bound gamma(K + 6) * sum |w x| and to the 1e-3 tolerance."""
    w = bf16_bits_to_f32(np.asarray(w_bits, np.uint16).reshape(rows, cols)).astype(np.float64)
    xv = _f32(x).reshape(-1, cols).astype(np.float64)
    return (xv @ w.T).astype(np.float32)


def gemv_f32w(w, rows: int, cols: int, x) -> np.ndarray:
    """F32-weight GEMV of the reference (gemv_b, engine/src/kernels.rs:97-115: the router projection): y[t][r] =
    sum_k w[r][k] * x[t][k].  As for gemv_bf16 the result is defined by the real-number sum: every f32 * f32 product is
    exact in f64 (48 significant bits), the f64 sum of K <= 2^20 of them is rounded once to f32.  The reference's own
    order (256 strided partial sums, then a halving tree) is one of the f32 orders the bound gamma(K) * sum |w x| covers."""
    wv = _f32(w).reshape(rows, cols).astype(np.float64)
    xv = _f32(x).reshape(-1, cols).astype(np.float64)
    return (xv @ wv.T).astype(np.float32)


def gemv_f32w_reference_order(w, rows: int, cols: int, x) -> np.ndarray:
    """The same product in the order the reference's kernel uses (engine/src/kernels.rs:104-114): thread t of 256 adds
    w[i] * x[i] for i = t, t + 256, ... in f32, each product and each add rounded on its own; then red[t] += red[t + st]
    for st = 128, 64, ..., 1."""
    wv = _f32(w).reshape(rows, cols)
    xv = _f32(x).reshape(-1, cols)
    out = np.zeros((xv.shape[0], rows), np.float32)
    pad = (-cols) % 256
    for t in range(xv.shape[0]):
        prod = (wv * xv[t][None, :]).astype(np.float32)                      # one rounding per product
        prod = np.pad(prod, ((0, 0), (0, pad))).reshape(rows, -1, 256)       # step j, thread t: column 256 j + t
        red = np.zeros((rows, 256), np.float32)
        for j in range(prod.shape[1]):
            live = min(256, cols - 256 * j)                                  # threads beyond K add nothing on the last step
            red[:, :live] = (red[:, :live] + prod[:, j, :live]).astype(np.float32)
        st = 128
        while st > 0:
            red[:, :st] = (red[:, :st] + red[:, st:2 * st]).astype(np.float32)
            st >>= 1
        out[t] = red[:, 0]
    return out
