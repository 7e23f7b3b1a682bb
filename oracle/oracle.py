"""numpy/ctypes front end of the C oracle (oracle/oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by
bench.py's cpu_baseline leg, never by the inductor_x_amd package.

bf16 arrays are numpy uint16 arrays holding the raw bits.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "_build", "liboracle.so")
_lib = None


def build(force: bool = False) -> str:
    if force or not os.path.exists(LIB_PATH) or os.path.getmtime(LIB_PATH) < os.path.getmtime(
        os.path.join(_HERE, "oracle.c")
    ):
        subprocess.run(["make", "-C", _HERE, "-B" if force else "-s", "all"], check=True, capture_output=True)
    return LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        l = ctypes.CDLL(LIB_PATH)
        vp, i64 = ctypes.c_void_p, ctypes.c_int64
        l.oracle_relu_sigmoid_rowsum_f32.argtypes = [vp, vp, i64, i64]
        l.oracle_relu_sigmoid_rowsum_f32.restype = None
        l.oracle_add_rmsnorm_bf16.argtypes = [vp, vp, vp, vp, vp, i64, i64, ctypes.c_float]
        l.oracle_add_rmsnorm_bf16.restype = None
        l.oracle_col_mean_var_argmax_f32.argtypes = [vp, vp, vp, vp, i64, i64, ctypes.c_double]
        l.oracle_col_mean_var_argmax_f32.restype = None
        l.oracle_gather_rows.argtypes = [vp, vp, vp, i64, i64, i64]
        l.oracle_gather_rows.restype = ctypes.c_int
        l.oracle_permute4.argtypes = [vp, vp, vp, vp, i64]
        l.oracle_permute4.restype = None
        l.oracle_attention_bf16.argtypes = [vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, ctypes.c_float, ctypes.c_int]
        l.oracle_attention_bf16.restype = None
        _lib = l
    return _lib


def _p(a: np.ndarray) -> ctypes.c_void_p:
    return ctypes.c_void_p(a.ctypes.data)


def _c(a, dtype) -> np.ndarray:
    a = np.ascontiguousarray(a)
    if a.dtype != dtype:
        raise TypeError(f"expected {dtype}, got {a.dtype}")
    return a


# bf16 helpers (numpy has no bf16): round-to-nearest-even, quiet NaNs
def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    r[nan] = ((u[nan] >> 16) | 0x40).astype(np.uint16)
    return r


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def relu_sigmoid_rowsum(x: np.ndarray) -> np.ndarray:
    x = _c(x, np.float32)
    cols = x.shape[-1]
    rows = x.size // cols if cols else 0
    y = np.zeros(x.shape[:-1], dtype=np.float32)
    if rows and cols:
        lib().oracle_relu_sigmoid_rowsum_f32(_p(x), _p(y), rows, cols)
    return y


def add_rmsnorm_bf16(h: np.ndarray, r: np.ndarray, w: np.ndarray, eps: float = 1e-6):
    """h, r: uint16 bf16 bits [..., cols]; w: [cols].  Returns (out, h_plus_r) as bf16 bits."""
    h, r, w = _c(h, np.uint16), _c(r, np.uint16), _c(w, np.uint16)
    cols = h.shape[-1]
    rows = h.size // cols if cols else 0
    out = np.zeros_like(h)
    s = np.zeros_like(h)
    if rows and cols:
        lib().oracle_add_rmsnorm_bf16(_p(h), _p(r), _p(w), _p(out), _p(s), rows, cols, eps)
    return out, s


def col_mean_var_argmax(x: np.ndarray, correction: float = 0.0):
    x = _c(x, np.float32)
    rows, cols = x.shape
    mean = np.zeros(cols, np.float32)
    var = np.zeros(cols, np.float32)
    arg = np.zeros(cols, np.int64)
    if cols:
        lib().oracle_col_mean_var_argmax_f32(_p(x), _p(mean), _p(var), _p(arg), rows, cols, float(correction))
    return mean, var, arg


def gather_rows(table: np.ndarray, idx: np.ndarray) -> np.ndarray:
    table = np.ascontiguousarray(table)
    idx = _c(idx, np.int64)
    out = np.zeros(idx.shape + table.shape[1:], dtype=table.dtype)
    row_bytes = table.dtype.itemsize * int(np.prod(table.shape[1:]))
    if idx.size and row_bytes:
        bad = lib().oracle_gather_rows(_p(table), _p(idx), _p(out), idx.size, row_bytes, table.shape[0])
        if bad:
            raise IndexError("gather index out of range")
    return out


def permute4(t: np.ndarray, perm) -> np.ndarray:
    t = np.ascontiguousarray(t)
    assert t.ndim == 4 and sorted(perm) == [0, 1, 2, 3]
    shape = np.array(t.shape, dtype=np.int64)
    p = np.array(perm, dtype=np.int32)
    out = np.zeros(tuple(t.shape[i] for i in perm), dtype=t.dtype)
    if t.size:
        lib().oracle_permute4(_p(t), _p(out), _p(shape), _p(p), t.dtype.itemsize)
    return out


def attention_bf16(q: np.ndarray, k: np.ndarray, v: np.ndarray, scale: float, causal: bool):
    """q [B,N,Sq,D], k/v [B,N,Sk,D] as bf16 bits.  Returns (out bits, softmax_max, softmax_sum)."""
    q, k, v = _c(q, np.uint16), _c(k, np.uint16), _c(v, np.uint16)
    B, N, Sq, D = q.shape
    Sk = k.shape[2]
    out = np.zeros_like(q)
    smax = np.zeros((B, N, Sq, 8), np.float32)
    ssum = np.zeros((B, N, Sq, 8), np.float32)
    if q.size:
        lib().oracle_attention_bf16(_p(q), _p(k), _p(v), _p(out), _p(smax), _p(ssum), B, N, Sq, Sk, D, scale, int(causal))
    return out, smax, ssum


def attention_bwd(q: np.ndarray, k: np.ndarray, v: np.ndarray, dout: np.ndarray, scale: float, causal: bool):
    """q, k, v, dout [B,N,S,D] as bf16 bits.  Returns (dq, dk, dv) as float64 arrays."""
    q, k, v, dout = _c(q, np.uint16), _c(k, np.uint16), _c(v, np.uint16), _c(dout, np.uint16)
    B, N, S, D = q.shape
    dq = np.zeros(q.shape, np.float64)
    dk = np.zeros(q.shape, np.float64)
    dv = np.zeros(q.shape, np.float64)
    if q.size:
        fn = lib().oracle_attention_bwd
        fn.argtypes = [ctypes.c_void_p] * 7 + [ctypes.c_int64] * 4 + [ctypes.c_double, ctypes.c_int]
        fn.restype = None
        fn(_p(q), _p(k), _p(v), _p(dout), _p(dq), _p(dk), _p(dv), B, N, S, D, float(scale), int(causal))
    return dq, dk, dv


def forward_update(prev_out, prev_max, prev_sum, cur_out, cur_max, cur_sum):
    """Ring-attention merge, (max, sum) statistics.  prev_out / cur_out [S, B, H] float32, statistics
    [B, N, S, 8] float32 (all contiguous).  Returns (out, max, sum) as float64 arrays."""
    prev_out, cur_out = _c(prev_out, np.float32), _c(cur_out, np.float32)
    prev_max, prev_sum = _c(prev_max, np.float32), _c(prev_sum, np.float32)
    cur_max, cur_sum = _c(cur_max, np.float32), _c(cur_sum, np.float32)
    S, B, H = prev_out.shape
    Bs, N, Ss, E = prev_max.shape
    assert (Bs, Ss, E) == (B, S, 8) and H % N == 0 and cur_out.shape == prev_out.shape
    assert prev_sum.shape == cur_max.shape == cur_sum.shape == prev_max.shape
    out = np.zeros(prev_out.shape, np.float64)
    mx = np.zeros(prev_max.shape, np.float64)
    sm = np.zeros(prev_max.shape, np.float64)
    fn = lib().oracle_forward_update
    fn.argtypes = [ctypes.c_void_p] * 9 + [ctypes.c_int64] * 8
    fn.restype = None
    fn(_p(prev_out), _p(prev_max), _p(prev_sum), _p(cur_out), _p(cur_max), _p(cur_sum), _p(out), _p(mx), _p(sm),
       S, B, N, H // N, B * H, N * S * 8, S * 8, 8)
    return out, mx, sm


def forward_update_lse(prev_out, prev_lse, cur_out, cur_lse):
    """Ring-attention merge, log-sum-exp statistics.  prev_out / cur_out [..., D] float32, lse [..., 1]
    float32.  Returns (out, lse) as float64 arrays."""
    prev_out, cur_out = _c(prev_out, np.float32), _c(cur_out, np.float32)
    prev_lse, cur_lse = _c(prev_lse, np.float32), _c(cur_lse, np.float32)
    D = prev_out.shape[-1]
    rows = prev_out.size // D
    assert prev_lse.size == rows and cur_lse.size == rows and cur_out.shape == prev_out.shape
    out = np.zeros(prev_out.shape, np.float64)
    lse = np.zeros(prev_lse.shape, np.float64)
    fn = lib().oracle_forward_update_lse
    fn.argtypes = [ctypes.c_void_p] * 6 + [ctypes.c_int64] * 2
    fn.restype = None
    fn(_p(prev_out), _p(prev_lse), _p(cur_out), _p(cur_lse), _p(out), _p(lse), rows, D)
    return out, lse


def add_bf16(dst: np.ndarray, src: np.ndarray) -> np.ndarray:
    """bf16(float(dst) + float(src)) element by element, on raw bf16 bits; returns a new array."""
    dst, src = _c(dst, np.uint16).copy(), _c(src, np.uint16)
    assert dst.shape == src.shape
    fn = lib().oracle_add_bf16
    fn.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64]
    fn.restype = None
    fn(_p(dst), _p(src), dst.size)
    return dst
