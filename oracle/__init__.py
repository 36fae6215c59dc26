"""numpy/ctypes front end of the CPU oracle (``librumus_oracle.so``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, by ``__graft_entry__.smoke``
and by the ``cpu_baseline`` leg of ``bench.py``.  Nothing under ``rumus_amd``
imports this package; the product path is the HIP library and fails loudly
without it.

Each wrapper allocates numpy outputs and forwards to the C function of the same
name in ``rumus_oracle.c`` (which cites the reference lines it follows).
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "librumus_oracle.so")


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (``make -C oracle``)."""
    if force and os.path.exists(_SO):
        os.remove(_SO)
    subprocess.check_call(["make", "-s", "-C", _HERE])
    return _SO


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = C.CDLL(_SO)
        _lib.orc_q8_buf_size.restype = C.c_uint64
        _lib.orc_q8_buf_size.argtypes = [C.c_uint64, C.c_uint32]
        _lib.orc_f32_to_f16_bits.restype = C.c_uint16
        _lib.orc_f32_to_f16_bits.argtypes = [C.c_float]
        _lib.orc_f16_bits_to_f32.restype = C.c_float
        _lib.orc_f16_bits_to_f32.argtypes = [C.c_uint16]
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


# --------------------------------------------------------------------------
# INT4 engine
# --------------------------------------------------------------------------

def w4_geometry(k: int, group_size: int):
    padded_k = ((k + group_size - 1) // group_size) * group_size
    return padded_k, padded_k // group_size


def w4_from_f32(w, group_size: int, symmetric: bool = False):
    """w [K,N] f32 -> (packed u32 [padded_k/8, N], scales, zp f32 [G, N])."""
    w = _f32(w)
    k, n = w.shape
    if group_size <= 0 or group_size % 8:
        raise ValueError("group_size must be a multiple of 8")
    padded_k, g = w4_geometry(k, group_size)
    packed = np.zeros((padded_k // 8, n), np.uint32)
    scales = np.zeros((g, n), np.float32)
    zp = np.zeros((g, n), np.float32)
    fn = lib().orc_w4_sym_from_f32 if symmetric else lib().orc_w4_from_f32
    rc = fn(_p(w), C.c_size_t(k), C.c_size_t(n), C.c_size_t(group_size),
            _p(packed), _p(scales), _p(zp))
    if rc != 0:
        raise RuntimeError(f"oracle w4_from_f32 failed: {rc}")
    return packed, scales, zp


def w4_awq_from_f32(w, group_size: int):
    """AWQ storage: w [K,N] -> (packed u32 [padded_k/8, N], scales f32 [G, N], qzeros u32 [G, N/8])."""
    w = _f32(w)
    k, n = w.shape
    if group_size <= 0 or group_size % 8 or n % 8:
        raise ValueError("group_size and n must be multiples of 8")
    padded_k, g = w4_geometry(k, group_size)
    packed = np.zeros((padded_k // 8, n), np.uint32)
    scales = np.zeros((g, n), np.float32)
    qzeros = np.zeros((g, n // 8), np.uint32)
    rc = lib().orc_w4_awq_from_f32(_p(w), C.c_size_t(k), C.c_size_t(n), C.c_size_t(group_size),
                                   _p(packed), _p(scales), _p(qzeros))
    if rc != 0:
        raise RuntimeError(f"oracle w4_awq_from_f32 failed: {rc}")
    return packed, scales, qzeros


def w4_qzeros_unpack(qzeros, n: int):
    """qzeros u32 [G, N/8] -> zero-points f32 [G, N] (column col in bits 4*(col%8) of word col/8)."""
    qzeros = np.ascontiguousarray(qzeros, np.uint32)
    cols = np.arange(n)
    return ((qzeros[:, cols // 8] >> (4 * (cols % 8)).astype(np.uint32)) & 0xF).astype(np.float32)


def qmatmul_int4(x, packed, scales, zp, k: int, group_size: int, bias=None,
                 g_idx=None, threads: int = 1):
    x = _f32(x)
    m = x.shape[0]
    assert x.shape[1] == k
    n = packed.shape[1]
    padded_k, g = w4_geometry(k, group_size)
    assert packed.shape[0] == padded_k // 8 and scales.shape == (g, n)
    packed = np.ascontiguousarray(packed, np.uint32)
    scales, zp = _f32(scales), _f32(zp)
    bias = None if bias is None else _f32(bias)
    g_idx = None if g_idx is None else np.ascontiguousarray(g_idx, np.int32)
    y = np.empty((m, n), np.float32)
    lib().orc_qmatmul_int4(_p(x), _p(packed), _p(scales), _p(zp), _p(bias), _p(g_idx),
                           _p(y), C.c_uint32(m), C.c_uint32(k), C.c_uint32(n),
                           C.c_uint32(padded_k), C.c_uint32(group_size), C.c_uint32(g),
                           C.c_int(threads))
    return y


def qmatmul_int4_t(a, packed, scales, zp, k: int, group_size: int, threads: int = 1):
    a = _f32(a)
    m, n = a.shape
    padded_k, g = w4_geometry(k, group_size)
    packed = np.ascontiguousarray(packed, np.uint32)
    scales, zp = _f32(scales), _f32(zp)
    out = np.empty((m, k), np.float32)
    lib().orc_qmatmul_int4_t(_p(a), _p(packed), _p(scales), _p(zp), _p(out),
                             C.c_uint32(m), C.c_uint32(k), C.c_uint32(n),
                             C.c_uint32(padded_k), C.c_uint32(group_size), C.c_uint32(g),
                             C.c_int(threads))
    return out


def w4_unpack(packed, k: int):
    """packed [padded_k/8, N] -> nibbles u8 [k, N] (row r = nibble r%8 of word r//8)."""
    packed = np.asarray(packed, np.uint32)
    shifts = (np.arange(8, dtype=np.uint32) * 4)[None, :, None]
    q = (packed[:, None, :] >> shifts) & np.uint32(15)
    return q.reshape(-1, packed.shape[1])[:k].astype(np.uint8)


# --------------------------------------------------------------------------
# INT8 engine, reference block format
# --------------------------------------------------------------------------

def q8_buf_size(numel: int, block_size: int) -> int:
    return int(lib().orc_q8_buf_size(numel, block_size))


def q8_stride_words(block_size: int) -> int:
    return (4 + block_size + 3) // 4


def q8_quantize(flat, block_size: int):
    flat = _f32(flat).reshape(-1)
    if block_size <= 0 or block_size % 4:
        raise ValueError("block_size must be > 0 and divisible by 4")
    numel = flat.size
    num_blocks = (numel + block_size - 1) // block_size
    out = np.zeros(num_blocks * q8_stride_words(block_size), np.uint32)
    rc = lib().orc_q8_quantize(_p(flat), _p(out), C.c_uint32(numel), C.c_uint32(block_size))
    if rc != 0:
        raise RuntimeError("oracle q8_quantize failed")
    return out


def q8_dequantize(words, numel: int, block_size: int):
    words = np.ascontiguousarray(words, np.uint32)
    out = np.empty(numel, np.float32)
    lib().orc_q8_dequantize(_p(words), _p(out), C.c_uint32(numel), C.c_uint32(block_size))
    return out


def tensor_quantize(w, block_size: int):
    """Tensor::quantize of a [K,N] weight: transpose to [N,K], flatten, block."""
    w = _f32(w)
    return q8_quantize(np.ascontiguousarray(w.T), block_size)


def matmul_q8(a, words, k: int, n: int, block_size: int, threads: int = 1):
    a = _f32(a)
    m = a.shape[0]
    assert a.shape[1] == k
    words = np.ascontiguousarray(words, np.uint32)
    c = np.empty((m, n), np.float32)
    lib().orc_matmul_q8(_p(a), _p(words), _p(c), C.c_uint32(m), C.c_uint32(k),
                        C.c_uint32(n), C.c_uint32(block_size), C.c_int(threads))
    return c


def add_bias(mat, bias):
    mat, bias = _f32(mat), _f32(bias)
    m, n = mat.shape
    out = np.empty_like(mat)
    lib().orc_add_bias(_p(mat), _p(bias), _p(out), C.c_size_t(m), C.c_size_t(n))
    return out


# --------------------------------------------------------------------------
# INT8 engine, W8A8 extension
# --------------------------------------------------------------------------

def i8_quantize_rows(x):
    x = _f32(x)
    rows, cols = x.shape
    xq = np.empty((rows, cols), np.int8)
    s = np.empty(rows, np.float32)
    lib().orc_i8_quantize_rows(_p(x), _p(xq), _p(s), C.c_size_t(rows), C.c_size_t(cols))
    return xq, s


def i8_gemm_i32(xq, wq, threads: int = 1):
    xq = np.ascontiguousarray(xq, np.int8)
    wq = np.ascontiguousarray(wq, np.int8)
    m, k = xq.shape
    n = wq.shape[0]
    assert wq.shape[1] == k
    acc = np.empty((m, n), np.int32)
    lib().orc_i8_gemm_i32(_p(xq), _p(wq), _p(acc), C.c_size_t(m), C.c_size_t(k),
                          C.c_size_t(n), C.c_int(threads))
    return acc


def i8_rescale_bias(acc, sx, sw, bias=None):
    acc = np.ascontiguousarray(acc, np.int32)
    m, n = acc.shape
    sx, sw = _f32(sx), _f32(sw)
    bias = None if bias is None else _f32(bias)
    y = np.empty((m, n), np.float32)
    lib().orc_i8_rescale_bias(_p(acc), _p(sx), _p(sw), _p(bias), _p(y),
                              C.c_size_t(m), C.c_size_t(n))
    return y


def i8_linear(x, w, bias=None, threads: int = 1):
    """INT8 QuantLinear forward: W [K,N] per-output-channel, X per-row."""
    w = _f32(w)
    wq, sw = i8_quantize_rows(np.ascontiguousarray(w.T))
    xq, sx = i8_quantize_rows(x)
    acc = i8_gemm_i32(xq, wq, threads)
    return i8_rescale_bias(acc, sx, sw, bias), acc, (xq, sx, wq, sw)


# --------------------------------------------------------------------------
# EXTENSION: the f32 operators around the projections of a decoder block, in
# float64 numpy.  Closed forms, no reference code behind them (the reference's
# flash_attention computes the same softmax(q k^T / sqrt(d)) v).
# --------------------------------------------------------------------------

def w4_dequant(packed, scales, zp, k: int, group_size: int):
    """float64 [k, n] matrix (q - zp) * scale of an INT4 weight."""
    q = w4_unpack(packed, k).astype(np.float64)
    g = np.arange(k) // group_size
    return (q - np.asarray(zp, np.float64)[g]) * np.asarray(scales, np.float64)[g]


def rmsnorm(x, weight, eps: float = 1e-6):
    x = np.asarray(x, np.float64)
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps) * np.asarray(weight, np.float64)


def swiglu(gate, up):
    gate = np.asarray(gate, np.float64)
    return gate / (1.0 + np.exp(-gate)) * np.asarray(up, np.float64)


def attention(q, k, v, causal: bool):
    """q [B, Nq, H, d], k, v [B, Nkv, H, d] -> [B, Nq, H, d]; query i is token Nkv - Nq + i."""
    q, k, v = (np.asarray(t, np.float64) for t in (q, k, v))
    nq, nkv, d = q.shape[1], k.shape[1], q.shape[3]
    s = np.einsum("bqhd,bkhd->bhqk", q, k) / np.sqrt(d)
    if causal:
        pos = np.arange(nq)[:, None] + (nkv - nq)
        s = np.where(np.arange(nkv)[None, :] <= pos, s, -np.inf)
    s = s - s.max(-1, keepdims=True)
    p = np.exp(s)
    p /= p.sum(-1, keepdims=True)
    return np.einsum("bhqk,bkhd->bqhd", p, v)


def decoder_block(x, wd: dict, heads: int, k_cache=None, v_cache=None, pos: int = 0, eps: float = 1e-6):
    """Pre-norm Llama-shaped block on dequantized float64 weights ``wd[name]`` ([in, out]), RMSNorm
    weights 1.  Returns (y, k, v); with caches the new key/value are placed at ``pos`` first."""
    x = np.asarray(x, np.float64)
    b, n, d = x.shape
    ones = np.ones(d)
    x2 = x.reshape(b * n, d)
    hn = rmsnorm(x2, ones, eps)
    q = (hn @ wd["q"]).reshape(b, n, heads, -1)
    k = (hn @ wd["k"]).reshape(b, n, heads, -1)
    v = (hn @ wd["v"]).reshape(b, n, heads, -1)
    if k_cache is None:
        att = attention(q, k, v, True)
    else:
        k_cache = np.array(k_cache, np.float64)
        v_cache = np.array(v_cache, np.float64)
        k_cache[:, pos] = k[:, 0]
        v_cache[:, pos] = v[:, 0]
        att = attention(q, k_cache[:, :pos + 1], v_cache[:, :pos + 1], False)
        k, v = k_cache, v_cache
    x1 = x2 + att.reshape(b * n, d) @ wd["o"]
    h2 = rmsnorm(x1, ones, eps)
    y = x1 + swiglu(h2 @ wd["gate"], h2 @ wd["up"]) @ wd["down"]
    return y.reshape(b, n, d), k, v
