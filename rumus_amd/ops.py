"""Thin Python front end of the C ABI: one function per entry point.

torch is used for device memory and streams only (``data_ptr()`` of CUDA/HIP
tensors, ``torch.cuda.current_stream()``); every computation happens inside
``librumus_hip.so``.  Shapes and dtypes are checked here because raw pointers
carry none; numeric preconditions are checked by the library itself.
"""
from __future__ import annotations

import torch

from . import _lib
from ._lib import RumusError, call

__all__ = [
    "q8_buf_size", "q8_quantize", "q8_dequantize", "q8_dequantize_kn", "matmul_q8", "q8_dense_layout", "matmul_q8_dense", "add_bias", "transpose_f32",
    "i8_quantize_rows", "i8_quantize_cols_t", "i8_gemm", "w4_quantize_pack", "qmatmul_int4", "matmul_q8_f16", "qmatmul_int4_f16",
    "qmatmul_int4_t", "w4_actorder_prepare", "qmatmul_int4_perm", "w4_geometry", "RumusError",
]


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _dev(t: torch.Tensor, dtype, name: str) -> int:
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise TypeError(f"{name}: expected a GPU tensor")
    if t.dtype != dtype:
        raise TypeError(f"{name}: expected {dtype}, got {t.dtype}")
    if not t.is_contiguous():
        raise ValueError(f"{name}: tensor must be contiguous")
    return t.data_ptr()


def _opt(t, dtype, name):
    return None if t is None else _dev(t, dtype, name)


def w4_geometry(k: int, group_size: int):
    padded_k = ((k + group_size - 1) // group_size) * group_size
    return padded_k, padded_k // group_size


# ---- INT8, reference block format -------------------------------------------

def q8_buf_size(numel: int, block_size: int) -> int:
    return int(_lib.lib().rumus_hip_q8_buf_size(numel, block_size))


def q8_quantize(flat: torch.Tensor, block_size: int) -> torch.Tensor:
    """f32 [numel] -> Q8 buffer as int32 words (header word + bs/4 data words per block)."""
    numel = flat.numel()
    nbytes = q8_buf_size(numel, block_size) if block_size > 0 else 4
    out = torch.empty(max(nbytes // 4, 1), dtype=torch.int32, device=flat.device)
    call("rumus_hip_q8_quantize", _dev(flat, torch.float32, "in"), out.data_ptr(), numel,
         block_size, _stream())
    return out


def q8_dequantize(words: torch.Tensor, numel: int, block_size: int) -> torch.Tensor:
    if block_size > 0 and block_size % 4 == 0 and words.numel() * 4 < q8_buf_size(numel, block_size):
        raise ValueError("q8_dequantize: the buffer is shorter than numel elements in blocks of block_size")
    out = torch.empty(numel, dtype=torch.float32, device=words.device)
    call("rumus_hip_q8_dequantize", _dev(words, torch.int32, "in"), out.data_ptr(), numel,
         block_size, _stream())
    return out


def q8_dequantize_kn(words: torch.Tensor, k: int, n: int, block_size: int) -> torch.Tensor:
    """The dequantized weight in its own ``[k, n]`` order (the buffer holds the transposed tensor)."""
    if block_size > 0 and block_size % 4 == 0 and words.numel() * 4 < q8_buf_size(k * n, block_size):
        raise ValueError("q8_dequantize_kn: the buffer is shorter than k * n elements in blocks of block_size")
    out = torch.empty((k, n), dtype=torch.float32, device=words.device)
    call("rumus_hip_q8_dequantize_kn", _dev(words, torch.int32, "in"), out.data_ptr(), k, n, block_size, _stream())
    return out


def matmul_q8(a: torch.Tensor, words: torch.Tensor, k: int, n: int, block_size: int, out=None) -> torch.Tensor:
    m = a.shape[0]
    if a.dim() != 2 or a.shape[1] != k:
        raise ValueError("matmul: inner dimension mismatch")
    # the kernel, like matmul_q8.wgsl:47-52, reads ceil(k / block_size) whole blocks per column; Tensor::quantize blocks
    # the flat transposed tensor, which is that many only when k % block_size == 0 (or one block holds it all)
    if block_size <= 0 or words.numel() < n * (-(-k // block_size)) * ((4 + block_size + 3) // 4):
        raise ValueError("matmul: the Q8 buffer is shorter than n columns of whole blocks (k % block_size != 0?)")
    c = torch.empty((m, n), dtype=torch.float32, device=a.device) if out is None else out
    if c.shape != (m, n) or c.dtype != torch.float32 or not c.is_contiguous():
        raise ValueError("matmul: out must be a contiguous f32 [m, n] tensor")
    call("rumus_hip_matmul_q8", _dev(a, torch.float32, "a"), _dev(words, torch.int32, "b"),
         c.data_ptr(), m, k, n, block_size, _stream())
    return c


def matmul_q8_f16(a: torch.Tensor, words: torch.Tensor, k: int, n: int, block_size: int, out=None) -> torch.Tensor:
    """:func:`matmul_q8` on half-precision activations: ``a`` and the result are ``torch.float16``; the product runs in
    the f32 kernels and is rounded to f16 once."""
    m = a.shape[0]
    if a.dim() != 2 or a.shape[1] != k:
        raise ValueError("matmul: inner dimension mismatch")
    if block_size <= 0 or words.numel() < n * (-(-k // block_size)) * ((4 + block_size + 3) // 4):
        raise ValueError("matmul: the Q8 buffer is shorter than n columns of whole blocks (k % block_size != 0?)")
    c = torch.empty((m, n), dtype=torch.float16, device=a.device) if out is None else out
    if c.shape != (m, n) or c.dtype != torch.float16 or not c.is_contiguous():
        raise ValueError("matmul: out must be a contiguous f16 [m, n] tensor")
    call("rumus_hip_matmul_q8_f16", _dev(a, torch.float16, "a"), _dev(words, torch.int32, "b"),
         c.data_ptr(), m, k, n, block_size, _stream())
    return c


def q8_dense_layout(words: torch.Tensor, k: int, n: int, block_size: int):
    """A Q8 buffer with one block per column (``block_size >= k``) as dense int8 ``[n, k]`` plus the ``n`` block
    scales: the operands of :func:`matmul_q8_dense`, made once per weight."""
    # (block_size < k, several blocks per column, is refused by the library itself)
    if block_size <= 0 or words.numel() < n * (-(-k // block_size)) * ((4 + block_size + 3) // 4):
        raise ValueError("q8_dense_layout: the Q8 buffer is shorter than n blocks")
    wq = torch.empty((n, k), dtype=torch.int8, device=words.device)
    sw = torch.empty(n, dtype=torch.float32, device=words.device)
    call("rumus_hip_q8_dense_layout", _dev(words, torch.int32, "b"), k, n, block_size, wq.data_ptr(), sw.data_ptr(),
         _stream())
    return wq, sw


def matmul_q8_dense(a: torch.Tensor, wq: torch.Tensor, sw: torch.Tensor, out=None) -> torch.Tensor:
    """``a @ W`` for a per-output-channel Q8 weight in the layout of :func:`q8_dense_layout`."""
    n, k = wq.shape
    m = a.shape[0]
    if a.dim() != 2 or a.shape[1] != k:
        raise ValueError("matmul: inner dimension mismatch")
    if sw.numel() != n:
        raise ValueError("matmul: one scale per output channel wanted")
    c = torch.empty((m, n), dtype=torch.float32, device=a.device) if out is None else out
    if c.shape != (m, n) or c.dtype != torch.float32 or not c.is_contiguous():
        raise ValueError("matmul: out must be a contiguous f32 [m, n] tensor")
    call("rumus_hip_matmul_q8_dense", _dev(a, torch.float32, "a"), _dev(wq, torch.int8, "wq"),
         _dev(sw, torch.float32, "sw"), c.data_ptr(), m, k, n, _stream())
    return c


def add_bias(mat: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    m, n = mat.shape
    if bias.numel() != n:
        raise ValueError("add_bias: bias length mismatch")
    out = torch.empty_like(mat)
    call("rumus_hip_add_bias", _dev(mat, torch.float32, "mat"), _dev(bias, torch.float32, "bias"),
         out.data_ptr(), m, n, _stream())
    return out


def transpose_f32(t: torch.Tensor) -> torch.Tensor:
    rows, cols = t.shape
    out = torch.empty((cols, rows), dtype=torch.float32, device=t.device)
    call("rumus_hip_transpose_f32", _dev(t, torch.float32, "in"), out.data_ptr(), rows, cols, _stream())
    return out


# ---- INT8, W8A8 ---------------------------------------------------------------

def i8_quantize_rows(x: torch.Tensor, out=None):
    """x f32 [rows, cols] -> (xq int8 [rows, cols], scale f32 [rows]); ``out`` = (xq, scale) to reuse buffers."""
    rows, cols = x.shape
    if out is not None:
        xq, s = out
        if xq.shape != (rows, cols) or xq.dtype != torch.int8 or s.shape != (rows,) or s.dtype != torch.float32 \
                or not (xq.is_cuda and s.is_cuda and xq.is_contiguous() and s.is_contiguous()):
            raise ValueError("i8_quantize_rows: out must be (int8 [rows, cols], float32 [rows]) on the device")
    else:
        xq = torch.empty((rows, cols), dtype=torch.int8, device=x.device)
        s = torch.empty(rows, dtype=torch.float32, device=x.device)
    call("rumus_hip_i8_quantize_rows", _dev(x, torch.float32, "x"), xq.data_ptr(), s.data_ptr(),
         rows, cols, _stream())
    return xq, s


def i8_quantize_cols_t(w: torch.Tensor):
    """w [k,n] -> wq int8 [n,k], sw f32 [n]."""
    k, n = w.shape
    wq = torch.empty((n, k), dtype=torch.int8, device=w.device)
    sw = torch.empty(n, dtype=torch.float32, device=w.device)
    call("rumus_hip_i8_quantize_cols_t", _dev(w, torch.float32, "w"), wq.data_ptr(), sw.data_ptr(),
         k, n, _stream())
    return wq, sw


def i8_gemm(xq, wq, sx=None, sw=None, bias=None, want_acc=False, want_y=True, out=None):
    m, k = xq.shape
    n = wq.shape[0]
    if xq.dim() != 2 or wq.dim() != 2 or wq.shape[1] != k:
        raise ValueError("i8_gemm: inner dimension mismatch")
    if (sx is not None and sx.numel() < m) or (sw is not None and sw.numel() < n) or (bias is not None and bias.numel() < n):
        raise ValueError("i8_gemm: sx must hold m scales, sw and bias n values")
    if out is not None and (tuple(out.shape) != (m, n) or out.dtype != torch.float32 or not out.is_contiguous()):
        raise ValueError("i8_gemm: out must be a contiguous f32 [m, n] tensor")
    acc = torch.empty((m, n), dtype=torch.int32, device=xq.device) if want_acc else None
    y = None
    if want_y:
        y = out if out is not None else torch.empty((m, n), dtype=torch.float32, device=xq.device)
    call("rumus_hip_i8_gemm", _dev(xq, torch.int8, "xq"), _dev(wq, torch.int8, "wq"),
         _opt(sx, torch.float32, "sx"), _opt(sw, torch.float32, "sw"), _opt(bias, torch.float32, "bias"),
         None if acc is None else acc.data_ptr(), None if y is None else _dev(y, torch.float32, "y"),
         m, k, n, _stream())
    return y, acc


# ---- INT4 -----------------------------------------------------------------------

def w4_quantize_pack(w: torch.Tensor, group_size: int, symmetric: bool = False):
    k, n = w.shape
    gs = max(group_size, 1)
    padded_k, groups = w4_geometry(k, gs)
    packed = torch.empty((max(padded_k // 8, 1), n), dtype=torch.int32, device=w.device)
    scales = torch.empty((groups, n), dtype=torch.float32, device=w.device)
    zp = torch.empty((groups, n), dtype=torch.float32, device=w.device)
    name = "rumus_hip_w4_quantize_pack_sym" if symmetric else "rumus_hip_w4_quantize_pack"
    call(name, _dev(w, torch.float32, "w"), k, n, group_size, packed.data_ptr(), scales.data_ptr(),
         zp.data_ptr(), _stream())
    return packed, scales, zp


def w4_quantize_pack_awq(w: torch.Tensor, group_size: int):
    """AWQ storage: (packed int32 [padded_k/8, n], scales f32 [groups, n], qzeros int32 [groups, n/8])."""
    k, n = w.shape
    padded_k, groups = w4_geometry(k, max(group_size, 1))
    packed = torch.empty((max(padded_k // 8, 1), n), dtype=torch.int32, device=w.device)
    scales = torch.empty((groups, n), dtype=torch.float32, device=w.device)
    qzeros = torch.empty((groups, max(n // 8, 1)), dtype=torch.int32, device=w.device)
    call("rumus_hip_w4_quantize_pack_awq", _dev(w, torch.float32, "w"), k, n, group_size, packed.data_ptr(),
         scales.data_ptr(), qzeros.data_ptr(), _stream())
    return packed, scales, qzeros


def f16_to_f32(t):
    """Half -> f32 (exact), same shape."""
    out = torch.empty(t.shape, dtype=torch.float32, device=t.device)
    call("rumus_hip_f16_to_f32", _dev(t, torch.float16, "in"), out.data_ptr(), t.numel(), _stream())
    return out


def w4_qzeros_unpack(qzeros, n):
    """u4 zero-points ``[groups, n/8]`` (eight per word) -> f32 ``[groups, n]``."""
    groups = qzeros.shape[0]
    if n % 8 != 0 or qzeros.shape[1] != n // 8:
        raise ValueError("w4_qzeros_unpack: qzeros must be [groups, n/8]")
    zp = torch.empty((groups, n), dtype=torch.float32, device=qzeros.device)
    call("rumus_hip_w4_qzeros_unpack", _dev(qzeros, torch.int32, "qzeros"), groups, n, zp.data_ptr(), _stream())
    return zp


def w4_decode_layout(packed, scales, zp, group_size):
    """Tile-major copies (16 columns per tile) of the three arrays of an INT4 weight."""
    rows, n = packed.shape
    _w4_sizes("w4_decode_layout", packed, scales, zp, rows * 8, group_size, 0)
    out = (torch.empty_like(packed), torch.empty_like(scales), torch.empty_like(zp))
    call("rumus_hip_w4_decode_layout", _dev(packed, torch.int32, "packed"), _dev(scales, torch.float32, "scales"),
         _dev(zp, torch.float32, "zero_points"), rows * 8, n, group_size, out[0].data_ptr(), out[1].data_ptr(),
         out[2].data_ptr(), _stream())
    return out


def qmatmul_int4_decode(x, packed_t, scales_t, zp_t, k, group_size, bias=None, perm=None, out=None):
    return _w4_call("rumus_hip_qmatmul_int4_decode", x, packed_t, scales_t, zp_t, bias, perm, k, group_size, out)


def qmatmul_int4_decode_max_rows(padded_k: int, n: int) -> int:
    """Rows up to which the decode entry points beat the matrix-core kernel for this weight."""
    return int(_lib.lib().rumus_hip_qmatmul_int4_decode_max_rows(padded_k, n))


def w4_decode_layout_zp4(packed, scales, qzeros, group_size):
    """Tile-major copies for AWQ storage: packed, scales as in w4_decode_layout, u4 zero-points with
    the two words of a tile side by side."""
    rows, n = packed.shape
    _w4_sizes("w4_decode_layout_zp4", packed, scales, qzeros, rows * 8, group_size, 0, zp4=True)
    out = (torch.empty_like(packed), torch.empty_like(scales), torch.empty_like(qzeros))
    call("rumus_hip_w4_decode_layout_zp4", _dev(packed, torch.int32, "packed"), _dev(scales, torch.float32, "scales"),
         _dev(qzeros, torch.int32, "qzeros"), rows * 8, n, group_size, out[0].data_ptr(), out[1].data_ptr(),
         out[2].data_ptr(), _stream())
    return out


def qmatmul_int4_decode_zp4(x, packed_t, scales_t, qzeros_t, k, group_size, bias=None, perm=None, out=None):
    m = x.shape[0]
    n = packed_t.shape[1]
    if x.dim() != 2 or x.shape[1] != k:
        raise ValueError("qmatmul_int4_decode_zp4: x must be [m, k]")
    _w4_sizes("qmatmul_int4_decode_zp4", packed_t, scales_t, qzeros_t, k, group_size, m, bias, perm, out, zp4=True)
    padded_k, groups = w4_geometry(k, group_size) if group_size > 0 else (k, 0)
    y = out if out is not None else torch.empty((m, n), dtype=torch.float32, device=x.device)
    call("rumus_hip_qmatmul_int4_decode_zp4", _dev(x, torch.float32, "x"), _dev(packed_t, torch.int32, "packed_t"),
         _dev(scales_t, torch.float32, "scales_t"), _dev(qzeros_t, torch.int32, "qzeros_t"),
         _opt(bias, torch.float32, "bias"), _opt(perm, torch.int32, "perm"),
         _dev(y, torch.float32, "y"), m, k, n, padded_k, group_size, groups, _stream())
    return y


def qmatmul_int4_decode_swiglu(gate_up, packed_t, scales_t, zp_t, k, group_size, bias=None, out=None):
    """``(silu(gate) * up) @ dequant(W)`` for ``gate_up`` ``[m, 2k]`` (gate | up), one launch."""
    m = gate_up.shape[0]
    n = packed_t.shape[1]
    if gate_up.dim() != 2 or gate_up.shape[1] != 2 * k:
        raise ValueError("qmatmul_int4_decode_swiglu: gate_up must be [m, 2k]")
    _w4_sizes("qmatmul_int4_decode_swiglu", packed_t, scales_t, zp_t, k, group_size, m, bias, None, out)
    padded_k, groups = w4_geometry(k, group_size) if group_size > 0 else (k, 0)
    y = out if out is not None else torch.empty((m, n), dtype=torch.float32, device=gate_up.device)
    call("rumus_hip_qmatmul_int4_decode_swiglu", _dev(gate_up, torch.float32, "gate_up"),
         _dev(packed_t, torch.int32, "packed_t"), _dev(scales_t, torch.float32, "scales_t"),
         _dev(zp_t, torch.float32, "zero_points_t"), _opt(bias, torch.float32, "bias"),
         _dev(y, torch.float32, "y"), m, k, n, padded_k, group_size, groups, _stream())
    return y


def qmatmul_int4_decode_block(x, packed_t, scales_t, zp_t, k, group_size, norm_weight=None, eps: float = 1e-6,
                              swiglu: bool = False, bias=None, residual=None, out=None):
    """The decode projection with a decoder block's neighbours folded in: ``x`` through RMSNorm with
    ``norm_weight`` (or, ``swiglu``, ``x`` = gate | up rows of ``2k``), ``residual`` ``[m, n]`` added to the result
    (it may be ``out``); one launch."""
    m = x.shape[0]
    n = packed_t.shape[1]
    if x.dim() != 2 or x.shape[1] != (2 * k if swiglu else k):
        raise ValueError("qmatmul_int4_decode_block: x must be [m, k] (gate | up: [m, 2k])")
    if norm_weight is not None and norm_weight.numel() < k:
        raise ValueError("qmatmul_int4_decode_block: norm_weight must hold k values")
    if residual is not None and (residual.dim() != 2 or tuple(residual.shape) != (m, n) or not residual.is_contiguous()):
        raise ValueError("qmatmul_int4_decode_block: residual must be a contiguous [m, n] tensor")
    _w4_sizes("qmatmul_int4_decode_block", packed_t, scales_t, zp_t, k, group_size, m, bias, None, out)
    padded_k, groups = w4_geometry(k, group_size) if group_size > 0 else (k, 0)
    y = out if out is not None else torch.empty((m, n), dtype=torch.float32, device=x.device)
    call("rumus_hip_qmatmul_int4_decode_block", _dev(x, torch.float32, "x"), _opt(norm_weight, torch.float32, "norm_weight"),
         float(eps), 1 if swiglu else 0, _dev(packed_t, torch.int32, "packed_t"), _dev(scales_t, torch.float32, "scales_t"),
         _dev(zp_t, torch.float32, "zero_points_t"), _opt(bias, torch.float32, "bias"),
         _opt(residual, torch.float32, "residual"), _dev(y, torch.float32, "y"), m, k, n, padded_k, group_size, groups,
         _stream())
    return y


def qmatmul_int4_zp4(x, packed, scales, qzeros, k, group_size, bias=None, perm=None, out=None):
    m = x.shape[0]
    n = packed.shape[1]
    if x.dim() != 2 or x.shape[1] != k:
        raise ValueError("qmatmul_int4_zp4: x must be [m, k]")
    _w4_sizes("qmatmul_int4_zp4", packed, scales, qzeros, k, group_size, m, bias, perm, out, zp4=True)
    padded_k, groups = w4_geometry(k, group_size) if group_size > 0 else (k, 0)
    y = out if out is not None else torch.empty((m, n), dtype=torch.float32, device=x.device)
    call("rumus_hip_qmatmul_int4_zp4", _dev(x, torch.float32, "x"), _dev(packed, torch.int32, "packed"),
         _dev(scales, torch.float32, "scales"), _dev(qzeros, torch.int32, "qzeros"),
         _opt(bias, torch.float32, "bias"), _opt(perm, torch.int32, "perm"),
         _dev(y, torch.float32, "y"), m, k, n, padded_k, group_size, groups, _stream())
    return y


def _w4_sizes(who, packed, scales, zp, k, group_size, rows, bias=None, index=None, out=None, out_cols=None, zp4=False,
              out_dtype=torch.float32):
    """The kernels take raw pointers: a short array would be read past its end on the device.  Checks the element
    counts the geometry implies (the library itself rejects a bad group size or alignment)."""
    if group_size <= 0 or packed.dim() != 2:
        return
    n = packed.shape[1]
    padded_k, groups = w4_geometry(k, group_size)
    zp_need = groups * (n // 8) if zp4 else groups * n
    if packed.numel() < max(padded_k // 8, 1) * n or scales.numel() < groups * n or zp.numel() < zp_need:
        raise ValueError(f"{who}: packed / scales / zero-points are smaller than k={k}, n={n}, group_size={group_size} needs")
    if bias is not None and bias.numel() < n:
        raise ValueError(f"{who}: bias must hold n = {n} values")
    if index is not None and index.numel() < k:
        raise ValueError(f"{who}: g_idx / perm must hold k = {k} entries")
    if out is not None:
        cols = n if out_cols is None else out_cols
        if tuple(out.shape) != (rows, cols) or out.dtype != out_dtype or not out.is_contiguous():
            raise ValueError(f"{who}: out must be a contiguous {out_dtype} [{rows}, {cols}] tensor")


def _w4_call(name, x, packed, scales, zp, bias, extra, k, group_size, out=None, act=torch.float32):
    m = x.shape[0]
    n = packed.shape[1]
    if x.dim() != 2 or x.shape[1] != k:
        raise ValueError("qmatmul_int4: x must be [m, k]")
    _w4_sizes(name, packed, scales, zp, k, group_size, m, bias, extra, out, out_dtype=act)
    padded_k, groups = w4_geometry(k, group_size) if group_size > 0 else (k, 0)
    y = out if out is not None else torch.empty((m, n), dtype=act, device=x.device)
    call(name, _dev(x, act, "x"), _dev(packed, torch.int32, "packed"),
         _dev(scales, torch.float32, "scales"), _dev(zp, torch.float32, "zero_points"),
         _opt(bias, torch.float32, "bias"), _opt(extra, torch.int32, "g_idx/perm"),
         _dev(y, act, "y"), m, k, n, padded_k, group_size, groups, _stream())
    return y


def qmatmul_int4(x, packed, scales, zp, k, group_size, bias=None, g_idx=None, out=None):
    return _w4_call("rumus_hip_qmatmul_int4", x, packed, scales, zp, bias, g_idx, k, group_size, out)


def qmatmul_int4_f16(x, packed, scales, zp, k, group_size, bias=None, g_idx=None, out=None):
    """:func:`qmatmul_int4` on half-precision activations: ``x`` and the result are ``torch.float16``; scales,
    zero-points and bias stay f32.  The product runs in the f32 kernels and is rounded to f16 once."""
    return _w4_call("rumus_hip_qmatmul_int4_f16", x, packed, scales, zp, bias, g_idx, k, group_size, out, torch.float16)


def qmatmul_int4_perm(x, packed_sorted, scales, zp, k, group_size, bias=None, perm=None, out=None):
    return _w4_call("rumus_hip_qmatmul_int4_perm", x, packed_sorted, scales, zp, bias, perm, k,
                    group_size, out)


def qmatmul_int4_perm_static(x, packed_sorted, scales, zp, k, group_size, bias=None, perm=None, out=None):
    """``qmatmul_int4_perm`` through the entry point that allocates nothing: temporaries live in the
    library's static 32 MiB device array; shapes that need more raise ``RumusError``.  Pass ``out``
    to keep this wrapper from allocating the result either."""
    return _w4_call("rumus_hip_qmatmul_int4_perm_static", x, packed_sorted, scales, zp, bias, perm, k,
                    group_size, out)


def qmatmul_int4_t(a, packed, scales, zp, k, group_size, out=None):
    m, n = a.shape
    if packed.shape[1] != n:
        raise ValueError("qmatmul_int4_t: a must be [m, n]")
    _w4_sizes("qmatmul_int4_t", packed, scales, zp, k, group_size, m)
    padded_k, groups = w4_geometry(k, group_size)
    if out is None:
        out = torch.empty((m, k), dtype=torch.float32, device=a.device)
    elif out.shape != (m, k) or out.dtype != torch.float32 or not out.is_contiguous():
        raise ValueError("qmatmul_int4_t: out must be a contiguous f32 [m, k] tensor")
    call("rumus_hip_qmatmul_int4_t", _dev(a, torch.float32, "a"), _dev(packed, torch.int32, "packed"),
         _dev(scales, torch.float32, "scales"), _dev(zp, torch.float32, "zero_points"),
         out.data_ptr(), m, k, n, padded_k, group_size, groups, _stream())
    return out


def w4_actorder_prepare(packed, g_idx, group_size):
    rows, n = packed.shape
    padded_k = rows * 8
    out = torch.empty_like(packed)
    perm = torch.empty(padded_k, dtype=torch.int32, device=packed.device)
    call("rumus_hip_w4_actorder_prepare", _dev(packed, torch.int32, "packed"),
         _dev(g_idx, torch.int32, "g_idx"), padded_k, n, group_size, out.data_ptr(), perm.data_ptr(),
         _stream())
    return out, perm


# ---- f32 operators between the projections of a decoder block ---------------------------------

def rmsnorm(x, weight, eps: float = 1e-6, out=None):
    rows, dim = x.shape
    y = out if out is not None else torch.empty_like(x)
    call("rumus_hip_rmsnorm", _dev(x, torch.float32, "x"), _dev(weight, torch.float32, "weight"),
         _dev(y, torch.float32, "y"), rows, dim, float(eps), _stream())
    return y


def add_rmsnorm(x, delta, weight, eps: float = 1e-6, sum_out=None, out=None):
    """``s = x + delta; y = rmsnorm(s)`` in one launch; returns ``(s, y)``.  ``sum_out`` may be x or delta."""
    rows, dim = x.shape
    s = sum_out if sum_out is not None else torch.empty_like(x)
    y = out if out is not None else torch.empty_like(x)
    call("rumus_hip_add_rmsnorm", _dev(x, torch.float32, "x"), _dev(delta, torch.float32, "delta"),
         _dev(weight, torch.float32, "weight"), _dev(s, torch.float32, "sum"), _dev(y, torch.float32, "y"),
         rows, dim, float(eps), _stream())
    return s, y


def swiglu(gate, up, out=None):
    y = out if out is not None else torch.empty_like(gate)
    call("rumus_hip_swiglu", _dev(gate, torch.float32, "gate"), _dev(up, torch.float32, "up"),
         _dev(y, torch.float32, "out"), gate.numel(), _stream())
    return y


def swiglu_rows(gate_up, out=None):
    """gate_up [rows, 2n] (gate | up side by side) -> silu(gate) * up, [rows, n]."""
    rows, n2 = gate_up.shape
    y = out if out is not None else torch.empty((rows, n2 // 2), dtype=torch.float32, device=gate_up.device)
    call("rumus_hip_swiglu_rows", _dev(gate_up, torch.float32, "gate_up"), _dev(y, torch.float32, "out"), rows,
         n2 // 2, _stream())
    return y


def add(a, b, out=None):
    y = out if out is not None else torch.empty_like(a)
    call("rumus_hip_add", _dev(a, torch.float32, "a"), _dev(b, torch.float32, "b"), _dev(y, torch.float32, "out"),
         a.numel(), _stream())
    return y


def attention(q, k, v, causal: bool, out=None):
    """q [B, Nq, H, 128], k and v [B, Nkv, H, 128] (any strides with the last dim contiguous) ->
    [B, Nq, H, 128]: softmax(q k^T / sqrt(128)) v per batch and head."""
    import ctypes
    b, nq, h, d = q.shape
    nkv = k.shape[1]
    o = out if out is not None else torch.empty((b, nq, h, d), dtype=torch.float32, device=q.device)
    for t, name in ((q, "q"), (k, "k"), (v, "v"), (o, "out")):
        if t.dtype != torch.float32 or not t.is_cuda or t.stride(3) != 1:
            raise ValueError(f"attention: {name} must be a float32 device tensor with a contiguous last dim")
    strides = (ctypes.c_uint64 * 12)(*[s for t in (q, k, v, o) for s in (t.stride(0), t.stride(2), t.stride(1))])
    call("rumus_hip_attention", q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), b, h, nq, nkv, d,
         strides, 1 if causal else 0, _stream())
    return o


def kv_append(k_new, v_new, k_cache, v_cache, pos: int):
    """Write the new tokens' keys / values ``[B, n, H, d]`` at positions ``pos .. pos+n-1`` of the
    caches ``[B, T, H, d]`` (any strides with the last dim contiguous; a ``[B, H, T, d]`` cache is
    passed as its ``transpose(1, 2)`` view), in one launch."""
    import ctypes
    b, n, h, d = k_new.shape
    t_len = k_cache.shape[1]
    for t, name in ((k_new, "k_new"), (v_new, "v_new"), (k_cache, "k_cache"), (v_cache, "v_cache")):
        if t.dtype != torch.float32 or not t.is_cuda or t.stride(3) != 1:
            raise ValueError(f"kv_append: {name} must be a float32 device tensor with a contiguous last dim")
    if v_new.shape != k_new.shape or k_cache.shape != v_cache.shape or k_cache.shape[0] != b or \
            k_cache.shape[2] != h or k_cache.shape[3] != d:
        raise ValueError("kv_append: shapes of the new entries and the caches do not match")
    strides = (ctypes.c_uint64 * 12)(*[s for t in (k_new, v_new, k_cache, v_cache)
                                       for s in (t.stride(0), t.stride(2), t.stride(1))])
    call("rumus_hip_kv_append", k_new.data_ptr(), v_new.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
         b, h, n, d, pos, t_len, strides, _stream())


def attention_decode_append(q, k_new, v_new, k_cache, v_cache, pos: int, out=None):
    """``kv_append`` of one new token per sequence at ``pos`` and ``attention`` of its query over positions
    ``0..pos``, without the launch for the append.  ``q``, ``k_new``, ``v_new`` ``[B, 1, H, 128]``, caches
    ``[B, T, H, 128]`` (any strides with the last dim contiguous); returns ``[B, 1, H, 128]``."""
    import ctypes
    b, n, h, d = q.shape
    if n != 1 or tuple(k_new.shape) != (b, 1, h, d) or tuple(v_new.shape) != (b, 1, h, d):
        raise ValueError("attention_decode_append: q, k_new and v_new must be [B, 1, H, d]")
    if k_cache.shape != v_cache.shape or k_cache.shape[0] != b or k_cache.shape[2] != h or k_cache.shape[3] != d:
        raise ValueError("attention_decode_append: shapes of the new entries and the caches do not match")
    o = out if out is not None else torch.empty((b, 1, h, d), dtype=torch.float32, device=q.device)
    ts = (q, k_new, v_new, k_cache, v_cache, o)
    for t, name in zip(ts, ("q", "k_new", "v_new", "k_cache", "v_cache", "out")):
        if t.dtype != torch.float32 or not t.is_cuda or t.stride(3) != 1:
            raise ValueError(f"attention_decode_append: {name} must be a float32 device tensor with a contiguous last dim")
    strides = (ctypes.c_uint64 * 18)(*[s for t in ts for s in (t.stride(0), t.stride(2), t.stride(1))])
    call("rumus_hip_attention_decode_append", q.data_ptr(), k_new.data_ptr(), v_new.data_ptr(), k_cache.data_ptr(),
         v_cache.data_ptr(), o.data_ptr(), b, h, d, pos, k_cache.shape[1], strides, _stream())
    return o
