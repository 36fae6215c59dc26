"""Host-side mirror of the reference's module API for the quantized-Linear path.

Same names, argument meaning and error behaviour as the reference (which
panics; here a failed precondition raises ``RumusError``/``ValueError``):

* ``Linear``             rumus/src/nn/linear.rs:44-104   (weight ``[in, out]``)
* ``QuantizedTensor``    rumus-vision/src/quant.rs:24-127
* ``QLinear``            rumus-vision/src/quant.rs:165-222
* ``Q8Tensor`` + ``quantize`` / ``dequantize`` / ``matmul``
                         rumus/src/tensor/ops.rs:516-545,2290-2357 (``DType::Q8``)
* ``Int8Linear``         the W8A8 engine (no reference counterpart)

torch tensors are only the device-memory handles; all arithmetic is done by the
HIP library through ``rumus_amd.ops``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

from . import ops


class Linear:
    """``y = x @ weight + bias`` with ``weight`` of shape ``[in_features, out_features]``."""

    def __init__(self, weight: torch.Tensor, bias: Optional[torch.Tensor] = None):
        if weight.dim() != 2:
            raise ValueError("Linear: weight must be 2-D [in, out]")
        self.weight = weight
        self.bias = bias

    @property
    def in_features(self) -> int:
        return self.weight.shape[0]

    @property
    def out_features(self) -> int:
        return self.weight.shape[1]


# ---- INT4 ------------------------------------------------------------------------

class QuantizedTensor:
    """INT4 weight with group-wise metadata (quant.rs:24-38)."""

    def __init__(self, k, n, padded_k, group_size, num_groups, packed, scales, zp,
                 perm: Optional[torch.Tensor] = None):
        self.k, self.n, self.padded_k = k, n, padded_k
        self.group_size, self.num_groups = group_size, num_groups
        self.packed_tensor, self.scales_tensor, self.zp_tensor = packed, scales, zp
        self.perm = perm  # act-order: original row held at each sorted position
        # tile-major copies for the decode kernel (same words in the order one workgroup reads
        # them); built once, costs a second copy of the weight in device memory
        self.decode = None
        if n % 16 == 0 and group_size % 32 == 0 and packed.is_cuda:
            self.decode = ops.w4_decode_layout(packed, scales, zp, group_size)
        # batches up to this many rows take the decode kernel (its cost grows with the rows, the
        # matrix-core kernel's hardly does; the library knows where they cross for this shape)
        self.decode_rows = ops.qmatmul_int4_decode_max_rows(padded_k, n) if self.decode is not None else 0

    def drop_decode_layout(self) -> None:
        """Give the second copy back: decode batches then run on the reference's arrays (about 15 % slower at
        4096 x 4096) and the weight costs its 4.5 bits per value only."""
        self.decode = None
        self.decode_rows = 0

    @classmethod
    def from_f32(cls, data: torch.Tensor, k: int, n: int, group_size: int,
                 symmetric: bool = False) -> "QuantizedTensor":
        """quant.rs:42-102 on the device.  ``data`` is ``[k, n]`` row-major (any shape with k*n elements)."""
        if group_size <= 0 or group_size % 8 != 0:
            raise ValueError("group_size must be a multiple of 8")
        if data.numel() != k * n:
            raise ValueError("data length mismatch")
        w = data.reshape(k, n).contiguous()
        packed, scales, zp = ops.w4_quantize_pack(w, group_size, symmetric)
        padded_k, groups = ops.w4_geometry(k, group_size)
        return cls(k, n, padded_k, group_size, groups, packed, scales, zp)

    @classmethod
    def from_packed(cls, packed, scales, zp, k: int, group_size: int,
                    g_idx: Optional[torch.Tensor] = None) -> "QuantizedTensor":
        """Adopt pre-quantized arrays (AWQ/GPTQ style).  With ``g_idx`` the rows are sorted once
        so that groups are contiguous (act-order)."""
        padded_k, groups = ops.w4_geometry(k, group_size)
        if packed.shape[0] * 8 != padded_k or scales.shape != (groups, packed.shape[1]):
            raise ValueError("from_packed: array shapes do not match k / group_size")
        perm = None
        if g_idx is not None:
            if k != padded_k:
                raise ValueError("act-order needs k to be a multiple of group_size")
            packed, perm = ops.w4_actorder_prepare(packed, g_idx, group_size)
        return cls(k, packed.shape[1], padded_k, group_size, groups, packed, scales, zp, perm)




class QLinear:
    """Linear layer with frozen INT4 weights and optional bias (quant.rs:165-222)."""

    def __init__(self, weight: QuantizedTensor, bias: Optional[torch.Tensor]):
        self.weight = weight
        self.bias = bias
        self.in_features = weight.k
        self.out_features = weight.n

    @classmethod
    def from_linear(cls, linear: Linear, group_size: int) -> "QLinear":
        k, n = linear.weight.shape
        return cls(QuantizedTensor.from_f32(linear.weight, k, n, group_size), linear.bias)

    def forward(self, x: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """``y = x @ dequant(W) + bias`` in one launch (the reference runs a second add_bias pass)."""
        w = self.weight
        if x.dtype == torch.float16:
            # the reference's kernels take f16 activations as they take f32 ones (qmatmul_int4.wgsl:33-38)
            if w.perm is not None:
                raise NotImplementedError("f16 activations with act-order weights")
            return ops.qmatmul_int4_f16(x, w.packed_tensor, w.scales_tensor, w.zp_tensor, w.k, w.group_size,
                                        bias=self.bias, out=out)
        if x.shape[0] <= w.decode_rows:
            return ops.qmatmul_int4_decode(x, *w.decode, w.k, w.group_size, bias=self.bias, perm=w.perm, out=out)
        return ops.qmatmul_int4_perm(x, w.packed_tensor, w.scales_tensor, w.zp_tensor, w.k,
                                     w.group_size, bias=self.bias, perm=w.perm, out=out)

    def backward_input(self, grad_output: torch.Tensor) -> torch.Tensor:
        """grad_x = grad_y @ dequant(W)^T (QLinearBackward, quant.rs:298-317)."""
        w = self.weight
        if w.perm is not None:
            raise NotImplementedError("grad_x for act-order weights")
        return ops.qmatmul_int4_t(grad_output, w.packed_tensor, w.scales_tensor, w.zp_tensor, w.k,
                                  w.group_size)

    __call__ = forward


# ---- INT8, reference block format -----------------------------------------------

@dataclass
class Q8Tensor:
    """A ``DType::Q8{block_size}`` tensor: fused header+data buffer, logical shape ``[K, N]``."""
    buffer: torch.Tensor
    shape: tuple
    block_size: int

    def numel(self) -> int:
        return self.shape[0] * self.shape[1]

    def prepare(self) -> "Q8Tensor":
        """For a weight with one block per column that meets batches of hundreds of rows more than once: keep a
        dense int8 copy beside the buffer (as many bytes again), which :func:`matmul` then multiplies against
        instead of unpacking the buffer on every call.  Same results, bit for bit."""
        k, n = self.shape
        if self.block_size < k or k % 16 != 0 or n > 65535:
            raise ValueError("prepare: wants one block per column (block_size >= k), k % 16 == 0 and n <= 65535")
        if getattr(self, "_dense", None) is None:
            object.__setattr__(self, "_dense", ops.q8_dense_layout(self.buffer, k, n, self.block_size))
        return self

    def data(self):
        """``Tensor::data()`` on a Q8 tensor (core.rs:612-691): dequantize on the GPU, download the
        f32 values (buffer order, as the reference does) and keep the host copy for later calls."""
        host = getattr(self, "_host", None)
        if host is None:
            host = ops.q8_dequantize(self.buffer, self.numel(), self.block_size).cpu().numpy()
            object.__setattr__(self, "_host", host)
        return host


def quantize(t, block_size: int) -> Q8Tensor:
    """``Tensor::quantize`` (ops.rs:2290-2327): transpose the last two dims, then block-quantize."""
    if isinstance(t, Q8Tensor):
        raise ValueError("quantize: input is already quantized")
    if block_size <= 0 or block_size % 4 != 0:
        raise ValueError("quantize: block_size must be > 0 and divisible by 4")
    if t.dim() != 2:
        raise ValueError("quantize: tensor must be 2-D for column-major repacking")
    tt = ops.transpose_f32(t.contiguous())
    return Q8Tensor(ops.q8_quantize(tt.reshape(-1), block_size), tuple(t.shape), block_size)


def dequantize(q: Q8Tensor) -> torch.Tensor:
    """``Tensor::dequantize`` (ops.rs:2332-2357).  Like the reference, the values come back in
    the transposed ``[N, K]`` order of the buffer under the original ``[K, N]`` shape."""
    if not isinstance(q, Q8Tensor):
        raise ValueError("dequantize: tensor is not Q8")
    return ops.q8_dequantize(q.buffer, q.numel(), q.block_size).reshape(q.shape)


def dequantize_kn(q: Q8Tensor) -> torch.Tensor:
    """The dequantized tensor with every value where its shape says it is (``[K, N]`` order):
    what ``Tensor::dequantize`` would return if it undid the transpose ``quantize`` applies."""
    if not isinstance(q, Q8Tensor):
        raise ValueError("dequantize: tensor is not Q8")
    if len(q.shape) != 2:
        raise ValueError("dequantize_kn: tensor is not 2-D")
    return ops.q8_dequantize_kn(q.buffer, q.shape[0], q.shape[1], q.block_size)


def matmul(lhs: torch.Tensor, rhs) -> torch.Tensor:
    """``Tensor::matmul`` with a Q8 right-hand side (ops.rs:516-545)."""
    if isinstance(lhs, Q8Tensor):
        raise ValueError("matmul: Q8 activations (lhs) not supported")
    if not isinstance(rhs, Q8Tensor):
        raise ValueError("matmul: this path handles Q8 weights only")
    if lhs.dim() != 2 or lhs.shape[1] != rhs.shape[0]:
        raise ValueError("matmul: inner dimension mismatch")
    if lhs.dtype == torch.float16:      # matmul_q8.wgsl:1-5: A and C are `scalar`, f32 or f16
        return ops.matmul_q8_f16(lhs.contiguous(), rhs.buffer, rhs.shape[0], rhs.shape[1], rhs.block_size)
    dense = getattr(rhs, "_dense", None)
    if dense is not None and lhs.shape[0] >= Q8_DENSE_MIN_ROWS:
        return ops.matmul_q8_dense(lhs.contiguous(), *dense)
    return ops.matmul_q8(lhs.contiguous(), rhs.buffer, rhs.shape[0], rhs.shape[1], rhs.block_size)


# below this many rows the kernels that read the Q8 buffer directly are the faster ones
Q8_DENSE_MIN_ROWS = 384


def linear_forward(linear: Linear, x: torch.Tensor, weight_q8: Q8Tensor) -> torch.Tensor:
    """``Linear::forward`` (nn/linear.rs:76-103) with the weight replaced by its Q8 form."""
    out = matmul(x, weight_q8)
    if linear.bias is not None and out.dtype != torch.float32:
        raise NotImplementedError("linear_forward: the bias pass is f32 only")
    return ops.add_bias(out, linear.bias) if linear.bias is not None else out


# ---- INT8, W8A8 -------------------------------------------------------------------

class Int8Linear:
    """Per-output-channel int8 weights, per-row dynamic int8 activations, i32 accumulate."""

    def __init__(self, wq: torch.Tensor, sw: torch.Tensor, bias: Optional[torch.Tensor]):
        self.wq, self.sw, self.bias = wq, sw, bias
        self.out_features, self.in_features = wq.shape

    @classmethod
    def from_linear(cls, linear: Linear) -> "Int8Linear":
        wq, sw = ops.i8_quantize_cols_t(linear.weight.contiguous())
        return cls(wq, sw, linear.bias)

    def forward(self, x: torch.Tensor, want_acc: bool = False):
        xq, sx = ops.i8_quantize_rows(x.contiguous())
        y, acc = ops.i8_gemm(xq, self.wq, sx, self.sw, self.bias, want_acc=want_acc)
        return (y, acc) if want_acc else y

    __call__ = forward


# ---- a decoder block built from the INT4 projections ---------------------------------------

class DecoderBlockW4:
    """Llama-shaped pre-norm decoder block whose seven projections are INT4 ``QLinear`` layers:
    RMSNorm -> q, k, v -> attention (f32, no rotary embedding) -> o -> residual ->
    RMSNorm -> gate, up -> SwiGLU -> down -> residual.  Activations stay ``[tokens, features]``
    between the layers; the attention reads the projection outputs through strides, so nothing
    is permuted or copied.  The K/V cache is token-major: ``[batch, positions, heads, 128]``."""

    NAMES = ("q", "k", "v", "o", "gate", "up", "down")

    def __init__(self, proj: dict, norm1: torch.Tensor, norm2: torch.Tensor, heads: int, eps: float = 1e-6):
        self.proj, self.norm1, self.norm2, self.heads, self.eps = proj, norm1, norm2, heads, eps
        self.dim = proj["q"].in_features
        if self.dim != heads * 128:
            raise ValueError("DecoderBlockW4: head_dim must be 128")
        # q|k|v and gate|up read the same activations: one launch each over the column-wise
        # concatenation of their weights (packed words, scales and zero-points are all [rows, n])
        self.qkv = self._concat([proj["q"], proj["k"], proj["v"]])
        self.gate_up = self._concat([proj["gate"], proj["up"]])

    @staticmethod
    def _concat(layers) -> QLinear:
        w0 = layers[0].weight
        for lin in layers:
            w = lin.weight
            if (w.k, w.group_size) != (w0.k, w0.group_size) or w.perm is not None or lin.bias is not None:
                raise ValueError("DecoderBlockW4: fused projections need equal k / group_size, no act-order, no bias")
        cat = lambda ts: torch.cat(ts, dim=1).contiguous()
        n = sum(lin.weight.n for lin in layers)
        return QLinear(QuantizedTensor(w0.k, n, w0.padded_k, w0.group_size, w0.num_groups,
                                       cat([lin.weight.packed_tensor for lin in layers]),
                                       cat([lin.weight.scales_tensor for lin in layers]),
                                       cat([lin.weight.zp_tensor for lin in layers])), None)

    @classmethod
    def from_f32(cls, weights: dict, group_size: int, heads: int, eps: float = 1e-6) -> "DecoderBlockW4":
        """``weights[name]`` is the f32 ``[in, out]`` matrix of projection ``name`` (on the device)."""
        proj = {}
        for name in cls.NAMES:
            w = weights[name]
            proj[name] = QLinear(QuantizedTensor.from_f32(w, w.shape[0], w.shape[1], group_size), None)
        d = weights["q"].shape[0]
        ones = torch.ones(d, dtype=torch.float32, device=weights["q"].device)
        return cls(proj, weights.get("norm1", ones), weights.get("norm2", ones), heads, eps)

    def forward(self, x: torch.Tensor, k_cache: Optional[torch.Tensor] = None,
                v_cache: Optional[torch.Tensor] = None, pos: int = 0):
        """``x`` is ``[batch, n, dim]``.  Without caches: causal self-attention over the n tokens
        (prefill); returns ``(y, k, v)`` with k, v ``[batch, n, heads, 128]`` (views of the fused
        q|k|v output).  With caches (``[batch, T, heads, 128]``, valid below ``pos``): n must be 1;
        the new key/value are written at ``pos`` and the token attends positions ``0..pos``;
        returns ``(y, k_cache, v_cache)``."""
        b, n, d = x.shape
        h = self.heads
        x2 = x.reshape(b * n, d)
        if k_cache is not None and n == 1 and self._folds(b):
            return self._decode_folded(x2, b, k_cache, v_cache, pos)
        hn = ops.rmsnorm(x2, self.norm1, self.eps)
        qkv = self.qkv(hn).view(b, n, 3, h, 128)
        q, k, v = qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2]
        if k_cache is None:
            att = ops.attention(q, k, v, causal=True)
            k_out, v_out = k, v
        else:
            if n != 1:
                raise ValueError("DecoderBlockW4: decode takes one token per sequence")
            att = ops.attention_decode_append(q, k, v, k_cache, v_cache, pos)
            k_out, v_out = k_cache, v_cache
        o = self.proj["o"](att.view(b * n, d))
        x1, h2 = ops.add_rmsnorm(x2, o, self.norm2, self.eps, sum_out=o, out=hn)
        gu = self.gate_up(h2)
        dw = self.proj["down"]
        if b * n <= dw.weight.decode_rows and dw.weight.perm is None:
            # decode rows: the SwiGLU happens while the down projection reads its input
            down = ops.qmatmul_int4_decode_swiglu(gu, *dw.weight.decode, dw.weight.k, dw.weight.group_size,
                                                  bias=dw.bias)
        else:
            down = dw(ops.swiglu_rows(gu))
        y = ops.add(x1, down, out=down)
        return y.view(b, n, d), k_out, v_out

    def _folds(self, rows: int) -> bool:
        """A decode step of few enough rows for every projection's decode kernel, plain weights: the norms, the
        SwiGLU and the residual adds then ride on the projections (``qmatmul_int4_decode_block``)."""
        layers = (self.qkv, self.proj["o"], self.gate_up, self.proj["down"])
        return all(rows <= lin.weight.decode_rows and lin.weight.perm is None and lin.weight.k % 8 == 0
                   for lin in layers)

    def _decode_folded(self, x2, b, k_cache, v_cache, pos):
        """The decode step in six launches: q|k|v on RMSNorm(x), attention with the cache append (two), o + x,
        gate|up on RMSNorm of that, down on SwiGLU + the residual."""
        h, d = self.heads, self.dim

        def project(lin, x, **kw):
            w = lin.weight
            return ops.qmatmul_int4_decode_block(x, *w.decode, w.k, w.group_size, bias=lin.bias, **kw)

        qkv = project(self.qkv, x2, norm_weight=self.norm1, eps=self.eps).view(b, 1, 3, h, 128)
        q, k, v = qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2]
        att = ops.attention_decode_append(q, k, v, k_cache, v_cache, pos)   # writes k, v at pos on its way
        x1 = project(self.proj["o"], att.view(b, d), residual=x2)
        gu = project(self.gate_up, x1, norm_weight=self.norm2, eps=self.eps)
        y = project(self.proj["down"], gu, swiglu=True, residual=x1, out=x1)
        return y.view(b, 1, d), k_cache, v_cache

    __call__ = forward
