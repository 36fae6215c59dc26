"""INT4 layers on disk: one safetensors file, loaded straight into device memory.

The reference keeps ``QuantizedTensor`` / ``QLinear`` (rumus-vision/src/quant.rs:24-38,165-170)
in memory only: ``QLinear`` is not a ``Module`` and has no state dict.  This is the stored form
of exactly those fields, with the tensor names GPTQ/AWQ checkpoints use, so that a file written
by another INT4 toolchain in the same bit layout loads unchanged:

    <name>.qweight  I32 [padded_k/8, n]  word (r, c) holds rows 8r..8r+7 of column c, row 8r+j in
                                         bits 4j..4j+3 (quant.rs:98-100; GPTQ's qweight)
    <name>.scales   F32 [groups, n]      (F16 is accepted and widened, which is exact)
    <name>.zeros    F32 [groups, n]      the reference's unrounded zero-points (quant.rs:77-79), or
    <name>.qzeros   I32 [groups, n/8]    u4 zero-points, column c in bits 4*(c%8) of word c/8
    <name>.bias     F32 [n]              optional
    <name>.perm     I32 [k]              optional: input feature held by each stored row (rows
                                         already sorted by group), or
    <name>.g_idx    I32 [k]              optional: group of each row, rows in their original order
                                         (GPTQ act-order); sorted once at load

``__metadata__`` carries ``format = rumus-w4``, ``version`` and, per layer, ``<name>.k`` and
``<name>.group_size`` (padding makes k unrecoverable from the shapes alone).

The file is read through two pinned staging buffers: while one chunk travels to the device the
next is read from disk.  Nothing is interpreted on the host except the JSON header.
"""
from __future__ import annotations

import json
import os
import struct
from typing import Dict, Optional

import numpy as np
import torch

from . import ops
from .nn import QLinear, QuantizedTensor

FORMAT = "rumus-w4"
VERSION = "1"
CHUNK_BYTES = 64 << 20

_DTYPES = {"F32": (np.float32, torch.float32), "F16": (np.float16, torch.float16),
           "I32": (np.int32, torch.int32)}
_NAMES = {np.dtype(np.float32): "F32", np.dtype(np.float16): "F16", np.dtype(np.int32): "I32"}


# ---- the container --------------------------------------------------------------------------

def write_safetensors(path: str, tensors: Dict[str, np.ndarray], metadata: Dict[str, str]) -> None:
    """8-byte little-endian header length, JSON header, tensor bytes back to back (row-major,
    little-endian), the layout the safetensors format fixes.  The header is padded with spaces so
    that the data start on a 64-byte boundary."""
    header = {"__metadata__": {str(k): str(v) for k, v in metadata.items()}}
    offset = 0
    order = sorted(tensors)
    for name in order:
        t = tensors[name]
        if t.dtype not in _NAMES:
            raise ValueError(f"{name}: dtype {t.dtype} is not stored by this format")
        nbytes = t.size * t.dtype.itemsize
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * (-(8 + len(blob)) % 64)
    tmp = path + ".tmp"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for name in order:
            f.write(np.ascontiguousarray(tensors[name]).tobytes())
    os.replace(tmp, path)


def read_header(path: str):
    """(entries, metadata, offset of the data region); entries: name -> (dtype, shape, begin, end).
    Rejects what a truncated or foreign file would show: offsets outside the file, sizes that do
    not match shape x dtype, unknown dtypes."""
    size = os.path.getsize(path)
    with open(path, "rb") as f:
        head = f.read(8)
        if len(head) != 8:
            raise ValueError(f"{path}: not a safetensors file (shorter than its length field)")
        (hlen,) = struct.unpack("<Q", head)
        if hlen > size - 8 or hlen > (100 << 20):
            raise ValueError(f"{path}: header length {hlen} does not fit the file")
        header = json.loads(f.read(hlen).decode("utf-8"))
    data_start = 8 + hlen
    metadata = header.pop("__metadata__", {}) or {}
    entries = {}
    for name, e in header.items():
        dtype, shape, (begin, end) = e["dtype"], tuple(int(v) for v in e["shape"]), e["data_offsets"]
        if dtype not in _DTYPES:
            raise ValueError(f"{path}: {name} has dtype {dtype}, which this loader does not read")
        want = int(np.prod(shape, dtype=np.int64)) * np.dtype(_DTYPES[dtype][0]).itemsize
        if begin < 0 or end < begin or end - begin != want or data_start + end > size:
            raise ValueError(f"{path}: {name} has offsets [{begin}, {end}) for {want} bytes in a file of {size}")
        entries[name] = (dtype, shape, int(begin), int(end))
    return entries, metadata, data_start


def read_tensor_host(path: str, name: str) -> np.ndarray:
    """One tensor of the file as a read-only memory map (inspection and tests; nothing is copied)."""
    entries, _, data_start = read_header(path)
    dtype, shape, begin, end = entries[name]
    return np.memmap(path, dtype=_DTYPES[dtype][0], mode="r", offset=data_start + begin, shape=shape)


class _Uploader:
    """File ranges -> device tensors through two pinned buffers, copies on the current stream."""

    def __init__(self, f, device):
        self.f, self.device = f, device
        self.pinned = [torch.empty(CHUNK_BYTES, dtype=torch.uint8, pin_memory=True) for _ in range(2)]
        self.done = [None, None]
        self.turn = 0

    def fetch(self, offset: int, nbytes: int) -> torch.Tensor:
        dst = torch.empty(nbytes, dtype=torch.uint8, device=self.device)
        self.f.seek(offset)
        pos = 0
        while pos < nbytes:
            n = min(CHUNK_BYTES, nbytes - pos)
            slot = self.turn
            self.turn ^= 1
            if self.done[slot] is not None:
                self.done[slot].synchronize()           # the copy that last used this buffer
            got = self.f.readinto(memoryview(self.pinned[slot].numpy())[:n])
            if got != n:
                raise ValueError(f"file ended {n - (got or 0)} bytes early")
            dst[pos:pos + n].copy_(self.pinned[slot][:n], non_blocking=True)
            self.done[slot] = torch.cuda.Event()
            self.done[slot].record()
            pos += n
        return dst

    def finish(self):
        for e in self.done:
            if e is not None:
                e.synchronize()


# ---- layers ---------------------------------------------------------------------------------

def _host(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().contiguous().numpy()


def save_w4(path: str, layers: Dict[str, QLinear], zero_points: str = "f32") -> None:
    """Write ``layers`` (name -> QLinear).  ``zero_points="u4"`` stores them eight per word, which
    needs every zero-point to be an integer in 0..15 (symmetric and AWQ-style weights are; the
    reference's asymmetric quantizer is not) and n % 8 == 0."""
    if zero_points not in ("f32", "u4"):
        raise ValueError("zero_points must be 'f32' or 'u4'")
    tensors, meta = {}, {"format": FORMAT, "version": VERSION}
    for name, layer in layers.items():
        w = layer.weight
        tensors[f"{name}.qweight"] = _host(w.packed_tensor).view(np.int32)
        tensors[f"{name}.scales"] = _host(w.scales_tensor)
        zp = _host(w.zp_tensor)
        if zero_points == "u4":
            finite = bool(np.isfinite(zp).all())              # a NaN cast to an integer is undefined
            zi = np.where(np.isfinite(zp), zp, 0).astype(np.int64)
            if w.n % 8 != 0 or not (finite and np.array_equal(zi.astype(np.float32), zp) and zi.min() >= 0
                                    and zi.max() <= 15):
                raise ValueError(f"{name}: zero-points are not integers in 0..15 over a multiple of 8 columns; "
                                 f"store them as f32")
            z8 = zi.reshape(w.num_groups, w.n // 8, 8).astype(np.uint32)
            words = np.zeros((w.num_groups, w.n // 8), dtype=np.uint32)
            for j in range(8):
                words |= z8[:, :, j] << np.uint32(4 * j)
            tensors[f"{name}.qzeros"] = words.view(np.int32)
        else:
            tensors[f"{name}.zeros"] = zp
        if layer.bias is not None:
            tensors[f"{name}.bias"] = _host(layer.bias)
        if w.perm is not None:
            tensors[f"{name}.perm"] = _host(w.perm).astype(np.int32)
        meta[f"{name}.k"] = w.k
        meta[f"{name}.group_size"] = w.group_size
    write_safetensors(path, tensors, meta)


def check_perm(perm: np.ndarray, k: int, what: str) -> None:
    """Raise ValueError unless ``perm`` holds every input feature 0..k-1 exactly once."""
    perm = np.asarray(perm)
    if perm.shape != (k,):
        raise ValueError(f"{what} has shape {perm.shape}, expected ({k},)")
    if perm.size and (perm.min() < 0 or perm.max() >= k):
        raise ValueError(f"{what} has entries outside [0, {k})")
    if not np.array_equal(np.sort(perm), np.arange(k, dtype=perm.dtype)):
        raise ValueError(f"{what} is not a permutation of 0..{k - 1}")


def load_w4(path: str, device="cuda:0") -> Dict[str, QLinear]:
    """Read every layer of the file into ``device`` memory and return name -> QLinear, ready to
    run (the tile-major decode copies are built here, as for a freshly quantized weight)."""
    device = torch.device(device)
    if device.type != "cuda":
        raise ValueError("load_w4: the layers live in GPU memory; pass a cuda device")
    entries, meta, data_start = read_header(path)
    if meta.get("format") != FORMAT:
        raise ValueError(f"{path}: not a {FORMAT} file (format = {meta.get('format')!r})")
    if meta.get("version") != VERSION:
        raise ValueError(f"{path}: version {meta.get('version')!r}, this loader reads {VERSION!r}")
    names = sorted(n[:-len(".qweight")] for n in entries if n.endswith(".qweight"))
    layers: Dict[str, QLinear] = {}
    with open(path, "rb") as f:
        up = _Uploader(f, device)

        def get(name: str, dtypes, shape=None) -> Optional[torch.Tensor]:
            if name not in entries:
                return None
            dtype, shp, begin, end = entries[name]
            if dtype not in dtypes:
                raise ValueError(f"{path}: {name} is {dtype}, expected {' or '.join(dtypes)}")
            if shape is not None and shp != shape:
                raise ValueError(f"{path}: {name} has shape {shp}, expected {shape}")
            return up.fetch(data_start + begin, end - begin).view(_DTYPES[dtype][1]).reshape(shp)

        for name in names:
            try:
                k, group_size = int(meta[f"{name}.k"]), int(meta[f"{name}.group_size"])
            except (KeyError, ValueError):
                raise ValueError(f"{path}: metadata lacks {name}.k / {name}.group_size") from None
            if group_size <= 0 or group_size % 8 != 0:
                raise ValueError(f"{path}: {name}.group_size {group_size} is not a multiple of 8")
            padded_k, groups = ops.w4_geometry(k, group_size)
            shp = entries[f"{name}.qweight"][1]
            if len(shp) != 2 or shp[0] * 8 != padded_k:
                raise ValueError(f"{path}: {name}.qweight has shape {shp}, expected [{padded_k // 8}, n]")
            n = shp[1]
            packed = get(f"{name}.qweight", ("I32",))
            scales = get(f"{name}.scales", ("F32", "F16"), (groups, n))
            if scales is None:
                raise ValueError(f"{path}: {name}.scales is missing")
            if scales.dtype == torch.float16:
                scales = ops.f16_to_f32(scales)
            zp = get(f"{name}.zeros", ("F32",), (groups, n))
            if zp is None:
                qz = get(f"{name}.qzeros", ("I32",), (groups, n // 8) if n % 8 == 0 else None)
                if qz is None or n % 8 != 0:
                    raise ValueError(f"{path}: {name} has neither zeros [groups, n] nor qzeros [groups, n/8]")
                zp = ops.w4_qzeros_unpack(qz, n)
            bias = get(f"{name}.bias", ("F32",), (n,))
            perm = get(f"{name}.perm", ("I32",), (k,))
            g_idx = get(f"{name}.g_idx", ("I32",), (k,))
            if perm is not None and g_idx is not None:
                raise ValueError(f"{path}: {name} has both perm and g_idx")
            if perm is not None:
                if k != padded_k:
                    raise ValueError(f"{path}: {name}.perm needs k to be a multiple of group_size")
                # the kernels gather activations through perm without a bounds check of their own:
                # an entry outside [0, k) in a damaged file would read outside x
                check_perm(perm.cpu().numpy(), k, f"{path}: {name}.perm")
                weight = QuantizedTensor(k, n, padded_k, group_size, groups, packed, scales, zp, perm)
            else:
                weight = QuantizedTensor.from_packed(packed, scales, zp, k, group_size, g_idx=g_idx)
            layers[name] = QLinear(weight, bias)
        up.finish()
    return layers
