"""INT4 layers through the on-disk form (rumus_amd.checkpoint) and back, on the GPU: the loaded
layer holds the same bits and computes the same outputs as the layer that was saved, and a file
written by another toolchain (the safetensors package, GPTQ tensor names) loads and matches the
CPU restatement."""
import numpy as np
import pytest
import torch

import oracle
from rumus_amd import checkpoint as ck
from rumus_amd.nn import QLinear, QuantizedTensor

from gpu_util import assert_close, dev, host, host_u32, say

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from rumus_amd import ops as o
    return o


def same_bits(a: torch.Tensor, b: torch.Tensor) -> bool:
    return a.shape == b.shape and a.dtype == b.dtype and bool(torch.equal(a.view(torch.int32), b.view(torch.int32)))


def layer(rng, k, n, g, bias=True, symmetric=False):
    w = dev((rng.standard_normal((k, n)) * 0.02).astype(np.float32))
    b = dev(rng.standard_normal(n).astype(np.float32)) if bias else None
    return QLinear(QuantizedTensor.from_f32(w, k, n, g, symmetric=symmetric), b)


@pytest.mark.parametrize("rows", [1, 16])
def test_round_trip_keeps_bits_and_outputs(tmp_path, rows):
    say(f"checkpoint round trip, {rows} rows")
    rng = np.random.default_rng(11)
    layers = {"blk.q_proj": layer(rng, 512, 256, 128), "blk.ragged": layer(rng, 200, 24, 64, bias=False),
              "blk.odd_n": layer(rng, 96, 20, 32)}
    path = str(tmp_path / "m.safetensors")
    ck.save_w4(path, layers)
    back = ck.load_w4(path)
    assert sorted(back) == sorted(layers)
    for name, a in layers.items():
        b = back[name]
        wa, wb = a.weight, b.weight
        assert (wa.k, wa.n, wa.padded_k, wa.group_size, wa.num_groups) == (wb.k, wb.n, wb.padded_k, wb.group_size, wb.num_groups)
        assert same_bits(wa.packed_tensor, wb.packed_tensor) and same_bits(wa.scales_tensor, wb.scales_tensor)
        assert same_bits(wa.zp_tensor, wb.zp_tensor)
        assert (a.bias is None) == (b.bias is None) and (a.bias is None or same_bits(a.bias, b.bias))
        assert (wa.decode is None) == (wb.decode is None)
        x = dev(rng.standard_normal((rows, wa.k)).astype(np.float32))
        assert same_bits(a(x), b(x)), name


def test_u4_zero_points_and_unpack_kernel(tmp_path, ops):
    say("checkpoint with u4 zero-points")
    rng = np.random.default_rng(12)
    # the kernel alone, against the CPU restatement
    qz = rng.integers(0, 2**32, size=(5, 13), dtype=np.uint64).astype(np.uint32)
    np.testing.assert_array_equal(host(ops.w4_qzeros_unpack(dev(qz), 104)), oracle.w4_qzeros_unpack(qz, 104))
    # symmetric weights (zero-point 8) stored eight per word
    lin = layer(rng, 256, 64, 64, symmetric=True)
    path = str(tmp_path / "s.safetensors")
    ck.save_w4(path, {"l": lin}, zero_points="u4")
    entries, _, _ = ck.read_header(path)
    assert "l.qzeros" in entries and "l.zeros" not in entries and entries["l.qzeros"][1] == (4, 8)
    assert np.all(np.asarray(ck.read_tensor_host(path, "l.qzeros")).view(np.uint32) == 0x88888888)
    back = ck.load_w4(path)["l"]
    assert same_bits(back.weight.zp_tensor, lin.weight.zp_tensor)
    x = dev(rng.standard_normal((3, 256)).astype(np.float32))
    assert same_bits(back(x), lin(x))
    # the reference's asymmetric quantizer leaves fractional zero-points: u4 storage must refuse them
    with pytest.raises(ValueError, match="store them as f32"):
        ck.save_w4(path, {"l": layer(rng, 256, 64, 64)}, zero_points="u4")


def test_act_order_layers(tmp_path, ops):
    say("checkpoint act-order: perm round trip and a g_idx file of another toolchain")
    from safetensors.numpy import save_file
    rng = np.random.default_rng(13)
    k, n, g = 512, 48, 128
    w = (rng.standard_normal((k, n)) * 0.02).astype(np.float32)
    packed, scales, zp = (host(t) for t in ops.w4_quantize_pack(dev(w), g))
    g_idx = (rng.permutation(k) // g).astype(np.int32)
    # rows in their original order + g_idx, f16 scales, written by the safetensors package
    s16 = scales.astype(np.float16)
    foreign = str(tmp_path / "gptq.safetensors")
    save_file({"m.qweight": packed.view(np.int32), "m.scales": s16, "m.zeros": zp, "m.g_idx": g_idx}, foreign,
              metadata={"format": ck.FORMAT, "version": ck.VERSION, "m.k": str(k), "m.group_size": str(g)})
    lin = ck.load_w4(foreign)["m"]
    assert lin.weight.perm is not None
    x = rng.standard_normal((4, k)).astype(np.float32)
    want = oracle.qmatmul_int4(x, packed.view(np.uint32), s16.astype(np.float32), zp, k, g, g_idx=g_idx)
    assert_close(host(lin(dev(x))), want)
    # saved again (sorted rows + perm) and reloaded: same bits, same outputs
    again = str(tmp_path / "sorted.safetensors")
    ck.save_w4(again, {"m": lin})
    back = ck.load_w4(again)["m"]
    assert same_bits(back.weight.packed_tensor, lin.weight.packed_tensor)
    assert torch.equal(back.weight.perm, lin.weight.perm)
    assert same_bits(back(dev(x)), lin(dev(x)))


def test_many_chunks_through_the_staging_buffers(tmp_path, monkeypatch):
    say("checkpoint upload in many chunks")
    monkeypatch.setattr(ck, "CHUNK_BYTES", 4096 + 64)      # 520 KB of words in 130 odd-sized pieces
    rng = np.random.default_rng(14)
    lin = layer(rng, 1024, 1040, 128)
    path = str(tmp_path / "c.safetensors")
    ck.save_w4(path, {"big": lin})
    back = ck.load_w4(path)["big"]
    assert same_bits(back.weight.packed_tensor, lin.weight.packed_tensor)
    assert same_bits(back.weight.scales_tensor, lin.weight.scales_tensor)
    np.testing.assert_array_equal(host_u32(back.weight.packed_tensor),
                                  np.asarray(ck.read_tensor_host(path, "big.qweight")).view(np.uint32))


def test_inconsistent_files_are_refused(tmp_path):
    say("checkpoint refusals")
    rng = np.random.default_rng(15)
    path = str(tmp_path / "r.safetensors")
    q = rng.integers(0, 2**31, size=(16, 8)).astype(np.int32)
    s = np.ones((1, 8), np.float32)
    base = {"format": ck.FORMAT, "version": ck.VERSION, "l.k": 128, "l.group_size": 128}
    cases = [
        ({"l.qweight": q, "l.scales": s, "l.zeros": s}, {**base, "format": "else"}, "not a rumus-w4 file"),
        ({"l.qweight": q, "l.scales": s, "l.zeros": s}, {**base, "version": "9"}, "version"),
        ({"l.qweight": q, "l.scales": s, "l.zeros": s}, {k: v for k, v in base.items() if k != "l.k"}, "metadata lacks"),
        ({"l.qweight": q, "l.scales": s, "l.zeros": s}, {**base, "l.group_size": 12}, "multiple of 8"),
        ({"l.qweight": q, "l.scales": s, "l.zeros": s}, {**base, "l.k": 300}, "qweight has shape"),
        ({"l.qweight": q, "l.scales": np.ones((2, 8), np.float32), "l.zeros": s}, base, "scales has shape"),
        ({"l.qweight": q, "l.scales": s}, base, "neither zeros"),
        ({"l.qweight": q, "l.zeros": s}, base, "scales is missing"),
        ({"l.qweight": q, "l.scales": s, "l.zeros": s, "l.perm": np.arange(128, dtype=np.int32),
          "l.g_idx": np.zeros(128, np.int32)}, base, "both perm and g_idx"),
        # gather indices are checked before any kernel reads through them
        ({"l.qweight": q, "l.scales": s, "l.zeros": s, "l.perm": np.arange(1, 129, dtype=np.int32)}, base,
         "entries outside"),
        ({"l.qweight": q, "l.scales": s, "l.zeros": s, "l.perm": -np.arange(128, dtype=np.int32)}, base,
         "entries outside"),
        ({"l.qweight": q, "l.scales": s, "l.zeros": s, "l.perm": np.zeros(128, dtype=np.int32)}, base,
         "not a permutation"),
    ]
    for tensors, meta, msg in cases:
        ck.write_safetensors(path, tensors, meta)
        with pytest.raises(ValueError, match=msg):
            ck.load_w4(path)
