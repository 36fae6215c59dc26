"""The safetensors container of rumus_amd.checkpoint, without a GPU: what it writes is what the
safetensors package reads, and the other way round; damaged headers are refused."""
import json
import os
import struct

import numpy as np
import pytest

from rumus_amd import checkpoint as ck


def sample():
    rng = np.random.default_rng(3)
    return {
        "a.qweight": rng.integers(-2**31, 2**31, size=(6, 24), dtype=np.int64).astype(np.int32),
        "a.scales": rng.standard_normal((3, 24)).astype(np.float32),
        "a.zeros": rng.standard_normal((3, 24)).astype(np.float32),
        "b.scales": rng.standard_normal((1, 8)).astype(np.float16),
        "b.bias": np.zeros((0,), np.float32),
    }


def test_written_file_is_read_by_the_safetensors_package(tmp_path):
    from safetensors import safe_open
    from safetensors.numpy import load_file
    path = str(tmp_path / "w.safetensors")
    tensors = sample()
    ck.write_safetensors(path, tensors, {"format": ck.FORMAT, "a.k": 44})
    got = load_file(path)
    assert set(got) == set(tensors)
    for name, t in tensors.items():
        assert got[name].dtype == t.dtype and got[name].shape == t.shape
        assert np.array_equal(got[name].view(np.uint8), t.view(np.uint8)), name
    with safe_open(path, "np") as f:
        assert f.metadata() == {"format": ck.FORMAT, "a.k": "44"}
    assert (8 + struct.unpack("<Q", open(path, "rb").read(8))[0]) % 64 == 0


def test_file_of_the_safetensors_package_is_read(tmp_path):
    from safetensors.numpy import save_file
    path = str(tmp_path / "p.safetensors")
    tensors = sample()
    save_file(tensors, path, metadata={"format": "other"})
    entries, meta, start = ck.read_header(path)
    assert meta == {"format": "other"} and set(entries) == set(tensors)
    for name, t in tensors.items():
        dtype, shape, begin, end = entries[name]
        assert shape == t.shape and end - begin == t.nbytes
        if t.size:
            assert np.array_equal(np.asarray(ck.read_tensor_host(path, name)).view(np.uint8), t.view(np.uint8)), name


def rewrite_header(path, edit):
    raw = open(path, "rb").read()
    (hlen,) = struct.unpack("<Q", raw[:8])
    header = json.loads(raw[8:8 + hlen])
    edit(header)
    blob = json.dumps(header).encode()
    open(path, "wb").write(struct.pack("<Q", len(blob)) + blob + raw[8 + hlen:])


def test_damaged_files_are_refused(tmp_path):
    path = str(tmp_path / "d.safetensors")
    tensors = sample()
    ck.write_safetensors(path, tensors, {})
    good = open(path, "rb").read()

    open(path, "wb").write(good[:5])
    with pytest.raises(ValueError, match="shorter than its length field"):
        ck.read_header(path)

    open(path, "wb").write(struct.pack("<Q", 1 << 40) + good[8:])
    with pytest.raises(ValueError, match="does not fit the file"):
        ck.read_header(path)

    open(path, "wb").write(good[:-10])                       # data cut short
    with pytest.raises(ValueError, match="offsets"):
        ck.read_header(path)

    open(path, "wb").write(good)
    rewrite_header(path, lambda h: h["a.scales"].update(shape=[3, 25]))
    with pytest.raises(ValueError, match="offsets"):
        ck.read_header(path)

    open(path, "wb").write(good)
    rewrite_header(path, lambda h: h["a.scales"].update(dtype="F64"))
    with pytest.raises(ValueError, match="does not read"):
        ck.read_header(path)


def test_unsupported_dtype_is_not_written(tmp_path):
    with pytest.raises(ValueError, match="not stored"):
        ck.write_safetensors(str(tmp_path / "x.safetensors"), {"t": np.zeros(3, np.float64)}, {})
    assert not os.path.exists(tmp_path / "x.safetensors")


def test_load_needs_a_gpu_device(tmp_path):
    path = str(tmp_path / "e.safetensors")
    ck.write_safetensors(path, {}, {"format": ck.FORMAT, "version": ck.VERSION})
    with pytest.raises(ValueError, match="cuda"):
        ck.load_w4(path, device="cpu")


def test_perm_check_accepts_permutations_only():
    rng = np.random.default_rng(3)
    ck.check_perm(rng.permutation(300).astype(np.int32), 300, "perm")
    ck.check_perm(np.zeros(0, np.int32), 0, "perm")
    bad = np.arange(300, dtype=np.int32)
    bad[7] = 300
    with pytest.raises(ValueError, match="outside"):
        ck.check_perm(bad, 300, "perm")
    bad[7] = -1
    with pytest.raises(ValueError, match="outside"):
        ck.check_perm(bad, 300, "perm")
    bad[7] = 8
    with pytest.raises(ValueError, match="not a permutation"):
        ck.check_perm(bad, 300, "perm")
    with pytest.raises(ValueError, match="shape"):
        ck.check_perm(np.arange(299, dtype=np.int32), 300, "perm")
