"""The C-ABI library loads without a GPU and exports exactly what the header declares."""
import os
import re
import subprocess

import pytest

from rumus_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "rumus_hip.h")


def _declared():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(rumus_hip_[a-z0-9_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def library():
    if not os.path.exists(_lib.LIB_PATH):
        _lib.build()
    return _lib.lib()


def test_header_is_plain_c(tmp_path):
    # the boundary is a C ABI: the header must compile as C99 with nothing but itself
    src = tmp_path / "c_abi.c"
    src.write_text('#include "rumus_hip.h"\nint main(void) { return rumus_hip_version() ? 0 : 1; }\n')
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-I", os.path.join(ROOT, "include"),
                    "-fsyntax-only", str(src)], check=True)


def test_header_and_binding_agree():
    assert _declared() == sorted(_lib.PROTOTYPES)


def test_every_declared_symbol_is_exported(library):
    out = subprocess.check_output(["nm", "-D", "--defined-only", _lib.LIB_PATH], text=True)
    exported = {line.split()[-1] for line in out.splitlines() if " T " in line}
    missing = [s for s in _declared() if s not in exported]
    assert not missing, missing
    for name in _declared():
        assert getattr(library, name) is not None


def test_version_and_pure_host_entry_points(library):
    assert library.rumus_hip_version().decode().endswith("gfx950")
    # tensor/core.rs:87-98
    assert library.rumus_hip_q8_buf_size(512 * 512, 512) == 512 * 516
    assert library.rumus_hip_q8_buf_size(10, 4) == 24


def test_preconditions_are_rejected_before_any_launch(library):
    # null pointers are fine here: validation runs first and nothing is launched
    rc = library.rumus_hip_q8_quantize(None, None, 16, 6, None)
    assert rc == _lib.EINVAL and b"divisible by 4" in library.rumus_hip_last_error()
    rc = library.rumus_hip_w4_quantize_pack(None, 16, 4, 12, None, None, None, None)
    assert rc == _lib.EINVAL and b"multiple of 8" in library.rumus_hip_last_error()
    rc = library.rumus_hip_qmatmul_int4(None, None, None, None, None, None, None,
                                        1, 100, 4, 128, 64, 3, None)
    assert rc == _lib.EINVAL and b"padded_k" in library.rumus_hip_last_error()
    rc = library.rumus_hip_i8_gemm(None, None, None, None, None, None, None, 4, 24, 4, None)
    assert rc == _lib.EINVAL
    with pytest.raises(_lib.RumusError):
        _lib.call("rumus_hip_matmul_q8", None, None, None, 1, 8, 1, 3, None)


def test_empty_calls_succeed_without_arrays_and_full_ones_need_them(library):
    """A call with no rows queues nothing and reads no array, so it may come without pointers (an empty tensor has
    none) and needs no GPU; the same call with rows is refused for its null pointers; scalar preconditions hold
    either way."""
    L = library
    assert L.rumus_hip_qmatmul_int4(None, None, None, None, None, None, None, 0, 128, 64, 128, 64, 2, None) == 0
    assert L.rumus_hip_qmatmul_int4(None, None, None, None, None, None, None, 2, 128, 64, 128, 64, 2, None) == _lib.EINVAL
    assert b"null buffer" in L.rumus_hip_last_error()
    assert L.rumus_hip_qmatmul_int4(None, None, None, None, None, None, None, 0, 128, 64, 128, 12, 2, None) == _lib.EINVAL
    assert L.rumus_hip_qmatmul_int4_t(None, None, None, None, None, 0, 128, 64, 128, 64, 2, None) == 0
    assert L.rumus_hip_qmatmul_int4_decode(None, None, None, None, None, None, None, 0, 128, 64, 128, 64, 2, None) == 0
    assert L.rumus_hip_qmatmul_int4_decode_block(None, None, 1e-6, 0, None, None, None, None, None, None,
                                                 0, 128, 64, 128, 64, 2, None) == 0
    assert L.rumus_hip_qmatmul_int4_decode_block(None, None, 1e-6, 0, None, None, None, None, None, None,
                                                 1, 128, 64, 128, 64, 2, None) == _lib.EINVAL
    assert L.rumus_hip_qmatmul_int4_decode_block(None, None, 1e-6, 0, None, None, None, None, None, None,
                                                 9, 128, 64, 128, 64, 2, None) == _lib.EINVAL
    assert L.rumus_hip_matmul_q8(None, None, None, 0, 64, 8, 32, None) == 0
    assert L.rumus_hip_matmul_q8(None, None, None, 1, 64, 8, 32, None) == _lib.EINVAL
    assert L.rumus_hip_matmul_q8(None, None, None, 0, 64, 8, 6, None) == _lib.EINVAL
    assert L.rumus_hip_matmul_q8_dense(None, None, None, None, 0, 64, 8, None) == 0
    # the half-precision entry points answer like the f32 ones they wrap
    assert L.rumus_hip_matmul_q8_f16(None, None, None, 0, 64, 8, 32, None) == 0
    assert L.rumus_hip_matmul_q8_f16(None, None, None, 1, 64, 8, 32, None) == _lib.EINVAL
    assert L.rumus_hip_matmul_q8_f16(None, None, None, 0, 64, 8, 6, None) == _lib.EINVAL
    assert L.rumus_hip_qmatmul_int4_f16(None, None, None, None, None, None, None, 0, 128, 64, 128, 64, 2, None) == 0
    assert L.rumus_hip_qmatmul_int4_f16(None, None, None, None, None, None, None, 2, 128, 64, 128, 64, 2, None) == _lib.EINVAL
    assert b"null buffer" in L.rumus_hip_last_error()
    assert L.rumus_hip_qmatmul_int4_f16(None, None, None, None, None, None, None, 2, 100, 4, 128, 64, 3, None) == _lib.EINVAL
    assert b"padded_k" in L.rumus_hip_last_error()
    assert L.rumus_hip_f16_staging_reserve(None, 0) == 0
    assert L.rumus_hip_q8_quantize(None, None, 0, 32, None) == 0
    assert L.rumus_hip_q8_dequantize(None, None, 0, 32, None) == 0
    assert L.rumus_hip_i8_quantize_rows(None, None, None, 0, 64, None) == 0
    assert L.rumus_hip_i8_quantize_rows(None, None, None, 3, 64, None) == _lib.EINVAL
    assert L.rumus_hip_i8_gemm(None, None, None, None, None, None, None, 0, 64, 8, None) == 0
    assert L.rumus_hip_i8_gemm(None, None, None, None, None, None, None, 0, 24, 8, None) == _lib.EINVAL
    assert L.rumus_hip_add_bias(None, None, None, 0, 8, None) == 0
    assert L.rumus_hip_transpose_f32(None, None, 0, 8, None) == 0
    assert L.rumus_hip_rmsnorm(None, None, None, 0, 64, 1e-6, None) == 0
    assert L.rumus_hip_rmsnorm(None, None, None, 2, 64, 1e-6, None) == _lib.EINVAL
    assert L.rumus_hip_swiglu(None, None, None, 0, None) == 0
    assert L.rumus_hip_add(None, None, None, 0, None) == 0
    assert L.rumus_hip_attention(None, None, None, None, 1, 4, 0, 8, 128, None, 0, None) == 0
    assert L.rumus_hip_kv_append(None, None, None, None, 1, 4, 0, 128, 3, 16, None, None) == 0
    assert L.rumus_hip_kv_append(None, None, None, None, 1, 4, 0, 128, 17, 16, None, None) == _lib.EINVAL


def test_matmul_q8_refuses_a_buffer_without_whole_blocks_per_column():
    # Tensor::quantize blocks the flat transposed tensor: with k % block_size != 0 the buffer holds fewer blocks than
    # matmul_q8's addressing (ceil(k / block_size) per column) walks, and the kernel would read past its end
    import torch
    from rumus_amd import ops
    k, n, bs = 1000, 100, 256
    flat_words = library_free_q8_words(k * n, bs)
    a = torch.zeros((2, k), dtype=torch.float32)
    with pytest.raises(ValueError, match="whole blocks"):
        ops.matmul_q8(a, torch.zeros(flat_words, dtype=torch.int32), k, n, bs)


def test_binding_refuses_arrays_shorter_than_the_geometry():
    # raw pointers go to the device: a short array would be read past its end there
    import torch
    from rumus_amd import ops
    k, n, g = 256, 64, 128
    x = torch.zeros((2, k))
    packed = torch.zeros((k // 8, n), dtype=torch.int32)
    scales = torch.zeros((k // g, n))
    with pytest.raises(ValueError, match="smaller than"):
        ops.qmatmul_int4(x, packed[:-1], scales, scales, k, g)
    with pytest.raises(ValueError, match="smaller than"):
        ops.qmatmul_int4(x, packed, scales[:-1], scales, k, g)
    with pytest.raises(ValueError, match="bias"):
        ops.qmatmul_int4(x, packed, scales, scales, k, g, bias=torch.zeros(n - 1))
    with pytest.raises(ValueError, match="perm"):
        ops.qmatmul_int4_perm(x, packed, scales, scales, k, g, perm=torch.zeros(k - 1, dtype=torch.int32))
    with pytest.raises(ValueError, match="out must be"):
        ops.qmatmul_int4(x, packed, scales, scales, k, g, out=torch.zeros((2, n + 1)))
    with pytest.raises(ValueError, match="smaller than"):
        ops.qmatmul_int4_t(torch.zeros((2, n)), packed, scales, scales[:-1], k, g)
    with pytest.raises(ValueError, match="sx must hold"):
        ops.i8_gemm(torch.zeros((4, 32), dtype=torch.int8), torch.zeros((8, 32), dtype=torch.int8), torch.zeros(3), torch.zeros(8))
    with pytest.raises(ValueError, match="shorter"):
        ops.q8_dequantize(torch.zeros(10, dtype=torch.int32), 1024, 32)
    # the dense copy of a per-channel Q8 weight walks n blocks of 1 + block_size / 4 words
    with pytest.raises(ValueError, match="shorter than n blocks"):
        ops.q8_dense_layout(torch.zeros(8 * 65 - 1, dtype=torch.int32), 256, 8, 256)


def library_free_q8_words(numel, bs):
    """Words of a flat-blocked Q8 buffer (tensor/core.rs:87-98) without loading the library."""
    blocks = -(-numel // bs)
    return blocks * ((4 + bs + 3) // 4)


def test_product_package_does_not_touch_the_oracle():
    pkg = os.path.join(ROOT, "rumus_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp", ".hpp")) or f == "Makefile":
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.replace("test oracle", ""), os.path.join(dirpath, f)
