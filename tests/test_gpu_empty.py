"""Empty inputs through the C ABI: zero rows (or zero elements) are accepted by every entry point that takes a batch,
return an empty result and leave the buffers they were given untouched."""
import numpy as np
import pytest
import torch

from gpu_util import dev, host, say

pytestmark = pytest.mark.gpu

K, N, G = 256, 64, 64


@pytest.fixture(scope="module")
def ops():
    from rumus_amd import ops as o
    return o


@pytest.fixture(scope="module")
def layer(ops):
    rng = np.random.default_rng(11)
    w = dev(rng.normal(0, 0.02, (K, N)).astype(np.float32))
    packed, scales, zp = ops.w4_quantize_pack(w, G)
    return w, packed, scales, zp


def no_rows(cols):
    return torch.empty((0, cols), dtype=torch.float32, device="cuda")


def test_w4_matmuls_take_zero_rows(ops, layer):
    _, packed, scales, zp = layer
    bias = torch.ones(N, device="cuda")
    say("qmatmul_int4, 0 rows")
    assert ops.qmatmul_int4(no_rows(K), packed, scales, zp, K, G, bias=bias).shape == (0, N)
    perm = torch.arange(K, dtype=torch.int32, device="cuda")
    say("qmatmul_int4_perm, 0 rows")
    assert ops.qmatmul_int4_perm(no_rows(K), packed, scales, zp, K, G, perm=perm).shape == (0, N)
    say("qmatmul_int4_perm_static, 0 rows")
    assert ops.qmatmul_int4_perm_static(no_rows(K), packed, scales, zp, K, G, perm=perm).shape == (0, N)
    say("qmatmul_int4_t, 0 rows")
    assert ops.qmatmul_int4_t(no_rows(N), packed, scales, zp, K, G).shape == (0, K)
    say("decode layout, 0 rows")
    pt, st, zt = ops.w4_decode_layout(packed, scales, zp, G)
    assert ops.qmatmul_int4_decode(no_rows(K), pt, st, zt, K, G).shape == (0, N)
    assert ops.qmatmul_int4_decode_swiglu(no_rows(2 * K), pt, st, zt, K, G).shape == (0, N)


def test_w4_packed_zero_points_take_zero_rows(ops, layer):
    w = layer[0]
    packed, scales, qzeros = ops.w4_quantize_pack_awq(w, G)
    say("qmatmul_int4_zp4, 0 rows")
    assert ops.qmatmul_int4_zp4(no_rows(K), packed, scales, qzeros, K, G).shape == (0, N)
    pt, st, qt = ops.w4_decode_layout_zp4(packed, scales, qzeros, G)
    say("qmatmul_int4_decode_zp4, 0 rows")
    assert ops.qmatmul_int4_decode_zp4(no_rows(K), pt, st, qt, K, G).shape == (0, N)


def test_int8_paths_take_zero_rows(ops, layer):
    w = layer[0]
    say("q8 quantize of nothing")
    assert ops.q8_quantize(torch.empty(0, device="cuda"), 32).numel() <= 1
    words = ops.q8_quantize(ops.transpose_f32(w).reshape(-1), 32)
    say("matmul_q8, 0 rows")
    assert ops.matmul_q8(no_rows(K), words, K, N, 32).shape == (0, N)
    per_channel = ops.q8_quantize(ops.transpose_f32(w).reshape(-1), K)     # one block per column
    wq, sw = ops.q8_dense_layout(per_channel, K, N, K)
    say("matmul_q8_dense, 0 rows")
    assert ops.matmul_q8_dense(no_rows(K), wq, sw).shape == (0, N)
    say("i8 quantize rows, 0 rows")
    xq, sx = ops.i8_quantize_rows(no_rows(K))
    assert xq.shape == (0, K) and sx.shape == (0,)
    wq8, sw8 = ops.i8_quantize_cols_t(w)
    say("i8 gemm, 0 rows")
    y, acc = ops.i8_gemm(xq, wq8, sx, sw8, want_acc=True)
    assert y.shape == (0, N) and acc.shape == (0, N)
    say("add_bias / transpose, 0 rows")
    assert ops.add_bias(no_rows(N), torch.ones(N, device="cuda")).shape == (0, N)
    assert ops.transpose_f32(no_rows(N)).shape == (N, 0)


def test_block_operators_take_zero_rows(ops):
    say("rmsnorm / swiglu / add, 0 rows")
    wt = torch.ones(K, device="cuda")
    assert ops.rmsnorm(no_rows(K), wt).shape == (0, K)
    assert ops.swiglu(no_rows(K), no_rows(K)).shape == (0, K)
    assert ops.swiglu_rows(no_rows(2 * K)).shape == (0, K)
    assert ops.add(no_rows(K), no_rows(K)).shape == (0, K)
    say("attention, no queries")
    q = torch.empty((1, 0, 4, 128), device="cuda")
    kv = torch.ones((1, 8, 4, 128), device="cuda")
    assert ops.attention(q, kv, kv, causal=False).shape == (1, 0, 4, 128)
    say("kv_append of no tokens leaves the cache alone")
    cache_k = torch.full((1, 16, 4, 128), 3.0, device="cuda")
    cache_v = torch.full((1, 16, 4, 128), 5.0, device="cuda")
    new = torch.empty((1, 0, 4, 128), device="cuda")
    ops.kv_append(new, new, cache_k, cache_v, 7)
    assert float(host(cache_k).min()) == 3.0 and float(host(cache_v).max()) == 5.0


def test_outputs_beside_an_empty_call_are_untouched(ops, layer):
    """A zero-row call between two real ones on the same stream changes nothing."""
    _, packed, scales, zp = layer
    rng = np.random.default_rng(12)
    x = dev(rng.normal(0, 1, (3, K)).astype(np.float32))
    say("real call, empty call, real call")
    before = host(ops.qmatmul_int4(x, packed, scales, zp, K, G))
    ops.qmatmul_int4(no_rows(K), packed, scales, zp, K, G)
    after = host(ops.qmatmul_int4(x, packed, scales, zp, K, G))
    assert np.array_equal(before, after)
