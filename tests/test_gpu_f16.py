"""GPU parity of the half-precision entry points: f16 activations in, f16 result out.

The oracle's f32 loops run on the f16-rounded activations (widening is exact); the entry points must return that
result rounded to f16 once: within the f32 tolerance of the other tests plus half an f16 ulp."""
import numpy as np
import pytest

import oracle

from gpu_util import ATOL, RTOL, dev, host, say

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from rumus_amd import ops as o
    return o


def assert_close_f16(got16, want32, what=""):
    assert got16.dtype == np.float16
    got = got16.astype(np.float32)
    # half an ulp of f16 is 2^-11 of the value (2^-25 below the normal range)
    tol = ATOL + RTOL * np.abs(want32) + np.maximum(np.abs(want32) * 2.0 ** -11, 2.0 ** -25)
    err = np.abs(got - want32)
    assert (err <= tol).all(), f"{what}: worst error {err.max()} over tolerance at {np.argmax(err - tol)}"


@pytest.mark.parametrize("m,k,n,bs", [(1, 512, 512, 512), (3, 256, 40, 64), (7, 96, 33, 12), (16, 1024, 352, 128),
                                      (70, 480, 40, 96), (300, 512, 700, 512)])
def test_matmul_q8_f16(ops, m, k, n, bs):
    say(f"matmul_q8_f16 m={m} k={k} n={n} bs={bs}")
    rng = np.random.default_rng(m * 7 + k + n)
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    a16 = rng.normal(0, 1, (m, k)).astype(np.float16)
    words = oracle.tensor_quantize(w, bs)
    want = oracle.matmul_q8(a16.astype(np.float32), words, k, n, bs, threads=8)
    got = host(ops.matmul_q8_f16(dev(a16), dev(words), k, n, bs))
    assert_close_f16(got, want, "matmul_q8_f16")
    # the same bits as the f32 entry point's result rounded to f16
    f32 = host(ops.matmul_q8(dev(a16.astype(np.float32)), dev(words), k, n, bs))
    np.testing.assert_array_equal(got, f32.astype(np.float16))


@pytest.mark.parametrize("m,k,n,g,act_order", [(1, 4096, 4096, 128, False), (1, 100, 24, 32, False), (4, 512, 352, 64, True),
                                               (16, 1024, 704, 128, False), (100, 1024, 352, 128, True),
                                               (300, 512, 256, 32, False)])
def test_qmatmul_int4_f16(ops, m, k, n, g, act_order):
    say(f"qmatmul_int4_f16 m={m} k={k} n={n} g={g} act_order={act_order}")
    rng = np.random.default_rng(m + k + n + g)
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    x16 = rng.normal(0, 1, (m, k)).astype(np.float16)
    bias = rng.normal(0, 0.01, n).astype(np.float32)
    packed, scales, zp = oracle.w4_from_f32(w, g)
    g_idx = None
    if act_order:
        padded_k, groups = oracle.w4_geometry(k, g)
        g_idx = rng.permutation(np.repeat(np.arange(groups, dtype=np.int32), g))[:k].astype(np.int32)
    want = oracle.qmatmul_int4(x16.astype(np.float32), packed, scales, zp, k, g, bias=bias, g_idx=g_idx)
    got = host(ops.qmatmul_int4_f16(dev(x16), dev(packed), dev(scales), dev(zp), k, g, bias=dev(bias),
                                    g_idx=None if g_idx is None else dev(g_idx)))
    assert_close_f16(got, want, "qmatmul_int4_f16")
    f32 = host(ops.qmatmul_int4(dev(x16.astype(np.float32)), dev(packed), dev(scales), dev(zp), k, g, bias=dev(bias),
                                g_idx=None if g_idx is None else dev(g_idx)))
    np.testing.assert_array_equal(got, f32.astype(np.float16))


def test_layers_take_f16_activations(ops):
    from rumus_amd import nn
    say("QLinear.forward and nn.matmul on f16 activations")
    rng = np.random.default_rng(9)
    k, n, g = 256, 96, 64
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    bias = rng.normal(0, 0.01, n).astype(np.float32)
    x16 = rng.normal(0, 1, (5, k)).astype(np.float16)
    layer = nn.QLinear.from_linear(nn.Linear(dev(w), dev(bias)), g)
    packed, scales, zp = oracle.w4_from_f32(w, g)
    assert_close_f16(host(layer(dev(x16))), oracle.qmatmul_int4(x16.astype(np.float32), packed, scales, zp, k, g, bias=bias))
    q8 = nn.quantize(dev(w), 64)
    assert_close_f16(host(nn.matmul(dev(x16), q8)), oracle.matmul_q8(x16.astype(np.float32), oracle.tensor_quantize(w, 64), k, n, 64))


def test_f16_overflow_and_empty(ops):
    import torch
    say("f16 entry points: a result beyond 65504 is an infinity; calls without rows or columns touch nothing")
    k, n, g = 64, 8, 32
    w = np.full((k, n), 1.0, np.float32)
    packed, scales, zp = oracle.w4_from_f32(w, g, symmetric=True)
    x16 = np.full((2, k), 2048.0, np.float16)
    x16[1] = -1.0
    want = oracle.qmatmul_int4(x16.astype(np.float32), packed, scales, zp, k, g)
    got = host(ops.qmatmul_int4_f16(dev(x16), dev(packed), dev(scales), dev(zp), k, g))
    assert want[0, 0] > 65504 and np.isinf(got[0]).all() and (got[0] > 0).all()
    assert_close_f16(got[1:], want[1:])
    empty = ops.qmatmul_int4_f16(torch.empty((0, k), dtype=torch.float16, device="cuda"), dev(packed), dev(scales), dev(zp), k, g)
    assert tuple(empty.shape) == (0, n) and empty.dtype == torch.float16
    words = oracle.tensor_quantize(w, 32)
    empty = ops.matmul_q8_f16(torch.empty((0, k), dtype=torch.float16, device="cuda"), dev(words), k, n, 32)
    assert tuple(empty.shape) == (0, n)


def test_f16_staging_reserved_then_captured_in_a_graph(ops):
    import torch
    from rumus_amd import _lib
    say("f16 entry point under HIP graph capture after reserving workspace and staging memory")
    m, k, n, g = 3, 512, 352, 128
    rng = np.random.default_rng(5)
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    packed, scales, zp = (dev(t) for t in oracle.w4_from_f32(w, g))
    x16 = dev(rng.normal(0, 1, (m, k)).astype(np.float16))
    eager = ops.qmatmul_int4_f16(x16, packed, scales, zp, k, g)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    y = torch.empty((m, n), dtype=torch.float16, device="cuda")
    with torch.cuda.stream(side):
        _lib.call("rumus_hip_workspace_reserve", side.cuda_stream, 8 << 20)
        _lib.call("rumus_hip_f16_staging_reserve", side.cuda_stream, 4 * m * (k + n) + 512)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        ops.qmatmul_int4_f16(x16, packed, scales, zp, k, g, out=y)
    for _ in range(3):
        y.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, eager)
