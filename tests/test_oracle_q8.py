"""Pins for the INT8 half of the CPU oracle.

Known answers (``tests/golden/q8_kat.json``) fix the rounding mode, the zero
block rule and the byte/header layout; numpy's own float16 fixes the header
conversion; numpy integer matmuls fix the i32 GEMM.
"""
import json
import os

import numpy as np
import pytest

import oracle

GOLD = os.path.join(os.path.dirname(__file__), "golden", "q8_kat.json")


def _kats():
    with open(GOLD) as f:
        return json.load(f)["cases"]


def _bytes_of(words):
    return np.asarray(words, np.uint32).view(np.int8)


@pytest.mark.parametrize("case", _kats(), ids=lambda c: c["name"])
def test_q8_quantize_known_answers(case):
    x = np.array(case["x"], np.float32)
    bs = case["block_size"]
    words = oracle.q8_quantize(x, bs)
    assert words.size == 1 + bs // 4                       # header word + data words
    assert f"{words[0]:08x}" == case["header_hex"]
    assert _bytes_of(words[1:]).tolist() == case["q"]       # little-endian bytes, element order
    # the W8A8 row quantizer is the same formula with an f32 scale
    xq, s = oracle.i8_quantize_rows(x.reshape(1, -1))
    assert xq[0].tolist() == case["q"]
    amax = np.abs(x).max()
    assert s[0] == (np.float32(1.0) if amax == 0 else np.float32(amax) / np.float32(127))


def test_q8_buffer_sizes():
    # num_blocks * (4 + bs), rounded up to 4 bytes (tensor/core.rs:87-98)
    assert oracle.q8_buf_size(512 * 512, 512) == 512 * 516
    assert oracle.q8_buf_size(4096 * 11008, 4096) == 11008 * 4100
    assert oracle.q8_buf_size(10, 4) == 3 * 8
    assert oracle.q8_stride_words(128) == 33
    with pytest.raises(ValueError):
        oracle.q8_quantize(np.zeros(8, np.float32), 6)


def test_f16_conversion_matches_numpy():
    rng = np.random.default_rng(0)
    vals = np.concatenate([
        rng.normal(0, 1, 4000), rng.normal(0, 1e-4, 4000), rng.normal(0, 1e-7, 2000),
        rng.normal(0, 3e4, 2000),
        [0.0, -0.0, 1.0, 65504.0, 65519.9, 65520.0, 2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0001,
         1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11, 2.0 ** -14, 2.0 ** -14 - 2.0 ** -25],
    ]).astype(np.float32)
    lib = oracle.lib()
    got = np.array([lib.orc_f32_to_f16_bits(float(v)) for v in vals], np.uint16)
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    np.testing.assert_array_equal(got, want)
    halves = np.arange(0, 0x7C00, 7, dtype=np.uint16)
    back = np.array([lib.orc_f16_bits_to_f32(int(h)) for h in halves], np.float32)
    np.testing.assert_array_equal(back, halves.view(np.float16).astype(np.float32))


def test_q8_quantize_invariants_and_tail():
    rng = np.random.default_rng(1)
    bs, numel = 64, 64 * 5 + 20                   # last block is partial
    x = rng.normal(0, 0.02, numel).astype(np.float32)
    words = oracle.q8_quantize(x, bs)
    stride = oracle.q8_stride_words(bs)
    assert words.size == 6 * stride
    blocks = words.reshape(6, stride)
    q = _bytes_of(np.ascontiguousarray(blocks[:, 1:])).reshape(6, bs).astype(np.int32)
    assert (np.abs(q[:5]).max(1) == 127).all()   # the abs-max element hits +-127
    assert q.min() >= -127                        # -128 is unreachable
    assert (q[5, 20:] == 0).all()                 # out-of-range elements pack as 0
    assert (blocks[:, 0] >> 16 == 0).all()        # upper half of the header is padding
    # independent formula in numpy float32 (rint = half-even)
    xb = np.zeros(6 * bs, np.float32)
    xb[:numel] = x
    xb = xb.reshape(6, bs)
    amax = np.abs(xb).max(1, keepdims=True)
    want = np.rint(xb * (np.float32(127) / amax)).astype(np.int32)
    np.testing.assert_array_equal(q, want)
    np.testing.assert_array_equal(
        (blocks[:, 0] & 0xFFFF).astype(np.uint16),
        (amax[:, 0] / np.float32(127)).astype(np.float16).view(np.uint16))


def test_q8_dequantize_exact():
    rng = np.random.default_rng(2)
    bs, numel = 32, 32 * 7
    x = rng.normal(0, 1, numel).astype(np.float32)
    words = oracle.q8_quantize(x, bs)
    deq = oracle.q8_dequantize(words, numel, bs)
    blocks = words.reshape(7, oracle.q8_stride_words(bs))
    q = _bytes_of(np.ascontiguousarray(blocks[:, 1:])).reshape(7, bs).astype(np.float32)
    sc = (blocks[:, 0] & 0xFFFF).astype(np.uint16).view(np.float16).astype(np.float32)
    np.testing.assert_array_equal(deq, (q * sc[:, None]).reshape(-1))
    assert np.abs(deq - x).max() <= np.abs(x).max() / 127 * 0.51 + 1e-3 * np.abs(x).max()


@pytest.mark.parametrize("m,k,n,bs", [(4, 64, 10, 64), (3, 96, 7, 32), (2, 40, 5, 8)])
def test_matmul_q8_matches_float64(m, k, n, bs):
    rng = np.random.default_rng(k + n)
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    a = rng.normal(0, 1, (m, k)).astype(np.float32)
    words = oracle.tensor_quantize(w, bs)
    c = oracle.matmul_q8(a, words, k, n, bs)
    # dequantized weight, put back in [K,N] order (the Q8 buffer is [N,K] blocked)
    wd = oracle.q8_dequantize(words, k * n, bs).reshape(n, k).T.astype(np.float64)
    np.testing.assert_allclose(c, a.astype(np.float64) @ wd, rtol=1e-3, atol=1e-4)
    assert np.abs(wd - w).max() <= np.abs(w).max() / 127
    np.testing.assert_array_equal(oracle.matmul_q8(a, words, k, n, bs, threads=3), c)


def test_matmul_q8_exact_integer_case():
    # every column's abs-max is 127 -> header scale is exactly 1.0, q == w
    rng = np.random.default_rng(4)
    k, n, m, bs = 64, 9, 3, 32
    w = rng.integers(-126, 127, (k, n)).astype(np.float32)
    w[0, :] = 127
    w[bs, :] = -127
    a = rng.integers(-4, 5, (m, k)).astype(np.float32)
    words = oracle.tensor_quantize(w, bs)
    c = oracle.matmul_q8(a, words, k, n, bs)
    np.testing.assert_array_equal(c.astype(np.int64), a.astype(np.int64) @ w.astype(np.int64))


def test_add_bias_exact():
    rng = np.random.default_rng(6)
    mat = rng.normal(0, 1, (5, 9)).astype(np.float32)
    b = rng.normal(0, 1, 9).astype(np.float32)
    np.testing.assert_array_equal(oracle.add_bias(mat, b), mat + b[None, :])


def test_i8_gemm_bit_exact_vs_numpy_int():
    rng = np.random.default_rng(8)
    m, k, n = 9, 200, 13
    xq = rng.integers(-127, 128, (m, k)).astype(np.int8)
    wq = rng.integers(-127, 128, (n, k)).astype(np.int8)
    acc = oracle.i8_gemm_i32(xq, wq)
    np.testing.assert_array_equal(acc, xq.astype(np.int64) @ wq.astype(np.int64).T)
    np.testing.assert_array_equal(oracle.i8_gemm_i32(xq, wq, threads=4), acc)
    # extreme values stay inside int32 at K=4096: 4096*127*127 < 2^31
    assert 4096 * 127 * 127 < 2 ** 31


def test_i8_linear_close_to_f32_linear():
    from rumus_amd import workloads
    w, x, b = workloads.int8_linear(0)
    y, acc, (xq, sx, wq, sw) = oracle.i8_linear(x, w, b)
    assert wq.shape == (512, 512) and sw.shape == (512,) and sx.shape == (32,)
    # closed form in float64 from the integer accumulators
    want = acc.astype(np.float64) * sx[:, None].astype(np.float64) * sw[None, :] + b
    np.testing.assert_allclose(y, want, rtol=1e-5, atol=1e-6)
    # and the whole thing approximates the f32 Linear it replaces
    full = x.astype(np.float64) @ w.astype(np.float64) + b
    assert np.abs(y - full).max() < 0.05 * np.abs(full).max()
