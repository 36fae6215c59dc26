"""Pins for the INT4 half of the CPU oracle.

The reference holds no test or fixture for this path, so the oracle is pinned
by hand-computed known answers (``tests/golden/w4_kat.json``), by invariants of
min/max quantization and by float64 / exact-integer matmuls done in numpy.
None of the expected values below is produced by re-typing the oracle's loop.
"""
import json
import os

import numpy as np
import pytest

import oracle

GOLD = os.path.join(os.path.dirname(__file__), "golden", "w4_kat.json")


def _kats():
    with open(GOLD) as f:
        return json.load(f)["cases"]


@pytest.mark.parametrize("case", _kats(), ids=lambda c: c["name"])
def test_from_f32_known_answers(case):
    w = np.array(case["w"], np.float32).reshape(case["k"], case["n"])
    packed, scales, zp = oracle.w4_from_f32(w, case["group_size"])
    assert [f"{v:08x}" for v in packed.reshape(-1)] == case["packed_hex"]
    np.testing.assert_array_equal(scales.reshape(-1), np.array(case["scales"], np.float32))
    np.testing.assert_array_equal(zp.reshape(-1), np.array(case["zp"], np.float32))


def test_from_f32_rejects_bad_group():
    with pytest.raises(ValueError):
        oracle.w4_from_f32(np.zeros((16, 4), np.float32), 12)


def test_from_f32_invariants_random():
    rng = np.random.default_rng(7)
    k, n, g = 256, 24, 64
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    packed, scales, zp = oracle.w4_from_f32(w, g)
    q = oracle.w4_unpack(packed, k).astype(np.int64)
    wg = w.reshape(k // g, g, n)
    qg = q.reshape(k // g, g, n)
    # the smallest element of each (group, column) maps to 0, the largest to 15
    amin, amax = wg.argmin(1), wg.argmax(1)
    gi, ci = np.meshgrid(np.arange(k // g), np.arange(n), indexing="ij")
    assert (qg[gi, amin, ci] == 0).all()
    assert (qg[gi, amax, ci] == 15).all()
    # scale is the spread / 15 and the dequantized value is within half a step
    np.testing.assert_allclose(scales, (wg.max(1) - wg.min(1)) / 15.0, rtol=1e-6)
    deq = (qg - zp[:, None, :].astype(np.float64)) * scales[:, None, :].astype(np.float64)
    assert (np.abs(deq - wg) <= 0.5 * scales[:, None, :] * (1 + 1e-4)).all()
    # columns are independent: quantizing one column alone gives the same words
    p1, s1, z1 = oracle.w4_from_f32(w[:, 5:6].copy(), g)
    np.testing.assert_array_equal(p1[:, 0], packed[:, 5])
    np.testing.assert_array_equal(s1[:, 0], scales[:, 5])


def test_sym_known_answers():
    # scale = max|w|/7 ; q = round_half_away(w/scale) + 8
    s = 2.0 ** -5
    col = np.array([7, -7, 0, 0.5, -0.5, 1.5, -2.5, 3], np.float32) * s
    packed, scales, zp = oracle.w4_from_f32(col.reshape(8, 1), 8, symmetric=True)
    assert scales[0, 0] == np.float32(s)
    assert zp[0, 0] == 8.0
    expect = [15, 1, 8, 9, 7, 10, 5, 11]  # ties away from zero
    assert oracle.w4_unpack(packed, 8)[:, 0].tolist() == expect
    # all-zero group: scale 1, every nibble 8
    p0, s0, _ = oracle.w4_from_f32(np.zeros((8, 1), np.float32), 8, symmetric=True)
    assert s0[0, 0] == 1.0 and p0[0, 0] == 0x88888888


def _dequant64(packed, scales, zp, k, g, g_idx=None):
    q = oracle.w4_unpack(packed, k).astype(np.float64)
    rows = (np.arange(k) // g) if g_idx is None else np.asarray(g_idx)
    return (q - zp.astype(np.float64)[rows]) * scales.astype(np.float64)[rows]


@pytest.mark.parametrize("m,k,n,g", [(1, 256, 40, 128), (5, 200, 17, 64), (16, 64, 8, 8)])
def test_qmatmul_matches_float64(m, k, n, g):
    rng = np.random.default_rng(m * 1000 + k)
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    x = rng.normal(0, 1, (m, k)).astype(np.float32)
    b = rng.normal(0, 0.01, n).astype(np.float32)
    packed, scales, zp = oracle.w4_from_f32(w, g)
    y = oracle.qmatmul_int4(x, packed, scales, zp, k, g, bias=b)
    ref = x.astype(np.float64) @ _dequant64(packed, scales, zp, k, g) + b
    np.testing.assert_allclose(y, ref, rtol=1e-3, atol=1e-4)
    # rows are independent: row 0 alone gives bit-identical output
    y0 = oracle.qmatmul_int4(x[:1], packed, scales, zp, k, g, bias=b)
    np.testing.assert_array_equal(y0[0], y[0])
    # OpenMP split over outputs does not change any bit
    y_mt = oracle.qmatmul_int4(x, packed, scales, zp, k, g, bias=b, threads=4)
    np.testing.assert_array_equal(y_mt, y)


def test_qmatmul_exact_integer_case():
    # scale 1, zp 0, small integer activations: every partial sum is an exact
    # integer below 2^24, so f32 must equal the integer matmul bit for bit.
    rng = np.random.default_rng(3)
    k, n, g, m = 128, 16, 32, 3
    q = rng.integers(0, 16, (k, n)).astype(np.uint32)
    packed = np.zeros((k // 8, n), np.uint32)
    for r in range(k):
        packed[r // 8] |= q[r] << np.uint32(4 * (r % 8))
    scales = np.ones((k // g, n), np.float32)
    zp = np.zeros((k // g, n), np.float32)
    x = rng.integers(-8, 9, (m, k)).astype(np.float32)
    y = oracle.qmatmul_int4(x, packed, scales, zp, k, g)
    np.testing.assert_array_equal(y.astype(np.int64), x.astype(np.int64) @ q.astype(np.int64))


def test_qmatmul_k_tail_ignores_padding():
    # K=20 padded to 24: nibbles of rows 20..23 must not contribute.
    rng = np.random.default_rng(11)
    k, n, g = 20, 6, 8
    w = rng.normal(0, 1, (k, n)).astype(np.float32)
    x = rng.normal(0, 1, (2, k)).astype(np.float32)
    packed, scales, zp = oracle.w4_from_f32(w, g)
    y = oracle.qmatmul_int4(x, packed, scales, zp, k, g)
    poisoned = packed.copy()
    poisoned[2] |= np.uint32(0xFFFF0000)  # rows 20..23 live in the top nibbles of word-row 2
    y2 = oracle.qmatmul_int4(x, poisoned, scales, zp, k, g)
    np.testing.assert_array_equal(y, y2)
    ref = x.astype(np.float64) @ _dequant64(packed, scales, zp, k, g)
    np.testing.assert_allclose(y, ref, rtol=1e-3, atol=1e-4)


def test_qmatmul_g_idx_extension():
    rng = np.random.default_rng(5)
    k, n, g, m = 128, 12, 32, 4
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    x = rng.normal(0, 1, (m, k)).astype(np.float32)
    packed, scales, zp = oracle.w4_from_f32(w, g, symmetric=True)
    # the trivial map reproduces the reference kernel bit for bit
    trivial = (np.arange(k) // g).astype(np.int32)
    np.testing.assert_array_equal(
        oracle.qmatmul_int4(x, packed, scales, zp, k, g, g_idx=trivial),
        oracle.qmatmul_int4(x, packed, scales, zp, k, g))
    # a scrambled map equals the float64 closed form
    g_idx = (rng.permutation(k) // g).astype(np.int32)
    y = oracle.qmatmul_int4(x, packed, scales, zp, k, g, g_idx=g_idx)
    ref = x.astype(np.float64) @ _dequant64(packed, scales, zp, k, g, g_idx)
    np.testing.assert_allclose(y, ref, rtol=1e-3, atol=1e-4)


def test_qmatmul_transpose_matches_float64():
    rng = np.random.default_rng(9)
    m, k, n, g = 3, 72, 20, 8
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    gy = rng.normal(0, 1, (m, n)).astype(np.float32)
    packed, scales, zp = oracle.w4_from_f32(w, g)
    gx = oracle.qmatmul_int4_t(gy, packed, scales, zp, k, g)
    ref = gy.astype(np.float64) @ _dequant64(packed, scales, zp, k, g).T
    np.testing.assert_allclose(gx, ref, rtol=1e-3, atol=1e-4)
    assert gx.shape == (m, k)
