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


def test_awq_known_answers():
    # Column c holds (k - c) * 2^-6 for k = 0..15: min = -c*s, max = (15-c)*s, so scale = s exactly,
    # zero-point = c, q[k] = k.  qzeros packs column c in bits 4*c.
    s = np.float32(2.0 ** -6)
    w = np.stack([(np.arange(16) - c) * s for c in range(8)], axis=1).astype(np.float32)
    packed, scales, qzeros = oracle.w4_awq_from_f32(w, 16)
    np.testing.assert_array_equal(scales, np.full((1, 8), s, np.float32))
    np.testing.assert_array_equal(qzeros, np.array([[0x76543210]], np.uint32))
    np.testing.assert_array_equal(packed, np.tile(np.array([[0x76543210], [0xFEDCBA98]], np.uint32), (1, 8)))
    np.testing.assert_array_equal(oracle.w4_qzeros_unpack(qzeros, 8), np.arange(8, dtype=np.float32)[None, :])
    # ties go to even (AutoAWQ rounds with torch.round): 0, 15s, 2.5s, 0.5s, 3.5s -> 2, 0, 4
    w = np.zeros((8, 8), np.float32)
    w[:5, 0] = np.array([0, 15, 2.5, 0.5, 3.5], np.float32) * s
    packed, scales, qzeros = oracle.w4_awq_from_f32(w, 8)
    assert scales[0, 0] == s and (qzeros[0, 0] & 0xF) == 0
    assert [(int(packed[0, 0]) >> (4 * j)) & 0xF for j in range(5)] == [0, 15, 2, 0, 4]
    # a constant group: range clamps to 1e-5, zero-point 0, everything saturates at 15
    w = np.full((8, 8), 0.02, np.float32)
    packed, scales, qzeros = oracle.w4_awq_from_f32(w, 8)
    assert scales[0, 0] == np.float32(1e-5) / np.float32(15) and qzeros[0, 0] == 0 and packed[0, 0] == 0xFFFFFFFF
    with pytest.raises(ValueError):
        oracle.w4_awq_from_f32(np.zeros((8, 4), np.float32), 8)       # n % 8 != 0


def test_awq_matches_vectorised_formula_and_bounds():
    rng = np.random.default_rng(21)
    k, n, g = 200, 24, 64
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    w[:, 3] = np.abs(w[:, 3])                       # all positive: zero-point clamps to 0
    packed, scales, qzeros = oracle.w4_awq_from_f32(w, g)
    pk, G = oracle.w4_geometry(k, g)
    wp = np.zeros((pk, n), np.float32)
    wp[:k] = w
    wg = wp.reshape(G, g, n)
    mn, mx = wg.min(1), wg.max(1)
    sc = (np.maximum(mx - mn, np.float32(1e-5)) / np.float32(15)).astype(np.float32)
    z = np.clip(-np.rint(mn / sc), 0, 15)
    q = np.clip(np.rint(wg / sc[:, None, :]) + z[:, None, :], 0, 15).astype(np.uint32).reshape(pk, n)
    np.testing.assert_array_equal(scales, sc)
    np.testing.assert_array_equal(oracle.w4_qzeros_unpack(qzeros, n), z.astype(np.float32))
    np.testing.assert_array_equal(oracle.w4_unpack(packed, pk), q.astype(np.uint8))
    # dequantised error is at most half a step wherever the zero-point did not clamp
    deq = (q.astype(np.float32).reshape(G, g, n) - z[:, None, :]) * sc[:, None, :]
    free = (mn <= 0) & (mx >= 0)
    err = np.abs(deq - wg).max(1)
    assert (err[free] <= sc[free] * 0.5001).all()
