"""GPU parity for the INT4 engine, through the C ABI (rumus_amd.ops -> librumus_hip.so)."""
import json
import os

import numpy as np
import pytest

import oracle
from rumus_amd import workloads

from gpu_util import assert_close, dev, host, host_u32, say

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(__file__), "golden", "w4_kat.json")


@pytest.fixture(scope="module")
def ops():
    from rumus_amd import ops as o
    return o


def test_quantize_pack_known_answers(ops):
    for case in json.load(open(GOLD))["cases"]:
        say(f"w4_quantize_pack KAT {case['name']}")
        w = np.array(case["w"], np.float32).reshape(case["k"], case["n"])
        packed, scales, zp = ops.w4_quantize_pack(dev(w), case["group_size"])
        assert [f"{v:08x}" for v in host_u32(packed).reshape(-1)] == case["packed_hex"]
        np.testing.assert_array_equal(host(scales).reshape(-1), np.array(case["scales"], np.float32))
        np.testing.assert_array_equal(host(zp).reshape(-1), np.array(case["zp"], np.float32))


@pytest.mark.parametrize("k,n,g,sym", [(256, 48, 64, False), (200, 17, 64, False), (4096, 512, 128, False),
                                       (512, 300, 128, True), (72, 5, 8, True)])
def test_quantize_pack_bit_exact(ops, k, n, g, sym):
    say(f"w4_quantize_pack k={k} n={n} g={g} sym={sym}")
    rng = np.random.default_rng(k * 7 + n)
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    w[:: max(k // 5, 1), :: max(n // 3, 1)] = 0.0
    if not sym and k >= 128:
        w[64:128, 0] = 0.02   # a constant group: range <= 1e-10 branch
    pw, sw_, zw = oracle.w4_from_f32(w, g, symmetric=sym)
    packed, scales, zp = ops.w4_quantize_pack(dev(w), g, symmetric=sym)
    np.testing.assert_array_equal(host_u32(packed), pw)
    np.testing.assert_array_equal(host(scales), sw_)
    np.testing.assert_array_equal(host(zp), zw)


def test_quantize_pack_rejects_bad_group(ops):
    say("w4_quantize_pack group_size=12")
    with pytest.raises(ops.RumusError):
        ops.w4_quantize_pack(dev(np.zeros((24, 4), np.float32)), 12)


def test_quantize_pack_non_finite_weights(ops):
    # quant.rs:69-73 compares with `<` and `>`, so a NaN never becomes min or max; `as i32`
    # (quant.rs:96) saturates and turns NaN into 0.  Cases: a NaN among finite values, +inf, -inf,
    # a group of NaNs only, and an inf whose quotient overflows the nibble range.
    say("w4_quantize_pack non-finite weights")
    nan, inf = np.float32(np.nan), np.float32(np.inf)
    cols = [
        [nan, 1, 2, 3, 0, 0, 0, 0],          # scale 0.2, zp 0 -> 0,5,10,15,0,...
        [inf, 1, 0, 0, 0, 0, 0, 0],          # scale inf, zp -0: every quotient is 0 or NaN -> 0
        [-inf, 1, 0, 0, 0, 0, 0, 0],         # scale inf, zp NaN -> 0
        [nan] * 8,                           # min stays f32::MAX, max f32::MIN: range < 0 -> scale 1, zp 0
        [nan, -3, 3, 1e30, 0, 0, 0, 0],
    ]
    w = np.array(cols, np.float32).T.copy()                 # [k = 8, n = 5]
    want = oracle.w4_from_f32(w, 8)
    assert [f"{v:08x}" for v in want[0].reshape(-1)[:4]] == ["0000fa50", "00000000", "00000000", "00000000"]
    assert want[1][0, 3] == 1.0 and want[2][0, 3] == 0.0 and np.isinf(want[1][0, 1]) and np.isnan(want[2][0, 2])
    got = ops.w4_quantize_pack(dev(w), 8)
    np.testing.assert_array_equal(host_u32(got[0]), want[0])
    for g, wv in ((host(got[1]), want[1]), (host(got[2]), want[2])):
        np.testing.assert_array_equal(np.isnan(g), np.isnan(wv))
        np.testing.assert_array_equal(g[~np.isnan(wv)].view(np.uint32), wv[~np.isnan(wv)].view(np.uint32))


SHAPES = [
    # m, k, n, g, bias
    (1, 256, 64, 128, False),     # gemv, one pass
    (1, 4096, 4096, 128, True),   # the headline decode shape
    (3, 1000, 52, 64, True),      # K tail (1000 -> 1024), n % 16 != 0
    (8, 512, 20, 8, False),       # smallest group, ragged columns
    (1, 128, 10, 32, True),       # n % 4 != 0 -> reference-order kernel
    (5, 72, 7, 8, False),         # reference-order kernel, odd everything
    (16, 512, 256, 128, True),    # m > 8: f16 MFMA kernel, one row tile
    (33, 384, 96, 64, False),     # 64-row tile with dead rows, group 64, ragged strip
    (9, 160, 40, 32, True),       # group 32, padded_k not a multiple of the 128-row stage
    (64, 1024, 1024, 128, True),
    (100, 2048, 520, 256, False), # group spans two stages
    (20, 1000, 64, 64, True),     # K tail
    (12, 256, 36, 8, False),      # group 8: not an MFMA case -> the f32 decode kernel, a few rows per launch
    (7, 512, 128, 128, True),     # 6..8 rows already take the MFMA kernel
    (16, 4096, 4096, 128, True),  # few tiles: K split 16 ways over workgroups, ordered reduction
    (40, 1001, 64, 64, False),    # k % 4 != 0: activations are copied into padded rows first
    (100, 160, 520, 32, True),    # group 32: four settlements per stage, two row tiles
    (24, 192, 48, 96, False),     # group 96 does not divide a stage -> the f32 decode kernel in row chunks
    (1536, 256, 8192, 128, True), # 384 tiles of 64 rows: four waves over 256 columns, two workgroups per CU
    (1500, 128, 8200, 64, False), # the same, group 64, ragged rows and columns
    (300, 160, 4100, 32, True),   # the same, group 32, K tail inside a stage
    (2048, 256, 8192, 128, True), # 512 tiles of 64 rows: two full rounds of eight-wave workgroups
    (1990, 192, 8200, 64, False), # 544 tiles: four-wave workgroups, group 64, ragged rows and columns
    (2100, 96, 8192, 32, True),   # 528 tiles: four-wave workgroups, group 32, K shorter than a stage
]


@pytest.mark.parametrize("m,k,n,g,with_bias", SHAPES)
def test_qmatmul_int4_vs_oracle(ops, m, k, n, g, with_bias):
    say(f"qmatmul_int4 m={m} k={k} n={n} g={g} bias={with_bias}")
    rng = np.random.default_rng(m * 131 + k + n)
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    x = rng.normal(0, 1, (m, k)).astype(np.float32)
    b = rng.normal(0, 0.01, n).astype(np.float32) if with_bias else None
    packed, scales, zp = oracle.w4_from_f32(w, g)
    want = oracle.qmatmul_int4(x, packed, scales, zp, k, g, bias=b, threads=8)
    got = host(ops.qmatmul_int4(dev(x), dev(packed), dev(scales), dev(zp), k, g,
                                bias=None if b is None else dev(b)))
    assert_close(got, want)


def test_zero_scale_group_contributes_nothing(ops):
    # the MFMA kernel keeps its accumulator in units of the current group's scale; a zero scale
    # must not poison the groups around it
    say("qmatmul_int4 zero scale")
    rng = np.random.default_rng(5)
    m, k, n, g = 16, 512, 64, 128
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    x = rng.normal(0, 1, (m, k)).astype(np.float32)
    packed, scales, zp = oracle.w4_from_f32(w, g)
    scales[1, ::2] = 0.0
    scales[3, 5] = 0.0
    want = oracle.qmatmul_int4(x, packed, scales, zp, k, g, threads=8)
    got = host(ops.qmatmul_int4(dev(x), dev(packed), dev(scales), dev(zp), k, g))
    assert np.isfinite(got).all()
    assert_close(got, want)


@pytest.mark.parametrize("m", [2, 16])
def test_non_finite_activations_poison_their_row_only(ops, m):
    # the reference accumulates a * w in f32, so a NaN activation makes its whole output row NaN
    # (NaN * 0 is NaN too) and leaves the other rows alone.  The decode kernel (m = 2) scales each
    # chunk by its largest magnitude and the MFMA kernel (m = 16) splits activations into two
    # halves: both must still deliver NaN, and both turn an infinite activation into NaN as well
    # (the reference would give an infinity where all weights of the column agree in sign).
    say(f"qmatmul_int4 non-finite activations m={m}")
    rng = np.random.default_rng(50 + m)
    k, n, g = 512, 64, 128
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    x = rng.normal(0, 1, (m, k)).astype(np.float32)
    packed, scales, zp = oracle.w4_from_f32(w, g)
    d = [dev(a) for a in (packed, scales, zp)]
    clean = host(ops.qmatmul_int4(dev(x), *d, k, g))
    for bad in (np.float32(np.nan), np.float32(np.inf)):
        xb = x.copy()
        xb[1, 300] = bad
        got = host(ops.qmatmul_int4(dev(xb), *d, k, g))
        assert np.isnan(got[1]).all()
        np.testing.assert_array_equal(np.delete(got, 1, axis=0), np.delete(clean, 1, axis=0))
    want = oracle.qmatmul_int4(np.where(np.isfinite(xb), xb, np.float32(np.nan)), packed, scales, zp, k, g)
    assert np.isnan(want[1]).all() and np.isfinite(np.delete(want, 1, axis=0)).all()


@pytest.mark.parametrize("m", [1, 5, 16, 100])
def test_weights_far_from_zero(ops, m):
    # all weights near +10: the reference's zero-point is about -10 / scale, in the thousands and
    # negative, and the zero-point term dwarfs the nibble term.  Every kernel forms
    # scale * (sum x q - zp * sum x) per group instead of the reference's per-element products.
    say(f"qmatmul_int4 offset weights m={m}")
    rng = np.random.default_rng(70 + m)
    k, n, g = 1024, 128, 128
    w = (10.0 + rng.normal(0, 0.02, (k, n))).astype(np.float32)
    w[:, 1] = -7.0 + rng.normal(0, 0.5, k)
    x = rng.normal(0, 1, (m, k)).astype(np.float32)
    packed, scales, zp = oracle.w4_from_f32(w, g)
    assert zp.min() < -1000 and zp.max() > 30
    want = oracle.qmatmul_int4(x, packed, scales, zp, k, g, threads=8)
    got = host(ops.qmatmul_int4(dev(x), dev(packed), dev(scales), dev(zp), k, g))
    # outputs reach +-500 here and some cancel to nearly zero, where abs 1e-4 is below what any f32
    # summation order can promise: measure both results against float64 in units of the terms
    # that were added up, and ask the kernels to be as accurate as the reference's own f32 loop
    wd = oracle.w4_dequant(packed, scales, zp, k, g)
    exact = x.astype(np.float64) @ wd
    terms = np.abs(x).astype(np.float64) @ np.abs(wd)
    err_ref = (np.abs(want - exact) / terms).max()
    err_got = (np.abs(got - exact) / terms).max()
    assert err_ref < 2e-6 and err_got < max(2e-7, 1.5 * err_ref), (err_got, err_ref)
    np.testing.assert_allclose(got, want, rtol=1e-3, atol=1e-3)


def test_reference_order_kernel_is_bit_exact(ops):
    # n % 4 != 0 routes to the one-thread-per-column kernel, which performs the oracle's
    # operations in the oracle's order: equality, not tolerance.
    say("qmatmul_int4 reference-order kernel bit-exact")
    rng = np.random.default_rng(17)
    m, k, n, g = 6, 200, 37, 8
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    x = rng.normal(0, 1, (m, k)).astype(np.float32)
    b = rng.normal(0, 0.01, n).astype(np.float32)
    packed, scales, zp = oracle.w4_from_f32(w, g)
    want = oracle.qmatmul_int4(x, packed, scales, zp, k, g, bias=b)
    got = host(ops.qmatmul_int4(dev(x), dev(packed), dev(scales), dev(zp), k, g, bias=dev(b)))
    np.testing.assert_array_equal(got, want)


def test_qmatmul_int4_exact_integer_case(ops):
    say("qmatmul_int4 integer special case")
    rng = np.random.default_rng(3)
    for m, k, n, g in [(1, 256, 64, 32), (16, 256, 64, 32)]:
        q = rng.integers(0, 16, (k, n)).astype(np.uint32)
        packed = np.zeros((k // 8, n), np.uint32)
        for r in range(k):
            packed[r // 8] |= q[r] << np.uint32(4 * (r % 8))
        scales = np.ones((k // g, n), np.float32)
        zp = np.zeros((k // g, n), np.float32)
        x = rng.integers(-8, 9, (m, k)).astype(np.float32)
        got = host(ops.qmatmul_int4(dev(x), dev(packed), dev(scales), dev(zp), k, g))
        np.testing.assert_array_equal(got.astype(np.int64), x.astype(np.int64) @ q.astype(np.int64))


def test_gemv_rows_match_gemm_rows_and_linearity(ops):
    say("qmatmul_int4 row independence / linearity")
    w, x = workloads.w4_gemv(1, m=4, k=1024, n=256)
    packed, scales, zp = oracle.w4_from_f32(w, 128)
    d = [dev(a) for a in (packed, scales, zp)]
    y4 = host(ops.qmatmul_int4(dev(x), *d, 1024, 128))
    y1 = host(ops.qmatmul_int4(dev(x[2:3]), *d, 1024, 128))
    assert_close(y1[0], y4[2])
    ysum = host(ops.qmatmul_int4(dev((x[0:1] + 2 * x[1:2]).astype(np.float32)), *d, 1024, 128))
    assert_close(ysum[0], y4[0] + 2 * y4[1])


@pytest.mark.parametrize("m", [1, 4, 16])
def test_act_order(ops, m):
    say(f"act-order m={m}")
    k, n, g = 512, 128, 128
    w, g_idx, x = workloads.w4_gemm_actorder(2, m=m, k=k, n=n, group_size=g)
    # symmetric zp=8 quantization of the rows as grouped by g_idx
    order = np.argsort(g_idx, kind="stable")
    ps, ss, zs = oracle.w4_from_f32(w[order], g, symmetric=True)     # sorted layout
    q_sorted = oracle.w4_unpack(ps, k)
    q = np.empty_like(q_sorted)
    q[order] = q_sorted                                             # original row order
    packed = np.zeros((k // 8, n), np.uint32)
    for r in range(k):
        packed[r // 8] |= q[r].astype(np.uint32) << np.uint32(4 * (r % 8))
    want = oracle.qmatmul_int4(x, packed, ss, zs, k, g, g_idx=g_idx, threads=8)
    # (a) g_idx passed straight to the reference-order kernel: bit-exact
    got_direct = host(ops.qmatmul_int4(dev(x), dev(packed), dev(ss), dev(zs), k, g, g_idx=dev(g_idx)))
    np.testing.assert_array_equal(got_direct, want)
    # (b) prepared once, then the fast kernels with a permuted activation gather
    p_sorted, perm = ops.w4_actorder_prepare(dev(packed), dev(g_idx), g)
    np.testing.assert_array_equal(host(perm), order.astype(np.int32))
    np.testing.assert_array_equal(host_u32(p_sorted), ps)
    got = host(ops.qmatmul_int4_perm(dev(x), p_sorted, dev(ss), dev(zs), k, g, perm=perm))
    assert_close(got, want)
    # (c) the trivial map reproduces the plain kernel bit for bit
    trivial = (np.arange(k) // g).astype(np.int32)
    pt, permt = ops.w4_actorder_prepare(dev(ps), dev(trivial), g)
    np.testing.assert_array_equal(host(permt), np.arange(k, dtype=np.int32))
    a = host(ops.qmatmul_int4_perm(dev(x), pt, dev(ss), dev(zs), k, g, perm=permt))
    b = host(ops.qmatmul_int4(dev(x), dev(ps), dev(ss), dev(zs), k, g))
    np.testing.assert_array_equal(a, b)


def test_act_order_rejects_unbalanced_groups(ops):
    say("act-order unbalanced g_idx")
    k, n, g = 64, 8, 32
    bad = np.zeros(k, np.int32)
    with pytest.raises(ops.RumusError):
        ops.w4_actorder_prepare(dev(np.zeros((k // 8, n), np.uint32)), dev(bad), g)


@pytest.mark.parametrize("m,k,n,g", [(3, 72, 20, 8), (16, 512, 300, 128), (1, 1000, 64, 64),
                                     # from 8 rows on and group % 128 == 0: the f16 matrix cores
                                     (8, 256, 64, 128),
                                     (64, 4096, 1100, 128),     # n shared over workgroups
                                     (130, 1000, 264, 128),     # k ends inside the last group, three row tiles
                                     (100, 256, 4100, 256),     # n ends 4 past a step of 32
                                     (2050, 256, 516, 128),     # many row tiles
                                     (16, 128, 4, 128),         # the smallest n
                                     (40, 512, 300, 64),        # groups of 64: two waves per workgroup
                                     (70, 256, 132, 32),        # groups of 32: one
                                     (300, 200, 64, 32),        # k ends inside a group of 32
                                     (9, 96, 40, 16),           # other group sizes: the vector kernel, four rows per pass
                                     (1, 4096, 1100, 128), (2, 1000, 68, 64), (4, 11008, 260, 128),   # two word rows per workgroup
                                     (7, 520, 36, 32), (12, 4104, 64, 128),   # k ends inside the last word row pair
                                     (5, 72, 22, 8), (3, 256, 50, 128)])    # n % 4 != 0, groups of 8: scalar loads
def test_qmatmul_int4_transpose(ops, m, k, n, g):
    say(f"qmatmul_int4_t m={m} k={k} n={n} g={g}")
    rng = np.random.default_rng(k + n)
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    gy = rng.normal(0, 1, (m, n)).astype(np.float32)
    packed, scales, zp = oracle.w4_from_f32(w, g)
    want = oracle.qmatmul_int4_t(gy, packed, scales, zp, k, g, threads=8)
    got = host(ops.qmatmul_int4_t(dev(gy), dev(packed), dev(scales), dev(zp), k, g))
    assert got.shape == (m, k)
    assert_close(got, want)


def test_qmatmul_int4_transpose_scaling_and_non_finite_rows(ops):
    # the matrix-core grad_x rescales every row of grad_y and the scales by powers of two: rows of very
    # different magnitude, tiny and huge scales, a zero row; inf / nan poison their own row only
    say("qmatmul_int4_t row scaling")
    rng = np.random.default_rng(11)
    m, k, n, g = 48, 256, 520, 128
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    w[:, :100] *= 1e-4                                       # scales over four decades
    w[:, 100:200] *= 50.0
    w[:128, 200:230] += 3.0                                  # weights far from zero: zero-points near -300
    w[:128, 230:240] = 1.0 + 1e-5 * w[:128, 230:240]         # and beyond -1000
    gy = rng.normal(0, 1, (m, n)).astype(np.float32)
    gy[1] *= 1e-12
    gy[2] *= 1e9
    gy[3, 7] = 2.0e4                                         # dwarfs the rest of its row
    gy[4] = 0.0
    packed, scales, zp = oracle.w4_from_f32(w, g)
    d = [dev(a) for a in (packed, scales, zp)]
    want = oracle.qmatmul_int4_t(gy, packed, scales, zp, k, g, threads=8)
    got = host(ops.qmatmul_int4_t(dev(gy), *d, k, g))
    # judged in units of the summed terms, like the forward kernels with wide-ranging operands
    deq = oracle.w4_dequant(packed, scales, zp, k, g).astype(np.float64)          # [k, n]
    exact = gy.astype(np.float64) @ deq.T
    terms = np.abs(gy).astype(np.float64) @ np.abs(deq).T + 1e-300
    assert (np.abs(want - exact) / terms).max() < 2e-6                            # the f32 loop itself
    assert (np.abs(got - exact) / terms).max() < 2e-6
    np.testing.assert_array_equal(got[4], np.zeros(k, np.float32))
    for bad in (np.float32(np.nan), np.float32(np.inf)):
        gb = gy.copy()
        gb[9, 33] = bad
        out = host(ops.qmatmul_int4_t(dev(gb), *d, k, g))
        assert np.isnan(out[9]).all()
        np.testing.assert_array_equal(np.delete(out, 9, axis=0), np.delete(got, 9, axis=0))
    # the same rows, few enough for the vector kernel (scale and zero-point applied per column: sum t q - sum t zp)
    few = host(ops.qmatmul_int4_t(dev(gy[:6]), *d, k, g))
    assert (np.abs(few - exact[:6]) / terms[:6]).max() < 2e-6
    np.testing.assert_array_equal(few[4], np.zeros(k, np.float32))
    for bad in (np.float32(np.nan), np.float32(np.inf)):
        gb = gy[:6].copy()
        gb[2, 33] = bad
        out = host(ops.qmatmul_int4_t(dev(gb), *d, k, g))
        assert np.isnan(out[2]).all()
        np.testing.assert_array_equal(np.delete(out, 2, axis=0), np.delete(few, 2, axis=0))


def test_gptq_actorder_config_full_size(ops):
    # benchmark configuration: M=16 and M=128, K=4096, N=11008, g128, symmetric zp=8, act-order g_idx
    for m in (16, 128):
        say(f"w4 gemm act-order {m}x4096x11008")
        k, n, g = 4096, 11008, 128
        w, g_idx, x = workloads.w4_gemm_actorder(0, m=m, k=k, n=n, group_size=g)
        order = np.argsort(g_idx, kind="stable")
        ps, ss, zs = oracle.w4_from_f32(w[order], g, symmetric=True)         # groups contiguous
        rows = slice(0, m) if m == 16 else [0, 1, 63, 64, 127]               # oracle rows (CPU time)
        xs = x[rows]
        want = oracle.qmatmul_int4(np.ascontiguousarray(xs[:, order]), ps, ss, zs, k, g, threads=8)
        got = host(ops.qmatmul_int4_perm(dev(x), dev(ps), dev(ss), dev(zs), k, g,
                                         perm=dev(order.astype(np.int32))))
        assert_close(got[rows], want)
        # every row through a size-independent property: linearity, y(2x) == 2 y(x)
        got2 = host(ops.qmatmul_int4_perm(dev((2 * x).astype(np.float32)), dev(ps), dev(ss), dev(zs), k, g,
                                          perm=dev(order.astype(np.int32))))
        assert_close(got2, 2 * got)


def test_qlinear_module_mirror(ops):
    say("QLinear.from_linear / forward")
    from rumus_amd import nn
    rng = np.random.default_rng(21)
    k, n, m, g = 512, 256, 4, 128
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    b = rng.normal(0, 0.01, n).astype(np.float32)
    x = rng.normal(0, 1, (m, k)).astype(np.float32)
    ql = nn.QLinear.from_linear(nn.Linear(dev(w), dev(b)), g)
    assert (ql.in_features, ql.out_features) == (k, n)
    assert (ql.weight.padded_k, ql.weight.num_groups) == (512, 4)
    packed, scales, zp = oracle.w4_from_f32(w, g)
    np.testing.assert_array_equal(host_u32(ql.weight.packed_tensor), packed)
    assert_close(host(ql.forward(dev(x))), oracle.qmatmul_int4(x, packed, scales, zp, k, g, bias=b))
    gy = rng.normal(0, 1, (m, n)).astype(np.float32)
    assert_close(host(ql.backward_input(dev(gy))), oracle.qmatmul_int4_t(gy, packed, scales, zp, k, g))
    with pytest.raises(ValueError):
        nn.QuantizedTensor.from_f32(dev(w), k, n, 12)
    # without the second (tile-major) copy of the weight: the same rows through the reference's arrays, same bits
    with_copy = host(ql.forward(dev(x)))
    assert ql.weight.decode is not None
    ql.weight.drop_decode_layout()
    assert ql.weight.decode is None
    np.testing.assert_array_equal(host(ql.forward(dev(x))), with_copy)


def test_headline_shape_properties(ops):
    # full benchmark size: compare with the oracle (all host cores) and check linearity
    say("w4 gemv 1x4096x4096 g128 full size")
    w, x = workloads.w4_gemv(0)
    pw, sw_, zw = oracle.w4_from_f32(w, 128)
    packed, scales, zp = ops.w4_quantize_pack(dev(w), 128)
    np.testing.assert_array_equal(host_u32(packed), pw)
    np.testing.assert_array_equal(host(scales), sw_)
    np.testing.assert_array_equal(host(zp), zw)
    y = host(ops.qmatmul_int4(dev(x), packed, scales, zp, 4096, 128))
    assert_close(y, oracle.qmatmul_int4(x, pw, sw_, zw, 4096, 128, threads=8))
    y2 = host(ops.qmatmul_int4(dev((-0.5 * x).astype(np.float32)), packed, scales, zp, 4096, 128))
    assert_close(y2, -0.5 * y)


def test_workspace_reserved_then_captured_in_a_graph(ops):
    # K-split GEMM inside a HIP graph: the workspace is reserved on the capture stream first
    # (the library must not allocate while capturing); every replay, with eager work in
    # between, must reproduce the eager result bit for bit (fixed-order reduction).
    say("qmatmul_int4 workspace + graph replay")
    import torch
    from rumus_amd import _lib
    rng = np.random.default_rng(11)
    m, k, n, g = 16, 1024, 512, 128
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    packed, scales, zp = oracle.w4_from_f32(w, g)
    d = [dev(a) for a in (packed, scales, zp)]
    g_idx = (rng.permutation(k) // g).astype(np.int32)
    ps, perm = ops.w4_actorder_prepare(d[0], dev(g_idx), g)
    xs = [dev(rng.normal(0, 1, (m, k)).astype(np.float32)) for _ in range(3)]
    x = torch.empty_like(xs[0])
    y = torch.empty((m, n), dtype=torch.float32, device="cuda")
    eager = []
    for xi in xs:
        eager.append(host(ops.qmatmul_int4_perm(xi, ps, d[1], d[2], k, g, perm=perm)))
    side = torch.cuda.Stream()
    _lib.call("rumus_hip_workspace_reserve", side.cuda_stream, (m * k + 16 * m * n) * 4 + 256)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        ops.qmatmul_int4_perm(x, ps, d[1], d[2], k, g, perm=perm, out=y)
    for xi, want in zip(xs, eager):
        x.copy_(xi)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        np.testing.assert_array_equal(host(y), want)
        # eager work between replays, on the default stream
        np.testing.assert_array_equal(host(ops.qmatmul_int4_perm(xi, ps, d[1], d[2], k, g, perm=perm)), want)
    # without a reservation a capture on a fresh stream is refused with a clear error
    fresh = torch.cuda.Stream()
    g2 = torch.cuda.CUDAGraph()
    with pytest.raises(Exception, match="workspace"):
        with torch.cuda.graph(g2, stream=fresh):
            ops.qmatmul_int4_perm(x, ps, d[1], d[2], k, g, perm=perm, out=y)


# ---- AWQ storage: integer zero-points, eight per word along n -------------------------------

@pytest.mark.parametrize("k,n,g", [(16, 8, 16), (200, 24, 64), (4096, 4096, 128), (1000, 264, 8)])
def test_awq_quantize_pack_bit_exact(ops, k, n, g):
    say(f"w4_quantize_pack_awq k={k} n={n} g={g}")
    rng = np.random.default_rng(k + n + g)
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    w[:, 3] = np.abs(w[:, 3])        # zero-point clamps to 0
    w[:, 5] = 0.02                   # constant column: range clamps to 1e-5
    want = oracle.w4_awq_from_f32(w, g)
    got = ops.w4_quantize_pack_awq(dev(w), g)
    np.testing.assert_array_equal(host_u32(got[0]), want[0])
    np.testing.assert_array_equal(host(got[1]), want[1])
    np.testing.assert_array_equal(host_u32(got[2]), want[2])


def test_awq_rejects_bad_shapes(ops):
    from rumus_amd._lib import RumusError
    with pytest.raises(RumusError):
        ops.w4_quantize_pack_awq(dev(np.zeros((16, 12), np.float32)), 8)      # n % 8 != 0
    with pytest.raises(RumusError):
        ops.w4_quantize_pack_awq(dev(np.zeros((24, 8), np.float32)), 12)      # group % 8 != 0


@pytest.mark.parametrize("m,k,n,g,with_bias", [
    (1, 4096, 4096, 128, True),     # decode kernel, the benchmark storage (u4 zero-points) to the letter
    (4, 1024, 264, 64, False),      # decode kernel, n % 16 != 0
    (3, 200, 24, 8, True),          # group 8 -> reference-order kernel
    (16, 4096, 4096, 128, True),    # MFMA kernel, K split
    (70, 512, 520, 32, False),      # MFMA kernel, group 32
    (300, 256, 8192, 128, True),    # MFMA kernel, eight-wave 64-row tiles
    (1536, 128, 8192, 128, False),  # MFMA kernel, four-wave 64-row tiles (384 tiles: a poorly filled second round)
])
def test_qmatmul_int4_zp4_vs_oracle(ops, m, k, n, g, with_bias):
    say(f"qmatmul_int4_zp4 m={m} k={k} n={n} g={g}")
    rng = np.random.default_rng(m * 7 + k + n)
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    x = rng.normal(0, 1, (m, k)).astype(np.float32)
    b = rng.normal(0, 0.01, n).astype(np.float32) if with_bias else None
    packed, scales, qzeros = oracle.w4_awq_from_f32(w, g)
    zp = oracle.w4_qzeros_unpack(qzeros, n)
    want = oracle.qmatmul_int4(x, packed, scales, zp, k, g, bias=b, threads=8)
    got = host(ops.qmatmul_int4_zp4(dev(x), dev(packed), dev(scales), dev(qzeros), k, g,
                                    bias=None if b is None else dev(b)))
    assert_close(got, want)
    # the packed zero-points and their f32 expansion are the same numbers: the two entry points
    # must agree bit for bit (same kernels, same arithmetic)
    same = host(ops.qmatmul_int4(dev(x), dev(packed), dev(scales), dev(zp), k, g,
                                 bias=None if b is None else dev(b)))
    if g % 32 == 0:
        np.testing.assert_array_equal(got, same)
    else:
        assert_close(got, same)


def test_zp4_act_order(ops):
    say("qmatmul_int4_zp4 with perm")
    rng = np.random.default_rng(33)
    m, k, n, g = 16, 512, 64, 128
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    x = rng.normal(0, 1, (m, k)).astype(np.float32)
    perm = rng.permutation(k).astype(np.int32)
    # a weight whose rows are already in act-order: sorted row j multiplies x[:, perm[j]]
    packed, scales, qzeros = oracle.w4_awq_from_f32(w, g)
    zp = oracle.w4_qzeros_unpack(qzeros, n)
    want = oracle.qmatmul_int4(x[:, perm], packed, scales, zp, k, g, threads=8)
    got = host(ops.qmatmul_int4_zp4(dev(x), dev(packed), dev(scales), dev(qzeros), k, g, perm=dev(perm)))
    assert_close(got, want)


# ---- decode layout: tile-major copies of the weight arrays -----------------------------------

@pytest.mark.parametrize("m,k,n,g", [(1, 4096, 4096, 128), (3, 1000, 48, 64), (8, 512, 11008, 32), (5, 256, 16, 256)])
def test_decode_layout_is_bit_identical(ops, m, k, n, g):
    say(f"qmatmul_int4_decode m={m} k={k} n={n} g={g}")
    rng = np.random.default_rng(m + k + n)
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    x = rng.normal(0, 1, (m, k)).astype(np.float32)
    b = rng.normal(0, 0.01, n).astype(np.float32)
    packed, scales, zp = oracle.w4_from_f32(w, g)
    d = [dev(a) for a in (packed, scales, zp)]
    pt, st, zt = ops.w4_decode_layout(*d, g)
    # the layout itself: tile c holds columns 16c .. 16c+15 of every row, row-major
    want_pt = packed.reshape(packed.shape[0], n // 16, 16).transpose(1, 0, 2).reshape(-1)
    np.testing.assert_array_equal(host_u32(pt).reshape(-1), want_pt)
    want_st = scales.reshape(scales.shape[0], n // 16, 16).transpose(1, 0, 2).reshape(-1)
    np.testing.assert_array_equal(host(st).reshape(-1), want_st)
    got = host(ops.qmatmul_int4_decode(dev(x), pt, st, zt, k, g, bias=dev(b)))
    assert_close(got, oracle.qmatmul_int4(x, packed, scales, zp, k, g, bias=b, threads=8))
    if m <= ops.qmatmul_int4_decode_max_rows(packed.shape[0] * 8, n):   # the row-major entry point runs the same kernel then
        np.testing.assert_array_equal(got, host(ops.qmatmul_int4(dev(x), *d, k, g, bias=dev(b))))


@pytest.mark.parametrize("m,k,n,g", [(1, 4096, 4096, 128), (3, 1000, 48, 64), (8, 512, 11008, 32), (5, 256, 16, 256),
                                     # one row: 256-thread workgroups, 64 rows per quad (groups of 64 and up)
                                     (1, 1000, 48, 64), (1, 11008, 272, 128), (1, 520, 16, 256), (1, 512, 64, 32)])
def test_decode_layout_u4_zero_points(ops, m, k, n, g):
    say(f"qmatmul_int4_decode_zp4 m={m} k={k} n={n} g={g}")
    rng = np.random.default_rng(m + k + n + 1)
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    x = rng.normal(0, 1, (m, k)).astype(np.float32)
    b = rng.normal(0, 0.01, n).astype(np.float32)
    packed, scales, qzeros = oracle.w4_awq_from_f32(w, g)
    d = [dev(a) for a in (packed, scales, qzeros)]
    pt, st, qt = ops.w4_decode_layout_zp4(*d, g)
    # the zero-point layout itself: the two words of a tile's 16 columns side by side per group
    want_qt = qzeros.reshape(qzeros.shape[0], n // 16, 2).transpose(1, 0, 2).reshape(-1)
    np.testing.assert_array_equal(host_u32(qt).reshape(-1), want_qt)
    got = host(ops.qmatmul_int4_decode_zp4(dev(x), pt, st, qt, k, g, bias=dev(b)))
    zp = oracle.w4_qzeros_unpack(qzeros, n)
    assert_close(got, oracle.qmatmul_int4(x, packed, scales, zp, k, g, bias=b, threads=8))
    # the row-major entry point runs the same kernel arithmetic then (one row on groups of 64 and up takes 64 rows
    # per quad on the tile-major copy: another fixed-point scale per chunk, so close but not the same bits)
    if m <= ops.qmatmul_int4_decode_max_rows(packed.shape[0] * 8, n) and not (m == 1 and g % 64 == 0):
        np.testing.assert_array_equal(got, host(ops.qmatmul_int4_zp4(dev(x), *d, k, g, bias=dev(b))))
    # act-order on top
    if k % g == 0:
        perm = rng.permutation(k).astype(np.int32)
        got_p = host(ops.qmatmul_int4_decode_zp4(dev(x), pt, st, qt, k, g, perm=dev(perm)))
        assert_close(got_p, oracle.qmatmul_int4(np.ascontiguousarray(x[:, perm]), packed, scales, zp, k, g, threads=8))


def test_decode_layout_rejects_bad_arguments(ops):
    from rumus_amd._lib import RumusError
    import torch
    p = torch.zeros((16, 24), dtype=torch.int32, device="cuda")
    s = torch.zeros((1, 24), dtype=torch.float32, device="cuda")
    with pytest.raises(RumusError):
        ops.w4_decode_layout(p, s, s, 128)                       # n % 16 != 0
    p = torch.zeros((16, 32), dtype=torch.int32, device="cuda")
    s = torch.zeros((1, 32), dtype=torch.float32, device="cuda")
    x = torch.zeros((9, 128), dtype=torch.float32, device="cuda")
    with pytest.raises(RumusError):
        ops.qmatmul_int4_decode(x, p, s, s, 128, 128)            # more than 8 rows
