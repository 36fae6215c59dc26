"""Forward INT4 matmul beyond 128 rows (f16 matrix cores) on rows of very different magnitude."""
import numpy as np
import pytest
import torch

import oracle
from gpu_util import dev, host, say

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from rumus_amd import ops as o
    return o


# the workgroup shapes of the f16 kernel: 32-row tiles that convert x themselves (plain, through the gathered copy,
# ragged), 64-row tiles on pre-converted planes (gathered through LDS, 128-bit reads, element-wise reads), and their
# four-wave form; the last two: more steps of K per thread of the kernel that converts plain x from registers
@pytest.mark.parametrize("m,k,n,g,act_order", [(160, 512, 1024, 128, False), (520, 1024, 1536, 128, False),
                                               (300, 512, 512, 64, True), (136, 520, 516, 32, False),
                                               (600, 1024, 2048, 128, True), (600, 1024, 2048, 128, False),
                                               (600, 1028, 2048, 128, False), (1024, 256, 11008, 128, False),
                                               (600, 8192, 2048, 128, False), (600, 14336, 2048, 128, False)])
def test_rows_of_any_magnitude(ops, m, k, n, g, act_order):
    """Batches beyond 128 rows split x into two f16 planes: every row is first scaled by a power of two into
    f16's range, so rows of 1e-12, rows of 1e9 and a row with one element of 2e5 (beyond f16's 65504) come
    out as accurate as ordinary ones, in units of the summed terms (for the dominated row: plus half a quantization
    step per term); multiplying x by 2^40 multiplies y by 2^40 exactly; an infinity or a NaN poisons its own row only."""
    say(f"w4 forward row scaling m={m} k={k} n={n} g={g} act_order={act_order}")
    rng = np.random.default_rng(m + n)
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    x = rng.normal(0, 1, (m, k)).astype(np.float32)
    x[1] *= 1e-12
    x[2] *= 1e9
    x[3, 7] = 2.0e5
    x[4] = 0.0
    x[5] *= 1e-30
    x[6] *= 3e33
    packed, scales, zp = oracle.w4_from_f32(w, g)
    padded_k = packed.shape[0] * 8
    d = [dev(a) for a in (packed, scales, zp)]
    perm = None
    if act_order:
        assert padded_k == k
        perm_np = rng.permutation(k).astype(np.int32)
        perm = dev(perm_np)
        xs = x[:, perm_np]                                   # what the kernel multiplies with the (sorted) rows
    else:
        xs = x
    call = (lambda t: ops.qmatmul_int4_perm(t, *d, k, g, perm=perm)) if act_order else (lambda t: ops.qmatmul_int4(t, *d, k, g))
    got = host(call(dev(x)))
    deq = oracle.w4_dequant(packed, scales, zp, k, g).astype(np.float64)
    exact = xs.astype(np.float64) @ deq
    terms = np.abs(xs).astype(np.float64) @ np.abs(deq) + 1e-300
    assert np.isfinite(got).all()
    rel = np.abs(got - exact) / terms
    assert np.delete(rel, 3, axis=0).max() < 2e-6
    # row 3: the kernels sum x (q - z) with z the zero-point's nearest integer, and add (zp - z) sum x per group, so the
    # dominating element weighs in with its own product plus at most half a step of its weight's scale: judged in
    # units of |x| (|q - z| + |zp - z|) scale
    q = oracle.w4_unpack(packed, k).astype(np.float64)                      # [k, n] nibbles
    rows_of_group = np.repeat(np.arange(scales.shape[0]), g)[:k]
    zr = np.rint(zp[rows_of_group]).astype(np.float64)
    factored = np.abs(xs[3]).astype(np.float64) @ ((np.abs(q - zr) + np.abs(zp[rows_of_group] - zr)) * scales[rows_of_group])
    assert (np.abs(got[3] - exact[3]) / factored).max() < 2e-6
    np.testing.assert_array_equal(got[4], np.zeros(n, np.float32))
    say("  times 2^40")
    x40 = x.copy()
    keep = [2, 6]                                            # would overflow f32: left as they are
    rows = [r for r in range(m) if r not in keep]
    x40[rows] *= np.float32(2.0 ** 40)
    big = host(call(dev(x40)))
    np.testing.assert_array_equal(big[rows], got[rows] * np.float32(2.0 ** 40))
    np.testing.assert_array_equal(big[keep], got[keep])
    for bad in (np.float32(np.nan), np.float32(np.inf)):
        say(f"  {bad} in row 9")
        xb = x.copy()
        xb[9, 33] = bad
        out = host(call(dev(xb)))
        assert np.isnan(out[9]).all()
        np.testing.assert_array_equal(np.delete(out, 9, axis=0), np.delete(got, 9, axis=0))


@pytest.mark.parametrize("m,k,n,g", [(160, 512, 1024, 128), (600, 1024, 2048, 32), (1100, 1024, 2048, 64)])
def test_integer_zero_points_and_one_that_is_not(ops, m, k, n, g):
    """The f16 kernel takes the nearest integer of a zero-point off inside its conversion of the weights and
    leaves out the update for the rest when the whole table holds integers (a small kernel looks first).  One
    entry that is no integer - anywhere in the table, here the last group's last column, then the first's first -,
    one beyond the range the conversion holds exactly, and a NaN each bring the update back: judged against the
    float64 product, in units of the summed terms; the NaN poisons its own column only."""
    say(f"w4 forward integer zero-points m={m} k={k} n={n} g={g}")
    rng = np.random.default_rng(m + g)
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    x = rng.normal(0, 1, (m, k)).astype(np.float32)
    packed, scales, zp = oracle.w4_from_f32(w, g, symmetric=True)
    assert (zp == np.rint(zp)).all()
    zp = rng.integers(0, 16, zp.shape).astype(np.float32)            # integers, not all the same
    cases = [("integers", None, None), ("last", (-1, -1), 7.25), ("first", (0, 0), 0.5), ("middle", (zp.shape[0] // 2, n // 2 + 1), -3.75),
             ("large", (0, 5), 5000.0), ("large negative", (-1, 6), -70000.0), ("nan", (0, 9), np.nan)]
    for name, at, value in cases:
        z = zp.copy()
        if at is not None:
            z[at] = value
        say(f"  {name}")
        got = host(ops.qmatmul_int4(dev(x), dev(packed), dev(scales), dev(z), k, g))
        deq = oracle.w4_dequant(packed, scales, z, k, g).astype(np.float64)
        exact = x.astype(np.float64) @ deq
        terms = np.abs(x).astype(np.float64) @ np.abs(deq) + 1e-300
        if name == "nan":
            col = at[1]
            assert np.isnan(got[:, col]).all()
            got, exact, terms = (np.delete(a, col, axis=1) for a in (got, exact, terms))
        assert np.isfinite(got).all()
        assert (np.abs(got - exact) / terms).max() < 2e-6


@pytest.mark.parametrize("m", [1, 4, 8, 16, 64, 128])
@pytest.mark.parametrize("act_order", [False, True])
def test_few_rows_of_any_magnitude(ops, m, act_order):
    """Up to 128 rows the kernels turn x into fixed point, 20 bits below the largest magnitude of a part of the row
    (32 consecutive k for up to 8 rows, an eighth of K beyond): uniformly scaled rows, 1e-30 to 3e33, are as
    accurate as ordinary ones; a row with one element that dominates its part stays within the bound
    max|x| 2^-19 sum|w| (such an element is multiplied in f32 on its own: test_outlier_columns_keep_the_tolerance)."""
    say(f"w4 forward row scaling m={m} act_order={act_order}")
    k, n, g = 1024, 1024, 128
    rng = np.random.default_rng(100 + m)
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    x = rng.normal(0, 1, (8 * m, k)).astype(np.float32)[:m]
    scale = np.ones(m, np.float32)
    for r, f in ((1, 1e-12), (2, 1e9), (5, 1e-30), (6, 3e33)):
        if r < m:
            scale[r] = f
    if m == 1:
        scale[0] = 1e-30
    x *= scale[:, None]
    dominated = 3 if m > 3 else None
    if dominated is not None:
        x[dominated, 7] = 2.0e5
    packed, scales, zp = oracle.w4_from_f32(w, g)
    d = [dev(a) for a in (packed, scales, zp)]
    if act_order:
        perm_np = rng.permutation(k).astype(np.int32)
        perm = dev(perm_np)
        xs = x[:, perm_np]
        got = host(ops.qmatmul_int4_perm(dev(x), *d, k, g, perm=perm))
    else:
        xs = x
        got = host(ops.qmatmul_int4(dev(x), *d, k, g))
    deq = oracle.w4_dequant(packed, scales, zp, k, g).astype(np.float64)
    exact = xs.astype(np.float64) @ deq
    terms = np.abs(xs).astype(np.float64) @ np.abs(deq) + 1e-300
    assert np.isfinite(got).all()
    rel = np.abs(got - exact) / terms
    plain = [r for r in range(m) if r != dominated]
    assert rel[plain].max() < 2e-6, rel[plain].max(axis=1)
    if dominated is not None:
        q = oracle.w4_unpack(packed, k).astype(np.float64)
        rows_of_group = np.repeat(np.arange(scales.shape[0]), g)[:k]
        factored = np.abs(xs[dominated]).astype(np.float64) @ ((q + np.abs(zp[rows_of_group])) * scales[rows_of_group])
        bound = 2.0e5 * 2.0 ** -19 * np.abs(deq).sum(axis=0) + 2e-6 * factored
        assert (np.abs(got[dominated] - exact[dominated]) <= bound).all()


@pytest.mark.parametrize("m", [1, 4, 8, 64, 512])
@pytest.mark.parametrize("bs", [32, 128, 1024])
def test_q8_matmul_rows_of_any_magnitude(ops, m, bs):
    """f32 x Q8 (matmul_q8.wgsl:37-98) through every route (vector kernels, digit planes on the int8 matrix cores,
    f16 matrix cores per block): rows from 1e-30 to 3e33 and a row with one element of 2e5, in units of the summed
    terms."""
    say(f"matmul_q8 row scaling m={m} bs={bs}")
    k, n = 1024, 1024
    rng = np.random.default_rng(200 + m + bs)
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    x = rng.normal(0, 1, (8 * m, k)).astype(np.float32)[:m]
    for r, f in ((1, 1e-12), (2, 1e9), (5, 1e-30), (6, 3e33)):
        if r < m:
            x[r] *= np.float32(f)
    if m == 1:
        x[0] *= np.float32(1e-30)
    if m > 3:
        x[3, 7] = 2.0e5
    words = ops.q8_quantize(ops.transpose_f32(dev(w)).reshape(-1), bs)
    wd = host(ops.q8_dequantize_kn(words, k, n, bs)).astype(np.float64)
    got = host(ops.matmul_q8(dev(x), words, k, n, bs))
    exact = x.astype(np.float64) @ wd
    terms = np.abs(x).astype(np.float64) @ np.abs(wd) + 1e-300
    assert np.isfinite(got).all()
    rel = np.abs(got - exact) / terms
    plain = [r for r in range(m) if r != 3]
    assert rel[plain].max() < 2e-6
    if m > 3:                                            # the dominated row: digit planes below the row part's maximum
        assert rel[3].max() < 2e-4


@pytest.mark.parametrize("m,n", [(1, 1024), (4, 1024), (16, 1024), (128, 1024), (256, 4096), (512, 4096), (768, 4096)])
@pytest.mark.parametrize("act_order", [False, True])
@pytest.mark.parametrize("big", [1000.0, 3000.0])
def test_outlier_columns_keep_the_tolerance(ops, m, n, act_order, big):
    """N(0,1) activations with outlier channels a thousand times larger, the way the hidden states of language
    models have them (4096 -> 1024, three lone channels per row and, in row 2, a run of six neighbours; 4096 -> 4096 at
    256, 512 and 768 rows, which the int8-path kernels take where the columns fill the chip): up to 128 rows, and in those
    larger batches, the kernels hold x in fixed point below the largest magnitude of a part of the row, and such elements
    would cost their neighbours the low bits.  They leave the fixed point instead - the decode kernel multiplies a
    chunk with a towering element in f32, element by element; the int8-path kernels multiply the towering elements
    on their own - so every output stays within rel 1e-3 / abs 1e-4 of the float64 product."""
    say(f"w4 forward with outlier channels m={m} n={n} act_order={act_order} big={big}")
    k, g = 4096, 128
    rng = np.random.default_rng(7000 + m)
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    x = rng.normal(0, 1, (m, k)).astype(np.float32)
    x[:, 7] = big
    x[:, 1234] = -3 * big
    x[:, 4000] = 0.5 * big
    if m > 2:
        x[2, 8:14] = np.array([2, -1, 1, 1, -2, 1], np.float32) * big
    packed, scales, zp = oracle.w4_from_f32(w, g)
    d = [dev(a) for a in (packed, scales, zp)]
    if act_order:
        perm_np = rng.permutation(k).astype(np.int32)
        xs = x[:, perm_np]
        got = host(ops.qmatmul_int4_perm(dev(x), *d, k, g, perm=dev(perm_np)))
    else:
        xs = x
        got = host(ops.qmatmul_int4(dev(x), *d, k, g))
    exact = xs.astype(np.float64) @ oracle.w4_dequant(packed, scales, zp, k, g).astype(np.float64)
    err = np.abs(got - exact)
    tol = 1e-4 + 1e-3 * np.abs(exact)
    assert (err <= tol).all(), f"worst error / tolerance {np.max(err / tol):.2f}"
    # for scale: the reference's own loop (f32, one element after the other) on two rows - at 3000 sigma it misses
    # this tolerance itself on outputs near zero, the kernels above do not
    rows = [0, min(2, m - 1)]
    ref = oracle.qmatmul_int4(xs[rows], packed, scales, zp, k, g).astype(np.float64)
    say(f"    kernels: worst error / tolerance {np.max(err / tol):.2f}; the f32 loop: {np.max(np.abs(ref - exact[rows]) / tol[rows]):.2f}")
