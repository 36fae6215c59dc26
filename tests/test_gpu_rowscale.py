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
# four-wave form
@pytest.mark.parametrize("m,k,n,g,act_order", [(160, 512, 1024, 128, False), (520, 1024, 1536, 128, False),
                                               (300, 512, 512, 64, True), (136, 520, 516, 32, False),
                                               (600, 1024, 2048, 128, True), (600, 1024, 2048, 128, False),
                                               (600, 1028, 2048, 128, False), (1024, 256, 11008, 128, False)])
def test_rows_of_any_magnitude(ops, m, k, n, g, act_order):
    """Batches beyond 128 rows split x into two f16 planes: every row is first scaled by a power of two into
    f16's range, so rows of 1e-12, rows of 1e9 and a row with one element of 2e5 (beyond f16's 65504) come
    out as accurate as ordinary ones, in units of the summed terms (of the two sums the kernels keep, for the
    dominated row); multiplying x by 2^40 multiplies y by
    2^40 exactly; an infinity or a NaN poisons its own row only."""
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
    # row 3: the kernels sum x q and x separately per group (scale (sum x q - zp sum x)), so where the dominating
    # element meets a weight that dequantizes to almost nothing the two sums cancel: judged in units of
    # |x| (q + zp) scale there
    q = oracle.w4_unpack(packed, k).astype(np.float64)                      # [k, n] nibbles
    rows_of_group = np.repeat(np.arange(scales.shape[0]), g)[:k]
    factored = np.abs(xs[3]).astype(np.float64) @ ((q + np.abs(zp[rows_of_group])) * scales[rows_of_group])
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
