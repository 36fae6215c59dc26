"""The entry point that allocates nothing (rumus_hip_qmatmul_int4_perm_static) against the entry point it is
a variant of (rumus_hip_qmatmul_int4_perm): same bits, on calls in a row that share the static device array,
the later ones smaller than the first; requests beyond the array are refused with a clear error."""
import numpy as np
import pytest

import oracle

from gpu_util import assert_close, dev, host, say

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from rumus_amd import ops as o
    return o


def test_static_scratch_entry_point_matches_the_allocating_one(ops):
    import torch
    from rumus_amd import _lib
    assert _lib.lib().rumus_hip_static_scratch_bytes() == 32 << 20
    rng = np.random.default_rng(41)
    k, n, g = 4096, 11008, 128
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    packed, scales, zp = oracle.w4_from_f32(w, g, symmetric=True)
    g_idx = (rng.permutation(k) // g).astype(np.int32)
    ps, perm = ops.w4_actorder_prepare(dev(packed), dev(g_idx), g)
    sd, zd = dev(scales), dev(zp)
    bias = dev(rng.normal(0, 0.01, n).astype(np.float32))
    # Calls in a row that share the array, each with the contents the one before left in it.  Up to 300 rows run the
    # int8-path kernels (digit planes, chunk sums, row scales and the lists of towering elements in the array); 1024
    # rows the f16 tiles without partial tiles (18 MB of converted activations).
    outs = []
    for m in (128, 192, 16, 300, 48, 1024, 16):
        say(f"qmatmul_int4_perm_static m={m} k={k} n={n} act-order")
        x = dev(rng.normal(0, 1, (m, k)).astype(np.float32))
        y = torch.empty((m, n), dtype=torch.float32, device="cuda")
        ops.qmatmul_int4_perm_static(x, ps, sd, zd, k, g, bias=bias, perm=perm, out=y)
        want = ops.qmatmul_int4_perm(x, ps, sd, zd, k, g, bias=bias, perm=perm)
        np.testing.assert_array_equal(host(y), host(want), err_msg=f"m={m}")
        outs.append((host(x), host(y)))
    # and against the CPU restatement on a few rows of the first and the last call
    unsorted_w = dict(packed=packed, scales=scales, zp=zp)
    for xs, ys in (outs[0], outs[1], outs[3], outs[-1]):
        rows = [0, xs.shape[0] - 1]
        want = oracle.qmatmul_int4(xs[rows], unsorted_w["packed"], unsorted_w["scales"], unsorted_w["zp"], k, g,
                                   bias=host(bias), g_idx=g_idx, threads=8)
        assert_close(ys[rows], want)
    # Groups of 32 are not for the int8 path: 192 and 300 rows run the f16 tiles with K shared over three and two
    # workgroups per tile, whose partial tiles (25-26 MB) fill most of the array behind the converted activations -
    # after calls that left other contents there.
    p32, s32, z32 = oracle.w4_from_f32(w, 32)
    pd, sd32, zd32 = dev(p32), dev(s32), dev(z32)
    for m in (192, 16, 300):
        say(f"qmatmul_int4_perm_static m={m} k={k} n={n} g=32")
        x = dev(rng.normal(0, 1, (m, k)).astype(np.float32))
        y = torch.empty((m, n), dtype=torch.float32, device="cuda")
        ops.qmatmul_int4_perm_static(x, pd, sd32, zd32, k, 32, bias=bias, out=y)
        want = ops.qmatmul_int4_perm(x, pd, sd32, zd32, k, 32, bias=bias)
        np.testing.assert_array_equal(host(y), host(want), err_msg=f"g=32 m={m}")
        rows = [0, m - 1]
        assert_close(host(y)[rows], oracle.qmatmul_int4(host(x)[rows], p32, s32, z32, k, 32, bias=host(bias), threads=8))
    say("qmatmul_int4_perm_static small weight, plain order, few rows (no scratch needed)")
    k2, n2 = 512, 256
    w2 = rng.normal(0, 0.02, (k2, n2)).astype(np.float32)
    p2, s2, z2 = (dev(a) for a in oracle.w4_from_f32(w2, 64))
    for m in (24, 2):
        x = dev(rng.normal(0, 1, (m, k2)).astype(np.float32))
        got = ops.qmatmul_int4_perm_static(x, p2, s2, z2, k2, 64)
        np.testing.assert_array_equal(host(got), host(ops.qmatmul_int4_perm(x, p2, s2, z2, k2, 64)))


def test_static_scratch_refuses_what_does_not_fit(ops):
    import torch
    from rumus_amd._lib import RumusError
    say("qmatmul_int4_perm_static: 2048 rows need more than the static array")
    k, n, g = 4096, 11008, 128
    padded_words = torch.zeros((k // 8, n), dtype=torch.int32, device="cuda")
    meta = torch.ones((k // g, n), dtype=torch.float32, device="cuda")
    x = torch.zeros((2048, k), dtype=torch.float32, device="cuda")
    with pytest.raises(RumusError, match="bytes of scratch memory"):
        ops.qmatmul_int4_perm_static(x, padded_words, meta, meta, k, g)
    # the refusal left nothing behind: the next call that fits runs
    y = ops.qmatmul_int4_perm_static(x[:16].contiguous(), padded_words, meta, meta, k, g)
    assert float(host(y).max()) == 0.0
