"""Seeded sweep over ragged shapes: every matmul entry point against the CPU restatement on the
same inputs.  The fixed shape lists of the other GPU tests pick the known corners; this one draws
sizes around the kernels' tile, group and vector widths so that an unlisted combination of tails
does not go untested.  Integer results must be equal, f32 results within rel 1e-3 / abs 1e-4."""
import numpy as np
import pytest

import oracle

from gpu_util import assert_close, dev, host, say

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from rumus_amd import ops as o
    return o


def draw(rng, around, spread):
    """A size near one of the widths in `around` (tile edges are where indexing breaks)."""
    base = int(rng.choice(around))
    return max(1, base + int(rng.integers(-spread, spread + 1)))


W4_CASES = 48


@pytest.mark.parametrize("case", range(W4_CASES))
def test_w4_entry_points(ops, case):
    rng = np.random.default_rng(1000 + case)
    g = int(rng.choice([8, 16, 32, 64, 128, 256]))
    m = draw(rng, [1, 4, 6, 8, 16, 32, 33, 64, 100, 130], 2)
    k = draw(rng, [g, 2 * g, 128, 256, 512, 640, 1024], 9)
    n = draw(rng, [8, 16, 48, 64, 512, 520, 1024, 1100], 5)
    if case % 3 == 0:
        n = (n + 15) // 16 * 16          # the decode layout and the vector kernels
    elif case % 3 == 1:
        n = (n + 7) // 8 * 8             # u4 zero-points
    if case % 4 == 0:
        k = max(g, k // g * g)           # act-order needs whole groups
    bias = rng.normal(0, 0.01, n).astype(np.float32) if case % 2 else None
    say(f"sweep w4 case={case} m={m} k={k} n={n} g={g} bias={bias is not None}")
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    x = rng.normal(0, 1, (m, k)).astype(np.float32)
    packed, scales, zp = oracle.w4_from_f32(w, g, symmetric=bool(case % 5 == 0))
    d = [dev(a) for a in (packed, scales, zp)]
    db = None if bias is None else dev(bias)
    want = oracle.qmatmul_int4(x, packed, scales, zp, k, g, bias=bias, threads=8)

    got = host(ops.qmatmul_int4(dev(x), *d, k, g, bias=db))
    assert_close(got, want, "qmatmul_int4")

    gy = rng.normal(0, 1, (m, n)).astype(np.float32)
    assert_close(host(ops.qmatmul_int4_t(dev(gy), *d, k, g)),
                 oracle.qmatmul_int4_t(gy, packed, scales, zp, k, g, threads=8), "qmatmul_int4_t")

    if k % g == 0:                       # act-order: rows sorted by a shuffled group index
        g_idx = (rng.permutation(k) // g).astype(np.int32)
        ps, perm = ops.w4_actorder_prepare(d[0], dev(g_idx), g)
        want_ao = oracle.qmatmul_int4(x, packed, scales, zp, k, g, bias=bias, g_idx=g_idx, threads=8)
        assert_close(host(ops.qmatmul_int4_perm(dev(x), ps, d[1], d[2], k, g, bias=db, perm=perm)), want_ao,
                     "qmatmul_int4_perm")
        # g_idx handed to the plain entry point takes the same route
        assert_close(host(ops.qmatmul_int4(dev(x), *d, k, g, bias=db, g_idx=dev(g_idx))), want_ao, "g_idx")

    if n % 8 == 0:                       # AWQ storage
        pa, sa, qz = oracle.w4_awq_from_f32(w, g)
        za = oracle.w4_qzeros_unpack(qz, n)
        got_awq = host(ops.qmatmul_int4_zp4(dev(x), dev(pa), dev(sa), dev(qz), k, g, bias=db))
        assert_close(got_awq, oracle.qmatmul_int4(x, pa, sa, za, k, g, bias=bias, threads=8), "qmatmul_int4_zp4")

    if n % 16 == 0 and g % 32 == 0 and m <= 8:
        pt, st, zt = ops.w4_decode_layout(*d, g)
        got_dec = host(ops.qmatmul_int4_decode(dev(x), pt, st, zt, k, g, bias=db))
        assert_close(got_dec, want, "qmatmul_int4_decode")
        if m <= ops.qmatmul_int4_decode_max_rows(packed.shape[0] * 8, n):
            np.testing.assert_array_equal(got_dec, got)


@pytest.mark.parametrize("case", range(24))
def test_w4_quantizers(ops, case):
    rng = np.random.default_rng(2000 + case)
    g = int(rng.choice([8, 16, 32, 64, 128]))
    k = draw(rng, [g, 3 * g, 256, 1000], 11)
    n = draw(rng, [1, 8, 64, 256, 300], 3)
    say(f"sweep w4 quantize case={case} k={k} n={n} g={g}")
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    if case % 4 == 0:
        w[:, 0] = 0.0                    # a constant column: range below the threshold
    if case % 6 == 0:
        w = np.round(w * 256) / 256      # ties in w / scale
    from gpu_util import host_u32
    for sym in (False, True):
        want = oracle.w4_from_f32(w, g, symmetric=sym)
        got = ops.w4_quantize_pack(dev(w), g, sym)
        np.testing.assert_array_equal(host_u32(got[0]), want[0])
        np.testing.assert_array_equal(host(got[1]), want[1])
        np.testing.assert_array_equal(host(got[2]), want[2])
    if n % 8 == 0:
        want = oracle.w4_awq_from_f32(w, g)
        got = ops.w4_quantize_pack_awq(dev(w), g)
        np.testing.assert_array_equal(host_u32(got[0]), want[0])
        np.testing.assert_array_equal(host(got[1]), want[1])
        np.testing.assert_array_equal(host_u32(got[2]), want[2])


@pytest.mark.parametrize("case", range(32))
def test_i8_engine(ops, case):
    rng = np.random.default_rng(3000 + case)
    m = draw(rng, [1, 16, 32, 64, 128, 130, 256, 300], 3)
    k = draw(rng, [16, 64, 128, 256, 512, 1000], 5)
    n = draw(rng, [8, 32, 128, 256, 352, 384, 700], 5)
    k = (k + 63) // 64 * 64 if case % 2 == 0 else (k + 15) // 16 * 16   # LDS-DMA kernels / the k % 16 contract
    say(f"sweep i8 case={case} m={m} k={k} n={n}")
    x = rng.normal(0, 1, (m, k)).astype(np.float32)
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    bias = rng.normal(0, 0.01, n).astype(np.float32) if case % 3 else None
    xq_want, sx_want = oracle.i8_quantize_rows(x)
    xq, sx = ops.i8_quantize_rows(dev(x))
    np.testing.assert_array_equal(host(xq), xq_want)
    np.testing.assert_array_equal(host(sx), sx_want)
    wq, sw = ops.i8_quantize_cols_t(dev(w))
    wq_h, sw_h = host(wq), host(sw)
    wq_want, sw_want = oracle.i8_quantize_rows(np.ascontiguousarray(w.T))
    np.testing.assert_array_equal(wq_h, wq_want)
    np.testing.assert_array_equal(sw_h, sw_want)
    y, acc = ops.i8_gemm(xq, wq, sx, sw, None if bias is None else dev(bias), want_acc=True)
    acc_want = oracle.i8_gemm_i32(xq_want, wq_h, threads=8)
    np.testing.assert_array_equal(host(acc), acc_want)
    assert_close(host(y), oracle.i8_rescale_bias(acc_want, sx_want, sw_h, bias), "i8_gemm y")


@pytest.mark.parametrize("case", range(32))
def test_q8_block_format(ops, case):
    rng = np.random.default_rng(4000 + case)
    bs = int(rng.choice([4, 8, 32, 64, 256, 512] if case < 16 else [32, 64, 96, 128, 1024]))
    blocks_per_col = int(rng.integers(1, 5))
    k = bs * blocks_per_col
    n = draw(rng, [1, 7, 64, 130], 2)
    m = draw(rng, [1, 5, 33] if case < 16 else [5, 33, 70, 390], 1)   # few-rows kernel / the matrix-core paths
    say(f"sweep q8 case={case} m={m} k={k} n={n} bs={bs}")
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    if case % 4 == 0:
        w[:bs, 0] = 0.0                  # an all-zero block
    a = rng.normal(0, 1, (m, k)).astype(np.float32)
    from gpu_util import host_u32
    want_words = oracle.tensor_quantize(w, bs)
    flat_t = np.ascontiguousarray(w.T).reshape(-1)
    words = ops.q8_quantize(dev(flat_t), bs)
    np.testing.assert_array_equal(host_u32(words)[:want_words.size], want_words)
    np.testing.assert_array_equal(host(ops.q8_dequantize(words, k * n, bs)),
                                  oracle.q8_dequantize(want_words, k * n, bs))
    assert_close(host(ops.matmul_q8(dev(a), words, k, n, bs)), oracle.matmul_q8(a, want_words, k, n, bs, threads=8))


@pytest.mark.parametrize("case", range(8))
def test_w4_many_tiles(ops, case):
    # enough output tiles for the wider workgroup shapes of the MFMA kernel; K kept short so that
    # the CPU restatement stays quick
    rng = np.random.default_rng(5000 + case)
    g = int(rng.choice([32, 64, 128]))
    m = draw(rng, [130, 300, 1000, 2050], 40)
    k = draw(rng, [g, 128, 256, 384], 6)
    n = draw(rng, [2048, 4100, 8192], 12) // 4 * 4
    if case % 2:
        k = max(g, k // g * g)
    say(f"sweep w4 many tiles case={case} m={m} k={k} n={n} g={g}")
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    x = rng.normal(0, 1, (m, k)).astype(np.float32)
    bias = rng.normal(0, 0.01, n).astype(np.float32)
    packed, scales, zp = oracle.w4_from_f32(w, g)
    d = [dev(a) for a in (packed, scales, zp)]
    want = oracle.qmatmul_int4(x, packed, scales, zp, k, g, bias=bias, threads=8)
    assert_close(host(ops.qmatmul_int4(dev(x), *d, k, g, bias=dev(bias))), want)
    if k % g == 0:
        g_idx = (rng.permutation(k) // g).astype(np.int32)
        want_ao = oracle.qmatmul_int4(x, packed, scales, zp, k, g, bias=bias, g_idx=g_idx, threads=8)
        assert_close(host(ops.qmatmul_int4(dev(x), *d, k, g, bias=dev(bias), g_idx=dev(g_idx))), want_ao)


@pytest.mark.parametrize("case", range(8))
def test_i8_many_tiles(ops, case):
    rng = np.random.default_rng(6000 + case)
    m = draw(rng, [256, 512, 1024, 2048], 20)
    k = draw(rng, [64, 128, 320], 0) if case % 2 else draw(rng, [80, 144, 272], 0)
    n = draw(rng, [2816, 4096, 5632, 11008], 9)
    say(f"sweep i8 many tiles case={case} m={m} k={k} n={n}")
    xq = rng.integers(-127, 128, (m, k)).astype(np.int8)
    wq = rng.integers(-127, 128, (n, k)).astype(np.int8)
    sx = rng.uniform(0.001, 0.1, m).astype(np.float32)
    sw = rng.uniform(0.001, 0.1, n).astype(np.float32)
    bias = rng.normal(0, 0.01, n).astype(np.float32)
    import torch
    y, acc = ops.i8_gemm(torch.from_numpy(xq).cuda(), torch.from_numpy(wq).cuda(), dev(sx), dev(sw), dev(bias),
                         want_acc=True)
    acc_want = oracle.i8_gemm_i32(xq, wq, threads=8)
    np.testing.assert_array_equal(host(acc), acc_want)
    assert_close(host(y), oracle.i8_rescale_bias(acc_want, sx, sw, bias))


# Few rows over long K: the kernel that keeps the activations in registers (5..64 rows, K steps shared by eight waves,
# up to three chunks of K per column tile) and its neighbours on either side of every limit.
@pytest.mark.parametrize("k", [3008, 3072, 3136, 4096, 4160, 8192, 8256, 11008, 12288, 12352])
def test_i8_few_rows_long_k(ops, k):
    import torch
    rng = np.random.default_rng(7000 + k)
    wq_all = rng.integers(-127, 128, (4100, k)).astype(np.int8)
    sw_all = rng.uniform(0.001, 0.1, 4100).astype(np.float32)
    bias_all = rng.normal(0, 0.01, 4100).astype(np.float32)
    for m, n in ((5, 4100), (16, 8), (17, 100), (31, 352), (32, 4100), (33, 16), (48, 1000), (49, 40), (64, 4100), (65, 352)):
        say(f"sweep i8 few rows m={m} k={k} n={n}")
        xq = rng.integers(-127, 128, (m, k)).astype(np.int8)
        sx = rng.uniform(0.001, 0.1, m).astype(np.float32)
        wq, sw, bias = wq_all[:n], sw_all[:n], bias_all[:n] if (m + n) % 2 else None
        y, acc = ops.i8_gemm(torch.from_numpy(xq).cuda(), torch.from_numpy(np.ascontiguousarray(wq)).cuda(), dev(sx), dev(sw),
                             None if bias is None else dev(bias), want_acc=True)
        acc_want = oracle.i8_gemm_i32(xq, wq, threads=8)
        np.testing.assert_array_equal(host(acc), acc_want)
        assert_close(host(y), oracle.i8_rescale_bias(acc_want, sx, sw, bias))
