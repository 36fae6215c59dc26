"""GPU parity for the INT8 engine: reference Q8 block format and the W8A8 extension."""
import json
import os

import numpy as np
import pytest

import oracle
from rumus_amd import workloads

from gpu_util import assert_close, dev, host, host_u32, say

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(__file__), "golden", "q8_kat.json")


@pytest.fixture(scope="module")
def ops():
    from rumus_amd import ops as o
    return o


def test_q8_quantize_known_answers(ops):
    for case in json.load(open(GOLD))["cases"]:
        say(f"q8_quantize KAT {case['name']}")
        x = np.array(case["x"], np.float32)
        words = host_u32(ops.q8_quantize(dev(x), case["block_size"]))
        assert f"{words[0]:08x}" == case["header_hex"]
        assert words[1:].view(np.int8).tolist() == case["q"]
        xq, s = ops.i8_quantize_rows(dev(x.reshape(1, -1)))
        assert host(xq)[0].tolist() == case["q"]


@pytest.mark.parametrize("numel,bs", [(64 * 5 + 20, 64), (512 * 512, 512), (4096 * 24, 4096),
                                      (1000, 8), (36, 4)])
def test_q8_quantize_dequantize_bit_exact(ops, numel, bs):
    say(f"q8 quantize/dequantize numel={numel} bs={bs}")
    rng = np.random.default_rng(numel + bs)
    x = rng.normal(0, 0.02, numel).astype(np.float32)
    x[: min(bs, numel) // 2] *= 50
    if numel > 3 * bs:
        x[2 * bs: 3 * bs] = 0.0          # an all-zero block
    want = oracle.q8_quantize(x, bs)
    got = ops.q8_quantize(dev(x), bs)
    assert got.numel() * 4 == ops.q8_buf_size(numel, bs) == oracle.q8_buf_size(numel, bs)
    np.testing.assert_array_equal(host_u32(got), want)
    np.testing.assert_array_equal(host(ops.q8_dequantize(got, numel, bs)),
                                  oracle.q8_dequantize(want, numel, bs))


@pytest.mark.parametrize("k,n,bs", [(512, 512, 512), (96, 7, 32), (100, 9, 20), (130, 33, 64), (4096, 264, 4096),
                                    (257, 70, 8)])
def test_q8_dequantize_kn_is_the_transposed_dequantize(ops, k, n, bs):
    # values in the order of the tensor's shape: bit-identical to the reference-order output, moved
    say(f"q8 dequantize_kn k={k} n={n} bs={bs}")
    from rumus_amd import nn
    rng = np.random.default_rng(k + n + bs)
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    words = oracle.tensor_quantize(w, bs)
    want = oracle.q8_dequantize(words, k * n, bs).reshape(n, k).T
    got = host(ops.q8_dequantize_kn(dev(words), k, n, bs))
    np.testing.assert_array_equal(got, want)
    wq = nn.quantize(dev(w), bs)
    np.testing.assert_array_equal(host(nn.dequantize_kn(wq)), want)
    # Tensor::data() on a Q8 tensor: the dequantized buffer (reference order), downloaded once
    np.testing.assert_array_equal(wq.data(), oracle.q8_dequantize(words, k * n, bs))
    assert wq.data() is wq.data()
    # and it is the weight again, to quantization error: half a step, plus the f16 rounding of the
    # block scale (2^-11 of the value); blocks line up with columns when bs divides k
    if k % bs == 0:
        scale = np.abs(w).reshape(k // bs, bs, n).max(axis=1).repeat(bs, axis=0) / 127.0
        assert (np.abs(got - w) <= scale * 0.501 + np.abs(w) * 6e-4 + 1e-12).all()


@pytest.mark.parametrize("rows,cols", [(64, 64), (4096, 264), (1000, 4100), (1001, 4101), (4, 8), (3, 1), (1, 7),
                                       (68, 132), (130, 64)])
def test_transpose_is_exact(ops, rows, cols):
    # the transpose in front of the block quantizer (ops.rs:2307); 64 x 64 tiles with 128-bit accesses
    # when both sides are multiples of 4, 32 x 32 tiles otherwise
    say(f"transpose rows={rows} cols={cols}")
    rng = np.random.default_rng(rows * 7 + cols)
    w = rng.normal(0, 1, (rows, cols)).astype(np.float32)
    np.testing.assert_array_equal(host(ops.transpose_f32(dev(w))), np.ascontiguousarray(w.T))


def test_q8_rejects_bad_block_size(ops):
    say("q8 bad block size")
    with pytest.raises(ops.RumusError):
        ops.q8_quantize(dev(np.zeros(16, np.float32)), 6)
    with pytest.raises(ops.RumusError):
        ops.q8_quantize(dev(np.zeros(16, np.float32)), 0)


@pytest.mark.parametrize("m,k,n,bs", [(32, 512, 512, 512), (4, 64, 10, 64), (3, 96, 7, 32),
                                      (2, 40, 5, 8), (70, 256, 130, 128), (5, 100, 9, 20),
                                      (1, 4096, 1100, 4096),   # few-rows kernel, per-channel blocks
                                      (4, 8192, 70, 128),      # two groups of two rows
                                      (3, 1008, 64, 16),       # smallest block the few-rows kernel takes
                                      (2, 11008, 40, 64),      # one row per launch
                                      (7, 2048, 33, 2048),
                                      (100, 1024, 300, 1024),  # digit planes on the int8 matrix cores, one block per column
                                      (8, 48, 20, 48),         # W8A8 kernel on a dense copy: the smallest batch that goes there
                                      (400, 512, 96, 512),     # and from 384 rows on
                                      (1000, 4096, 264, 4096),
                                      (400, 8192, 256, 8192),  # the int8 GEMM inside shares K eight ways: its partial sums sit
                                      (384, 2048, 128, 2048),  # behind this call's planes in the workspace (two ways here)
                                      # block scales inside the MFMA loop: f16 planes for blocks up to 64 ...
                                      (5, 64, 64, 32),         # the smallest batch that goes there
                                      (11, 96, 20, 32),        # a fold per 32 k, K ends mid-step
                                      (100, 1024, 300, 32),
                                      (33, 512, 100, 64),
                                      (1030, 256, 2050, 32),
                                      # ... and for more than 64 rows
                                      (70, 480, 40, 96),       # blocks that straddle the K steps, K ends mid-step
                                      (1024, 512, 2048, 128),  # the largest tile
                                      # four int8 digit planes for larger blocks and up to 64 rows
                                      (12, 192, 40, 96),
                                      (40, 4096, 64, 2048),    # two folds per block, K shared over workgroups
                                      (6, 1184, 16, 1184)])    # 37 K halves per block: a fold at every half
def test_matmul_q8_vs_oracle(ops, m, k, n, bs):
    say(f"matmul_q8 m={m} k={k} n={n} bs={bs}")
    from rumus_amd import nn
    rng = np.random.default_rng(m + k + n)
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    a = rng.normal(0, 1, (m, k)).astype(np.float32)
    b = rng.normal(0, 0.01, n).astype(np.float32)
    words = oracle.tensor_quantize(w, bs)
    wq = nn.quantize(dev(w), bs)                       # transpose + quantize on the GPU
    np.testing.assert_array_equal(host_u32(wq.buffer), words)
    want = oracle.add_bias(oracle.matmul_q8(a, words, k, n, bs, threads=8), b)
    got = host(nn.linear_forward(nn.Linear(dev(w), dev(b)), dev(a), wq))
    assert_close(got, want)
    # Tensor::dequantize returns the buffer order ([N,K]) under the [K,N] shape
    deq = host(nn.dequantize(wq))
    np.testing.assert_array_equal(deq.reshape(-1), oracle.q8_dequantize(words, k * n, bs))


def test_matmul_q8_row_split_inside_on_a_fresh_stream(ops):
    # 520 rows become 2080 rows of digit planes; the int8 GEMM inside splits them into 2048 rows of wide
    # blocks and 32 rows that share K over workgroups, whose partial sums must fit behind this call's own
    # buffers.  A stream that has never run anything has no workspace yet, so the reservation is exact.
    import torch
    from rumus_amd import nn
    m, k, n, bs = 520, 4096, 11008, 4096
    say(f"matmul_q8 m={m} k={k} n={n} bs={bs} on a fresh stream")
    rng = np.random.default_rng(520)
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    a = rng.normal(0, 1, (m, k)).astype(np.float32)
    wq = nn.quantize(dev(w), bs)
    ad = dev(a)
    torch.cuda.synchronize()
    fresh = torch.cuda.Stream()
    with torch.cuda.stream(fresh):
        got = nn.matmul(ad, wq)
    fresh.synchronize()
    rows = [0, 1, 255, 511, 512, 513, 519]                  # both sides of the split at plane row 2048
    words = host_u32(wq.buffer)
    want = oracle.matmul_q8(a[rows], words, k, n, bs, threads=8)
    assert_close(host(got)[rows], want)
    # rows are independent: the whole product equals the product computed 104 rows at a time
    parts = torch.cat([nn.matmul(ad[i:i + 104].contiguous(), wq) for i in range(0, m, 104)])
    assert_close(host(got), host(parts))


@pytest.mark.parametrize("m,k,n", [(1024, 256, 2048),     # planes added in the epilogue of the 256 x 256 blocks
                                   (1501, 192, 2801),     # ... of the wide blocks, ragged on both sides
                                   (1536, 128, 4096),     # ... rows split over two launches of those kernels
                                   (3000, 64, 2050),      # rows split with a part on kernels without that epilogue:
                                   (400, 512, 96),        # ... those and small shapes add the planes in a pass
                                   (100, 1024, 300), (8, 48, 20), (1, 16, 5)])
def test_matmul_q8_dense_copy(ops, m, k, n):
    # a per-output-channel weight prepared once (Q8Tensor.prepare) against the same weight unpacked on every call
    say(f"matmul_q8_dense m={m} k={k} n={n}")
    from rumus_amd import nn
    rng = np.random.default_rng(m * 3 + k + n)
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    a = rng.normal(0, 1, (m, k)).astype(np.float32)
    a[m // 2, 3] = 2.0e4
    if m > 4:
        a[4] = 0.0
    words = oracle.tensor_quantize(w, k)
    wq, sw = ops.q8_dense_layout(dev(words), k, n, k)
    blocks = words.reshape(n, 1 + k // 4)                  # a header word, then k / 4 data words per column
    np.testing.assert_array_equal(host(wq).view(np.uint8), np.ascontiguousarray(blocks[:, 1:]).view(np.uint8))
    np.testing.assert_array_equal(host(sw), (blocks[:, 0] & 0xFFFF).astype(np.uint16).view(np.float16).astype(np.float32))
    got = host(ops.matmul_q8_dense(dev(a), wq, sw))
    want = oracle.matmul_q8(a, words, k, n, k, threads=8)
    assert_close(got, want)
    if m > 4:
        np.testing.assert_array_equal(got[4], np.zeros(n, np.float32))
    if m >= 384:                                           # there matmul_q8 takes the same route on a copy it makes itself
        np.testing.assert_array_equal(got, host(ops.matmul_q8(dev(a), dev(words), k, n, k)))
    q = nn.Q8Tensor(dev(words), (k, n), k).prepare()
    via_nn = host(nn.matmul(dev(a), q))
    if m >= nn.Q8_DENSE_MIN_ROWS:
        np.testing.assert_array_equal(via_nn, got)
    else:
        assert_close(via_nn, want)
    ab = a.copy()
    ab[m - 1, 7] = np.float32(np.inf)                      # poisons its own row only
    gb = host(ops.matmul_q8_dense(dev(ab), wq, sw))
    assert np.isnan(gb[m - 1]).all()
    np.testing.assert_array_equal(gb[:m - 1], got[:m - 1])


def test_q8_dense_rejects(ops):
    say("q8 dense rejects")
    import torch
    from rumus_amd import nn
    with pytest.raises(ValueError):                        # blocks smaller than a column have no dense form
        nn.Q8Tensor(dev(oracle.tensor_quantize(np.ones((64, 8), np.float32), 32)), (64, 8), 32).prepare()
    with pytest.raises(ops.RumusError):                    # more columns than the layout kernel's grid takes
        ops.q8_dense_layout(torch.zeros(70000 * 5, dtype=torch.int32, device="cuda"), 16, 70000, 16)
    words = dev(oracle.tensor_quantize(np.ones((64, 8), np.float32), 32))
    with pytest.raises(ops.RumusError):                    # two blocks per column
        ops.q8_dense_layout(words, 64, 8, 32)
    wq = torch.zeros((8, 24), dtype=torch.int8, device="cuda")
    with pytest.raises(ops.RumusError):                    # k % 16
        ops.matmul_q8_dense(torch.zeros((4, 24), device="cuda"), wq, torch.ones(8, device="cuda"))
    with pytest.raises(ValueError):
        ops.matmul_q8_dense(torch.zeros((4, 32), device="cuda"), wq, torch.ones(8, device="cuda"))


@pytest.mark.parametrize("bs,m", [(512, 64), (32, 64), (128, 64), (128, 100), (512, 400)])
def test_matmul_q8_batch_accuracy_and_non_finite_rows(ops, bs, m):
    # batches: activations go through four 7-bit digit planes and the int8 matrix cores (block scales
    # inside the loop; 400 rows and one block per column: the W8A8 kernel on a dense copy) or, for
    # 32-element blocks and for 100 rows, through two f16 planes and the f16 matrix cores.
    # Judged against float64 in units of the summed terms (the digit planes keep 28 bits below the
    # row maximum, so a row with one huge entry is the hard case; the f16 planes keep 22 bits of
    # every entry), and a NaN or infinite activation must poison its own row only.
    say(f"matmul_q8 digit-plane path bs={bs}")
    rng = np.random.default_rng(77)
    k, n = 512, 96
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    a = rng.normal(0, 1, (m, k)).astype(np.float32)
    a[3, 17] = 3.0e4                                        # dwarfs the rest of its row
    a[5] *= 1e-30
    a[6] = 0.0
    words = oracle.tensor_quantize(w, bs)
    got = host(ops.matmul_q8(dev(a), dev(words), k, n, bs))
    want = oracle.matmul_q8(a, words, k, n, bs, threads=8)
    deq = oracle.q8_dequantize(words, k * n, bs).reshape(n, k).T.astype(np.float64)
    exact = a.astype(np.float64) @ deq
    terms = np.abs(a).astype(np.float64) @ np.abs(deq) + 1e-300
    err_ref = (np.abs(want - exact) / terms).max()
    err_got = (np.abs(got - exact) / terms).max()
    # ordinary rows come out at least as accurate as the f32 loop; the row with the outlier lands
    # within a few times the f32 loop's own error
    assert err_ref < 2e-6 and err_got < 1e-5, (err_got, err_ref)
    assert (np.abs(np.delete(got, 3, axis=0) - np.delete(exact, 3, axis=0)) / np.delete(terms, 3, axis=0)).max() < 1e-7
    assert_close(got, want)
    np.testing.assert_array_equal(got[6], np.zeros(n, np.float32))
    for bad in (np.float32(np.nan), np.float32(np.inf)):
        ab = a.copy()
        ab[9, 100] = bad
        gb = host(ops.matmul_q8(dev(ab), dev(words), k, n, bs))
        assert np.isnan(gb[9]).all()
        np.testing.assert_array_equal(np.delete(gb, 9, axis=0), np.delete(got, 9, axis=0))


def test_matmul_q8_naive_kernel_is_bit_exact(ops):
    # block_size % 16 != 0 routes to the one-thread-per-output kernel (the reference's loop)
    say("matmul_q8 naive kernel bit-exact")
    rng = np.random.default_rng(5)
    m, k, n, bs = 5, 100, 9, 20
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    a = rng.normal(0, 1, (m, k)).astype(np.float32)
    words = oracle.tensor_quantize(w, bs)
    got = host(ops.matmul_q8(dev(a), dev(words), k, n, bs))
    np.testing.assert_array_equal(got, oracle.matmul_q8(a, words, k, n, bs))


def test_api_errors_mirror_reference_asserts(ops):
    say("module-level asserts")
    from rumus_amd import nn
    w = dev(np.zeros((8, 8), np.float32))
    q = nn.quantize(w, 8)
    with pytest.raises(ValueError):
        nn.quantize(q, 8)                       # already quantized (ops.rs:2292)
    with pytest.raises(ValueError):
        nn.quantize(w, 6)                       # block_size % 4 (ops.rs:2291)
    with pytest.raises(ValueError):
        nn.matmul(q, q)                         # Q8 lhs (ops.rs:519)
    with pytest.raises(ValueError):
        nn.matmul(dev(np.zeros((2, 4), np.float32)), q)   # inner dim (ops.rs:523)


# ---- W8A8 extension -------------------------------------------------------------

@pytest.mark.parametrize("rows,cols", [(32, 512), (7, 100), (3, 4096), (1, 5), (130, 1024),
                                       (3, 6000), (5, 11008), (2, 12288),   # rows held in registers: 8 and 12 K
                                       (2, 12292), (2, 20001)])             # longer rows are read twice
def test_i8_quantize_rows_bit_exact(ops, rows, cols):
    say(f"i8_quantize_rows {rows}x{cols}")
    rng = np.random.default_rng(rows * cols)
    x = rng.normal(0, 1, (rows, cols)).astype(np.float32)
    if rows > 2:
        x[1] = 0.0
    wq, ws = oracle.i8_quantize_rows(x)
    xq, s = ops.i8_quantize_rows(dev(x))
    np.testing.assert_array_equal(host(xq), wq)
    np.testing.assert_array_equal(host(s), ws)


@pytest.mark.parametrize("k,n", [(512, 512), (100, 37), (4096, 200), (64, 1), (208, 130), (72, 64), (1024, 2052)])
def test_i8_quantize_cols_t_bit_exact(ops, k, n):
    say(f"i8_quantize_cols_t k={k} n={n}")
    rng = np.random.default_rng(k + n)
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    if n > 3:
        w[:, 2] = 0.0
    want_q, want_s = oracle.i8_quantize_rows(np.ascontiguousarray(w.T))
    wq, sw = ops.i8_quantize_cols_t(dev(w))
    np.testing.assert_array_equal(host(wq), want_q)
    np.testing.assert_array_equal(host(sw), want_s)


@pytest.mark.parametrize("m,k,n", [(32, 512, 512), (1, 16, 1), (77, 208, 133), (256, 1024, 384),
                                   (300, 4096, 260), (2048, 256, 2304),
                                   # few tiles, K % 64 == 0: one-wave tiles, K shared over workgroups
                                   (32, 4096, 1100),          # eight shares
                                   (6, 4096, 64), (128, 1088, 70),   # 17 K steps in two shares of 9 and 8
                                   # 5 to 32 rows, K % 256 == 0: MFMA tiles fed straight from global memory
                                   (5, 256, 16), (16, 1024, 100), (17, 1024, 40), (32, 2816, 70), (9, 11008, 30),
                                   (12, 256, 20490), (8, 512, 22016),   # the same with two column tiles per workgroup
                                   # up to 4 rows: the dot4 decode kernel
                                   (1, 4096, 1100), (2, 11008, 130), (3, 5008, 67), (4, 4096, 260), (4, 48, 5),
                                   (5, 576, 200),             # 9 steps: a single share
                                   (300, 8192, 130),          # 128 x 128 tiles, six of them, K in eight shares
                                   (129, 1024, 129),          # the same tiles, four, ragged both ways, one share
                                   (200, 4160, 384),          # 65 K steps in four shares of 17, 17, 17 and 14
                                   (1000, 8192, 1100),        # 72 tiles, three shares of 43, 43 and 42 steps
                                   (300, 208, 260), (2048, 208, 2304),   # K % 64 != 0: the register-staged tiles
                                   (2250, 128, 4096)])        # 144 blocks of 256 x 256: one partly filled round
def test_i8_gemm_accumulators_bit_exact(ops, m, k, n):
    check_i8_gemm(ops, m, k, n)


# Shapes that take the wide-block kernel (256 x 32*W blocks in whole rounds over 256 CUs),
# one per block width W = 8..12, with K of 1, 2, 3 and 5 steps of 64 (fewer steps than
# pipeline stages included), a ragged last row block and N that is not a multiple of 32.
@pytest.mark.parametrize("m,k,n", [(4096, 192, 4096), (2048, 64, 9216), (2048, 128, 10240),
                                   (2048, 320, 11008), (2000, 64, 10990), (2048, 64, 12288),
                                   (1990, 128, 12281),
                                   # whole rounds and the rest launched apart: 4096 + 2048 rows, 1024 + 512 rows
                                   (6144, 64, 4096), (1536, 64, 16384), (1500, 128, 16300)])
def test_i8_gemm_wide_blocks_bit_exact(ops, m, k, n):
    check_i8_gemm(ops, m, k, n)


def check_i8_gemm(ops, m, k, n):
    say(f"i8_gemm m={m} k={k} n={n}")
    rng = np.random.default_rng(m + k + n)
    xq = rng.integers(-127, 128, (m, k)).astype(np.int8)
    wq = rng.integers(-127, 128, (n, k)).astype(np.int8)
    sx = rng.uniform(0.001, 0.05, m).astype(np.float32)
    sw = rng.uniform(0.0001, 0.001, n).astype(np.float32)
    b = rng.normal(0, 0.01, n).astype(np.float32)
    want_acc = oracle.i8_gemm_i32(xq, wq, threads=8)
    y, acc = ops.i8_gemm(dev(xq), dev(wq), dev(sx), dev(sw), dev(b), want_acc=True)
    np.testing.assert_array_equal(host(acc), want_acc)
    # the epilogue uses the oracle's association, so it is bit-exact too
    np.testing.assert_array_equal(host(y), oracle.i8_rescale_bias(want_acc, sx, sw, b))
    y2, _ = ops.i8_gemm(dev(xq), dev(wq), dev(sx), dev(sw), None)
    np.testing.assert_array_equal(host(y2), oracle.i8_rescale_bias(want_acc, sx, sw, None))
    _, acc_only = ops.i8_gemm(dev(xq), dev(wq), want_acc=True, want_y=False)
    np.testing.assert_array_equal(host(acc_only), want_acc)


def test_i8_gemm_extreme_values(ops):
    say("i8_gemm extremes")
    m, k, n = 64, 4096, 64
    xq = np.full((m, k), 127, np.int8)
    wq = np.full((n, k), -128, np.int8)
    wq[::2] = 127
    _, acc = ops.i8_gemm(dev(xq), dev(wq), want_acc=True, want_y=False)
    want = xq.astype(np.int64) @ wq.astype(np.int64).T
    np.testing.assert_array_equal(host(acc), want)


def test_int8_quantlinear_config(ops):
    # smallest benchmark configuration: W [512,512] N(0,0.02), X [32,512] N(0,1), b N(0,0.01), seed 0
    say("Int8Linear 32x512x512 seed 0")
    from rumus_amd import nn
    w, x, b = workloads.int8_linear(0)
    want_y, want_acc, (xq, sx, wq, sw) = oracle.i8_linear(x, w, b)
    layer = nn.Int8Linear.from_linear(nn.Linear(dev(w), dev(b)))
    np.testing.assert_array_equal(host(layer.wq), wq)
    np.testing.assert_array_equal(host(layer.sw), sw)
    y, acc = layer.forward(dev(x), want_acc=True)
    np.testing.assert_array_equal(host(acc), want_acc)
    assert_close(host(y), want_y)


def test_i8_gemm_prefill_shape_properties(ops):
    # the INT8 benchmark shape at full size: 2048 x 4096 x 11008.  The oracle checks a
    # sample of rows exactly; the rest is pinned by a row/column checksum
    # identity computed in int64 on the host.
    say("i8_gemm 2048x4096x11008")
    x, w = workloads.int8_gemm(0)
    xq_t, sx_t = ops.i8_quantize_rows(dev(x))
    wq_t, sw_t = ops.i8_quantize_cols_t(dev(w))
    xq, wq = host(xq_t), host(wq_t)
    rows = [0, 1, 777, 2047]
    wq_o, sw_o = oracle.i8_quantize_rows(np.ascontiguousarray(w.T[:64]))
    np.testing.assert_array_equal(wq[:64], wq_o)
    xq_o, sx_o = oracle.i8_quantize_rows(x[rows])
    np.testing.assert_array_equal(xq[rows], xq_o)
    y, acc = ops.i8_gemm(xq_t, wq_t, sx_t, sw_t, None, want_acc=True)
    acc = host(acc)
    np.testing.assert_array_equal(acc[rows], oracle.i8_gemm_i32(xq[rows], wq, threads=8))
    # checksum of checksums: sum_m acc[m,:] == (sum_m xq[m,:]) @ wq^T, and the same by columns
    np.testing.assert_array_equal(acc.sum(0, dtype=np.int64),
                                  xq.sum(0, dtype=np.int64) @ wq.astype(np.int64).T)
    np.testing.assert_array_equal(acc.sum(1, dtype=np.int64),
                                  xq.astype(np.int64) @ wq.sum(0, dtype=np.int64))
    yh = host(y)
    np.testing.assert_array_equal(yh[rows], oracle.i8_rescale_bias(acc[rows], host(sx_t)[rows], host(sw_t), None))
