"""Two host threads inside the library at once, on ONE stream (the reference runs ops from several threads,
rumus/src/nn/parallel.rs:84).  Calls that queue several kernels talking through the stream's workspace
must come out as if they had been made one after the other."""
import threading

import numpy as np
import pytest

import oracle

from gpu_util import assert_close, dev, host, say

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from rumus_amd import ops as o
    return o


def _run_threads(workers):
    errors = []

    def guard(fn):
        def run():
            try:
                fn()
            except BaseException as exc:     # report in the main thread
                errors.append(exc)
        return run

    threads = [threading.Thread(target=guard(w)) for w in workers]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    if errors:
        raise errors[0]


def test_two_threads_share_one_stream(ops):
    import torch
    from rumus_amd import nn
    say("threads: K-split qmatmul_int4 (m=16), qmatmul_int4_t and matmul_q8 from two threads on one stream")
    rng = np.random.default_rng(77)
    k, n, g = 4096, 1024, 128
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    packed, scales, zp = oracle.w4_from_f32(w, g)
    pd, sd, zd = dev(packed), dev(scales), dev(zp)
    xs = [dev(rng.normal(0, 1, (16, k)).astype(np.float32)) for _ in range(4)]
    gys = [dev(rng.normal(0, 1, (16, n)).astype(np.float32)) for _ in range(4)]
    k8, n8, bs = 2048, 512, 2048
    w8 = rng.normal(0, 0.02, (k8, n8)).astype(np.float32)
    wq = nn.quantize(dev(w8), bs)
    a8 = [dev(rng.normal(0, 1, (32 + 8 * i, k8)).astype(np.float32)) for i in range(4)]
    stream = torch.cuda.current_stream()

    # serial results first (also warms the workspace to its largest size on this stream)
    want_fw = [host(ops.qmatmul_int4(x, pd, sd, zd, k, g)) for x in xs]
    want_bw = [host(ops.qmatmul_int4_t(gy, pd, sd, zd, k, g)) for gy in gys]
    want_q8 = [host(nn.matmul(a, wq)) for a in a8]
    assert_close(want_fw[0], oracle.qmatmul_int4(host(xs[0]), packed, scales, zp, k, g, threads=8))

    rounds = 60
    got_fw = [[None] * rounds for _ in xs]
    got_bw = [[None] * rounds for _ in gys]
    got_q8 = [[None] * rounds for _ in a8]
    start = threading.Barrier(2)

    def w4_worker():
        with torch.cuda.stream(stream):
            start.wait()
            for r in range(rounds):
                for i, x in enumerate(xs):
                    got_fw[i][r] = ops.qmatmul_int4(x, pd, sd, zd, k, g)
                    got_bw[i][r] = ops.qmatmul_int4_t(gys[i], pd, sd, zd, k, g)

    def q8_worker():
        with torch.cuda.stream(stream):
            start.wait()
            for r in range(rounds):
                for i, a in enumerate(a8):
                    got_q8[i][r] = nn.matmul(a, wq)

    _run_threads([w4_worker, q8_worker])
    torch.cuda.synchronize()
    for i in range(4):
        for r in range(rounds):
            np.testing.assert_array_equal(host(got_fw[i][r]), want_fw[i], err_msg=f"qmatmul_int4 x{i} round {r}")
            np.testing.assert_array_equal(host(got_bw[i][r]), want_bw[i], err_msg=f"qmatmul_int4_t gy{i} round {r}")
            np.testing.assert_array_equal(host(got_q8[i][r]), want_q8[i], err_msg=f"matmul_q8 a{i} round {r}")


def test_two_threads_on_their_own_streams(ops):
    import torch
    say("threads: one stream each, workspaces grown inside the threads")
    rng = np.random.default_rng(78)
    k, n, g = 2048, 2048, 128
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    packed, scales, zp = oracle.w4_from_f32(w, g)
    pd, sd, zd = dev(packed), dev(scales), dev(zp)
    xs = [dev(rng.normal(0, 1, (m, k)).astype(np.float32)) for m in (16, 48)]
    want = [host(ops.qmatmul_int4(x, pd, sd, zd, k, g)) for x in xs]
    torch.cuda.synchronize()
    outs = [[], []]

    def worker(i):
        def run():
            s = torch.cuda.Stream()
            with torch.cuda.stream(s):
                for _ in range(40):
                    outs[i].append(ops.qmatmul_int4(xs[i], pd, sd, zd, k, g))
            s.synchronize()
        return run

    _run_threads([worker(0), worker(1)])
    for i in range(2):
        for y in outs[i]:
            np.testing.assert_array_equal(host(y), want[i])
