"""GPU parity of the f32 operators around the projections and of a whole INT4 decoder block."""
import numpy as np
import pytest

import oracle
from rumus_amd import workloads

from gpu_util import dev, host, say

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from rumus_amd import ops as o
    return o


def close(got, want, rtol=1e-3, atol=1e-4):
    np.testing.assert_allclose(got, want, rtol=rtol, atol=atol)


@pytest.mark.parametrize("rows,dim", [(1, 4096), (7, 100), (130, 11008)])
def test_rmsnorm(ops, rows, dim):
    say(f"rmsnorm {rows}x{dim}")
    rng = np.random.default_rng(rows + dim)
    x = rng.normal(0, 2, (rows, dim)).astype(np.float32)
    w = rng.normal(1, 0.1, dim).astype(np.float32)
    close(host(ops.rmsnorm(dev(x), dev(w), 1e-6)), oracle.rmsnorm(x, w, 1e-6), atol=1e-5)


def test_swiglu_and_add(ops):
    say("swiglu / add")
    rng = np.random.default_rng(2)
    g = rng.normal(0, 3, (5, 1001)).astype(np.float32)
    u = rng.normal(0, 1, (5, 1001)).astype(np.float32)
    g[0, :4] = [-100.0, 100.0, 0.0, -20.0]
    close(host(ops.swiglu(dev(g), dev(u))), oracle.swiglu(g, u), atol=1e-6)
    close(host(ops.swiglu_rows(dev(np.concatenate([g, u], axis=1)))), oracle.swiglu(g, u), atol=1e-6)
    np.testing.assert_array_equal(host(ops.add(dev(g), dev(u))), g + u)


@pytest.mark.parametrize("rows,dim", [(1, 4096), (7, 100), (3, 8200), (130, 11008)])
def test_add_rmsnorm_is_add_then_rmsnorm(ops, rows, dim):
    say(f"add_rmsnorm {rows}x{dim}")
    rng = np.random.default_rng(rows * 3 + dim)
    x = rng.normal(0, 2, (rows, dim)).astype(np.float32)
    d = rng.normal(0, 1, (rows, dim)).astype(np.float32)
    w = rng.normal(1, 0.1, dim).astype(np.float32)
    s, y = ops.add_rmsnorm(dev(x), dev(d), dev(w), 1e-6)
    np.testing.assert_array_equal(host(s), x + d)
    close(host(y), oracle.rmsnorm(x + d, w, 1e-6), atol=1e-5)
    # the same bits as the two separate launches
    s2 = ops.add(dev(x), dev(d))
    np.testing.assert_array_equal(host(y), host(ops.rmsnorm(s2, dev(w), 1e-6)))
    # the sum written over the delta (the residual stream updated in place)
    dd = dev(d)
    s3, y3 = ops.add_rmsnorm(dev(x), dd, dev(w), 1e-6, sum_out=dd)
    assert s3.data_ptr() == dd.data_ptr()
    np.testing.assert_array_equal(host(s3), x + d)
    np.testing.assert_array_equal(host(y3), host(y))
    with pytest.raises(Exception, match="must not alias"):
        ops.add_rmsnorm(dd, dd, dev(w), 1e-6, out=dd)


@pytest.mark.parametrize("m,k,n,g", [(1, 11008, 4096, 128), (3, 512, 48, 64), (5, 264, 16, 256), (8, 1024, 272, 32)])
def test_decode_gemv_with_swiglu_input(ops, m, k, n, g):
    say(f"qmatmul_int4_decode_swiglu m={m} k={k} n={n} g={g}")
    rng = np.random.default_rng(m + k + n)
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    gu = rng.normal(0, 2, (m, 2 * k)).astype(np.float32)
    gu[0, :3] = [-100.0, 100.0, 0.0]
    b = rng.normal(0, 0.01, n).astype(np.float32)
    packed, scales, zp = oracle.w4_from_f32(w, g)
    pt, st, zt = ops.w4_decode_layout(dev(packed), dev(scales), dev(zp), g)
    got = host(ops.qmatmul_int4_decode_swiglu(dev(gu), pt, st, zt, k, g, bias=dev(b)))
    x = oracle.swiglu(gu[:, :k], gu[:, k:]).astype(np.float32)
    close(got, oracle.qmatmul_int4(x, packed, scales, zp, k, g, bias=b, threads=8))
    # the same bits as the SwiGLU kernel followed by the decode kernel
    act = ops.swiglu_rows(dev(gu))
    np.testing.assert_array_equal(got, host(ops.qmatmul_int4_decode(act, pt, st, zt, k, g, bias=dev(b))))
    with pytest.raises(Exception, match="gate_up must be"):
        ops.qmatmul_int4_decode_swiglu(dev(gu[:, :k]), pt, st, zt, k, g)


@pytest.mark.parametrize("m,k,n,g", [(1, 4096, 4096, 128), (1, 11008, 1024, 128), (3, 512, 48, 64), (5, 264, 16, 256),
                                     (8, 1024, 272, 32), (2, 5120, 640, 128)])
def test_decode_projection_with_the_block_folded_in(ops, m, k, n, g):
    """qmatmul_int4_decode_block: RMSNorm or SwiGLU on the way in, residual on the way out, one launch; against
    the operators one after the other (oracle), and against the separate kernels."""
    say(f"qmatmul_int4_decode_block m={m} k={k} n={n} g={g}")
    rng = np.random.default_rng(3 * m + k + n)
    w = rng.normal(0, 0.02, (k, n)).astype(np.float32)
    x = rng.normal(0, 2, (m, k)).astype(np.float32)
    if m > 1:
        x[1] *= 1e-3                                          # rows of different size: the norm is per row
    nw = rng.normal(1, 0.2, k).astype(np.float32)
    b = rng.normal(0, 0.01, n).astype(np.float32)
    r = rng.normal(0, 1, (m, n)).astype(np.float32)
    packed, scales, zp = oracle.w4_from_f32(w, g)
    pt, st, zt = ops.w4_decode_layout(dev(packed), dev(scales), dev(zp), g)
    # RMSNorm -> projection -> + bias + residual
    hn = oracle.rmsnorm(x, nw, 1e-5).astype(np.float32)
    want = oracle.qmatmul_int4(hn, packed, scales, zp, k, g, bias=b, threads=8) + r
    got = host(ops.qmatmul_int4_decode_block(dev(x), pt, st, zt, k, g, norm_weight=dev(nw), eps=1e-5, bias=dev(b),
                                             residual=dev(r)))
    close(got, want)
    # the norm alone, against the two kernels it replaces (the factor meets the sum instead of x: rounding only)
    two = host(ops.qmatmul_int4_decode(ops.rmsnorm(dev(x), dev(nw), 1e-5), pt, st, zt, k, g))
    one = host(ops.qmatmul_int4_decode_block(dev(x), pt, st, zt, k, g, norm_weight=dev(nw), eps=1e-5))
    np.testing.assert_allclose(one, two, rtol=2e-5, atol=2e-5)
    # SwiGLU -> projection -> residual accumulated in place
    gu = rng.normal(0, 2, (m, 2 * k)).astype(np.float32)
    acc = dev(r)
    out = ops.qmatmul_int4_decode_block(dev(gu), pt, st, zt, k, g, swiglu=True, residual=acc, out=acc)
    assert out.data_ptr() == acc.data_ptr()
    plain = host(ops.qmatmul_int4_decode_swiglu(dev(gu), pt, st, zt, k, g))
    np.testing.assert_array_equal(host(out), plain + r)       # one add per element: the same bits
    # nothing folded in: the decode kernel itself
    np.testing.assert_array_equal(host(ops.qmatmul_int4_decode_block(dev(x), pt, st, zt, k, g)),
                                  host(ops.qmatmul_int4_decode(dev(x), pt, st, zt, k, g)))
    with pytest.raises(Exception, match="exclude each other"):
        ops.qmatmul_int4_decode_block(dev(gu), pt, st, zt, k, g, norm_weight=dev(nw), swiglu=True)
    with pytest.raises(Exception, match="residual must be"):
        ops.qmatmul_int4_decode_block(dev(x), pt, st, zt, k, g, residual=dev(r[:, :n - 1]))


@pytest.mark.parametrize("b,h,nq,nkv,causal", [
    (1, 2, 64, 64, True), (2, 3, 100, 100, True), (1, 2, 70, 70, False), (1, 4, 33, 97, True),
    (2, 32, 1, 2048, False), (3, 2, 1, 1, False), (1, 2, 1, 300, True), (1, 1, 512, 512, True),
    (1, 2, 200, 333, True), (2, 2, 130, 130, True), (1, 3, 64, 500, False), (1, 1, 129, 160, True)])
def test_attention_vs_float64(ops, b, h, nq, nkv, causal):
    say(f"attention b={b} h={h} nq={nq} nkv={nkv} causal={causal}")
    rng = np.random.default_rng(b * 1000 + nq + nkv)
    q = rng.normal(0, 1, (b, nq, h, 128)).astype(np.float32)
    k = rng.normal(0, 1, (b, nkv, h, 128)).astype(np.float32)
    v = rng.normal(0, 1, (b, nkv, h, 128)).astype(np.float32)
    close(host(ops.attention(dev(q), dev(k), dev(v), causal)), oracle.attention(q, k, v, causal), atol=2e-5)


def test_attention_reads_strided_views(ops):
    # operands as slices of wider buffers (a fused qkv output, a longer cache): only strides change
    say("attention strided")
    rng = np.random.default_rng(4)
    b, n, h = 2, 40, 3
    qkv = rng.normal(0, 1, (b, n, 3, h, 128)).astype(np.float32)
    t = dev(qkv)
    got = host(ops.attention(t[:, :, 0], t[:, :, 1], t[:, :, 2], True))
    close(got, oracle.attention(qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2], True), atol=2e-5)


def test_attention_rejects_bad_arguments(ops):
    import torch
    from rumus_amd._lib import RumusError
    q = torch.zeros((1, 4, 2, 64), device="cuda")
    with pytest.raises(RumusError):
        ops.attention(q, q, q, True)                       # head_dim != 128
    q = torch.zeros((1, 4, 2, 128), device="cuda")
    with pytest.raises(RumusError):
        ops.attention(q, q[:, :2], q[:, :2], True)         # more queries than keys


@pytest.mark.parametrize("layout", ["token_major", "reference"])
@pytest.mark.parametrize("b,h,n,pos,cache_len", [(1, 32, 1, 2047, 2048), (3, 2, 1, 0, 5), (2, 3, 20, 7, 40),
                                                 (8, 4, 64, 0, 64)])
def test_kv_append_is_an_exact_copy(ops, layout, b, h, n, pos, cache_len):
    # the reference's cache is [batch, heads, cached_len, head_dim] (rumus-serve/src/model.rs:11-14); the
    # block here keeps it token-major.  Both are the same call with other strides.  The new entries are
    # the k and v slices of a fused q|k|v projection output, read in place.
    say(f"kv_append {layout} b={b} h={h} n={n} pos={pos} T={cache_len}")
    import torch
    rng = np.random.default_rng(b * 100 + n + pos)
    qkv = rng.normal(0, 1, (b, n, 3, h, 128)).astype(np.float32)
    shape = (b, cache_len, h, 128) if layout == "token_major" else (b, h, cache_len, 128)
    kc0 = rng.normal(0, 1, shape).astype(np.float32)
    vc0 = rng.normal(0, 1, shape).astype(np.float32)
    t, kc, vc = dev(qkv), dev(kc0), dev(vc0)
    view = (lambda c: c) if layout == "token_major" else (lambda c: c.transpose(1, 2))
    ops.kv_append(t[:, :, 1], t[:, :, 2], view(kc), view(vc), pos)
    want_k, want_v = kc0.copy(), vc0.copy()
    if layout == "token_major":
        want_k[:, pos:pos + n], want_v[:, pos:pos + n] = qkv[:, :, 1], qkv[:, :, 2]
    else:
        want_k[:, :, pos:pos + n] = qkv[:, :, 1].transpose(0, 2, 1, 3)
        want_v[:, :, pos:pos + n] = qkv[:, :, 2].transpose(0, 2, 1, 3)
    np.testing.assert_array_equal(host(kc), want_k)          # new rows in place, every other entry untouched
    np.testing.assert_array_equal(host(vc), want_v)
    torch.cuda.synchronize()


@pytest.mark.parametrize("layout", ["token_major", "reference"])
@pytest.mark.parametrize("b,h,pos,cache_len", [(1, 32, 2047, 2048), (3, 2, 0, 5), (2, 3, 255, 300), (2, 3, 256, 300),
                                               (1, 4, 4, 5),
                                               # slices of 256 keys (batch * heads * slices >= 512): the last slice
                                               # full, and the last slice holding the new key alone
                                               (2, 32, 2047, 2048), (2, 32, 1792, 1800)])
def test_attention_decode_append_is_append_then_attention(ops, layout, b, h, pos, cache_len):
    """One call for the cache write of the newest token and the attention of its query: the same bits in the output
    and in the caches as kv_append followed by attention, on both cache layouts, at the first and the last
    position, across a slice boundary of the decode kernel and with slices of 64, 128 and 256 keys."""
    say(f"attention_decode_append {layout} b={b} h={h} pos={pos} T={cache_len}")
    rng = np.random.default_rng(7 * b + h + pos)
    qkv = rng.normal(0, 1, (b, 1, 3, h, 128)).astype(np.float32)
    shape = (b, cache_len, h, 128) if layout == "token_major" else (b, h, cache_len, 128)
    kc0 = rng.normal(0, 1, shape).astype(np.float32)
    vc0 = rng.normal(0, 1, shape).astype(np.float32)
    view = (lambda c: c) if layout == "token_major" else (lambda c: c.transpose(1, 2))
    t = dev(qkv)
    q, k, v = t[:, :, 0], t[:, :, 1], t[:, :, 2]
    kc, vc = dev(kc0), dev(vc0)
    ops.kv_append(k, v, view(kc), view(vc), pos)
    want = host(ops.attention(q, view(kc)[:, :pos + 1], view(vc)[:, :pos + 1], causal=False))
    kc2, vc2 = dev(kc0), dev(vc0)
    got = host(ops.attention_decode_append(q, k, v, view(kc2), view(vc2), pos))
    np.testing.assert_array_equal(got, want)
    np.testing.assert_array_equal(host(kc2), host(kc))
    np.testing.assert_array_equal(host(vc2), host(vc))
    # against float64 as well
    kk = host(view(kc))[:, :pos + 1]
    vv = host(view(vc))[:, :pos + 1]
    close(got, oracle.attention(qkv[:, :, 0], kk, vv, False), atol=2e-5)


def test_attention_decode_append_rejects_bad_arguments(ops):
    import torch
    from rumus_amd._lib import RumusError
    q = torch.zeros((1, 1, 2, 128), device="cuda")
    cache = torch.zeros((1, 4, 2, 128), device="cuda")
    with pytest.raises(RumusError, match="does not fit"):
        ops.attention_decode_append(q, q, q, cache, cache.clone(), 4)
    with pytest.raises(ValueError, match="must be"):
        ops.attention_decode_append(torch.zeros((1, 2, 2, 128), device="cuda"), q, q, cache, cache.clone(), 0)
    with pytest.raises(ValueError, match="do not match"):
        ops.attention_decode_append(q, q, q, torch.zeros((1, 4, 3, 128), device="cuda"), cache, 0)


def test_kv_append_rejects_bad_arguments(ops):
    import torch
    from rumus_amd._lib import RumusError
    new = torch.zeros((1, 2, 2, 128), device="cuda")
    cache = torch.zeros((1, 8, 2, 128), device="cuda")
    with pytest.raises(RumusError, match="do not fit"):
        ops.kv_append(new, new, cache, cache, 7)               # positions 7..8 of a cache of 8
    with pytest.raises(ValueError):
        ops.kv_append(new, new, cache[:, :, :1], cache[:, :, :1], 0)   # head counts differ
    odd = torch.zeros((1, 2, 2, 130), device="cuda")
    with pytest.raises(RumusError, match="multiple of 4"):
        ops.kv_append(odd, odd, torch.zeros((1, 8, 2, 130), device="cuda"), torch.zeros((1, 8, 2, 130), device="cuda"), 0)


def _block(ops, dim, ffn, heads, g):
    import torch
    from rumus_amd import nn
    w = workloads.decoder_block(dim, ffn)
    blk = nn.DecoderBlockW4.from_f32({k: dev(v) for k, v in w.items()}, g, heads)
    wd = {}
    for name, lin in blk.proj.items():
        qt = lin.weight
        wd[name] = oracle.w4_dequant(host(qt.packed_tensor).view(np.uint32), host(qt.scales_tensor),
                                     host(qt.zp_tensor), qt.k, g)
    torch.cuda.synchronize()
    return blk, wd


def test_decoder_block_small(ops):
    say("decoder block 256/704, prefill then decode")
    dim, ffn, heads, g = 256, 704, 2, 64
    blk, wd = _block(ops, dim, ffn, heads, g)
    x, _, _ = workloads.decoder_block_inputs(3, 20, dim)
    y, k, v = blk(dev(x))
    want_y, want_k, want_v = oracle.decoder_block(x, wd, heads)
    close(host(y), want_y, atol=1e-4)
    close(host(k), want_k, atol=1e-4)
    # decode the next token against the cache the prefill produced
    import torch
    kc = torch.zeros((3, 32, heads, 128), device="cuda")
    vc = torch.zeros_like(kc)
    kc[:, :20].copy_(k)
    vc[:, :20].copy_(v)
    x1, _, _ = workloads.decoder_block_inputs(3, 1, dim, seed=8)
    y1, _, _ = blk(dev(x1), kc, vc, pos=20)
    kc_ref = np.zeros((3, 32, heads, 128))
    vc_ref = np.zeros_like(kc_ref)
    kc_ref[:, :20], vc_ref[:, :20] = want_k, want_v
    want_y1, _, _ = oracle.decoder_block(x1, wd, heads, kc_ref, vc_ref, pos=20)
    close(host(y1), want_y1, atol=1e-4)


def test_decoder_block_llama7b_shape(ops):
    # the benchmark's decoder-block configuration at full width: decode at position 2047 against a
    # 2047-entry cache, and a (shortened) prefill of 2 x 192 tokens.
    say("decoder block 4096/11008, decode at 2047 and prefill 2x192")
    import torch
    dim, ffn, heads, g = 4096, 11008, 32, 128
    blk, wd = _block(ops, dim, ffn, heads, g)
    x, kc, vc = workloads.decoder_block_inputs(1, 1, dim, cache_len=2048, heads=heads)
    y, _, _ = blk(dev(x), dev(kc), dev(vc), pos=2047)
    want, _, _ = oracle.decoder_block(x, wd, heads, kc, vc, pos=2047)
    err = np.abs(host(y) - want).max()
    say(f"  decode max abs err {err:.2e} (|y| max {np.abs(want).max():.2f})")
    close(host(y), want, atol=1e-4)
    xp, _, _ = workloads.decoder_block_inputs(2, 192, dim, seed=9)
    yp, _, _ = blk(dev(xp))
    wantp, _, _ = oracle.decoder_block(xp, wd, heads)
    err = np.abs(host(yp) - wantp).max()
    say(f"  prefill max abs err {err:.2e} (|y| max {np.abs(wantp).max():.2f})")
    close(host(yp), wantp, atol=1e-4)
    torch.cuda.synchronize()


def test_decoder_block_llama7b_full_prefill(ops):
    # the benchmark's prefill at its full size: 8 sequences of 512 tokens, 4096 rows through every
    # projection (other tile and round plans than a few hundred rows take), checked in full against
    # the float64 block on the dequantized weights; then each sequence's last token is decoded again
    # against the cache the prefill filled (kv_append at position 511) and must reproduce its row.
    say("decoder block 4096/11008, prefill 8x512")
    import torch
    dim, ffn, heads, g = 4096, 11008, 32, 128
    blk, wd = _block(ops, dim, ffn, heads, g)
    xp, _, _ = workloads.decoder_block_inputs(8, 512, dim, seed=9)
    yp, kp, vp = blk(dev(xp))
    got, got_k, got_v = host(yp), host(kp), host(vp)
    want, want_k, want_v = oracle.decoder_block(xp, wd, heads)
    err = np.abs(got - want).max()
    say(f"  prefill max abs err {err:.2e} (|y| max {np.abs(want).max():.2f})")
    close(got, want, atol=1e-4)
    close(got_k, want_k, atol=1e-4)
    close(got_v, want_v, atol=1e-4)
    # linearity in the batch: sequences do not see each other, so a block of two of them gives the same rows
    y2, _, _ = blk(dev(xp[5:7]))
    close(host(y2), got[5:7], atol=2e-4)
    # decode of token 511 against the prefilled cache: same row as the prefill computed
    kc = torch.zeros((8, 512, heads, 128), device="cuda")
    vc = torch.zeros_like(kc)
    ops.kv_append(kp[:, :511], vp[:, :511], kc, vc, 0)
    yd, kc2, vc2 = blk(dev(xp[:, 511:512]), kc, vc, pos=511)
    close(host(yd)[:, 0], want[:, 511], atol=1e-4)
    close(host(kc2), want_k, atol=1e-4)
    torch.cuda.synchronize()
