"""Runs the C++ host-mirror test (tests/host_cpp/test_host.cpp) on the GPU, and exchanges stored
INT4 layers with it: a file written by either side loads on the other and computes the same bits."""
import os
import subprocess

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))
BIN = os.path.join(HERE, "host_cpp", "test_host")


def test_cpp_host_mirror_matches_oracle(tmp_path):
    print("[gpu-case] C++ host mirror: QLinear / Q8 / Int8Linear / stored layers", flush=True)
    if not os.path.exists(BIN):
        import __graft_entry__
        __graft_entry__.build_host_cpp_test()
    import torch
    from safetensors.numpy import load_file, save_file
    from rumus_amd import checkpoint as ck, ops
    from gpu_util import dev, host

    # what the Python side leaves for the C++ loader: a GPTQ-style file written by the safetensors
    # package (f16 scales, u4 zero-points, g_idx) and a plain layer written by save_w4
    rng = np.random.default_rng(41)
    k, n, g, m = 256, 48, 64, 2
    w = (rng.standard_normal((k, n)) * 0.02).astype(np.float32)
    packed, scales, qzeros = (host(t) for t in ops.w4_quantize_pack_awq(dev(w), g))
    g_idx = (rng.permutation(k) // g).astype(np.int32)
    foreign = {"a.qweight": packed.view(np.int32), "a.scales": scales.astype(np.float16),
               "a.qzeros": qzeros.view(np.int32), "a.g_idx": g_idx,
               "a.bias": rng.standard_normal(n).astype(np.float32)}
    meta = {"format": ck.FORMAT, "version": ck.VERSION, "a.k": str(k), "a.group_size": str(g)}
    save_file(foreign, str(tmp_path / "py.safetensors"), metadata=meta)
    x = rng.standard_normal((m, k)).astype(np.float32)
    x.tofile(tmp_path / "py_x.bin")

    # a decoder block for the C++ mirror of DecoderBlockW4: seven stored layers, a prefill input and one
    # decode token; small enough for a test, large enough for the matrix-core attention (64 rows or more)
    from rumus_amd import nn
    heads, ffn, gs, batch, ntok, cache_len = 2, 512, 64, 2, 70, 96
    dim = heads * 128
    shapes = {"q": (dim, dim), "k": (dim, dim), "v": (dim, dim), "o": (dim, dim), "gate": (dim, ffn),
              "up": (dim, ffn), "down": (ffn, dim)}
    wts = {name: dev((rng.standard_normal(sh) * 0.05).astype(np.float32)) for name, sh in shapes.items()}
    blk = nn.DecoderBlockW4.from_f32(wts, gs, heads)
    ck.save_w4(str(tmp_path / "block.safetensors"), blk.proj)
    bx = rng.standard_normal((batch, ntok, dim)).astype(np.float32)
    bx1 = rng.standard_normal((batch, 1, dim)).astype(np.float32)
    bx.tofile(tmp_path / "block_x.bin")
    bx1.tofile(tmp_path / "block_x1.bin")
    (tmp_path / "block_cfg.txt").write_text(f"{batch} {ntok} {heads} {cache_len}\n")

    out = subprocess.run([BIN, str(tmp_path)], capture_output=True, text=True, timeout=300)
    print(out.stdout)
    print(out.stderr)
    assert out.returncode == 0, out.stdout[-2000:]
    assert "all passed" in out.stdout

    # the C++ loader on the Python-side file: same output bits as the Python loader
    mine = ck.load_w4(str(tmp_path / "py.safetensors"))["a"]
    y_cpp = np.fromfile(tmp_path / "py_y_a.bin", dtype=np.float32).reshape(m, n)
    np.testing.assert_array_equal(y_cpp, host(mine(dev(x))))

    # the C++ writer's file: valid for the safetensors package, and the Python loader computes
    # the bits the C++ side computed before saving
    raw = load_file(str(tmp_path / "cpp.safetensors"))
    assert {"blk.plain.qweight", "blk.plain.scales", "blk.plain.zeros", "blk.plain.bias",
            "blk.act_order.qweight", "blk.act_order.perm"} <= set(raw)
    layers = ck.load_w4(str(tmp_path / "cpp.safetensors"))
    plain = layers["blk.plain"]
    xc = np.fromfile(tmp_path / "cpp_x.bin", dtype=np.float32).reshape(-1, plain.in_features)
    yc = np.fromfile(tmp_path / "cpp_y.bin", dtype=np.float32).reshape(xc.shape[0], plain.out_features)
    np.testing.assert_array_equal(host(plain(dev(xc))), yc)
    assert layers["blk.act_order"].weight.perm is not None
    assert torch.equal(layers["blk.act_order"].weight.scales_tensor, plain.weight.scales_tensor)

    # the C++ decoder block on the stored layers: the bits of the Python block, prefill and decode step
    y_py, k_py, v_py = blk(dev(bx))
    kc = torch.zeros((batch, cache_len, heads, 128), dtype=torch.float32, device="cuda")
    vc = torch.zeros_like(kc)
    kc[:, :ntok] = k_py
    vc[:, :ntok] = v_py
    y1_py, kc, vc = blk(dev(bx1), kc, vc, pos=ntok)
    y_cpp = np.fromfile(tmp_path / "block_y.bin", dtype=np.float32).reshape(batch, ntok, dim)
    y1_cpp = np.fromfile(tmp_path / "block_y1.bin", dtype=np.float32).reshape(batch, 1, dim)
    k_cpp = np.fromfile(tmp_path / "block_k.bin", dtype=np.float32).reshape(batch, cache_len, heads, 128)
    np.testing.assert_array_equal(y_cpp, host(y_py))
    np.testing.assert_array_equal(k_cpp, host(kc))
    np.testing.assert_array_equal(y1_cpp, host(y1_py))
