"""The loader: an fp32 payload in .bin tensor order (run.cpp:194-233) goes through the engine's
pinned, double-buffered staging pipeline into the kernels' device layouts.  Every tensor of the
device image is compared, byte for byte, with what the op-level entry points make of the same
tensor (gptoss_pack_weight, whose layout has a test of its own, and plain bf16 conversion), for the
tiny .bin and for a payload with the GPT-OSS-20B dimensions (11 GB, several staging chunks per
tensor, chunk boundaries inside the expert tensors)."""
import dataclasses
import time

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _expected(ops, name, t):
    """Device bytes the engine must hold for payload tensor `t` (numpy fp32, one layer's share)."""
    g = torch.from_numpy(np.ascontiguousarray(t)).cuda()
    if name in ("embedding", "gate_weight"):
        return g.to(torch.bfloat16).contiguous().view(torch.uint8).flatten()
    if name in ("unembedding", "qkv_weight", "out_weight", "mlp2_weight"):
        return ops.pack_weight(g).view(torch.uint8).flatten()
    if name == "mlp1_weight":
        return ops.pack_weight(g, glu=True).view(torch.uint8).flatten()
    return g.contiguous().view(torch.uint8).flatten()          # fp32 vectors


def _check_image(ops, binfmt, cfg, flat, eng):
    off = 0
    n_cmp = 0
    for name, shape in binfmt.tensor_shapes(cfg).items():
        n = int(np.prod(shape))
        t = flat[off:off + n].reshape(shape)
        off += n
        if name in ("embedding", "unembedding", "final_norm"):
            got, want = eng.tensor(name), _expected(ops, name, t)
            assert got.numel() == want.numel() and torch.equal(got, want), name
            n_cmp += 1
            continue
        for l in range(cfg.n_layers):
            got, want = eng.tensor(name, l), _expected(ops, name, t[l])
            assert got.numel() == want.numel() and torch.equal(got, want), (name, l)
            n_cmp += 1
            del got, want
    assert off == flat.size
    return n_cmp


def test_device_image_of_the_tiny_bin(ops, binfmt, synth, tmp_path):
    cfg = synth.tiny_config(2048)
    path = str(tmp_path / "tiny.bin")
    binfmt.write_bin(path, cfg, synth.random_tensors(cfg, 8))
    flat = np.fromfile(path, dtype="<f4", offset=binfmt.HEADER_BYTES)
    eng = ops.Engine(cfg, flat, max_batch=2, max_seq=16)
    assert _check_image(ops, binfmt, cfg, flat, eng) == 3 + 13 * cfg.n_layers
    eng.close()


def test_device_image_at_20b_dimensions_and_load_rate(ops, binfmt, synth):
    from test_fullsize_gpu import _payload_20b
    cfg = dataclasses.replace(synth.gptoss20b_config(max_seq_len=64), n_layers=2)
    flat = _payload_20b(binfmt, cfg, 77)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    eng = ops.Engine(cfg, flat, max_batch=2, max_seq=16, prefill=False)
    dt = time.perf_counter() - t0
    print(f"loaded {flat.nbytes / 1e9:.1f} GB of fp32 payload in {dt:.2f} s = {flat.nbytes / dt / 1e9:.1f} GB/s")
    _check_image(ops, binfmt, cfg, flat, eng)
    eng.close()
    del flat
    torch.cuda.empty_cache()
