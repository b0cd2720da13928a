"""gptoss_attn_decode_static (the decode attention on the library's built-in scratch array, no
workspace and no allocation) against gptoss_attn_decode, through the C ABI: bit-identical output on
two calls in a row, the second smaller than the first, then a size beyond the array's limit."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_attn_decode_static_equals_attn_decode(ops):
    from conftest import load_pkg
    lib = load_pkg("lib")
    n_q, n_kv, D, S = 64, 8, 64, 4096
    g = torch.Generator(device="cuda").manual_seed(41)
    B1, B2 = 200, 37
    cache = ops.KVCache(B1, n_kv, D, S)
    cache.kv.copy_(torch.randn(cache.kv.numel(), device="cuda", generator=g).to(torch.bfloat16))
    sinks = torch.randn(n_q, device="cuda", generator=g)
    rng = np.random.default_rng(2)
    attn = ops.AttnDecode(B1, n_q, n_kv, D, S)
    assert attn.ws_bytes <= lib.load().gptoss_attn_decode_static_max_bytes()
    # first call: 200 sequences of up to 4096 positions (up to 9 chunks each go through the scratch);
    # second call: 37 sequences of up to 1500 positions, on what the first call left in the array
    for B, hi, window in ((B1, S, 0), (B2, 1500, 0), (B2, 3000, 128)):
        lens_np = rng.integers(1, hi + 1, size=B).astype(np.int32)
        lens_np[0] = hi
        lens = torch.from_numpy(lens_np).cuda()
        q = torch.randn(B, n_q, D, device="cuda", generator=g)
        small = cache.first(B)
        want = attn.forward(q, small, lens, sinks, window=window, max_len=hi)
        out = torch.full((B, n_q, D), float("nan"), dtype=torch.bfloat16, device="cuda")
        got = ops.attn_decode_static(q, small, lens, n_q, sinks, window=window, max_len=hi, out=out)
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), (B, hi, window)
    # beyond the array: refused with a workspace error, nothing launched
    big_b = 1024
    lens = torch.ones(big_b, dtype=torch.int32, device="cuda")
    q = torch.zeros(big_b, n_q, D, device="cuda")
    assert lib.load().gptoss_attn_workspace_bytes(big_b, n_q, n_kv, D, S) > lib.load().gptoss_attn_decode_static_max_bytes()
    with pytest.raises(lib.GptossError) as ei:
        ops.attn_decode_static(q, ops.KVCache(4, n_kv, D, S), lens, n_q, sinks, max_len=S)
    assert ei.value.code == 4 and "scratch" in str(ei.value)
