"""GPU parity of decode attention (sinks, sliding window, GQA, ragged lengths, ring cache)
against the CPU oracle, through the C ABI."""
import numpy as np
import pytest
import torch

from conftest import TOL_MAX, TOL_MEAN, rel_errors

pytestmark = pytest.mark.gpu


def _mk(B, S, n_q, n_kv, D, seed):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, n_q, D, generator=g)
    K = torch.randn(B, S, n_kv, D, generator=g).to(torch.bfloat16)
    V = torch.randn(B, S, n_kv, D, generator=g).to(torch.bfloat16)
    sinks = torch.randn(n_q, generator=g)
    return q, K, V, sinks


def _run(ops, q, K, V, lens, sinks, window, capacity=None, max_len=None):
    B, S, n_kv, D = K.shape
    n_q = q.shape[1]
    cap = capacity or ((S + 63) // 64 * 64)
    cache = ops.KVCache(B, n_kv, D, cap)
    # never-written slots keep whatever the allocator left there, NaN patterns included
    cache.kv.view(torch.int16).fill_(0x7FC1)
    cache.write(K.cuda(), V.cuda(), 0)
    attn = ops.AttnDecode(B, n_q, n_kv, D, max_len or int(lens.max()))
    out = attn.forward(q.cuda(), cache, torch.as_tensor(lens, dtype=torch.int32).cuda(),
                       None if sinks is None else sinks.cuda(), window=window)
    torch.cuda.synchronize()
    return out.float().cpu().numpy()


@pytest.mark.parametrize("B,n_q,n_kv,D,lens,window", [
    (3, 8, 2, 32, [1, 2, 63], 0),                    # tiny-model heads, very short contexts
    (4, 8, 2, 32, [64, 65, 127, 128], 0),
    (4, 8, 2, 32, [100, 129, 200, 300], 128),        # window smaller than the context
    (5, 64, 8, 64, [1, 17, 256, 257, 700], 0),       # 20B heads, one and several chunks
    (3, 64, 8, 64, [512, 1500, 4096], 0),            # long contexts: 512-token chunks + merge
    (4, 64, 8, 64, [100, 128, 129, 4000], 128),      # sliding window on a full-length cache
    (2, 16, 1, 64, [333, 90], 0),                    # 16 query heads per kv head
    (2, 4, 4, 64, [70, 5], 0),                       # no sharing (MHA)
])
def test_attn_matches_oracle(ops, orc, B, n_q, n_kv, D, lens, window):
    lens = np.asarray(lens, np.int32)
    S = int(lens.max())
    q, K, V, sinks = _mk(B, S, n_q, n_kv, D, seed=S + n_q)
    got = _run(ops, q, K, V, lens, sinks, window)
    want = orc.attn_decode(q.numpy(), K.float().numpy(), V.float().numpy(), lens, sinks.numpy(), window)
    assert np.isfinite(got).all()
    mx, mean = rel_errors(got, want)
    assert mx <= TOL_MAX and mean <= TOL_MEAN, (mx, mean)


def test_attn_no_sink_equals_sdpa(ops):
    """sinks=None reduces to plain softmax attention (checked against torch SDPA)."""
    B, n_q, n_kv, D, S = 2, 64, 8, 64, 300
    q, K, V, _ = _mk(B, S, n_q, n_kv, D, seed=11)
    lens = np.array([S, S], np.int32)
    got = _run(ops, q, K, V, lens, None, 0)
    Kf = K.float().permute(0, 2, 1, 3).repeat_interleave(n_q // n_kv, dim=1)
    Vf = V.float().permute(0, 2, 1, 3).repeat_interleave(n_q // n_kv, dim=1)
    want = torch.nn.functional.scaled_dot_product_attention(q.unsqueeze(2), Kf, Vf).squeeze(2).numpy()
    mx, mean = rel_errors(got, want)
    assert mx <= TOL_MAX and mean <= TOL_MEAN, (mx, mean)


def test_attn_ring_cache_wrapped(ops, orc):
    """A cache of capacity == window holds position p in slot p % capacity; after wrapping the
    result equals attention over the last `window` positions."""
    B, n_q, n_kv, D, W = 3, 8, 2, 32, 128
    total = [130, 256, 301]
    S = max(total)
    q, K, V, sinks = _mk(B, S, n_q, n_kv, D, seed=5)
    cache = ops.KVCache(B, n_kv, D, W)
    Kc, Vc = K.cuda(), V.cuda()
    for p0 in range(0, S, 64):                          # stream the positions through the ring
        n = min(64, S - p0)
        cache.write(Kc[:, p0:p0 + n], Vc[:, p0:p0 + n], p0)
    torch.cuda.synchronize()
    # sequences shorter than S saw extra writes; rebuild per-sequence caches for exactness
    outs = []
    for b in range(B):
        cb = ops.KVCache(1, n_kv, D, W)
        for p0 in range(0, total[b], 50):
            n = min(50, total[b] - p0)
            cb.write(Kc[b:b + 1, p0:p0 + n], Vc[b:b + 1, p0:p0 + n], p0)
        attn = ops.AttnDecode(1, n_q, n_kv, D, max_len=2048)
        o = attn.forward(q[b:b + 1].cuda(), cb, torch.tensor([total[b]], dtype=torch.int32).cuda(),
                         sinks.cuda(), window=W)
        outs.append(o.float().cpu().numpy())
    got = np.concatenate(outs)
    want = orc.attn_decode(q.numpy(), K.float().numpy(), V.float().numpy(),
                           np.asarray(total, np.int32), sinks.numpy(), W)
    mx, mean = rel_errors(got, want)
    assert mx <= TOL_MAX and mean <= TOL_MEAN, (mx, mean)


def test_attn_len1_closed_form(ops):
    """One cached position: o = v * e^s / (e^s + e^sink)."""
    B, n_q, n_kv, D = 2, 8, 2, 32
    q, K, V, sinks = _mk(B, 1, n_q, n_kv, D, seed=3)
    got = _run(ops, q, K, V, np.array([1, 1], np.int32), sinks, 0)
    Kf, Vf = K.float().numpy(), V.float().numpy()
    for b in range(B):
        for h in range(n_q):
            g = h // (n_q // n_kv)
            s = float(q[b, h].numpy() @ Kf[b, 0, g]) / np.sqrt(D)
            w = np.exp(s) / (np.exp(s) + np.exp(float(sinks[h])))
            np.testing.assert_allclose(got[b, h], w * Vf[b, 0, g], rtol=1e-2, atol=1e-2)


def test_attn_without_lengths_means_every_row_has_max_len(ops):
    """lens = NULL (lock-step decoding: the host knows the one length) gives the bits of an array filled
    with max_len, in both launch forms."""
    for B, n_q, n_kv, D, S, L in ((5, 8, 2, 32, 256, 200), (70, 64, 8, 64, 640, 601)):
        q, K, V, sinks = _mk(B, S, n_q, n_kv, D, seed=21)
        cache = ops.KVCache(B, n_kv, D, S)
        cache.write(K.cuda(), V.cuda(), 0)
        attn = ops.AttnDecode(B, n_q, n_kv, D, S)
        lens = torch.full((B,), L, dtype=torch.int32, device="cuda")
        for window in (0, 128):
            a = attn.forward(q.cuda(), cache, lens, sinks.cuda(), window=window, max_len=L).clone()
            b = attn.forward(q.cuda(), cache, None, sinks.cuda(), window=window, max_len=L)
            assert torch.equal(a, b), (B, window)


def test_attn_output_rows_kept_back_equal_rows_stored_at_once(ops):
    """One query row per sequence and contexts of one chunk run on a resident grid that keeps its
    output rows in LDS and writes them 16 bytes at a time after its last row; an output buffer that
    is only 8-byte aligned gets the plain launch, which stores every row as it is finished.  Same bits
    for a few rows (less than one round of the grid), for 1200 and for 8000 workgroup indices (several
    rounds; the last case fills a workgroup's 16 slots and makes it write them in between), with
    ragged lengths, empty rows and both head sizes."""
    for B, n_q, n_kv, D, S in ((3, 8, 2, 32, 128), (600, 16, 8, 64, 192), (4000, 8, 8, 32, 128)):
        q, K, V, sinks = _mk(B, S, n_q, n_kv, D, seed=33)
        cache = ops.KVCache(B, n_kv, D, S)
        cache.write(K.cuda(), V.cuda(), 0)
        attn = ops.AttnDecode(B, n_q, n_kv, D, S)
        g = torch.Generator().manual_seed(7)
        lens = torch.randint(0, S + 1, (B,), generator=g, dtype=torch.int32)
        lens[0] = S
        lens = lens.cuda()
        flat = torch.zeros(B * n_q * D + 8, dtype=torch.bfloat16, device="cuda")
        for window in (0, 64):
            a = attn.forward(q.cuda(), cache, lens, sinks.cuda(), window=window)
            off = flat[4:4 + B * n_q * D].view(B, n_q, D)   # 8 bytes past a 16-byte boundary
            assert off.data_ptr() % 16 == 8
            attn.forward(q.cuda(), cache, lens, sinks.cuda(), window=window, out=off)
            assert torch.equal(a, off), (B, D, window)


def test_attn_bad_arguments(ops):
    import ctypes as C
    from conftest import load_pkg
    lib = load_pkg("lib")
    L = lib.load(strict=False)
    q = torch.zeros(1, 8, 48, device="cuda")
    rc = L.gptoss_attn_decode(C.c_void_p(q.data_ptr()), C.c_void_p(q.data_ptr()), C.c_void_p(q.data_ptr()),
                              None, C.c_void_p(q.data_ptr()), 1, 8, 2, 48, 64, 0,
                              10, C.c_void_p(q.data_ptr()), 1 << 20, None)
    assert rc == 2 and "head_dim" in lib.last_error()
    rc = L.gptoss_attn_decode(None, None, None, None, None, 1, 8, 2, 64, 64, 0, 10, None, 0, None)
    assert rc == 1


def test_attn_many_long_sequences_static_and_ticket_rounds(ops, orc):
    """160 sequences x 8 kv heads: enough for the workgroup-per-row kernel (long rows: four waves
    interleave 64-slot blocks, longest rows first) next to the one-wave kernel (rows of up to 512
    slots); lengths from 0 to the full 4096, the result twice in a row from the same workspace."""
    B, n_q, n_kv, D, S = 160, 16, 8, 64, 4096
    rng = np.random.default_rng(42)
    lens = rng.integers(1, S + 1, size=B).astype(np.int32)
    lens[:4] = [0, 1, S, 513]
    q, K, V, sinks = _mk(B, S, n_q, n_kv, D, seed=3)
    cache = ops.KVCache(B, n_kv, D, S)
    cache.kv.view(torch.int16).fill_(0x7FC1)
    cache.write(K.cuda(), V.cuda(), 0)
    attn = ops.AttnDecode(B, n_q, n_kv, D, S)
    lens_d = torch.as_tensor(lens).cuda()
    a = attn.forward(q.cuda(), cache, lens_d, sinks.cuda(), window=0).float().cpu().numpy()
    b = attn.forward(q.cuda(), cache, lens_d, sinks.cuda(), window=0).float().cpu().numpy()
    assert np.array_equal(a, b)                       # whatever order the rows were dealt in
    want = orc.attn_decode(q.numpy(), K.float().numpy(), V.float().numpy(), lens, sinks.numpy(), 0)
    assert np.isfinite(a).all()
    mx, mean = rel_errors(a, want)
    assert mx <= TOL_MAX and mean <= TOL_MEAN, (mx, mean)
    # the same rows through the other launch form: 32 sequences x 8 kv heads is below the switch, so
    # long rows are 512-slot chunks merged by the reduce kernel.  Rows of one chunk take the same
    # path in both calls (equal bits); longer rows are summed in another order and may differ by a
    # last-bit rounding of the bf16 output here and there.
    n = 32
    few = ops.AttnDecode(n, n_q, n_kv, D, S)
    c = few.forward(q[:n].cuda().contiguous(), cache.first(n), lens_d[:n].contiguous(), sinks.cuda(),
                    window=0).float().cpu().numpy()
    short = lens[:n] <= 512
    assert short.any() and (~short).any()
    assert np.array_equal(a[:n][short], c[short])
    diff = np.abs(a[:n] - c)
    assert diff.max() <= 2.0 ** -7 * np.abs(c).max(), diff.max()
    assert (diff > 0).mean() < 0.02, (diff > 0).mean()


def test_attn_batch_larger_than_one_launch_slice(ops, orc):
    """More sequences than one launch keeps in LDS (2048): the call is sliced internally."""
    B, n_q, n_kv, D, S = 2100, 2, 1, 32, 64
    rng = np.random.default_rng(7)
    lens = rng.integers(1, S + 1, size=B).astype(np.int32)
    q, K, V, sinks = _mk(B, S, n_q, n_kv, D, seed=9)
    got = _run(ops, q, K, V, lens, sinks, 0)
    want = orc.attn_decode(q.numpy(), K.float().numpy(), V.float().numpy(), lens, sinks.numpy(), 0)
    mx, mean = rel_errors(got, want)
    assert mx <= TOL_MAX and mean <= TOL_MEAN, (mx, mean)


@pytest.mark.parametrize("B,T,pos0,n_q,n_kv,D,window", [
    (3, 40, 0, 8, 2, 32, 0),          # tiny-model heads, whole prompt from position 0
    (2, 128, 0, 64, 8, 64, 128),      # 20B heads, the window exactly as long as the prompt
    (2, 300, 0, 64, 8, 64, 128),      # prompt longer than the window (linear cache)
    (2, 70, 500, 64, 8, 64, 0),       # a later slice of a long context: two chunks per row
    (1, 200, 1000, 64, 8, 64, 0),     # rows on both sides of the 1024-position chunk-size change
    (2, 65, 60, 64, 8, 64, 128),      # odd row count (the last row of a sequence has no partner), window edges
    (3, 41, 0, 8, 2, 32, 0),          # odd row count, four query heads per kv head
    (1, 66, 480, 64, 8, 64, 0),       # partners on either side of a chunk boundary (512 / 513 positions)
    (1, 1024, 0, 64, 8, 64, 0),       # the reference's longest prompt: 16 blocks per row group
    (2, 1024, 0, 8, 2, 32, 128),      # the same with the window, head_dim 32
    (1, 1000, 24, 16, 2, 64, 128),    # row groups that start inside a block, 8 query heads per kv head, ragged end
    (2, 20, 0, 8, 2, 32, 0),          # fewer than 32 positions: the row-pair form
])
def test_attn_prefill_rows_equal_decode_calls(ops, orc, B, T, pos0, n_q, n_kv, D, window):
    """Prompt attention = the decode attention of every position at once: row (b, t) must equal, bit
    for bit, the decode call with lens = pos0 + t + 1 on the same cache (whatever else is in the
    launch) while the row's slot range fits one 512-slot chunk; a longer row is summed block by
    block in one pass where the decode call merges chunk partials, so it may differ from it by a
    last-bit rounding of a few outputs.  A sample of rows must match the oracle."""
    S = pos0 + T
    g = torch.Generator().manual_seed(S + n_q)
    q = torch.randn(B, T, n_q, D, generator=g)
    K = torch.randn(B, S, n_kv, D, generator=g).to(torch.bfloat16)
    V = torch.randn(B, S, n_kv, D, generator=g).to(torch.bfloat16)
    sinks = torch.randn(n_q, generator=g)
    cap = (S + 63) // 64 * 64
    cache = ops.KVCache(B, n_kv, D, cap)
    cache.kv.view(torch.int16).fill_(0x7FC1)
    cache.write(K.cuda(), V.cuda(), 0)
    pre = ops.AttnPrefill(B, T, n_q, n_kv, D, S)
    got = pre.forward(q.cuda(), cache, pos0=pos0, sinks=sinks.cuda(), window=window)
    torch.cuda.synchronize()
    assert torch.isfinite(got.float()).all()
    dec = ops.AttnDecode(B, n_q, n_kv, D, S)
    # every row of the short prompts (two consecutive rows share a wave), a sample of the long ones
    for t in (range(T) if T <= 70 else sorted({0, 1, T // 3, T // 2, T - 2, T - 1})):
        lens = torch.full((B,), pos0 + t + 1, dtype=torch.int32)
        one = dec.forward(q[:, t].contiguous().cuda(), cache, lens.cuda(), sinks.cuda(), window=window,
                          max_len=pos0 + t + 1)
        length = pos0 + t + 1
        first_slot = (max(0, length - window) if window else 0) // 64 * 64
        if length - first_slot <= 512:
            assert torch.equal(got[:, t], one), t
        else:
            a, b = got[:, t].float(), one.float()
            assert (a - b).abs().max() <= 2.0 ** -7 * b.abs().max(), t        # one bf16 step at the largest output
            assert (a != b).float().mean() < 0.05, t
        want = orc.attn_decode(q[:, t].numpy(), K.float().numpy(), V.float().numpy(), lens.numpy(), sinks.numpy(),
                               window)
        mx, mean = rel_errors(got[:, t].float().cpu().numpy(), want)
        assert mx <= TOL_MAX and mean <= TOL_MEAN, (t, mx, mean)


def test_attn_prefill_refuses_a_wrapped_window_ring(ops):
    from conftest import load_pkg
    lib = load_pkg("lib")
    cache = ops.KVCache(1, 8, 64, 128)
    pre = ops.AttnPrefill(1, 200, 64, 8, 64, 200)
    with pytest.raises(lib.GptossError):
        pre.forward(torch.zeros(1, 200, 64, 64).cuda(), cache, window=128)
