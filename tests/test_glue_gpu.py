"""The glue ops of a decode step through their own C-ABI entry points, each against the CPU oracle
or a closed form: embedding gather, RMSNorm (with and without the residual add), dense GEMM at
every row-tile regime, fused classifier arg-max, row arg-max with ties, rotary tables, and the
q/k/v split + rotation + KV-cache store for head dimensions 32 and 64."""
import numpy as np
import pytest
import torch

from conftest import TOL_MAX, TOL_MEAN, rel_errors

pytestmark = pytest.mark.gpu


def test_embedding_lookup(ops):
    g = torch.Generator().manual_seed(1)
    V, H = 1000, 2880
    table = torch.randn(V, H, generator=g).to(torch.bfloat16)
    ids = torch.tensor([0, 999, 5, 5, 123, -3, 4000], dtype=torch.int32)        # out of range: clamped
    got = ops.embedding_lookup(table.cuda(), ids.cuda()).cpu()
    want = table.float()[ids.clamp(0, V - 1).long()]
    assert torch.equal(got, want)


@pytest.mark.parametrize("B,H", [(1, 256), (7, 2880), (300, 2880), (5, 5000), (3, 100)])
def test_rmsnorm_matches_oracle(ops, orc, B, H):
    rng = np.random.default_rng(B + H)
    x = rng.standard_normal((B, H)).astype(np.float32) * 3
    r = rng.standard_normal((B, H)).astype(np.float32)
    w = (1 + 0.1 * rng.standard_normal(H)).astype(np.float32)
    for residual in (None, r):
        xd = torch.from_numpy(x.copy()).cuda()
        t = ops.rmsnorm(xd, torch.from_numpy(w).cuda(), None if residual is None else torch.from_numpy(r).cuda())
        xin = x if residual is None else x + r
        assert np.array_equal(xd.cpu().numpy(), xin)                            # x += residual, in place
        want = np.stack([orc.rmsnorm(xin[b], w) for b in range(B)])
        want_bf16 = torch.from_numpy(want).to(torch.bfloat16).float().numpy()
        got = t.float().cpu().numpy()
        # the CPU arithmetic restated (double sum, float rsqrt): equal up to one bf16 rounding step
        assert np.abs(got - want_bf16).max() <= 2.0 ** -7 * np.abs(want).max()
        assert (got == want_bf16).mean() > 0.999


@pytest.mark.parametrize("B,N,K,bias", [(1, 64, 64, True), (33, 5120, 2880, True), (130, 2880, 4096, True),
                                        (600, 2880, 4096, True), (1024, 5120, 2880, False),
                                        (700, 4096, 256, True), (2304, 1056, 512, True)])
def test_dense_gemm(ops, B, N, K, bias):
    """Every regime of the dispatch: row tiles of 32..160 rows chosen from the batch size, 256-row
    tiles from 2048 rows on, ragged last row tile and last column tile."""
    g = torch.Generator(device="cuda").manual_seed(B + N)
    a = torch.randn(B, K, device="cuda", generator=g).to(torch.bfloat16)
    w = (torch.randn(N, K, device="cuda", generator=g) * 0.05).to(torch.bfloat16)
    b = (torch.randn(N, device="cuda", generator=g)).to(torch.bfloat16).float() if bias else None
    got = ops.dense_gemm(a, ops.pack_weight(w), N, b).cpu().numpy()
    want = (a.double() @ w.double().T + (b.double() if bias else 0)).cpu().numpy()
    assert np.abs(got - want).max() <= 2e-5 * np.abs(want).max() + 1e-6 * np.sqrt(K)


@pytest.mark.parametrize("B,N,K", [(2500, 2880, 4096), (2049, 5120, 2880), (4096, 288, 256)])
def test_dense_gemm_of_a_prompt_pass_equals_the_same_rows_in_small_batches(ops, B, N, K):
    """From 2048 rows on the fp32 GEMM runs the kernel with 256-row tiles and both operands through
    LDS: same bits per row as the streaming kernels, which run the batches of a fifth of the rows."""
    g = torch.Generator(device="cuda").manual_seed(B + N)
    a = torch.randn(B, K, device="cuda", generator=g).to(torch.bfloat16)
    w = (torch.randn(N, K, device="cuda", generator=g) * 0.05).to(torch.bfloat16)
    b = (torch.randn(N, device="cuda", generator=g)).to(torch.bfloat16).float()
    wp = ops.pack_weight(w)
    full = ops.dense_gemm(a, wp, N, b)
    step = B // 5 + 1
    for r0 in range(0, B, step):
        assert torch.equal(full[r0:r0 + step], ops.dense_gemm(a[r0:r0 + step].contiguous(), wp, N, b)), r0


@pytest.mark.parametrize("B,V,K", [(5, 4096, 256), (130, 201088, 2880), (1024, 50304, 512), (515, 9984, 256),
                                   (256, 9984, 512), (255, 4128, 320)])
def test_classifier_argmax_equals_argmax_of_logits(ops, B, V, K):
    g = torch.Generator(device="cuda").manual_seed(V)
    a = torch.randn(B, K, device="cuda", generator=g).to(torch.bfloat16)
    w = (torch.randn(V, K, device="cuda", generator=g) * 0.05).to(torch.bfloat16)
    w[V - 1] = w[7]                                   # the same logit in the first and in the last, partly filled tile
    wp = ops.pack_weight(w)
    logits = ops.dense_gemm(a, wp, V)
    ids = ops.classifier_argmax(a, wp, V).cpu().numpy()
    assert np.array_equal(ids, logits.cpu().numpy().argmax(axis=1))
    assert np.array_equal(ops.argmax(logits).cpu().numpy(), ids)


@pytest.mark.parametrize("B", [130, 600])
@pytest.mark.parametrize("cols", [(7, 11, 40, 135, 300, 4127), (11, 40, 135), (135, 300), (200, 250), (259, 263)])
def test_classifier_argmax_ties_pick_the_lowest_column(ops, B, cols):
    """Equal maxima in the two half-waves of a lane pair, in two column blocks of a wave, in the two
    waves that share a row, in two column tiles and in the last, partly filled tile: the lowest
    column wins (run.cpp:739-750), on the streaming kernel (130 rows) and the 256-row kernel (600)."""
    V, K = 4128, 256
    g = torch.Generator(device="cuda").manual_seed(B)
    a = torch.randn(B, K, device="cuda", generator=g).to(torch.bfloat16)
    w = (torch.randn(V, K, device="cuda", generator=g) * 0.05).to(torch.bfloat16)
    big = (w[cols[0]].float() * 8).to(torch.bfloat16)
    for c in cols:
        w[c] = big
    ids = ops.classifier_argmax(a, ops.pack_weight(w), V).cpu().numpy()
    logits = (a.float() @ w.float().T).cpu().numpy()
    wins = logits[:, cols[0]] >= logits.max(axis=1)               # rows where the repeated column is the maximum
    assert wins.sum() > B // 10
    assert (ids[wins] == min(cols)).all()


def test_argmax_ties_lowest_index(ops):
    x = np.full((4, 4096), -1.0, np.float32)
    x[0, [4095, 17, 2000]] = 3.0
    x[1, :] = 0.0
    x[2, 4095] = 1.0
    x[3, :] = -np.inf
    assert ops.argmax(torch.from_numpy(x).cuda()).cpu().tolist() == [17, 0, 4095, 0]


def test_rope_tables_match_oracle(ops, orc, synth):
    for cfg in (synth.tiny_config(2048), synth.gptoss20b_config(1024)):
        cs, sn = ops.rope_tables(cfg, 300)
        ocs, osn = orc.rope_tables(cfg, 300)
        assert np.array_equal(cs, ocs) and np.array_equal(sn, osn)


@pytest.mark.parametrize("D,n_q,n_kv", [(32, 8, 2), (64, 64, 8)])
def test_rope_kv_store_then_attention(ops, orc, synth, D, n_q, n_kv):
    """Positions are fed one by one through the rotation + store op, every sequence at its own
    position; q must be the half-split rotation of run.cpp:480-499 and attention over the cache the
    op filled must be the oracle's attention over the rotated keys and the values."""
    import dataclasses
    cfg = dataclasses.replace(synth.tiny_config(2048), head_dim=D, n_attn_heads=n_q, n_kv_heads=n_kv)
    B, S, cap = 3, 70, 128
    lens_final = np.array([70, 33, 1], np.int32)
    rng = np.random.default_rng(D)
    qkv_dim = (n_q + 2 * n_kv) * D
    qkv = rng.standard_normal((S, B, qkv_dim)).astype(np.float32)
    cs, sn = orc.rope_tables(cfg, S)
    cs_d, sn_d = torch.from_numpy(cs).cuda(), torch.from_numpy(sn).cuda()

    def rot(x, pos):                                  # x [..., D]
        h = D // 2
        x1, x2 = x[..., :h], x[..., h:]
        return np.concatenate([x1 * cs[pos] - x2 * sn[pos], x2 * cs[pos] + x1 * sn[pos]], -1)

    cache = ops.KVCache(B, n_kv, D, cap)
    cache.kv.view(torch.int16).fill_(0x7FC1)
    K = np.zeros((B, S, n_kv, D), np.float32)
    V = np.zeros((B, S, n_kv, D), np.float32)
    q_last = np.zeros((B, n_q, D), np.float32)
    for step in range(S):
        pos = np.minimum(step, lens_final - 1)        # a finished sequence rewrites its last position
        lens = torch.from_numpy((pos + 1).astype(np.int32)).cuda()
        q = ops.rope_kv_store(torch.from_numpy(qkv[step]).cuda(), cache, cs_d, sn_d, lens, n_q).cpu().numpy()
        for b in range(B):
            row = qkv[step, b]
            want_q = rot(row[: n_q * D].reshape(n_q, D), pos[b])
            np.testing.assert_allclose(q[b], want_q, rtol=1e-6, atol=1e-6)
            K[b, pos[b]] = rot(row[n_q * D:(n_q + n_kv) * D].reshape(n_kv, D), pos[b])
            V[b, pos[b]] = row[(n_q + n_kv) * D:].reshape(n_kv, D)
            q_last[b] = want_q
    bf = lambda a: torch.from_numpy(a).to(torch.bfloat16).float().numpy()
    sinks = rng.standard_normal(n_q).astype(np.float32)
    attn = ops.AttnDecode(B, n_q, n_kv, D, S)
    got = attn.forward(torch.from_numpy(q_last).cuda(), cache, torch.from_numpy(lens_final).cuda(),
                       torch.from_numpy(sinks).cuda()).float().cpu().numpy()
    want = orc.attn_decode(q_last, bf(K), bf(V), lens_final, sinks, 0)
    assert np.isfinite(got).all()
    mx, mean = rel_errors(got, want)
    assert mx <= TOL_MAX and mean <= TOL_MEAN, (mx, mean)


def test_rope_kv_store_skips_empty_sequences(ops, orc, synth):
    """lens[b] == 0 is an empty sequence, as for the attention call: its q row comes back zero and
    nothing is written to its part of the cache; the other rows are unaffected."""
    cfg = synth.tiny_config(2048)
    D, n_q, n_kv, cap, B = cfg.head_dim, cfg.n_attn_heads, cfg.n_kv_heads, 64, 3
    rng = np.random.default_rng(9)
    qkv = torch.from_numpy(rng.standard_normal((B, (n_q + 2 * n_kv) * D)).astype(np.float32)).cuda()
    cs, sn = orc.rope_tables(cfg, 8)
    cs_d, sn_d = torch.from_numpy(cs).cuda(), torch.from_numpy(sn).cuda()
    both = []
    for lens in ([3, 0, 5], [3, 2, 5]):
        cache = ops.KVCache(B, n_kv, D, cap)
        cache.kv.view(torch.int16).fill_(0x1234)
        q = ops.rope_kv_store(qkv, cache, cs_d, sn_d, torch.tensor(lens, dtype=torch.int32).cuda(), n_q)
        torch.cuda.synchronize()
        both.append((q.cpu().numpy(), cache.kv.view(torch.int16).cpu().numpy().reshape(B, -1)))
    (q0, kv0), (q1, kv1) = both
    assert (q0[1] == 0).all() and (kv0[1] == 0x1234).all()           # empty row: zero q, cache untouched
    assert (kv1[1] != 0x1234).any()                                   # the same row with a length does store
    for b in (0, 2):
        assert np.array_equal(q0[b], q1[b]) and np.array_equal(kv0[b], kv1[b])
