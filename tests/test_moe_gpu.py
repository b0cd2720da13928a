"""GPU parity of the MoE path against the CPU oracle, through the C ABI."""
import numpy as np
import pytest
import torch

from conftest import TOL_MAX, TOL_MEAN, rel_errors

pytestmark = pytest.mark.gpu


def _bf16(t):
    return t.to(torch.bfloat16)


def _rand_layer(E, H, I, seed, std=0.02, dev="cuda"):
    g = torch.Generator(device="cpu").manual_seed(seed)
    def n(*shape, s=std):
        return _bf16(torch.randn(*shape, generator=g) * s)
    return dict(w_router=n(E, H), b_router=n(E), w1=n(E, 2 * I, H), b1=n(E, 2 * I),
                w2=n(E, H, I), b2=n(E, H))


def _f32np(t):
    return t.float().cpu().numpy()


# ---------------------------------------------------------------- routing: bit-exact integers
@pytest.mark.parametrize("B,E,k", [(1, 8, 4), (7, 8, 4), (64, 32, 4), (1024, 32, 4), (333, 128, 4),
                                   (4096, 128, 4), (100, 256, 8), (65, 40, 3), (0, 32, 4)])
def test_route_matches_oracle(ops, orc, B, E, k):
    rng = np.random.default_rng(1000 + B + E)
    logits = rng.standard_normal((B, E)).astype(np.float32)
    tw, ti, off, srt, inv, tiles = ops.moe_route(torch.from_numpy(logits).cuda(), k, rows_per_tile=128)
    torch.cuda.synchronize()
    if B == 0:
        assert off.cpu().numpy().tolist() == [0] * (E + 1)
        assert int(tiles[0]) == 0
        return
    ov, oi = orc.topk_softmax(logits, k)
    ooff, osrt, oinv = orc.group(oi, E)
    np.testing.assert_array_equal(ti.cpu().numpy(), oi)
    np.testing.assert_array_equal(off.cpu().numpy(), ooff)
    np.testing.assert_array_equal(srt.cpu().numpy(), osrt)
    np.testing.assert_array_equal(inv.cpu().numpy(), oinv)
    np.testing.assert_allclose(tw.cpu().numpy(), ov, rtol=2e-6, atol=1e-7)
    # tile list: every expert's rows cut into tiles of 128, in expert order
    t = tiles.cpu().numpy()
    exp = []
    for e in range(E):
        r0, r1 = int(ooff[e]), int(ooff[e + 1])
        for s in range(r0, r1, 128):
            exp.append((e, s, min(128, r1 - s)))
    assert t[0] == len(exp)
    assert [tuple(x) for x in t[1:1 + 3 * len(exp)].reshape(-1, 3)] == exp


def test_route_ties_lowest_expert_first(ops, orc):
    logits = np.zeros((5, 32), np.float32)
    logits[1, [3, 9, 20, 31]] = 1.0
    logits[2, :] = np.arange(32) % 4            # many equal values
    logits[3, 7] = -np.inf
    logits[4, :] = -1.0
    logits[4, [30, 2]] = 5.0
    tw, ti, off, srt, inv, _ = ops.moe_route(torch.from_numpy(logits).cuda(), 4)
    ov, oi = orc.topk_softmax(logits, 4)
    np.testing.assert_array_equal(ti.cpu().numpy(), oi)
    assert ti.cpu().numpy()[0].tolist() == [0, 1, 2, 3]
    assert ti.cpu().numpy()[1].tolist() == [3, 9, 20, 31]
    assert ti.cpu().numpy()[4].tolist()[:2] == [2, 30]
    np.testing.assert_allclose(tw.cpu().numpy(), ov, rtol=2e-6)


def test_route_skewed_all_to_one_expert(ops, orc):
    B, E, k = 2048, 32, 4
    logits = np.random.default_rng(5).standard_normal((B, E)).astype(np.float32)
    logits[:, 5] += 100.0
    logits[:, 17] += 50.0
    tw, ti, off, srt, inv, _ = ops.moe_route(torch.from_numpy(logits).cuda(), k)
    ov, oi = orc.topk_softmax(logits, k)
    ooff, osrt, oinv = orc.group(oi, E)
    np.testing.assert_array_equal(off.cpu().numpy(), ooff)
    np.testing.assert_array_equal(srt.cpu().numpy(), osrt)
    np.testing.assert_array_equal(inv.cpu().numpy(), oinv)


# ---------------------------------------------------------------- router GEMM
@pytest.mark.parametrize("B,H,E", [(1, 256, 8), (37, 256, 8), (1024, 2880, 32), (100, 2880, 128)])
def test_router_gemm(ops, B, H, E):
    g = torch.Generator().manual_seed(B + E)
    t = _bf16(torch.randn(B, H, generator=g)).cuda()
    w = _bf16(torch.randn(E, H, generator=g) * 0.02).cuda()
    b = _bf16(torch.randn(E, generator=g) * 0.02).float().cuda()
    got = ops.router_gemm(t, w, b).cpu().numpy()
    want = (t.double().cpu() @ w.double().cpu().T + b.double().cpu()).numpy()
    assert np.abs(got - want).max() <= 1e-4 * max(1.0, np.abs(want).max())


# ---------------------------------------------------------------- weight packing
def test_pack_weight_layout(ops):
    n_mat, N, K = 2, 128, 128
    w = torch.arange(n_mat * N * K, dtype=torch.float32).reshape(n_mat, N, K) % 251
    wp = ops.pack_weight(w.to(torch.bfloat16).cuda()).float().cpu().numpy().reshape(n_mat, N // 32, K // 16, 64, 8)
    wp32 = ops.pack_weight(w.cuda()).float().cpu().numpy().reshape(n_mat, N // 32, K // 16, 64, 8)
    wn = w.numpy()
    for m, nb, ks, lane in [(0, 0, 0, 0), (1, 3, 7, 63), (0, 2, 5, 33), (1, 1, 1, 31)]:
        row, k0 = nb * 32 + lane % 32, ks * 16 + (lane // 32) * 8
        np.testing.assert_array_equal(wp[m, nb, ks, lane], wn[m, row, k0:k0 + 8])
        np.testing.assert_array_equal(wp32[m, nb, ks, lane], wn[m, row, k0:k0 + 8])
    # GLU pairing: virtual row v of a 32-row block -> pair (v//32)*16 + v%16, 16 gates then 16 ups
    wg = ops.pack_weight(w.to(torch.bfloat16).cuda(), glu=True).float().cpu().numpy().reshape(n_mat, N // 32, K // 16, 64, 8)
    for m, nb, ks, lane in [(0, 0, 0, 0), (0, 1, 2, 5), (1, 3, 7, 63), (1, 2, 0, 40)]:
        v = nb * 32 + lane % 32
        row = 2 * ((v // 32) * 16 + v % 16) + (v // 16) % 2
        k0 = ks * 16 + (lane // 32) * 8
        np.testing.assert_array_equal(wg[m, nb, ks, lane], wn[m, row, k0:k0 + 8])


# ---------------------------------------------------------------- whole MoE block vs oracle
@pytest.mark.parametrize("B,E,H,I,seed", [
    (8, 8, 256, 256, 1),        # tiny-model shape, decode batch
    (1, 8, 256, 256, 2),
    (96, 8, 256, 256, 3),       # 48 rows per expert
    (300, 8, 256, 256, 4),      # >128 rows per expert: 256-row tiles
    (700, 8, 256, 256, 5),      # >256 rows per expert: several tiles per expert
    (64, 32, 2880, 2880, 6),    # 20B shape, few tokens
])
def test_moe_forward_matches_oracle(ops, orc, B, E, H, I, seed):
    L = _rand_layer(E, H, I, seed)
    g = torch.Generator().manual_seed(100 + seed)
    t = _bf16(torch.randn(B, H, generator=g))
    layer = ops.MoeLayer(*[L[n].cuda() for n in ("w_router", "b_router", "w1", "b1", "w2", "b2")],
                         max_tokens=max(B, 1))
    out = layer.forward(t.cuda())
    torch.cuda.synchronize()
    logits, tw, ti, off, srt, inv = [x.cpu().numpy() for x in layer.routing_views()]
    want, ologits, otv, oti = orc.moe_layer(_f32np(t), *[_f32np(L[n]) for n in
                                            ("w_router", "b_router", "w1", "b1", "w2", "b2")],
                                            k=4, limit=7.0, stage=orc.STAGE_SWIGLU, want_routing=True)
    np.testing.assert_allclose(logits, ologits, atol=2e-5 * max(1.0, np.abs(ologits).max()))
    # grouping is bit-exact given the GPU's own logits
    ov, oi = orc.topk_softmax(logits, 4)
    ooff, osrt, oinv = orc.group(oi, E)
    np.testing.assert_array_equal(ti, oi)
    np.testing.assert_array_equal(off, ooff)
    np.testing.assert_array_equal(srt, osrt)
    np.testing.assert_array_equal(inv, oinv)
    # rows whose GPU routing equals the oracle's routing (ties in the 1e-6 range may differ)
    same = (oti == ti).all(axis=1)
    assert same.mean() > 0.98
    mx, mean = rel_errors(out.cpu().numpy()[same], want[same])
    assert mx <= TOL_MAX and mean <= TOL_MEAN, (mx, mean)


def test_moe_forward_accumulate_and_determinism(ops):
    E, H, I, B = 8, 256, 256, 200
    L = _rand_layer(E, H, I, 9)
    t = _bf16(torch.randn(B, H, generator=torch.Generator().manual_seed(3))).cuda()
    layer = ops.MoeLayer(*[L[n].cuda() for n in ("w_router", "b_router", "w1", "b1", "w2", "b2")],
                         max_tokens=B)
    a = layer.forward(t).clone()
    b = layer.forward(t).clone()
    assert torch.equal(a, b)                      # run-to-run bit reproducible
    x = torch.randn(B, H, device="cuda")
    y = x.clone()
    layer.forward(t, out=y, accumulate=True)
    assert torch.equal(y, x + a)


@pytest.mark.parametrize("B,E,H,I", [(3000, 16, 256, 512), (1500, 64, 512, 256)])
def test_moe_forward_skewed_routing_is_batch_invariant(ops, orc, B, E, H, I):
    """Zipf-skewed routing (experts with many row tiles next to experts with a few rows): the work
    list is then cut into per-XCD parts by estimated cost, with cuts that fall inside tiles.  Every
    token's output must not depend on what else is in the batch: the full batch equals, bit for bit,
    the same tokens run in two halves (other tiles, other cuts), and a sample equals the oracle."""
    L = _rand_layer(E, H, I, 21)
    ranks = np.random.default_rng(B).permutation(E) + 1
    L["b_router"] = torch.from_numpy((1.5 * np.log(1.0 / ranks ** 1.1)).astype(np.float32))
    g = torch.Generator().manual_seed(B)
    t = _bf16(torch.randn(B, H, generator=g))
    layer = ops.MoeLayer(*[L[n].cuda() for n in ("w_router", "b_router", "w1", "b1", "w2", "b2")],
                         max_tokens=B)
    full = layer.forward(t.cuda()).clone()
    logits, tw, ti, off, srt, inv = [x.cpu().numpy() for x in layer.routing_views()]
    counts = np.diff(off)
    assert counts.max() >= 4 * counts.mean() and counts.max() > 3 * 160   # several tiles for one expert
    h = B // 2 + 7
    first = layer.forward(t[:h].cuda()).clone()
    second = layer.forward(t[h:].cuda()).clone()
    assert torch.equal(full[:h], first)
    assert torch.equal(full[h:], second)
    n_chk = 40
    want, _, _, oti = orc.moe_layer(_f32np(t)[:n_chk], *[_f32np(L[n]) for n in
                                    ("w_router", "b_router", "w1", "b1", "w2", "b2")],
                                    k=4, limit=7.0, stage=orc.STAGE_SWIGLU, want_routing=True)
    same = (oti == ti[:n_chk]).all(axis=1)
    assert same.mean() > 0.9
    mx, mean = rel_errors(full.cpu().numpy()[:n_chk][same], want[same])
    assert mx <= TOL_MAX and mean <= TOL_MEAN, (mx, mean)


# ---------------------------------------------------------------- SwiGLU epilogue and bias order, alone
def test_swiglu_special_cases_and_bias_order_through_a_one_expert_layer(ops, orc):
    """One expert, top-1, w2 = identity: the layer's output is the bf16-rounded clamped SwiGLU of
    chosen (gate, up) values plus b2, so the epilogue of GEMM1 (run.cpp:669-686: gate = min(g, 7),
    up = clamp(u, -7, 7), g * sigmoid(1.702 g) * (up + 1)), the (gate, up) interleave of mlp1's rows
    and the order of both bias vectors are checked on their own, special cases included:
    g > 7, u > 7, u < -7 (up + 1 = -6), g -> -inf (0)."""
    H = I = 64
    B = 4
    gv = np.array([8.0, 7.0, 6.5, -100.0, 0.5, -0.5, 30.0, -8.0], np.float32)
    uv = np.array([-8.0, 8.0, 0.25, 7.0, -7.0, -6.5, 100.0, -1.0], np.float32)
    j = np.arange(I)
    g_j, u_j = gv[j % 8], uv[(j // 8) % 8]
    w1 = np.zeros((1, 2 * I, H), np.float32)
    w1[0, 0::2, 0] = g_j                       # row 2j = gate of pair j, row 2j+1 = its up
    w1[0, 1::2, 0] = u_j
    b1 = np.zeros((1, 2 * I), np.float32)
    b1[0, 0::2] = 0.125 * (j % 3)
    b1[0, 1::2] = -0.25 * (j % 5)
    b2 = (0.5 * (j % 7) - 1.0).astype(np.float32)[None]
    w2 = np.eye(H, I, dtype=np.float32)[None]
    s = np.array([1.0, 0.5, -1.0, 2.0], np.float32)
    t = np.zeros((B, H), np.float32)
    t[:, 0] = s
    t[:, 5] = 3.0                              # a column no weight reads
    tt = lambda a: torch.from_numpy(a).to(torch.bfloat16).cuda()
    mk = lambda bias2: ops.MoeLayer(torch.zeros(1, H, dtype=torch.bfloat16).cuda(), torch.zeros(1).cuda(), tt(w1),
                                    torch.from_numpy(b1).cuda(), tt(w2), torch.from_numpy(bias2).cuda(), top_k=1,
                                    max_tokens=B)
    got = mk(np.zeros_like(b2)).forward(tt(t)).cpu().numpy()
    with_b2 = mk(b2).forward(tt(t)).cpu().numpy()
    np.testing.assert_allclose(with_b2 - got, np.broadcast_to(b2, got.shape), atol=1e-5)   # b2[j] lands on column j
    gate = s[:, None] * g_j[None, :] + b1[0, 0::2][None, :]
    up = s[:, None] * u_j[None, :] + b1[0, 1::2][None, :]
    pre = np.empty((B, 2 * I), np.float32)
    pre[:, 0::2], pre[:, 1::2] = gate, up
    want = orc.swiglu(pre, 7.0)
    # closed form in float64, independent of the oracle
    gc_, uc_ = np.minimum(gate.astype(np.float64), 7.0), np.clip(up.astype(np.float64), -7.0, 7.0)
    closed = gc_ / (1.0 + np.exp(-1.702 * gc_)) * (uc_ + 1.0)
    np.testing.assert_allclose(want, closed, rtol=1e-5, atol=1e-30)
    # the GPU result is bf16-rounded (2^-9 relative) after exp2/reciprocal of a few ulp
    np.testing.assert_allclose(got, closed, rtol=5e-3, atol=1e-30)
    # the special cases, by value
    big_g = gate > 7.0
    assert big_g.any() and (up < -7.0).any() and (up > 7.0).any() and (gate < -50).any()
    sig7 = 7.0 / (1.0 + np.exp(-1.702 * 7.0))
    np.testing.assert_allclose(got[big_g], (sig7 * (uc_ + 1.0))[big_g], rtol=5e-3)
    np.testing.assert_allclose(got[big_g & (up < -7.0)], sig7 * -6.0, rtol=5e-3)
    assert (got[gate < -50] == 0).all()


@pytest.mark.parametrize("B,E,k,skew", [(2048, 8, 4, 0.0), (2300, 40, 4, 2.0), (4096, 128, 4, 3.0), (3000, 256, 8, 0.0),
                                        (9000, 32, 1, 1.0)])
def test_grouping_by_many_workgroups(ops, orc, B, E, k, skew):
    """From 8192 (token, expert) pairs on, the layer sorts them with one workgroup per 1024 pairs
    (counts per workgroup, then offsets + scatter) instead of a single workgroup: offsets,
    permutation and inverse must still be the stable counting sort, bit for bit, and the layer
    output (which follows the tile list the same kernels write) must match the oracle."""
    H = I = 64
    g = torch.Generator().manual_seed(B + E)
    n = lambda *s: _bf16(torch.randn(*s, generator=g) * 0.05)
    br = _bf16(n(E).float() - skew * torch.arange(E) / E)
    L = dict(w_router=n(E, H), b_router=br, w1=n(E, 2 * I, H), b1=n(E, 2 * I), w2=n(E, H, I), b2=n(E, H))
    names = ("w_router", "b_router", "w1", "b1", "w2", "b2")
    t = _bf16(torch.randn(B, H, generator=g))
    layer = ops.MoeLayer(*[L[x].cuda() for x in names], top_k=k, max_tokens=B)
    out = layer.forward(t.cuda())
    torch.cuda.synchronize()
    logits, tw, ti, off, srt, inv = [x.cpu().numpy() for x in layer.routing_views()]
    assert B * k >= 8192
    _, oi = orc.topk_softmax(logits, k)
    ooff, osrt, oinv = orc.group(oi, E)
    np.testing.assert_array_equal(ti, oi)
    np.testing.assert_array_equal(off, ooff)
    np.testing.assert_array_equal(srt, osrt)
    np.testing.assert_array_equal(inv, oinv)
    want, _, _, oti = orc.moe_layer(_f32np(t), *[_f32np(L[x]) for x in names], k=k, limit=7.0,
                                    stage=orc.STAGE_SWIGLU, want_routing=True)
    same = (oti == ti).all(axis=1)
    assert same.mean() > 0.95
    mx, mean = rel_errors(out.cpu().numpy()[same], want[same])
    assert mx <= TOL_MAX and mean <= TOL_MEAN, (mx, mean)


# ---------------------------------------------------------------- prompt-pass sizes: 256-row tiles
@pytest.mark.parametrize("B,E,H,I,skew", [
    (2100, 8, 320, 320, 0.0),      # K = 320: ten stages; N = 640 and 320: a partial column tile each
    (2600, 16, 256, 512, 1.1),     # skewed: experts of many tiles beside experts of a few rows
    (1300, 4, 512, 256, 0.0),      # an expert's last tile of a few rows
    (4100, 32, 2880, 2880, 0.0),   # the 20B layer at 4100 tokens
])
def test_moe_forward_of_a_prompt_pass_equals_the_same_tokens_in_small_batches(ops, orc, B, E, H, I, skew):
    """From 512 rows per expert on average the block runs kernels of their own (256-row tiles, both
    operands through LDS).  They must give every token the bits that the streaming kernels give it:
    the full batch equals the same tokens run in batches of 1/8 of the size, and a sample equals the oracle."""
    L = _rand_layer(E, H, I, 31)
    if skew:
        ranks = np.random.default_rng(B).permutation(E) + 1
        L["b_router"] = torch.from_numpy((1.5 * np.log(1.0 / ranks ** skew)).astype(np.float32))
    t = _bf16(torch.randn(B, H, generator=torch.Generator().manual_seed(B)))
    layer = ops.MoeLayer(*[L[n].cuda() for n in ("w_router", "b_router", "w1", "b1", "w2", "b2")],
                         max_tokens=B)
    assert B * 4 >= 512 * E
    full = layer.forward(t.cuda()).clone()
    ti = layer.routing_views()[2].cpu().numpy()
    step = B // 8 + 3
    assert step * 4 < 512 * E
    for r0 in range(0, B, step):
        part = layer.forward(t[r0:r0 + step].cuda())
        assert torch.equal(full[r0:r0 + step], part), r0
    n_chk = 24
    rows = np.r_[0:n_chk // 2, B - n_chk // 2:B]
    want, _, _, oti = orc.moe_layer(_f32np(t)[rows], *[_f32np(L[n]) for n in
                                    ("w_router", "b_router", "w1", "b1", "w2", "b2")],
                                    k=4, limit=7.0, stage=orc.STAGE_SWIGLU, want_routing=True)
    same = (oti == ti[rows]).all(axis=1)
    assert same.mean() > 0.9
    mx, mean = rel_errors(full.cpu().numpy()[rows][same], want[same])
    assert mx <= TOL_MAX and mean <= TOL_MEAN, (mx, mean)
