"""Randomised shapes and model configurations (fixed seeds): the MoE layer, decode attention and the
engine against the CPU oracle on dimensions no hand-picked case covers - odd token counts, one to 64
experts, top-1 to top-8, skewed routing, every supported head grouping, ring caches that have
wrapped, ragged lengths with empty rows."""
import numpy as np
import pytest
import torch

from conftest import TOL_MAX, TOL_MEAN, rel_errors

pytestmark = pytest.mark.gpu


def test_moe_random_shapes(ops, orc):
    rng = np.random.default_rng(20240)
    worst = [0.0, 0.0]
    for case in range(48):
        E = int(rng.choice([1, 2, 4, 8, 16, 32, 40, 64]))
        k = int(min(E, rng.choice([1, 2, 4, 4, 4, 8])))
        H = int(rng.choice([64, 128, 192, 256, 320, 512]))
        I = int(rng.choice([64, 128, 192, 256, 384]))
        B = int(rng.choice([1, 2, 3, 17, 31, 33, 64, 100, 129, 257, 500, 1000, 1500]))
        skew = float(rng.choice([0.0, 0.0, 1.0, 3.0]))
        g = torch.Generator().manual_seed(int(rng.integers(1 << 30)))
        n = lambda *s: (torch.randn(*s, generator=g) * 0.05).to(torch.bfloat16)
        br = (n(E).float() - skew * torch.arange(E) / max(E, 1)).to(torch.bfloat16)   # skew: a few hot experts
        L = dict(w_router=n(E, H), b_router=br, w1=n(E, 2 * I, H), b1=n(E, 2 * I), w2=n(E, H, I), b2=n(E, H))
        names = ("w_router", "b_router", "w1", "b1", "w2", "b2")
        t = torch.randn(B, H, generator=g).to(torch.bfloat16)
        layer = ops.MoeLayer(*[L[x].cuda() for x in names], top_k=k, max_tokens=B)
        out = layer.forward(t.cuda()).clone()
        assert torch.equal(out, layer.forward(t.cuda())), (case, "not reproducible")
        logits, tw, ti, off, srt, inv = [x.cpu().numpy() for x in layer.routing_views()]
        f = lambda x: x.float().cpu().numpy()
        want, _, _, oti = orc.moe_layer(f(t), *[f(L[x]) for x in names], k=k, limit=7.0,
                                        stage=orc.STAGE_SWIGLU, want_routing=True)
        _, oi = orc.topk_softmax(logits, k)
        ooff, osrt, oinv = orc.group(oi, E)
        assert np.array_equal(ti, oi) and np.array_equal(off, ooff), case
        assert np.array_equal(srt, osrt) and np.array_equal(inv, oinv), case
        same = (oti == ti).all(axis=1)           # near-ties of the router may go the other way
        assert same.mean() > 0.9, (case, same.mean())
        if same.any():
            mx, mean = rel_errors(out.cpu().numpy()[same], want[same])
            worst = [max(worst[0], mx), max(worst[1], mean)]
            assert mx <= TOL_MAX and mean <= TOL_MEAN, (case, E, k, H, I, B, mx, mean)
    print("random MoE shapes: worst max-rel / mean-rel", worst)


def test_attn_random_shapes(ops, orc):
    rng = np.random.default_rng(20241)
    worst = [0.0, 0.0]
    for case in range(64):
        D = int(rng.choice([32, 64]))
        n_kv = int(rng.choice([1, 2, 4, 8]))
        n_q = n_kv * int(rng.choice([1, 2, 4, 8, 16]))
        B = int(rng.choice([1, 2, 5, 16, 63, 64, 65, 130]))
        cap = int(rng.choice([64, 128, 192, 512, 1024, 2048]))
        window = int(rng.choice([0, 0, 16, 64, 128, 200]))
        wrapped = 0 < window <= cap and rng.random() < 0.4
        max_len = int(rng.integers(cap + 1, 3 * cap)) if wrapped else int(rng.integers(1, cap + 1))
        # a ring holds the last positions written, so every row of a wrapped cache is at the end
        lens = np.full(B, max_len, np.int32) if wrapped else rng.integers(0, max_len + 1, size=B).astype(np.int32)
        g = torch.Generator().manual_seed(int(rng.integers(1 << 30)))
        q = torch.randn(B, n_q, D, generator=g)
        K = torch.randn(B, max_len, n_kv, D, generator=g).to(torch.bfloat16)
        V = torch.randn(B, max_len, n_kv, D, generator=g).to(torch.bfloat16)
        sinks = torch.randn(n_q, generator=g)
        cache = ops.KVCache(B, n_kv, D, cap)
        cache.kv.view(torch.int16).fill_(0x7FC1)
        for p0 in range(0, max_len, cap):
            m = min(cap, max_len - p0)
            cache.write(K[:, p0:p0 + m].contiguous().cuda(), V[:, p0:p0 + m].contiguous().cuda(), p0)
        attn = ops.AttnDecode(B, n_q, n_kv, D, max_len)
        got = attn.forward(q.cuda(), cache, torch.as_tensor(lens).cuda(), sinks.cuda(),
                           window=window).float().cpu().numpy()
        want = orc.attn_decode(q.numpy(), K.float().numpy(), V.float().numpy(), lens, sinks.numpy(), window)
        live = lens > 0
        if live.any():
            assert np.isfinite(got[live]).all(), case
            mx, mean = rel_errors(got[live], want[live])
            worst = [max(worst[0], mx), max(worst[1], mean)]
            assert mx <= TOL_MAX and mean <= TOL_MEAN, (case, B, n_q, n_kv, D, cap, window, max_len, mx, mean)
    print("random attention shapes: worst max-rel / mean-rel", worst)


#: a router decision of the staged CPU model closer than this (k-th against (k+1)-th score) may fall
#: the other way on the GPU or under a different summation order: the criterion by which the
#: lock-step comparison above drops rows.  (Observed flips: gaps of 3.1e-4, 5.3e-3 and 1.56e-2; the
#: last one in a model whose logits sit 0.5-1 % of their scale from the staged CPU model's at every
#: position, so its router scores, of unit scale, carry an error of that order.)
ROUTER_NEAR_TIE = 2e-2


def _engine_case(ops, orc, binfmt, D, nq, nkv, H, E, k, I, L, V, win, B, T, seed, tok_cols):
    """One model configuration through lock-step steps, the prompt pass and one ragged step.
    Returns the worst max-rel of the lock-step rows against the staged CPU model and the rows of
    the prompt pass that a router near-tie excused."""
    cfg = binfmt.Config(vocab_size=V, hidden_dim=H, n_experts=E, experts_per_token=k, intermediate_dim=I,
                        n_layers=L, head_dim=D, n_attn_heads=nq, n_kv_heads=nkv, seq_len=2048,
                        initial_context_length=4096, rope_theta=150000.0, rope_scaling_factor=32.0,
                        sliding_window=win, swiglu_limit=7.0)
    g = np.random.default_rng(seed)
    flat = np.empty(binfmt.n_weight_floats(cfg), np.float32)
    off = 0
    for name, shape in binfmt.tensor_shapes(cfg).items():
        m = int(np.prod(shape))
        x = g.standard_normal(m).astype(np.float32) * 0.05
        if name in ("attn_norm", "mlp_norm", "final_norm"):
            x = x * 0.4 + 1.0
        flat[off:off + m] = torch.from_numpy(x).to(torch.bfloat16).float().numpy()
        off += m
    toks = g.integers(0, V, size=(B, tok_cols)).astype(np.int32)
    a = ops.Engine(cfg, flat, max_batch=B, max_seq=128, keep_logits=True)
    b = ops.Engine(cfg, flat, max_batch=B, max_seq=128, keep_logits=True)
    rows = sorted({0, B // 2, B - 1})
    cpu = {r: orc.Model(cfg, flat, stage=orc.STAGE_GPU) for r in rows}
    live = set(rows)
    worst = 0.0
    for pos in range(T):
        ids = a.step(toks[:, pos], pos)
        got = a.last_logits(B)
        assert np.array_equal(ids, got.argmax(axis=1)), (pos, cfg)
        for r in rows:
            want = cpu[r].forward(int(toks[r, pos]), pos)
            if cpu[r].last_router_gap() < ROUTER_NEAR_TIE:
                live.discard(r)
            if r in live:
                mx, _ = rel_errors(got[r], want)
                worst = max(worst, mx)
                assert mx <= 2e-2, (pos, r, mx, cfg)
    b.prefill(toks[:, :T])
    lb = b.last_logits(B)
    excused = []
    if T <= win:
        assert np.array_equal(lb, got), ("prompt pass differs from lock step", cfg)
    else:
        # A ring has wrapped: the prompt pass sums the window in position order, the lock-step
        # step in slot order, so the two differ by fp32 summation order and, through the bf16
        # roundings, by a last bit here and there.  Every row must stay within the bf16 bound
        # unless, on the positions where the orders differ, the staged CPU model shows a router
        # decision of that row close enough to fall the other way.
        per = np.abs(lb - got).max(axis=1) / np.abs(got).max(axis=1)
        tie = {}
        for r in np.nonzero(per > 5e-3)[0]:
            m = orc.Model(cfg, flat, stage=orc.STAGE_GPU)
            gaps = []
            for pos in range(T):
                m.forward(int(toks[r, pos]), pos)
                gaps.append(m.last_router_gap())
            m.close()
            tie[int(r)] = (float(min(gaps[win:])), win + int(np.argmin(gaps[win:])))
        # rows without a near-tie stay tight (a near-tie that falls the same way still moves a row by
        # up to a percent: one expert's weight shifts); rows beyond the bound must have one
        # (a median needs a few rows: single rows without a near-tie reach 5.4e-3 and are held to the
        # bf16 bound below, like every row)
        clear = [r for r in range(B) if r not in tie or tie[r][0] >= ROUTER_NEAR_TIE]
        if len(clear) >= 3:
            assert np.median(per[clear]) <= 5e-3, (per, cfg)
        for r in range(B):
            if per[r] > TOL_MAX:
                assert r in tie and tie[r][0] < ROUTER_NEAR_TIE, (
                    "prompt pass row beyond bf16 tolerance without a router near-tie", r, float(per[r]), tie.get(r), cfg)
                excused.append((r, float(per[r]), tie[r][0], tie[r][1]))
        assert len(excused) <= max(1, B // 8), (excused, cfg)
    posv = np.array([T - (i % 2) for i in range(B)], np.int32)   # every other row repeats its last position
    a.step_ragged(np.array([toks[i, posv[i]] for i in range(B)], np.int32), posv)
    lr = a.last_logits(B)
    for r in rows:
        if r in live and posv[r] == T:
            want = cpu[r].forward(int(toks[r, T]), T)
            if cpu[r].last_router_gap() >= ROUTER_NEAR_TIE:
                mx, _ = rel_errors(lr[r], want)
                assert mx <= 2e-2, ("ragged", r, mx, cfg)
    a.close()
    b.close()
    for m in cpu.values():
        m.close()
    return worst, excused


def test_engine_random_configs(ops, orc, binfmt):
    """Lock-step steps against the CPU model that rounds where the GPU dataflow rounds (rows are
    dropped once a router decision comes closer than ROUTER_NEAR_TIE: the two may then pick different
    experts), the prompt pass against the lock-step steps (bit for bit while no sliding-window ring
    has wrapped; per row within the bf16 bound after, router near-ties excepted), and one step
    with per-sequence positions."""
    rng = np.random.default_rng(20242)
    done = 0
    worst = 0.0
    while done < 10:
        D = int(rng.choice([32, 64]))
        nkv = int(rng.choice([1, 2, 4]))
        nq = nkv * int(rng.choice([1, 2, 4, 8]))
        H = int(rng.choice([128, 192, 256, 320]))
        E = int(rng.choice([4, 8, 16, 32]))
        k = int(min(E, rng.choice([1, 2, 4])))
        I = int(rng.choice([64, 128, 192, 256]))
        L = int(rng.choice([1, 2, 3]))
        V = int(rng.choice([256, 512, 1088, 1024, 4096]))
        win = int(rng.choice([64, 128]))
        seed = int(rng.integers(1 << 30))
        B = int(rng.choice([1, 3, 8, 33]))
        T = int(rng.choice([3, 9, 70 if win == 64 else 20]))
        if ((nq + 2 * nkv) * D) % 64 or (nq * D) % 64:
            continue                                         # the engine wants these multiples of 64
        w, _ = _engine_case(ops, orc, binfmt, D, nq, nkv, H, E, k, I, L, V, win, B, T, seed, T + 1)
        worst = max(worst, w)
        done += 1
    print("random engine configurations: worst max-rel against the staged CPU model", worst)


def test_prompt_pass_past_the_window_differs_from_lock_step_only_at_router_near_ties(ops, orc, binfmt):
    """A case a long run of the generator above turned up: 33 sequences, 70-token prompt, window 64,
    top-2 of 32 experts.  One row's logits after the prompt pass differ from the lock-step ones by
    most of their scale.  The staged CPU model puts that row's 2nd and 3rd router scores at
    position 69 only 3.1e-4 apart (row 19; the next closest decision at that position in the whole
    batch is ten times wider), so the two summation orders of the wrapped window pick different
    experts there; every other row agrees within the bf16 bound."""
    _, excused = _engine_case(ops, orc, binfmt, D=32, nq=2, nkv=2, H=320, E=32, k=2, I=128, L=2, V=512, win=64,
                              B=33, T=70, seed=355231429, tok_cols=72)
    print("rows excused by a router near-tie (row, max-rel, gap, position):", excused)
    assert [e[0] for e in excused] in ([19], []), excused


def test_prompt_pass_of_a_single_row_with_a_near_tie_below_the_bound(ops, orc, binfmt):
    """Another case of a long run: ONE sequence, 100-token prompt, window 64, three blocks, top-4 of 32
    experts.  Its logits after the prompt pass differ from the lock-step ones by 1.7e-2 of their
    scale, inside the bf16 bound but far above what rows without a close router decision show (a
    median over one row is that row).  The staged CPU model puts two router scores 2.7e-4 apart at
    position 90, past the ring: the row is counted as a near-tie row, not as a loose one."""
    _, excused = _engine_case(ops, orc, binfmt, D=64, nq=2, nkv=2, H=256, E=32, k=4, I=128, L=3, V=4096, win=64,
                              B=1, T=100, seed=480297126, tok_cols=102)
    assert excused == []


def test_lock_step_row_that_parts_from_the_cpu_model_at_a_gap_of_1_56e_2(ops, orc, binfmt):
    """A third case of a long run: 33 sequences, 70-token prompt, window 64, three blocks, top-2 of 16
    experts, hidden size 320.  Prompt pass and lock-step steps agree bit for bit for prompts of up to
    68 tokens and to 4e-3 at 69; at 70 row 15 differs by a third of the logits' scale.  It is the
    lock-step engine that leaves the staged CPU model there (0.34 against 1.1e-2 for the prompt pass):
    the CPU model's 2nd and 3rd router scores at position 69 are 1.56e-2 apart, the closest decision
    of that row past the window, in a model whose engine logits are 0.5-1 % of their scale away from
    the CPU model's at every position before.  The row counts as a near-tie row."""
    _, excused = _engine_case(ops, orc, binfmt, D=32, nq=8, nkv=2, H=320, E=16, k=2, I=64, L=3, V=512, win=64,
                              B=33, T=70, seed=12359588, tok_cols=72)
    print("rows excused by a router near-tie (row, max-rel, gap, position):", excused)
    assert [e[0] for e in excused] in ([15], []), excused
    for e in excused:
        assert e[3] == 69 and 1.5e-2 < e[2] < 1.6e-2, excused
