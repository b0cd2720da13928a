"""Pins of the CPU oracle (no GPU): against the reference's own compiled CPU model where it is
built (oracle/_ref), against the committed golden ids, and against closed forms, invariants and
brute force chosen so that a dropped term, a wrong sign or a swapped index fails."""
import ctypes as C
import hashlib
import json
import os

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
GOLDEN = os.path.join(HERE, "golden", "tiny_e2e.json")


# ------------------------------------------------------------------ basic blocks: closed forms
def test_rmsnorm_closed_form(orc):
    rng = np.random.default_rng(0)
    x = rng.standard_normal(256).astype(np.float32) * 3
    w = rng.standard_normal(256).astype(np.float32)
    want = w.astype(np.float64) * x / np.sqrt(np.mean(x.astype(np.float64) ** 2) + 1e-5)
    np.testing.assert_allclose(orc.rmsnorm(x, w), want, rtol=2e-6)
    # eps sits inside the square root: a zero vector maps to zero, not NaN
    assert np.all(orc.rmsnorm(np.zeros(8, np.float32), np.ones(8, np.float32)) == 0)


def test_softmax_and_matmul(orc):
    rng = np.random.default_rng(1)
    x = rng.standard_normal(37).astype(np.float32) * 5
    e = np.exp(x.astype(np.float64) - x.max())
    np.testing.assert_allclose(orc.softmax(x), e / e.sum(), rtol=1e-6)
    w = rng.standard_normal((5, 37)).astype(np.float32)
    np.testing.assert_allclose(orc.matmul(x, w), w.astype(np.float64) @ x, rtol=1e-6)
    # (out,in) orientation: a one-hot input picks a column
    onehot = np.zeros(37, np.float32); onehot[3] = 1
    np.testing.assert_array_equal(orc.matmul(onehot, w), w[:, 3])


def test_topk_softmax(orc):
    rng = np.random.default_rng(2)
    logits = rng.standard_normal((200, 32)).astype(np.float32)
    v, i = orc.topk_softmax(logits, 4)
    order = np.argsort(-logits, axis=1, kind="stable")[:, :4]
    np.testing.assert_array_equal(i, order)                       # descending, distinct values
    picked = np.take_along_axis(logits, order, 1).astype(np.float64)
    e = np.exp(picked - picked[:, :1])
    np.testing.assert_allclose(v, e / e.sum(1, keepdims=True), rtol=1e-6)
    np.testing.assert_allclose(v.sum(1), 1.0, rtol=1e-6)
    assert (np.diff(v, axis=1) <= 0).all()
    # ties: lowest expert id first
    tie = np.zeros((1, 8), np.float32); tie[0, [6, 2, 5]] = 1.0
    _, ti = orc.topk_softmax(tie, 4)
    assert ti[0].tolist() == [2, 5, 6, 0]


def test_topk_matches_reference_cpu(orc):
    if not orc.have_ref():
        pytest.skip("oracle/_ref not built (reference tree absent)")
    R = orc.ref()
    rng = np.random.default_rng(3)
    for _ in range(50):
        s = rng.standard_normal(32).astype(np.float32)
        vals = np.zeros(4, np.float32); idx = np.zeros(4, np.int32)
        sc = s.copy()
        R.ref_topk(vals.ctypes.data_as(C.c_void_p), idx.ctypes.data_as(C.c_void_p),
                   sc.ctypes.data_as(C.c_void_p), 32, 4)
        v, i = orc.topk_softmax(s[None], 4)
        np.testing.assert_array_equal(i[0], idx)
        np.testing.assert_array_equal(v[0], vals)                 # bit-identical


def test_group_is_stable_counting_sort(orc):
    rng = np.random.default_rng(4)
    for B, k, E in [(1, 4, 8), (17, 4, 8), (1024, 4, 32), (300, 8, 128), (5, 1, 3)]:
        ti = np.stack([rng.permutation(E)[:k] for _ in range(B)]).astype(np.int32)
        off, srt, inv = orc.group(ti, E)
        flat = ti.ravel()
        np.testing.assert_array_equal(off, np.concatenate([[0], np.cumsum(np.bincount(flat, minlength=E))]))
        np.testing.assert_array_equal(srt, np.argsort(flat, kind="stable"))
        np.testing.assert_array_equal(inv[srt], np.arange(B * k))  # bijection and inverse
        for e in range(E):
            seg = srt[off[e]:off[e + 1]]
            assert (flat[seg] == e).all() and (np.diff(seg) > 0).all()
    # brute force on a tiny case
    off, srt, inv = orc.group(np.array([[2, 0], [0, 1], [2, 1]], np.int32), 3)
    assert off.tolist() == [0, 2, 4, 6] and srt.tolist() == [1, 2, 3, 5, 0, 4]
    assert inv.tolist() == [4, 0, 1, 2, 5, 3]


def test_swiglu_closed_form_and_clamps(orc):
    rng = np.random.default_rng(5)
    m = (rng.standard_normal((4, 64)) * 6).astype(np.float32)
    g, u = m[:, 0::2].astype(np.float64), m[:, 1::2].astype(np.float64)
    gc, uc = np.minimum(g, 7.0), np.clip(u, -7.0, 7.0)
    want = gc / (1 + np.exp(-1.702 * gc)) * (uc + 1)
    np.testing.assert_allclose(orc.swiglu(m, 7.0), want, rtol=3e-6, atol=1e-6)
    # special cases: gate > limit, up > limit, up < -limit (u+1 = -6), very negative gate -> 0
    cases = np.array([[9, 0.5], [1, 9], [1, -9], [-60, 3], [0, 5]], np.float32).reshape(1, -1)
    out = orc.swiglu(cases, 7.0)[0]
    sig = lambda x: 1 / (1 + np.exp(-1.702 * x))
    np.testing.assert_allclose(out, [7 * sig(7) * 1.5, sig(1) * 8, sig(1) * -6, 0.0, 0.0],
                               rtol=1e-6, atol=1e-30)
    # gate is the EVEN element: swapping the pair changes the result
    assert not np.allclose(orc.swiglu(np.array([[2.0, 0.5]], np.float32)),
                           orc.swiglu(np.array([[0.5, 2.0]], np.float32)))


def test_moe_layer_dense_one_hot_formulation(orc):
    rng = np.random.default_rng(6)
    B, H, I, E, k = 9, 32, 48, 6, 3
    t = rng.standard_normal((B, H)).astype(np.float32)
    wr = rng.standard_normal((E, H)).astype(np.float32) * 0.3
    br = rng.standard_normal(E).astype(np.float32) * 0.1
    w1 = rng.standard_normal((E, 2 * I, H)).astype(np.float32) * 0.2
    b1 = rng.standard_normal((E, 2 * I)).astype(np.float32) * 0.1
    w2 = rng.standard_normal((E, H, I)).astype(np.float32) * 0.2
    b2 = rng.standard_normal((E, H)).astype(np.float32) * 0.1
    out, logits, tv, ti = orc.moe_layer(t, wr, br, w1, b1, w2, b2, k=k, limit=7.0, want_routing=True)
    T = t.astype(np.float64)
    lg = T @ wr.T.astype(np.float64) + br
    np.testing.assert_allclose(logits, lg, rtol=1e-5, atol=1e-6)
    order = np.argsort(-lg, axis=1)[:, :k]
    np.testing.assert_array_equal(ti, order)
    G = np.zeros((B, E))
    sel = np.take_along_axis(lg, order, 1)
    wts = np.exp(sel - sel.max(1, keepdims=True)); wts /= wts.sum(1, keepdims=True)
    np.put_along_axis(G, order, wts, 1)
    want = np.zeros((B, H))
    for e in range(E):
        y1 = T @ w1[e].T.astype(np.float64) + b1[e]
        g, u = np.minimum(y1[:, 0::2], 7.0), np.clip(y1[:, 1::2], -7.0, 7.0)
        a = g / (1 + np.exp(-1.702 * g)) * (u + 1)
        want += G[:, [e]] * (a @ w2[e].T.astype(np.float64) + b2[e])
    np.testing.assert_allclose(out, want, rtol=2e-5, atol=2e-6)


def _naive_attn(q, K, V, lens, sinks, window):
    B, n_q, D = q.shape
    n_kv = K.shape[2]
    out = np.zeros((B, n_q, D))
    for b in range(B):
        L = int(lens[b]); lo = max(0, L - window) if window > 0 else 0
        for h in range(n_q):
            g = h // (n_q // n_kv)
            s = K[b, lo:L, g].astype(np.float64) @ q[b, h].astype(np.float64) / np.sqrt(D)
            z = np.concatenate([s, [sinks[h]]])                   # the sink is one more logit ...
            p = np.exp(z - z.max()); p /= p.sum()
            out[b, h] = p[:-1] @ V[b, lo:L, g].astype(np.float64)  # ... whose value row is zero
    return out


def test_attn_decode_against_naive_softmax(orc):
    rng = np.random.default_rng(7)
    B, S, n_q, n_kv, D = 3, 40, 8, 2, 16
    q = rng.standard_normal((B, n_q, D)).astype(np.float32)
    K = rng.standard_normal((B, S, n_kv, D)).astype(np.float32)
    V = rng.standard_normal((B, S, n_kv, D)).astype(np.float32)
    sinks = rng.standard_normal(n_q).astype(np.float32)
    lens = np.array([1, 17, 40], np.int32)
    for window in (0, 8, 100):
        np.testing.assert_allclose(orc.attn_decode(q, K, V, lens, sinks, window),
                                   _naive_attn(q, K, V, lens, sinks, window), rtol=2e-5, atol=2e-6)
    # window >= len is full attention; a very negative sink is plain softmax attention (SDPA)
    np.testing.assert_array_equal(orc.attn_decode(q, K, V, lens, sinks, 40),
                                  orc.attn_decode(q, K, V, lens, sinks, 0))
    import torch
    full = np.array([S] * B, np.int32)
    got = orc.attn_decode(q, K, V, full, np.full(n_q, -1e30, np.float32), 0)
    Kt = torch.from_numpy(K).permute(0, 2, 1, 3).repeat_interleave(n_q // n_kv, 1)
    Vt = torch.from_numpy(V).permute(0, 2, 1, 3).repeat_interleave(n_q // n_kv, 1)
    want = torch.nn.functional.scaled_dot_product_attention(torch.from_numpy(q).unsqueeze(2), Kt, Vt)
    np.testing.assert_allclose(got, want.squeeze(2).numpy(), rtol=2e-5, atol=2e-6)


def test_rope_tables(orc, synth):
    cfg = synth.tiny_config(64)
    cs, sn = orc.rope_tables(cfg, 64)
    conc = 0.1 * np.log(32.0) + 1.0
    np.testing.assert_allclose(cs ** 2 + sn ** 2, conc ** 2, rtol=1e-5)
    np.testing.assert_allclose(cs[0], conc, rtol=1e-6)            # position 0: no rotation
    assert np.all(sn[0] == 0)
    # highest frequency pair (i=0) rotates by exactly pos radians (extrapolation side of the ramp)
    np.testing.assert_allclose(cs[5, 0], conc * np.cos(5.0), rtol=1e-5)
    # lowest frequency pair is fully interpolated: angle = pos / (32 * theta^((D-2)/D))
    ang = 5.0 / (32.0 * 150000.0 ** (30.0 / 32.0))
    np.testing.assert_allclose(sn[5, -1], conc * np.sin(ang), rtol=1e-4)
    if orc.have_ref():
        R = orc.ref()
        c = np.zeros(16, np.float32); s = np.zeros(16, np.float32)
        for pos in (0, 1, 17, 63):
            R.ref_rope(pos, C.c_float(cfg.rope_theta), cfg.head_dim, C.c_float(cfg.rope_scaling_factor),
                       C.c_float(cfg.initial_context_length), c.ctypes.data_as(C.c_void_p),
                       s.ctypes.data_as(C.c_void_p))
            np.testing.assert_array_equal(cs[pos], c)
            np.testing.assert_array_equal(sn[pos], s)


def test_mxfp4_dequant_brute_force(orc):
    lut = [0, .5, 1, 1.5, 2, 3, 4, 6, -0.0, -.5, -1, -1.5, -2, -3, -4, -6]
    for scale in range(0, 256, 5):
        blocks = np.zeros((1, 16), np.uint8)
        for j in range(16):
            blocks[0, j] = j | ((15 - j) << 4)                     # low nibble j, high nibble 15-j
        got = orc.mxfp4_dequant(blocks, np.array([scale], np.uint8))[0]
        want = np.empty(32, np.float64)
        want[0::2] = [lut[j] for j in range(16)]                    # low nibble -> even element
        want[1::2] = [lut[15 - j] for j in range(16)]
        with np.errstate(over="ignore", under="ignore"):
            want = np.ldexp(want, scale - 127).astype(np.float32)
        np.testing.assert_array_equal(got, want)


# ------------------------------------------------------------------ whole model
@pytest.fixture(scope="module")
def tiny(synth, binfmt, tmp_path_factory):
    fx = json.load(open(GOLDEN))
    cfg = binfmt.Config(**fx["config"])
    path = str(tmp_path_factory.mktemp("tiny") / "tiny.bin")
    binfmt.write_bin(path, cfg, synth.random_tensors(cfg, fx["weight_seed"]))
    return fx, cfg, path


def test_bin_roundtrip_and_fixture_checkpoint(tiny, binfmt):
    fx, cfg, path = tiny
    assert hashlib.sha256(open(path, "rb").read()).hexdigest() == fx["bin_sha256"], \
        "the seeded checkpoint differs from the one the golden ids were made with"
    c2, tensors = binfmt.read_bin(path)
    assert c2 == cfg and binfmt.HEADER_BYTES == 60
    assert os.path.getsize(path) == 60 + 4 * binfmt.n_weight_floats(cfg)
    assert tensors["mlp1_weight"].shape == (4, 8, 512, 256) and tensors["sinks"].shape == (4, 8)


def test_oracle_generate_matches_golden_ids(tiny, orc, synth):
    fx, cfg, path = tiny
    flat = np.fromfile(path, dtype="<f4", offset=60)
    prompts = np.asarray(fx["prompts"], np.int32)
    np.testing.assert_array_equal(prompts, synth.random_prompts(cfg, fx["n_req"], fx["n_prompt"], fx["prompt_seed"]))
    out, n = orc.generate(cfg, flat, prompts, fx["max_seq_len"])
    np.testing.assert_array_equal(out[:, :fx["n_prompt"]], np.asarray(fx["expected_ids"]))
    assert (out[:, fx["terminator_index"]] == -1).all() and n == fx["n_generated"]
    m = orc.Model(cfg, flat)
    lg = m.forward(int(prompts[0, 0]), 0)
    assert int(lg.argmax()) == fx["first_logits_req0"]["argmax"]
    np.testing.assert_allclose(lg[:8], fx["first_logits_req0"]["head"], rtol=1e-6)
    np.testing.assert_allclose(lg.astype(np.float64).sum(), fx["first_logits_req0"]["sum"], rtol=1e-6)


def test_oracle_forward_bit_identical_to_reference_cpu(tiny, orc):
    if not orc.have_ref():
        pytest.skip("oracle/_ref not built (reference tree absent)")
    fx, cfg, path = tiny
    flat = np.fromfile(path, dtype="<f4", offset=60)
    R = orc.ref()
    assert R.ref_sizeof_config() == 60
    h = C.c_void_p(R.ref_open(path.encode()))
    m = orc.Model(cfg, flat)
    for pos, tok in enumerate([5, 99, 1000, 4000, 17, 17, 2048]):
        lr = np.ctypeslib.as_array(R.ref_forward(h, tok, pos), shape=(cfg.vocab_size,)).copy()
        np.testing.assert_array_equal(m.forward(tok, pos), lr)
    R.ref_close(h)
    prompts = np.asarray(fx["prompts"], np.int32)[:2]
    ro, rn = orc.ref_generate(path, prompts, fx["max_seq_len"])
    oo, on = orc.generate(cfg, flat, prompts, fx["max_seq_len"])
    np.testing.assert_array_equal(ro, oo)
    assert rn == on


def test_sliding_window_layers_are_the_even_ones(orc, synth):
    """run.cpp:582-584 masks positions `pos - t >= window` on layers with `l % 2 == 0`.  Two-layer
    model, window 4, 7 positions.  With the output projection of layer 1 zeroed only layer 0's
    attention reaches the logits: they must change with the window (layer 0 is windowed).  With the
    output projection of layer 0 zeroed instead only layer 1's attention does: they must not change
    (layer 1 sees every position).  An oracle that windowed the odd layers fails both halves."""
    import dataclasses
    base = dataclasses.replace(synth.tiny_config(16), n_layers=2, vocab_size=64, sliding_window=4)
    from conftest import load_pkg
    binfmt = load_pkg("binfmt")

    def run(cfg, mute_layer=None, n_pos=7):
        T = synth.random_tensors(base, 3, std=0.2)
        if mute_layer is not None:
            T["out_weight"][mute_layer] = 0
            T["out_bias"][mute_layer] = 0
        flat = np.concatenate([np.asarray(T[n], np.float32).ravel() for n in binfmt.tensor_shapes(base)])
        m = orc.Model(cfg, flat)
        for pos in range(n_pos):
            lg = m.forward(pos + 1, pos)
        return lg

    no_window = dataclasses.replace(base, sliding_window=0)
    a = run(base)
    b = run(no_window)
    c = run(dataclasses.replace(base, sliding_window=16))
    assert not np.allclose(a, b) and np.array_equal(b, c)
    assert not np.allclose(run(base, mute_layer=1), run(no_window, mute_layer=1))      # layer 0: windowed
    assert np.array_equal(run(base, mute_layer=0), run(no_window, mute_layer=0))       # layer 1: not
    # the mask is `pos - t >= window`: at position window-1 nothing is masked yet, at position window
    # exactly one position is
    assert np.array_equal(run(base, 1, n_pos=4), run(no_window, 1, n_pos=4))
    assert not np.array_equal(run(base, 1, n_pos=5), run(no_window, 1, n_pos=5))


WINDOW_GOLDEN = os.path.join(HERE, "golden", "window_e2e.json")


@pytest.fixture(scope="module")
def windowed(synth, binfmt, tmp_path_factory):
    fx = json.load(open(WINDOW_GOLDEN))
    cfg = binfmt.Config(**fx["config"])
    path = str(tmp_path_factory.mktemp("window") / "window.bin")
    binfmt.write_bin(path, cfg, synth.random_tensors(cfg, fx["weight_seed"], std=fx["weight_std"], gate_scale=fx["gate_scale"]))
    assert hashlib.sha256(open(path, "rb").read()).hexdigest() == fx["bin_sha256"]
    return fx, cfg, path


def test_oracle_matches_the_reference_ids_past_the_window(windowed, orc):
    """tests/golden/window_e2e.json: ids and logit probes the reference's own CPU model produced for
    a 3-layer model with window 8 over 79 positions (248 of the 256 ids change when the window is
    taken away, so the mask and the even-layer rule decide them)."""
    fx, cfg, path = windowed
    flat = np.fromfile(path, dtype="<f4", offset=60)
    prompts = np.asarray(fx["prompts"], np.int32)
    out, n = orc.generate(cfg, flat, prompts, fx["max_seq_len"])
    gold = np.asarray(fx["expected_ids"], np.int32)
    np.testing.assert_array_equal(out[:, :gold.shape[1]], gold)
    assert (out[:, fx["terminator_index"]] == -1).all() and n == fx["n_generated"]
    m = orc.Model(cfg, flat)
    seq = list(prompts[0]) + list(gold[0])
    probes = {p["pos"]: p for p in fx["logits_req0"]}
    for pos in range(fx["max_seq_len"] - 1):
        lg = m.forward(int(seq[pos]), pos)
        if pos in probes:
            assert int(lg.argmax()) == probes[pos]["argmax"]
            assert float(lg.max()) == probes[pos]["max"]
            np.testing.assert_allclose(lg.astype(np.float64).sum(), probes[pos]["sum"], rtol=1e-9)


def test_oracle_forward_bit_identical_to_reference_cpu_past_the_window(orc, synth, binfmt, tmp_path):
    """The reference's own compiled forward() against the oracle, logits bit for bit, on models that
    run well past their sliding window (run.cpp:157-164,582-584): windows 4..8, 3 and 4 layers,
    24 positions."""
    if not orc.have_ref():
        pytest.skip("oracle/_ref not built (reference tree absent)")
    import dataclasses
    R = orc.ref()
    rng = np.random.default_rng(12)
    for window, layers in ((4, 3), (6, 4), (8, 3)):
        cfg = dataclasses.replace(synth.tiny_config(2048), n_layers=layers, hidden_dim=128, n_attn_heads=4,
                                  n_kv_heads=2, intermediate_dim=64, vocab_size=256, sliding_window=window)
        path = str(tmp_path / f"w{window}.bin")
        binfmt.write_bin(path, cfg, synth.random_tensors(cfg, 40 + window, std=0.08))
        flat = np.fromfile(path, dtype="<f4", offset=60)
        h = C.c_void_p(R.ref_open(path.encode()))
        m = orc.Model(cfg, flat)
        for pos in range(24):
            tok = int(rng.integers(cfg.vocab_size))
            lr = np.ctypeslib.as_array(R.ref_forward(h, tok, pos), shape=(cfg.vocab_size,)).copy()
            np.testing.assert_array_equal(m.forward(tok, pos), lr, err_msg=f"window {window} pos {pos}")
        R.ref_close(h)
        m.close()
