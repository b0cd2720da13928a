"""End-to-end parity of the decode engine on the tiny GPT-OSS configuration: a flat .bin written
from seeds, loaded by the engine, compared with the CPU oracle and with the golden ids that the
reference's own CPU model produced (tests/golden/tiny_e2e.json)."""
import json
import os

import numpy as np
import pytest

from conftest import rel_errors

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "tiny_e2e.json")


@pytest.fixture(scope="module")
def tiny(synth, binfmt, tmp_path_factory):
    fx = json.load(open(GOLDEN))
    cfg = binfmt.Config(**fx["config"])
    path = str(tmp_path_factory.mktemp("tiny") / "tiny.bin")
    binfmt.write_bin(path, cfg, synth.random_tensors(cfg, fx["weight_seed"]))
    cfg2, _ = binfmt.read_bin(path)
    flat = np.fromfile(path, dtype="<f4", offset=binfmt.HEADER_BYTES)
    return fx, cfg2, flat


def test_first_steps_logits_match_oracle(ops, orc, tiny):
    """Teacher-forced logits of 40 positions against the fp32 CPU model and against the same CPU
    model rounded where the GPU dataflow rounds (bf16 activations into every GEMM, bf16 KV).
    A step in which some layer's 4th and 5th router scores are closer than the bf16 noise of this
    dataflow may legitimately pick another expert; those steps are counted, not compared."""
    fx, cfg, flat = tiny
    prompts = np.asarray(fx["prompts"], np.int32)
    B, T = 4, 40
    seqs = np.concatenate([prompts[:B], np.asarray(fx["expected_ids"], np.int32)[:B]], axis=1)[:, :T]
    eng = ops.Engine(cfg, flat, max_batch=B, max_seq=64)
    exact = [orc.Model(cfg, flat) for _ in range(B)]
    staged = [orc.Model(cfg, flat, stage=orc.STAGE_GPU) for _ in range(B)]
    worst_exact = worst_staged = 0.0
    compared = 0
    for pos in range(T):
        eng.step(seqs[:, pos], pos)
        got = eng.last_logits(B)
        for b in range(B):
            we = exact[b].forward(int(seqs[b, pos]), pos)
            ws = staged[b].forward(int(seqs[b, pos]), pos)
            if pos == 0:
                # one cached position, the same rounding points: what is left is fp32 summation
                # order plus the few-ulp difference of the hardware exp2/reciprocal in the SwiGLU,
                # which now and then moves one bf16 rounding of an activation (~1e-3 on the logits)
                assert rel_errors(got[b], ws)[0] <= 5e-3
            if min(exact[b].last_router_gap(), staged[b].last_router_gap()) < 3e-3:
                continue
            compared += 1
            worst_exact = max(worst_exact, rel_errors(got[b], we)[0])
            worst_staged = max(worst_staged, rel_errors(got[b], ws)[0])
    assert compared >= 0.8 * B * T, compared
    # bf16 tolerance (max rel err 2e-2) against the fp32 model and the equally-staged model
    assert worst_exact <= 2e-2, worst_exact
    assert worst_staged <= 2e-2, worst_staged
    print("compared", compared, "of", B * T, "worst vs fp32", worst_exact, "vs staged", worst_staged)
    eng.close()


def test_teacher_forced_ids_match_golden_where_margin_is_clear(ops, orc, tiny):
    """Feed the golden sequences; the engine's arg-max must be the golden id at every position
    where the reference's own decision is not a near-tie at bf16 precision: top-1/top-2 logit
    margin above 5e-3 and every layer's 4th/5th router score at least 3e-3 apart."""
    fx, cfg, flat = tiny
    prompts = np.asarray(fx["prompts"], np.int32)
    gold = np.asarray(fx["expected_ids"], np.int32)
    margins = np.asarray(fx["logit_margins"], np.float32)
    n_req, n_prompt = prompts.shape
    seqs = np.concatenate([prompts, gold], axis=1)
    eng = ops.Engine(cfg, flat, max_batch=n_req, max_seq=fx["max_seq_len"])
    cpu = [orc.Model(cfg, flat) for _ in range(n_req)]
    pred = np.zeros_like(gold)
    gaps = np.zeros(gold.shape, np.float32)
    for pos in range(fx["max_seq_len"] - 1):
        nxt = eng.step(seqs[:, pos], pos)
        for r in range(n_req):
            lg = cpu[r].forward(int(seqs[r, pos]), pos)
            if pos >= n_prompt - 1:
                assert int(lg.argmax()) == gold[r, pos - (n_prompt - 1)]   # the fixture is consistent
                gaps[r, pos - (n_prompt - 1)] = cpu[r].last_router_gap()
        if pos >= n_prompt - 1:
            pred[:, pos - (n_prompt - 1)] = nxt
    eng.close()
    clear = (margins > 5e-3) & (gaps > 3e-3)
    print("teacher-forced agreement: all positions", float((pred == gold).mean()),
          "clear positions", int(clear.sum()), "of", clear.size)
    assert clear.mean() > 0.6
    bad = np.argwhere((pred != gold) & clear)
    assert len(bad) == 0, [(int(r), int(i), float(margins[r, i]), float(gaps[r, i])) for r, i in bad]


def test_generate_follows_getp_loop_semantics(ops, orc, tiny):
    """Free-running greedy generation on the production (bf16-staged, MFMA) engine.

    Layout, terminator and count are the harness's.  The ids cannot equal the fp32 golden ids
    everywhere (top-1/top-2 logit margins and 4th/5th router gaps of this model reach 2e-4, below
    the noise of six bf16 roundings per layer); what must hold instead, and is asserted:

    1. every request's FIRST divergence from the golden ids sits at a position where the reference's
       own decision is a near-tie: logit margin < 5e-3 or a router gap < 3e-3 in the forward call
       that produced that id (both stored in the fixture; up to that position the engine has seen
       exactly the golden history);
    2. fed the engine's own output as history, the CPU model with the GPU dataflow's rounding points
       (STAGE_GPU) picks the engine's id at every position that is not such a near-tie for it: the
       engine's trajectory is a greedy trajectory of that model up to near-ties;
    3. hence the STAGE_GPU model's free-running ids equal the engine's up to each request's first
       near-tie position, which is checked directly as well.
    """
    fx, cfg, flat = tiny
    prompts = np.asarray(fx["prompts"], np.int32)
    eng = ops.Engine(cfg, flat, max_batch=4, max_seq=fx["max_seq_len"])   # 8 requests, 2 batches
    out, n = eng.generate(prompts, fx["max_seq_len"])
    eng.close()
    n_req, n_prompt = prompts.shape
    n_gen = fx["n_prompt"]
    assert n == fx["n_generated"]
    assert (out[:, fx["terminator_index"]] == -1).all()
    assert ((out[:, :n_gen] >= 0) & (out[:, :n_gen] < cfg.vocab_size)).all()
    gold = np.asarray(fx["expected_ids"], np.int32)
    margins = np.asarray(fx["logit_margins"], np.float32)
    gaps = np.asarray(fx["router_gaps"], np.float32)
    MARGIN, GAP = 5e-3, 3e-3

    # 1. against the reference's fp32 ids
    agree = out[:, :n_gen] == gold
    first_diff = [int(np.argmin(a)) if not a.all() else n_gen for a in agree]
    for r, d in enumerate(first_diff):
        if d < n_gen:
            assert margins[r, d] < MARGIN or gaps[r, d] < GAP, (r, d, float(margins[r, d]), float(gaps[r, d]))
    print("free-running agreement with the fp32 golden ids:", float(agree.mean()), first_diff)

    # 2. and 3. against the CPU model rounded where the GPU dataflow rounds
    clear_total = pinned_total = 0
    for r in range(n_req):
        seq = np.concatenate([prompts[r], out[r, :n_gen]])
        forced = orc.Model(cfg, flat, stage=orc.STAGE_GPU)       # sees the engine's history
        free = orc.Model(cfg, flat, stage=orc.STAGE_GPU)         # feeds back its own ids
        tok_free, free_alive = int(prompts[r, 0]), True
        for pos in range(fx["max_seq_len"] - 1):
            lg = forced.forward(int(seq[pos]), pos)
            i = pos - (n_prompt - 1)
            if free_alive:
                lf = free.forward(tok_free, pos)
                tok_free = int(prompts[r, pos + 1]) if i < 0 else int(lf.argmax())
            if i < 0:
                continue
            top2 = np.partition(lg, -2)[-2:]
            near = (top2[1] - top2[0]) < MARGIN or forced.last_router_gap() < GAP
            if not near:
                clear_total += 1
                assert int(lg.argmax()) == out[r, i], (r, i, float(top2[1] - top2[0]), forced.last_router_gap())
            if free_alive:
                if near:
                    free_alive = False          # from here on the two may legitimately part
                else:
                    pinned_total += 1
                    assert tok_free == out[r, i], (r, i)
        forced.close()
        free.close()
    print("positions where the staged CPU model's decision is clear:", clear_total, "of", n_req * n_gen,
          "; ids pinned before each request's first near-tie:", pinned_total)
    assert clear_total >= 0.6 * n_req * n_gen
    assert pinned_total >= n_req                 # not vacuous: about one clear id per request at least


def test_precise_engine_reproduces_the_golden_ids_exactly(ops, orc, tiny):
    """GPTOSS_ENGINE_PRECISE runs the reference CPU model's arithmetic on the GPU (fp32 weights and
    KV cache, double-accumulated dot products): free-running greedy generation must give exactly the
    ids the reference's own CPU model produced (tests/golden/tiny_e2e.json, 8 x 32 ids), with the
    getp loop's layout and count, and its logits must equal the CPU oracle's to fp32 rounding."""
    fx, cfg, flat = tiny
    prompts = np.asarray(fx["prompts"], np.int32)
    gold = np.asarray(fx["expected_ids"], np.int32)
    eng = ops.Engine(cfg, flat, max_batch=8, max_seq=fx["max_seq_len"], precise=True)
    out, n = eng.generate(prompts, fx["max_seq_len"])
    n_gen = gold.shape[1]
    assert n == fx["n_generated"]
    assert (out[:, fx["terminator_index"]] == -1).all()
    assert np.array_equal(out[:, :n_gen], gold)
    eng.close()
    # teacher-forced logits against the fp32 oracle (bit-identical to the compiled reference)
    B, T = 4, 40
    seqs = np.concatenate([prompts[:B], gold[:B]], axis=1)[:, :T]
    eng = ops.Engine(cfg, flat, max_batch=B, max_seq=64, precise=True)
    cpu = [orc.Model(cfg, flat) for _ in range(B)]
    worst = 0.0
    for pos in range(T):
        eng.step(seqs[:, pos], pos)
        got = eng.last_logits(B)
        for b in range(B):
            want = cpu[b].forward(int(seqs[b, pos]), pos)
            worst = max(worst, rel_errors(got[b], want)[0])
    eng.close()
    print("precise engine vs fp32 oracle, worst max-rel logit error:", worst)
    assert worst <= 2e-5, worst


def test_precise_engine_needs_host_weights(ops, tiny):
    from conftest import load_pkg
    lib = load_pkg("lib")
    fx, cfg, flat = tiny
    with pytest.raises(lib.GptossError):
        ops.Engine(cfg, None, max_batch=2, max_seq=16, synthetic=True, precise=True)


def test_engine_rejects_bad_arguments(ops, tiny):
    from conftest import load_pkg
    lib = load_pkg("lib")
    fx, cfg, flat = tiny
    import dataclasses
    with pytest.raises(lib.GptossError) as ei:
        ops.Engine(dataclasses.replace(cfg, head_dim=48), flat, max_batch=2, max_seq=16)
    assert ei.value.code == 2
    eng = ops.Engine(cfg, flat, max_batch=2, max_seq=16)
    with pytest.raises(lib.GptossError):
        eng.step(np.zeros(3, np.int32), 0)            # batch larger than max_batch
    with pytest.raises(lib.GptossError):
        eng.step(np.zeros(2, np.int32), 16)           # position beyond max_seq
    eng.close()


def test_fused_argmax_equals_argmax_of_logits(ops, tiny):
    """Without GPTOSS_ENGINE_LOGITS the classifier GEMM keeps only each row's arg-max (two stages:
    per column tile in the GEMM epilogue, then across tiles); the ids must equal those of the
    engine that writes the logits and arg-maxes them, step for step, ties included."""
    fx, cfg, flat = tiny
    prompts = np.asarray(fx["prompts"], np.int32)
    a = ops.Engine(cfg, flat, max_batch=8, max_seq=48, keep_logits=True)
    b = ops.Engine(cfg, flat, max_batch=8, max_seq=48, keep_logits=False)
    tok = prompts[:, 0].copy()
    for pos in range(40):
        na, nb = a.step(tok, pos), b.step(tok, pos)
        assert np.array_equal(na, nb), pos
        assert np.array_equal(na, a.last_logits(8).argmax(axis=1))
        tok = na
    with pytest.raises(RuntimeError):
        b.last_logits(8)
    a.close()
    b.close()


def test_prefill_equals_lockstep_steps(ops, tiny):
    """One prompt pass over T positions must leave the engine where T lock-step steps leave it:
    the same next ids, and bit-identical logits on the decode steps that follow (T below the
    sliding window, so no ring has wrapped)."""
    fx, cfg, flat = tiny
    prompts = np.asarray(fx["prompts"], np.int32)
    gold = np.asarray(fx["expected_ids"], np.int32)
    seqs = np.concatenate([prompts, gold], axis=1)
    B, T = 8, 32
    a = ops.Engine(cfg, flat, max_batch=B, max_seq=64)
    b = ops.Engine(cfg, flat, max_batch=B, max_seq=64)
    for pos in range(T):
        na = a.step(seqs[:, pos], pos)
    la = a.last_logits(B).copy()
    nb = b.prefill(seqs[:, :T])
    assert np.array_equal(na, nb)
    assert np.array_equal(la, b.last_logits(B))
    for pos in range(T, T + 12):
        na, nb = a.step(seqs[:, pos], pos), b.step(seqs[:, pos], pos)
        assert np.array_equal(na, nb), pos
        assert np.array_equal(a.last_logits(B), b.last_logits(B)), pos
    a.close()
    b.close()


def test_prefill_longer_than_the_window_and_in_several_passes(ops, orc, tiny):
    """200-token prompts: longer than the 128-position ring of the sliding-window layers (they read
    a linear copy during the pass and keep the last 128 positions), and with 48 sequences more rows
    (9600) than one pass holds (8192), so the last 8 sequences go through in a second pass.
    Compared with lock-step steps (equal to rounding: a wrapped ring sums in another order) and,
    for sequences of both passes, with the fp32 oracle."""
    fx, cfg, flat = tiny
    rng = np.random.default_rng(11)
    B, T, S = 48, 200, 212
    seqs = rng.integers(0, cfg.vocab_size, size=(B, S)).astype(np.int32)
    a = ops.Engine(cfg, flat, max_batch=B, max_seq=S)
    b = ops.Engine(cfg, flat, max_batch=B, max_seq=S)
    for pos in range(T):
        na = a.step(seqs[:, pos], pos)
    nb = b.prefill(seqs[:, :T])
    lb = b.last_logits(B).copy()
    mx, _ = rel_errors(lb, a.last_logits(B))
    assert mx <= 5e-3, mx
    assert (na == nb).mean() >= 0.9
    for r in (0, 39, 40, 47):
        cpu = orc.Model(cfg, flat)
        for pos in range(T):
            want = cpu.forward(int(seqs[r, pos]), pos)
        mx, _ = rel_errors(lb[r], want)
        assert mx <= 2e-2, (r, mx)
    # decode steps after the pass, per sequence: equal to bf16 rounding, except where that rounding
    # moves a near-tie of the router to another expert (a handful of sequence-steps)
    diffs = []
    for pos in range(T, S):
        a.step(seqs[:, pos], pos)
        b.step(seqs[:, pos], pos)
        la, lb = a.last_logits(B), b.last_logits(B)
        diffs.append(np.abs(lb - la).max(axis=1) / np.abs(la).max(axis=1))
    diffs = np.concatenate(diffs)
    print("prefill vs lock-step after a wrapped window: median", float(np.median(diffs)),
          "sequence-steps above 5e-3:", int((diffs > 5e-3).sum()), "of", diffs.size)
    assert np.median(diffs) <= 5e-3
    assert (diffs > 5e-3).mean() <= 0.03
    a.close()
    b.close()


def test_generate_with_prefill_equals_generate_without(ops, tiny):
    """gptoss_engine_generate sends the prompt positions all sequences of a batch share through one
    pass; its output must be the lock-step loop's, ragged prompt lengths included."""
    fx, cfg, flat = tiny
    prompts = np.asarray(fx["prompts"], np.int32)
    ragged = np.asarray([32, 20, 32, 9, 32, 32, 2, 32], np.int32)   # shared prefixes of 9 and of 2
    outs = []
    for prefill in (True, False):
        eng = ops.Engine(cfg, flat, max_batch=4, max_seq=fx["max_seq_len"], prefill=prefill)
        outs.append(eng.generate(prompts, fx["max_seq_len"], n_prompt=ragged))
        outs.append(eng.generate(prompts, fx["max_seq_len"]))          # all 32 prompt tokens in one pass
        eng.close()
    assert np.array_equal(outs[0][0], outs[2][0]) and outs[0][1] == outs[2][1]
    assert np.array_equal(outs[1][0], outs[3][0]) and outs[1][1] == outs[3][1]
    with pytest.raises(Exception):
        ops.Engine(cfg, flat, max_batch=2, max_seq=16, prefill=False).prefill(prompts[:2, :8])


def test_step_ragged_equals_lockstep_per_sequence(ops, tiny):
    """Sequences at different positions in one step: each must get, bit for bit, the logits it gets
    when the whole batch is at its position (sequence i runs i steps behind sequence 0)."""
    fx, cfg, flat = tiny
    prompts = np.asarray(fx["prompts"], np.int32)
    gold = np.asarray(fx["expected_ids"], np.int32)
    seqs = np.concatenate([prompts, gold], axis=1)
    B, n_steps = 6, 30
    a = ops.Engine(cfg, flat, max_batch=B, max_seq=64)
    ref = []
    for pos in range(n_steps):
        a.step(seqs[:B, pos], pos)
        ref.append(a.last_logits(B).copy())
    a.close()
    b = ops.Engine(cfg, flat, max_batch=B, max_seq=64)
    lag = np.arange(B)
    for step in range(n_steps + B - 1):
        pos = np.clip(step - lag, 0, n_steps - 1)
        live = (step - lag >= 0) & (step - lag < n_steps)
        b.step_ragged(seqs[np.arange(B), pos], pos)
        got = b.last_logits(B)
        for i in np.nonzero(live)[0]:
            assert np.array_equal(got[i], ref[pos[i]][i]), (step, i)
    b.close()


def test_continuous_schedule_gives_the_lockstep_output(ops, tiny):
    """20 requests with ragged prompts and ragged length limits over 4 slots: slots are refilled as
    their sequences end.  Every request's output must be what it gets when run the reference's way
    (lock-step batches; a request with a smaller limit produces a prefix), and the token count must
    be the sum of the per-request counts."""
    fx, cfg, flat = tiny
    rng = np.random.default_rng(5)
    n_req, S = 20, fx["max_seq_len"]
    prompts = rng.integers(0, cfg.vocab_size, size=(n_req, 24)).astype(np.int32)
    n_prompt = rng.integers(1, 25, size=n_req).astype(np.int32)
    max_len = rng.integers(2, S + 1, size=n_req).astype(np.int32)
    max_len[3] = 1                                              # a request that may not take a step
    ref = ops.Engine(cfg, flat, max_batch=4, max_seq=S, prefill=False)
    want, _ = ref.generate(prompts, S, n_prompt=n_prompt)        # everyone runs to the common limit
    ref.close()
    eng = ops.Engine(cfg, flat, max_batch=4, max_seq=S)
    got, n = eng.generate(prompts, S, n_prompt=n_prompt, max_len=max_len)
    same, n_same = eng.generate(prompts, S, n_prompt=n_prompt)
    eng.close()
    assert np.array_equal(same, want)                            # no limits: the lock-step output
    total = 0
    for r in range(n_req):
        gen = max(0, int(max_len[r]) - 1 - int(n_prompt[r]))     # positions left after the prompt
        total += gen + 1
        assert got[r, gen + 1] == -1, r
        assert np.array_equal(got[r, :gen + 1], want[r, :gen + 1]) or gen == 0, r
        if gen > 0:
            assert np.array_equal(got[r, :gen], want[r, :gen]), r
    assert n == total


def test_continuous_schedule_runs_admitted_prompts_as_rows_of_a_step(ops, tiny):
    """40 requests with prompts of 1..100 tokens and ragged limits over 6 slots.  A request admitted
    into a slot that has become free runs all the prompt positions it has left as consecutive rows
    of the next step, next to the single rows of the sequences that are decoding (every row's K/V
    is stored before any row attends).  Outputs and token count must be exactly the lock-step
    schedule's (rows are bit-equal to their lock-step steps: contexts below 512 positions, prompts
    inside the first lap of the 128-slot ring), and the schedule must take far fewer steps than one
    per position."""
    fx, cfg, flat = tiny
    rng = np.random.default_rng(17)
    n_req, S = 40, 140
    prompts = rng.integers(0, cfg.vocab_size, size=(n_req, 100)).astype(np.int32)
    n_prompt = rng.integers(2, 101, size=n_req).astype(np.int32)
    n_prompt[[4, 9]] = 1                                         # no stretch to run
    max_len = np.minimum(S, n_prompt + rng.integers(1, 30, size=n_req)).astype(np.int32)
    ref = ops.Engine(cfg, flat, max_batch=6, max_seq=S, prefill=False)
    want, _ = ref.generate(prompts, S, n_prompt=n_prompt)
    ref.close()
    eng = ops.Engine(cfg, flat, max_batch=6, max_seq=S)
    with ops.KernelTrace(capacity=16384) as tr:
        got, n = eng.generate(prompts, S, n_prompt=n_prompt, max_len=max_len)
    eng.close()
    total = 0
    for r in range(n_req):
        gen = max(0, int(max_len[r]) - 1 - int(n_prompt[r]))
        total += gen + 1
        assert got[r, gen + 1] == -1, r
        if gen > 0:
            assert np.array_equal(got[r, :gen], want[r, :gen]), r
    assert n == total
    steps = sum(1 for name, _ in tr.results() if name == "embedding")   # one per step or pass
    positions = int((max_len - 1).sum())
    print("continuous schedule:", steps, "steps and passes for", positions, "positions on 6 slots")
    assert steps < 0.5 * positions / 6, (steps, positions)


def test_step_rows_stop_at_the_ring_capacity(ops, tiny, binfmt):
    """Prompts longer than the sliding-window ring (here 64 slots holding a window of 8): a stretch
    of rows may only cover the ring's first lap, the rest of the prompt is forced one position per
    step.  The continuous schedule must still give the lock-step output."""
    import dataclasses
    fx, cfg0, flat = tiny
    cfg = dataclasses.replace(cfg0, sliding_window=8)            # same tensors, a short window
    rng = np.random.default_rng(23)
    n_req, S = 10, 120
    prompts = rng.integers(0, cfg.vocab_size, size=(n_req, 90)).astype(np.int32)
    n_prompt = rng.integers(60, 91, size=n_req).astype(np.int32)
    n_prompt[:3] = (40, 50, 45)        # the first three share a prompt pass: keep it inside the ring too
    max_len = (n_prompt + rng.integers(2, 20, size=n_req)).astype(np.int32)
    ref = ops.Engine(cfg, flat, max_batch=3, max_seq=S, prefill=False)
    want, _ = ref.generate(prompts, S, n_prompt=n_prompt)
    ref.close()
    eng = ops.Engine(cfg, flat, max_batch=3, max_seq=S)
    got, n = eng.generate(prompts, S, n_prompt=n_prompt, max_len=max_len)
    eng.close()
    for r in range(n_req):
        gen = int(max_len[r]) - 1 - int(n_prompt[r])
        assert got[r, gen + 1] == -1, r
        assert np.array_equal(got[r, :gen], want[r, :gen]), r


def test_stop_ids_in_prompts_and_schedules_agree(ops, orc, binfmt, synth):
    """A model with the real vocabulary size (so that the stop ids 199999 and 200002 exist) and
    prompts that contain them: a forced stop id ends its sequence in the reference's loop
    (getp_run_submit.cpp:75-83, run.cpp:939-941).  The continuous schedule with the prompt pass,
    the lock-step schedule and the fp32-faithful engine must all end every sequence where the CPU
    oracle ends it and report its token count; the two bf16 schedules must agree id for id, and the
    fp32-faithful engine must reproduce the oracle's ids."""
    cfg = binfmt.Config(vocab_size=200064, hidden_dim=64, n_experts=4, experts_per_token=2,
                        intermediate_dim=64, n_layers=2, head_dim=32, n_attn_heads=2, n_kv_heads=1,
                        seq_len=2048, initial_context_length=4096, rope_theta=150000.0,
                        rope_scaling_factor=32.0, sliding_window=128, swiglu_limit=7.0)
    tensors = synth.random_tensors(cfg, 3)
    flat = np.concatenate([np.asarray(t, np.float32).ravel() for t in tensors.values()])
    rng = np.random.default_rng(4)
    n_req, stride, S = 7, 12, 24
    prompts = rng.integers(0, 199000, size=(n_req, stride)).astype(np.int32)
    prompts[1, 5] = 199999          # ends in the middle of its prompt
    prompts[2, 1] = 200002          # ends at the first forced token
    prompts[3, stride - 1] = 199999  # ends at the last prompt token
    prompts[5, 0] = 200002          # the first token is never checked
    prompts[6, 3] = 200002
    prompts[6, 7] = 199999
    want, n_want = orc.generate(cfg, flat, prompts, S)
    ends = (want < 0).argmax(axis=1)
    outs = {}
    for name, kw in (("continuous", {}), ("lockstep", {"prefill": False}), ("precise", {"precise": True})):
        eng = ops.Engine(cfg, flat, max_batch=3, max_seq=S, **kw)      # 7 requests over 3 slots
        outs[name] = eng.generate(prompts, S)
        eng.close()
        got, n = outs[name]
        assert n == n_want, name
        assert np.array_equal((got < 0).argmax(axis=1), ends), name
    assert np.array_equal(outs["continuous"][0], outs["lockstep"][0])
    assert np.array_equal(outs["precise"][0], want)
    assert sorted(set(ends.tolist())) != [S - stride + 1]              # some sequences did end early


def test_mxfp4_expert_storage_is_bit_identical_to_bf16_storage(ops, orc, tiny, synth, binfmt):
    """GPT-OSS expert weights are MXFP4 at the source and the .bin holds their dequantised values.
    With such a payload GPTOSS_ENGINE_MXFP4_EXPERTS converts the experts back to MXFP4 exactly, and
    every step must give the logits of the bf16 storage bit for bit (same bf16 operands, same MFMA
    order), in lock step, through the prompt pass and in generation (the bf16 storage is what the
    other tests hold against the oracle).  A payload that is not representable must be refused."""
    fx, cfg, _ = tiny
    lib = __import__("conftest").load_pkg("lib")
    rng = np.random.default_rng(21)
    tensors = synth.random_tensors(cfg, 5)
    L, E, H, I = cfg.n_layers, cfg.n_experts, cfg.hidden_dim, cfg.intermediate_dim
    for name, (n_out, n_in) in (("mlp1_weight", (2 * I, H)), ("mlp2_weight", (H, I))):
        blocks = rng.integers(0, 256, size=(L * E * n_out * n_in // 32, 16), dtype=np.uint8)
        scales = (127 + rng.integers(-9, -3, size=L * E * n_out * n_in // 32)).astype(np.uint8)
        blocks[:7] = 0                                     # an all-zero block, zeros next to large codes
        tensors[name] = orc.mxfp4_dequant(blocks, scales).reshape(L, E, n_out, n_in)
    flat = np.concatenate([np.asarray(tensors[n], np.float32).ravel() for n in binfmt.tensor_shapes(cfg)])
    prompts = np.asarray(fx["prompts"], np.int32)
    B, T = 8, 20
    a = ops.Engine(cfg, flat, max_batch=B, max_seq=64)
    b = ops.Engine(cfg, flat, max_batch=B, max_seq=64, mxfp4_experts=True)
    assert b.device_bytes() < a.device_bytes()
    for pos in range(T):
        na, nb = a.step(prompts[:, pos], pos), b.step(prompts[:, pos], pos)
        assert np.array_equal(na, nb), pos
        assert np.array_equal(a.last_logits(B), b.last_logits(B)), pos
    assert np.array_equal(a.prefill(prompts[:, :T]), b.prefill(prompts[:, :T]))
    assert np.array_equal(a.last_logits(B), b.last_logits(B))
    ga, gb = a.generate(prompts, fx["max_seq_len"]), b.generate(prompts, fx["max_seq_len"])
    assert np.array_equal(ga[0], gb[0]) and ga[1] == gb[1]
    a.close()
    b.close()
    # the golden model's experts are bf16-rounded normals: no exact MXFP4 form
    with pytest.raises(lib.GptossError) as ei:
        ops.Engine(cfg, tiny[2], max_batch=2, max_seq=16, mxfp4_experts=True)
    assert ei.value.code == 6 or "MXFP4" in str(ei.value)


def test_prefill_and_ragged_step_edge_cases(ops, tiny):
    """One position, one sequence, the whole context in one pass; arguments out of range."""
    from conftest import load_pkg
    lib = load_pkg("lib")
    fx, cfg, flat = tiny
    prompts = np.asarray(fx["prompts"], np.int32)
    a = ops.Engine(cfg, flat, max_batch=3, max_seq=32)
    b = ops.Engine(cfg, flat, max_batch=3, max_seq=32)
    # T = 1 is one lock-step step
    assert np.array_equal(a.prefill(prompts[:3, :1]), b.step(prompts[:3, 0], 0))
    assert np.array_equal(a.last_logits(3), b.last_logits(3))
    # a single sequence, the whole context (T = max_seq) in one pass
    na = a.prefill(prompts[5:6, :32])
    for pos in range(32):
        nb = b.step(prompts[5:6, pos], pos)
    assert np.array_equal(na, nb) and np.array_equal(a.last_logits(1), b.last_logits(1))
    # ragged step with equal positions is the lock-step step
    a.step(prompts[:3, 0], 0), b.step(prompts[:3, 0], 0)
    assert np.array_equal(a.step_ragged(prompts[:3, 1], [1, 1, 1]), b.step(prompts[:3, 1], 1))
    assert np.array_equal(a.last_logits(3), b.last_logits(3))
    wide = np.concatenate([prompts[:3], prompts[:3, :1]], axis=1)     # 33 positions
    for bad in (lambda: a.prefill(wide),                              # more positions than max_seq
                lambda: a.prefill(prompts[:4, :4]),                   # more sequences than max_batch
                lambda: a.step_ragged(prompts[:3, 0], [0, 32, 0]),    # a position beyond max_seq
                lambda: a.step_ragged(prompts[:3, 0], [0, -1, 0]),
                lambda: a.generate(prompts[:3, :4], 40)):             # longer than the engine holds
        with pytest.raises(lib.GptossError):
            bad()
    a.close()
    b.close()
    c = ops.Engine(cfg, flat, max_batch=2, max_seq=16, precise=True)
    with pytest.raises(lib.GptossError):
        c.step_ragged(prompts[:2, 0], [0, 0])
    with pytest.raises(lib.GptossError):
        c.prefill(prompts[:2, :4])
    with pytest.raises(lib.GptossError):
        c.generate(prompts[:2, :4], 12, max_len=[8, 8])              # limits need the continuous schedule
    c.close()


# ------------------------------------------------------------------ ten windows past the window
WINDOW_GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "window_e2e.json")


@pytest.fixture(scope="module")
def windowed(synth, binfmt):
    fx = json.load(open(WINDOW_GOLDEN))
    cfg = binfmt.Config(**fx["config"])
    T = synth.random_tensors(cfg, fx["weight_seed"], std=fx["weight_std"], gate_scale=fx["gate_scale"])
    flat = np.concatenate([np.asarray(T[n], np.float32).ravel() for n in binfmt.tensor_shapes(cfg)])
    return fx, cfg, flat


def test_precise_engine_reproduces_the_reference_ids_past_the_window(ops, windowed):
    """tests/golden/window_e2e.json holds what the reference's own CPU model generated for a 3-layer
    model with a sliding window of 8 over 79 positions; 248 of the 256 ids change without the
    window, so its mask (`pos - t >= window`) and the even-layer rule (run.cpp:157-164,582-584)
    decide them.  The fp32-faithful engine must reproduce every id."""
    fx, cfg, flat = windowed
    prompts = np.asarray(fx["prompts"], np.int32)
    gold = np.asarray(fx["expected_ids"], np.int32)
    eng = ops.Engine(cfg, flat, max_batch=fx["n_req"], max_seq=fx["max_seq_len"], precise=True)
    out, n = eng.generate(prompts, fx["max_seq_len"])
    eng.close()
    assert n == fx["n_generated"]
    assert (out[:, fx["terminator_index"]] == -1).all()
    assert np.array_equal(out[:, :gold.shape[1]], gold)


def test_engine_past_the_window_matches_the_reference_ids_where_margin_is_clear(ops, orc, windowed):
    """The same fixture through the production (bf16-staged, MFMA) engine, teacher-forced with the
    reference's ids: lock-step steps through a 64-slot ring that holds the window of 8 (masked
    blocks; the ring wraps at position 64), and the prompt pass over the first 70 positions (longer
    than the ring: the linear K/V copy) followed by steps.  The fixture's weights were picked so that
    no router decision of the fp32 or of the bf16-staged CPU model comes closer than 5e-3, so the
    engine follows the same experts throughout and EVERY position is compared: logits within the
    bf16 bound of the staged CPU model, and the reference's id wherever its top-1 margin exceeds
    that bound on the logits (0.06 = 2e-2 of a logit scale of 2-3)."""
    fx, cfg, flat = windowed
    prompts = np.asarray(fx["prompts"], np.int32)
    gold = np.asarray(fx["expected_ids"], np.int32)
    margins = np.asarray(fx["logit_margins"], np.float32)
    n_req, n_prompt = prompts.shape
    seqs = np.concatenate([prompts, gold], axis=1)
    assert fx["min_router_gap_fp32_and_staged_all_positions"] > 5e-3
    clear = margins > 0.06
    assert clear.mean() > 0.8
    last = fx["max_seq_len"] - 1

    def check(pred, what):
        bad = np.argwhere((pred != gold) & clear & (pred >= 0))
        assert len(bad) == 0, (what, [(int(r), int(i), float(margins[r, i])) for r, i in bad])

    # lock step
    eng = ops.Engine(cfg, flat, max_batch=n_req, max_seq=fx["max_seq_len"], keep_logits=True)
    cpu = [orc.Model(cfg, flat, stage=orc.STAGE_GPU) for _ in range(n_req)]
    want = np.zeros((last, n_req, cfg.vocab_size), np.float32)
    pred = np.full_like(gold, -1)
    worst = 0.0
    for pos in range(last):
        nxt = eng.step(seqs[:, pos], pos)
        got = eng.last_logits(n_req)
        for r in range(n_req):
            want[pos, r] = cpu[r].forward(int(seqs[r, pos]), pos)
            worst = max(worst, rel_errors(got[r], want[pos, r])[0])
        if pos >= n_prompt - 1:
            pred[:, pos - (n_prompt - 1)] = nxt
    eng.close()
    assert worst <= 2e-2, worst
    check(pred, "lock step")
    # prompt pass over 70 positions (the window layers' ring has 64 slots), then steps
    T = 70
    eng = ops.Engine(cfg, flat, max_batch=n_req, max_seq=fx["max_seq_len"], keep_logits=True)
    pred = np.full_like(gold, -1)
    pred[:, T - n_prompt] = eng.prefill(seqs[:, :T])
    worst_pf = rel_errors(eng.last_logits(n_req), want[T - 1])[0]
    for pos in range(T, last):
        pred[:, pos - (n_prompt - 1)] = eng.step(seqs[:, pos], pos)
        worst_pf = max(worst_pf, rel_errors(eng.last_logits(n_req), want[pos])[0])
    eng.close()
    assert worst_pf <= 2e-2, worst_pf
    check(pred, "prompt pass")
    print("window fixture: ids compared", int(clear.sum()), "of", clear.size, "; worst max-rel vs the staged CPU model:",
          "lock step", worst, "prompt pass + steps", worst_pf)


@pytest.mark.parametrize("head_dim,n_q,n_kv", [(32, 8, 2), (64, 4, 2)])
def test_prefill_of_1024_positions(ops, orc, tiny, synth, binfmt, head_dim, n_q, n_kv):
    """The reference's longest prompt (1024 positions, getp-csrc/src/alloc.cpp:1047) in one pass:
    the tiled prompt attention walks up to 16 K/V blocks per row group on the full layers and a
    linear copy of the prompt on the window layers (their 128-slot ring has wrapped seven times).
    Against 1024 lock-step steps of the same engine (equal to bf16 rounding: rows of more than 512
    positions are summed in another order) and against the fp32 CPU model."""
    import dataclasses
    fx, cfg0, flat0 = tiny
    if head_dim == cfg0.head_dim:
        cfg, flat = cfg0, flat0
    else:
        cfg = dataclasses.replace(cfg0, head_dim=head_dim, n_attn_heads=n_q, n_kv_heads=n_kv)
        T_ = synth.random_tensors(cfg, 21)
        flat = np.concatenate([np.asarray(T_[n], np.float32).ravel() for n in binfmt.tensor_shapes(cfg)])
    rng = np.random.default_rng(head_dim)
    B, T, S = 4, 1024, 1032
    seqs = rng.integers(0, cfg.vocab_size, size=(B, S)).astype(np.int32)
    a = ops.Engine(cfg, flat, max_batch=B, max_seq=S, keep_logits=True)
    b = ops.Engine(cfg, flat, max_batch=B, max_seq=S, keep_logits=True)
    for pos in range(T):
        a.step(seqs[:, pos], pos)
    b.prefill(seqs[:, :T])
    la, lb = a.last_logits(B).copy(), b.last_logits(B).copy()
    per = np.abs(lb - la).max(axis=1) / np.abs(la).max(axis=1)
    cpu = orc.Model(cfg, flat)
    for pos in range(T):
        want = cpu.forward(int(seqs[0, pos]), pos)
    vs_cpu = rel_errors(lb[0], want)[0], rel_errors(la[0], want)[0]
    print("1024-position prompt pass vs lock step, per row:", per, "; row 0 vs fp32 CPU model (pass, lock step):", vs_cpu)
    assert np.median(per) <= 5e-3 and np.sort(per)[-2] <= 2e-2, per   # at most one row may hit a router near-tie
    assert vs_cpu[0] <= max(2e-2, 1.5 * vs_cpu[1]), vs_cpu
    # and the steps that follow read what the pass left in the caches
    diffs = []
    for pos in range(T, S):
        a.step(seqs[:, pos], pos)
        b.step(seqs[:, pos], pos)
        x, y = a.last_logits(B), b.last_logits(B)
        diffs.append(np.abs(y - x).max(axis=1) / np.abs(x).max(axis=1))
    diffs = np.concatenate(diffs)
    assert np.median(diffs) <= 5e-3, float(np.median(diffs))
    a.close()
    b.close()


def test_step_rows_equals_single_steps(ops, tiny):
    """gptoss_engine_step_rows directly: sequence 0 decodes at position 20, sequence 2 runs positions
    0..11 of a prompt as twelve rows of the same step, slot 1 takes no part.  The sampled ids and the
    logits must be those of the lock-step engine fed the same positions one by one, and bad row lists
    are refused."""
    from conftest import load_pkg
    lib = load_pkg("lib")
    fx, cfg, flat = tiny
    rng = np.random.default_rng(31)
    seq = rng.integers(0, cfg.vocab_size, size=(3, 40)).astype(np.int32)
    a = ops.Engine(cfg, flat, max_batch=3, max_seq=64, keep_logits=True)
    b = ops.Engine(cfg, flat, max_batch=3, max_seq=64, keep_logits=True)
    for pos in range(20):                                    # sequence 0 up to position 19 in both engines
        a.step(seq[:, pos], pos)
        b.step(seq[:, pos], pos)
    # lock-step reference: sequence 0 at position 20; sequence 2 restarted with a new prompt, 12 positions
    prompt = rng.integers(0, cfg.vocab_size, size=12).astype(np.int32)
    a.step_ragged(np.array([seq[0, 20], 0, prompt[0]], np.int32), np.array([20, 0, 0], np.int32))
    want0 = a.last_logits(3)[0].copy()
    for pos in range(1, 12):
        a.step_ragged(np.array([seq[0, 20], 0, prompt[pos]], np.int32), np.array([20, 0, pos], np.int32))
    want2 = a.last_logits(3)[2].copy()
    tokens = np.concatenate([[seq[0, 20]], prompt]).astype(np.int32)
    slots = np.array([0] + [2] * 12, np.int32)
    poss = np.array([20] + list(range(12)), np.int32)
    nxt = b.step_rows(tokens, slots, poss, sample=[0, 12])
    lg = b.last_logits(3)
    assert np.array_equal(lg[0], want0) and np.array_equal(lg[2], want2)
    assert nxt.tolist() == [int(want0.argmax()), int(want2.argmax())]
    with pytest.raises(lib.GptossError):                     # a stretch with a gap
        b.step_rows(np.zeros(2, np.int32), np.array([1, 1], np.int32), np.array([0, 2], np.int32), sample=[1])
    with pytest.raises(lib.GptossError):                     # slot outside the engine
        b.step_rows(np.zeros(1, np.int32), np.array([3], np.int32), np.array([0], np.int32), sample=[0])
    with pytest.raises(lib.GptossError):                     # sampled row outside the list
        b.step_rows(np.zeros(1, np.int32), np.array([0], np.int32), np.array([0], np.int32), sample=[1])
    a.close()
    b.close()
