"""The reference's own `run` executable (CPU model, getp harness, tokenizer, main, compiled from
/root/reference where it lies) with this repository's hook file in place of its GPU engine, run end
to end on the GPU: `run model.bin -m getp -i in.txt -o out.txt`.  The executable is built on the
machine that has the reference tree (oracle/Makefile target `getp`) and only run here.

Checked: the ids the harness writes to its output file are exactly those of
gptoss_engine_generate on the ids the reference's tokenizer produced, in the harness's own format
(one line per request, generated ids only), and the token count it reports."""
import os
import re
import struct
import subprocess

import json
import numpy as np
import pytest

from conftest import ROOT

pytestmark = pytest.mark.gpu
RUN = os.path.join(ROOT, "oracle", "_ref", "run_getp")
GOLDEN = os.path.join(ROOT, "tests", "golden", "tiny_e2e.json")


def _write_byte_tokenizer(path, vocab_size):
    """A tokenizer file in the reference's format (tokenizer.cpp:49-101: int max_token_length, then
    per token float score, int length, bytes) whose tokens 0..255 are the single bytes and whose
    other tokens never occur in text, so encode() maps a prompt to its byte values."""
    with open(path, "wb") as f:
        f.write(struct.pack("<i", 8))
        for i in range(vocab_size):
            tok = bytes([i]) if i < 256 else b"\xff\xfe" + ("%06d" % i).encode()
            f.write(struct.pack("<fi", 0.0, len(tok)) + tok)


@pytest.mark.parametrize("env", [{}, {"GPTOSS_NO_PREFILL": "1"}])
def test_reference_harness_runs_on_the_hooks(ops, binfmt, synth, tmp_path, env):
    if not os.path.exists(RUN):
        pytest.skip("oracle/_ref/run_getp was not built (needs the reference tree at build time)")
    fx = json.load(open(GOLDEN))
    cfg = binfmt.Config(**fx["config"])
    model = str(tmp_path / "tiny.bin")
    binfmt.write_bin(model, cfg, synth.random_tensors(cfg, fx["weight_seed"]))
    tok = str(tmp_path / "tokenizer.bin")
    _write_byte_tokenizer(tok, cfg.vocab_size)
    prompts = ["The quick brown fox", "x", "1234567 tokens of 89", "MoE routing: top-4 of 8 experts",
               "a", "sliding window = 128; sinks", "Zipf", "decode", "q", "rope theta 150000", "kv"]
    inp, out = str(tmp_path / "in.txt"), str(tmp_path / "out.txt")
    with open(inp, "w") as f:
        f.write("%d\n" % len(prompts) + "\n".join(prompts) + "\n")
    steps = 48
    r = subprocess.run([RUN, model, "-m", "getp", "-i", inp, "-o", out, "-n", str(steps), "-z", tok],
                       capture_output=True, text=True, timeout=100,
                       env=dict(os.environ, GPTOSS_BATCH="4", **env))
    assert r.returncode == 0, (r.stdout[-1500:], r.stderr[-1500:])
    got = [[int(t) for t in line.split()] for line in open(out).read().splitlines()]
    assert len(got) == len(prompts)
    # the same requests through the Python front end of the same library
    flat = np.fromfile(model, dtype="<f4", offset=binfmt.HEADER_BYTES)
    ids = [list(p.encode()) for p in prompts]
    stride = max(len(i) for i in ids)
    arr = np.zeros((len(ids), stride), np.int32)
    for i, t in enumerate(ids):
        arr[i, :len(t)] = t
    eng = ops.Engine(cfg, flat, max_batch=4, max_seq=steps)
    want, n = eng.generate(arr, steps, n_prompt=np.asarray([len(t) for t in ids], np.int32))
    eng.close()
    for i, row in enumerate(want):
        end = int(np.argmax(row < 0))
        assert got[i] == [int(t) for t in row[:end]], i
        assert len(got[i]) == steps - len(ids[i])       # positions left after the prompt, as run.cpp counts
    m = re.search(r"achieved throughput TPS \(tok/s\): ([0-9.]+)", r.stdout)
    assert m and float(m.group(1)) > 0
    elapsed = float(re.search(r"\nelapsed time\(s\): ([0-9.]+)", r.stdout).group(1))
    assert abs(float(m.group(1)) * elapsed - n) <= max(2.0, 0.02 * n)   # tokens = TPS x seconds
