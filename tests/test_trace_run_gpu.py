"""bin/trace_run as a user drives it: a child process, steps on its standard input one JSON line at a
time (the next only after `done <step>`), logits read back from OUT/<step>.f32 and compared with the
plain implementation."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

from conftest import ROOT, TINY
from helpers import compare, last_one_by_one, make_requests, mixed, plain_logits, portions, whole

pytestmark = pytest.mark.gpu


def replay(folder, dtype, steps, max_tokens, out_dir, vocab):
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
           "--out", out_dir, "--max-tokens", str(max_tokens)]
    proc = subprocess.Popen(cmd, stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True, bufsize=1)
    got, position = {}, {}
    try:
        for s in steps:
            proc.stdin.write(json.dumps(s) + "\n")
            proc.stdin.flush()
            line = proc.stdout.readline().strip()
            assert line == f"done {s['step']}", line
            keys = []
            for e in s["entries"]:
                p0 = position.get(e["id"], 0)
                keys += [(e["id"], p0 + w) for w in e["want"]]
                position[e["id"]] = p0 + len(e["tokens"])
            path = os.path.join(out_dir, f"{s['step']}.f32")
            if keys:
                rows = np.fromfile(path, dtype="<f4").reshape(len(keys), vocab)
                for key, row in zip(keys, rows):
                    got[key] = row.astype(np.float64)
            else:
                assert not os.path.exists(path)
        proc.stdin.close()
        assert proc.wait(timeout=60) == 0
    finally:
        if proc.poll() is None:
            proc.kill()
    return got


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replay_matches_the_plain_implementation(model_folders, plain_models, tmp_path, dtype):
    name = "B"
    vocab = TINY[name]["vocab_size"]
    reqs = make_requests(vocab, [70, 40, 100, 17, 64], seed=21)
    want = plain_logits(plain_models[name], reqs)
    steps, peak = mixed(reqs, seed=6)
    # whole, last 32 one by one, portions, and mixed, as one long trace through one process
    trace = []
    for part in (whole(reqs), last_one_by_one(reqs), portions(reqs), steps):
        base = len(trace)
        trace += [dict(s, step=base + i) for i, s in enumerate(part)]
    got_all = {}
    # replay part by part so that each position is compared once per way of cutting
    at = 0
    for label, part in (("whole", whole(reqs)), ("last32", last_one_by_one(reqs)), ("portions", portions(reqs)),
                        ("mixed", steps)):
        out_dir = str(tmp_path / f"{dtype}-{label}")
        got = replay(model_folders[name], dtype, part, max(peak, 128), out_dir, vocab)
        compare(got, want, dtype)
        got_all[label] = got
    scale = max(float(np.abs(v).max()) for v in want.values())
    limit = 2e-5 if dtype == "float32" else 0.03 * scale        # bfloat16: rounding between kernels for few and many rows
    for label in ("last32", "portions", "mixed"):
        assert max(np.abs(got_all["whole"][k] - got_all[label][k]).max() for k in want) <= limit


def test_steps_without_wanted_logits_and_unfinished_requests(model_folders, plain_models, tmp_path):
    vocab = TINY["A"]["vocab_size"]
    toks = make_requests(vocab, [30], seed=1)["r0"]
    steps = [dict(step=7, entries=[dict(id="x", tokens=toks[:20], want=[])], end=[]),
             dict(step=8, entries=[], end=[]),
             dict(step=9, entries=[dict(id="x", tokens=toks[20:], want=[9])], end=[])]
    got = replay(model_folders["A"], "float32", steps, 64, str(tmp_path / "o"), vocab)
    assert sorted(os.listdir(tmp_path / "o")) == ["9.f32"]
    np.testing.assert_allclose(got[("x", 29)], plain_models["A"].logits(toks, [29])[0], atol=2e-4, rtol=2e-4)


def test_the_input_digest_knows_the_steps_boundaries(model_folders, tmp_path):
    """The digest on standard error is the same for the same steps and differs when the same tokens are cut
    differently (the reference digests its replayed batches with their boundaries,
    tests/cuda_validation_support.h:81-91)."""
    vocab = TINY["A"]["vocab_size"]
    toks = make_requests(vocab, [24], seed=2)["r0"]

    def digest(cuts, label):
        lines, at = [], 0
        for i, n in enumerate(cuts):
            lines.append(json.dumps(dict(step=i, entries=[dict(id="x", tokens=toks[at:at + n], want=[n - 1])], end=[])))
            at += n
        cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model_folders["A"], "--dtype", "float32",
               "--out", str(tmp_path / label), "--max-tokens", "64"]
        done = subprocess.run(cmd, input="\n".join(lines) + "\n", capture_output=True, text=True, timeout=120)
        assert done.returncode == 0, done.stderr
        found = [l.split()[-1] for l in done.stderr.splitlines() if l.startswith("[trace_run] input digest")]
        assert len(found) == 1 and len(found[0]) == 64
        return found[0]
    a, b, c = digest([24], "a"), digest([24], "b"), digest([20, 4], "c")
    assert a == b and a != c
