"""bin/trace_run as a user runs it: a subprocess that reads steps from a pipe, one at a
time, and writes logits.  The same requests whole, with the last 32 tokens one by one, and
in batches of unequal lengths, in float32 and bfloat16, against the plain implementation."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from helpers import CONFIGS, TOL, max_err, model_folder, plain_logits, tokens_for

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


class Replay:
    def __init__(self, name, dtype, max_tokens, out_dir):
        self.vocab = CONFIGS[name][0]["vocab_size"]
        self.out = str(out_dir)
        self.proc = subprocess.Popen(
            [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model_folder(name), "--dtype", dtype,
             "--out", self.out, "--max-tokens", str(max_tokens)],
            stdin=subprocess.PIPE, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
        self.n = 0

    def step(self, entries, end=()):
        """entries: (id, tokens, want).  Returns float32 [wanted, vocab] or None."""
        rec = {"step": self.n, "entries": [{"id": i, "tokens": t, "want": w} for i, t, w in entries],
               "end": list(end)}
        self.proc.stdin.write(json.dumps(rec) + "\n")
        self.proc.stdin.flush()
        line = self.proc.stdout.readline().strip()
        assert line == f"done {self.n}", (line, self.proc.stderr.read() if self.proc.poll() is not None else "")
        path = os.path.join(self.out, f"{self.n}.f32")
        self.n += 1
        if not any(w for _, _, w in entries):
            assert not os.path.exists(path)
            return None
        return torch.from_numpy(np.fromfile(path, dtype="<f4").reshape(-1, self.vocab))

    def close(self):
        self.proc.stdin.close()
        assert self.proc.wait(timeout=60) == 0, self.proc.stderr.read()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_replay_whole_tail_and_batched(name, dtype, tmp_path):
    lengths = {"A": [5, 17, 70, 33], "B": [1, 9, 40, 77]}[name]
    reqs = {f"r{i}": tokens_for(name, n, 90 + i) for i, n in enumerate(lengths)}
    want = {k: plain_logits(name, tuple(v)) for k, v in reqs.items()}
    pages = sum((n + 63) // 64 for n in lengths)
    rp = Replay(name, dtype, 64 * pages, tmp_path)
    tol = TOL[dtype]
    # whole, each alone
    for k, toks in reqs.items():
        got = rp.step([(k, toks, list(range(len(toks))))], end=[k])
        assert max_err(got, want[k]) < tol, ("whole", k)
    # last 32 tokens one by one; nothing wanted from the head of the longest
    for k, toks in reqs.items():
        head = max(0, len(toks) - 32)
        rows = []
        if head:
            r = rp.step([(k, toks[:head], [] if k == "r2" else list(range(head)))])
            rows.append(r if r is not None else want[k][:head].float())
        for j in range(head, len(toks)):
            rows.append(rp.step([(k, [toks[j]], [0])], end=[k] if j == len(toks) - 1 else []))
        assert max_err(torch.cat(rows), want[k]) < tol, ("tail", k)
    # batches of unequal lengths, twice, so that slots and pages are used again
    for _ in range(2):
        prompt = {k: max(1, len(v) - 4 - 3 * i) for i, (k, v) in enumerate(reqs.items())}
        got = {k: [] for k in reqs}
        first = rp.step([(k, v[:prompt[k]], [prompt[k] - 1]) for k, v in reqs.items()],
                        end=[k for k, v in reqs.items() if prompt[k] == len(v)])
        for i, k in enumerate(reqs):
            got[k].append((prompt[k] - 1, first[i]))
        at = dict(prompt)
        live = [k for k in reqs if at[k] < len(reqs[k])]
        while live:
            ending = [k for k in live if at[k] + 1 == len(reqs[k])]
            r = rp.step([(k, [reqs[k][at[k]]], [0]) for k in live], end=ending)
            for i, k in enumerate(live):
                got[k].append((at[k], r[i]))
                at[k] += 1
            live = [k for k in live if at[k] < len(reqs[k])]
        for k in reqs:
            idx = [p for p, _ in got[k]]
            rows = torch.stack([r for _, r in got[k]])
            assert max_err(rows, want[k][idx]) < tol, ("batched", k)
    rp.close()


@pytest.mark.parametrize("mode", ["whole", "tail", "batched"])
def test_replay_of_whole_requests(mode, tmp_path):
    """`rbitnet replay --requests`: a file of requests, every position's logits per request as .npy
    and an index; the three ways of cutting give the plain implementation's logits.  Five requests in
    groups of two: the last group is smaller, and every group takes the slots the one before freed."""
    name, dtype = "B", "float32"
    lengths = [3, 50, 33, 70, 34]
    reqs = {f"q{i}": tokens_for(name, n, 40 + i) for i, n in enumerate(lengths)}
    trace = tmp_path / "requests.jsonl"
    with open(trace, "w") as f:
        for i, (k, v) in enumerate(reqs.items()):
            rec = {"id": k, "tokens": v}
            if i == 3:
                rec["prefill"] = 11                      # its own cut, used by the batched mode
            f.write(json.dumps(rec) + "\n")
    out = tmp_path / "out"
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "rbitnet"), "replay", "--model", model_folder(name),
                        "--dtype", dtype, "--out", str(out), "--max-tokens", str(64 * 4), "--requests", str(trace),
                        "--mode", mode, "--batch-size", "2"], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    with open(out / "index.json") as f:
        index = json.load(f)
    assert index["mode"] == mode and sorted(index["requests"]) == sorted(reqs)
    for k, toks in reqs.items():
        got = torch.from_numpy(np.load(out / index["requests"][k]))
        assert got.dtype == torch.float32 and got.shape == (len(toks), CONFIGS[name][0]["vocab_size"])
        assert max_err(got, plain_logits(name, tuple(toks))) < TOL[dtype], (mode, k)


def test_replay_reports_errors(tmp_path):
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", str(tmp_path),
                          "--dtype", "float32", "--out", str(tmp_path / "o"), "--max-tokens", "64"],
                         input="", capture_output=True, text=True)
    assert out.returncode == 1 and out.stderr.startswith("error: ")
