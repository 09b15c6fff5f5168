"""How whole requests are cut into steps by `replay_requests`, with an engine that only records:
which tokens each step brings, that a request's logits come back in order, and that every slot
is freed exactly once and used again by the next group."""
import json

import numpy as np
import pytest
import torch

from rbitnet_amd.errors import RbitnetError
from rbitnet_amd.replay import replay_requests

VOCAB = 5


class RecordingEngine:
    """The logits of a token are its id and its position in the request, so that a misplaced row shows."""

    def __init__(self):
        self.free = [2, 1, 0]
        self.length = {}
        self.steps = []
        self.freed = []

    def alloc_slot(self):
        s = self.free.pop()
        self.length[s] = 0
        return s

    def free_slot(self, s):
        assert s in self.length, "freed twice"
        del self.length[s]
        self.freed.append(s)
        self.free.append(s)

    def step(self, entries, want):
        self.steps.append([(s, list(t)) for s, t in entries])
        rows = []
        for s, toks in entries:
            mine = []
            for t in toks:
                mine.append([float(t), float(self.length[s])] + [0.0] * (VOCAB - 2))
                self.length[s] += 1
            rows += mine if want == "all" else mine[-1:]
        return torch.tensor(rows)


REQS = [{"id": "a", "tokens": list(range(10, 50))}, {"id": "b", "tokens": [7]},
        {"id": "c", "tokens": list(range(100, 135)), "prefill": 30}, {"id": "d", "tokens": [1, 2, 3]}]


@pytest.mark.parametrize("mode", ["whole", "tail", "batched"])
def test_every_position_once_and_in_order(mode, tmp_path):
    eng = RecordingEngine()
    index = replay_requests(eng, REQS, mode, str(tmp_path), batch_size=3)
    assert sorted(index) == ["a", "b", "c", "d"]
    for r in REQS:
        got = np.load(tmp_path / index[r["id"]])
        assert got.dtype == np.float32 and got.shape == (len(r["tokens"]), VOCAB)
        assert got[:, 0].tolist() == [float(t) for t in r["tokens"]]
        assert got[:, 1].tolist() == [float(i) for i in range(len(r["tokens"]))]
    assert len(eng.freed) == 4 and not eng.length
    with open(tmp_path / "index.json") as f:
        assert json.load(f) == {"mode": mode, "requests": index}


def test_cuts():
    import tempfile
    with tempfile.TemporaryDirectory() as d:
        eng = RecordingEngine()
        replay_requests(eng, REQS, "whole", d)
        assert [len(s) for s in eng.steps] == [1, 1, 1, 1] and [len(s[0][1]) for s in eng.steps] == [40, 1, 35, 3]
        eng = RecordingEngine()
        replay_requests(eng, REQS[:1], "tail", d)
        assert [len(s[0][1]) for s in eng.steps] == [8] + [1] * 32
        eng = RecordingEngine()
        replay_requests(eng, REQS, "batched", d, batch_size=3)
        first = eng.steps[0]
        assert [len(t) for _, t in first] == [8, 1, 30]              # all but 32; the only token; its own count
        assert [len(s) for s in eng.steps[1:6]] == [2] * 5           # b has left, then c after five more
        assert [len(s) for s in eng.steps[6:33]] == [1] * 27
        last_group = eng.steps[33:]
        assert [len(t) for _, t in last_group[0]] == [1] and len(last_group) == 3
        assert last_group[0][0][0] in (0, 1, 2)                      # a slot that the first group gave back


def test_refusals(tmp_path):
    with pytest.raises(RbitnetError, match="mode"):
        replay_requests(RecordingEngine(), REQS, "sideways", str(tmp_path))
    with pytest.raises(RbitnetError, match="no tokens"):
        replay_requests(RecordingEngine(), [{"id": "x", "tokens": []}], "whole", str(tmp_path))
