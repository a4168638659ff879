"""The trace replay's handling of its input and output, with a stand-in for the model runner (no GPU needed): which
tokens reach the step function at which positions, where logits are written, when requests are given back."""
import io
import json
import os

import numpy as np
import torch

from atoma_infer_amd.engine import replay as replay_mod


class FakeRunner:
    """Keeps the books a runner keeps and returns logits that name (request, position): row = [id, position, want]."""

    def __init__(self):
        self.live, self.log = {}, []

    def add_request(self, rid):
        assert rid not in self.live
        self.live[rid] = 0
        self.log.append(("add", rid))

    def computed_len(self, rid):
        return self.live[rid]

    def free_request(self, rid):
        del self.live[rid]
        self.log.append(("free", rid))

    def step(self, entries):
        rows = []
        for e in entries:
            assert e.start == self.live[e.request]
            for w in e.want:
                rows.append([float(e.request), float(e.start + w), float(e.tokens[w])])
            self.live[e.request] += len(e.tokens)
        self.log.append(("step", [(e.request, list(e.tokens), e.start, list(e.want)) for e in entries]))
        return torch.tensor(rows, dtype=torch.float32) if rows else None


def run(lines, tmp_path, monkeypatch):
    monkeypatch.setattr(torch.cuda, "synchronize", lambda *a, **k: None)
    runner, report = FakeRunner(), io.StringIO()
    rc = replay_mod.replay(runner, io.StringIO("\n".join(json.dumps(x) for x in lines) + "\n"), str(tmp_path), report)
    return rc, runner, report.getvalue().split()


def test_steps_files_and_requests(tmp_path, monkeypatch):
    lines = [
        {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []},
        {"step": 1, "entries": [{"id": "b", "tokens": [9, 9], "want": []}], "end": []},           # nothing wanted: no file
        {"step": 2, "entries": [{"id": "a", "tokens": [4], "want": [0]}, {"id": "b", "tokens": [1, 2, 3], "want": [2, 0]}],
         "end": ["a"]},
        {"step": 7, "entries": [{"id": "a", "tokens": [8, 8], "want": [1]}], "end": ["a", "b", "never-seen"]},
    ]
    rc, runner, said = run(lines, tmp_path, monkeypatch)
    assert rc == 0 and said == ["done", "0", "done", "1", "done", "2", "done", "7"]
    assert sorted(os.listdir(tmp_path)) == ["0.f32", "2.f32", "7.f32"]
    read = lambda n: np.fromfile(os.path.join(tmp_path, n), dtype="<f4").reshape(-1, 3).tolist()
    assert read("0.f32") == [[0, 0, 5], [0, 2, 3]]
    # the order of the entries and, inside an entry, of `want` as given
    assert read("2.f32") == [[0, 3, 4], [1, 4, 3], [1, 2, 1]]
    # "a" ended after step 2: the name now stands for a new request, which starts at position 0
    assert read("7.f32") == [[2, 1, 8]]
    assert runner.live == {}
    assert [x for x in runner.log if x[0] != "step"] == [("add", 0), ("add", 1), ("free", 0), ("add", 2), ("free", 2),
                                                         ("free", 1)]


def test_blank_lines_and_steps_without_entries(tmp_path, monkeypatch):
    monkeypatch.setattr(torch.cuda, "synchronize", lambda *a, **k: None)
    runner, report = FakeRunner(), io.StringIO()
    text = '\n{"step": 3, "entries": [], "end": []}\n\n{"step": 4, "entries": [{"id": 1, "tokens": [2], "want": [0]}], "end": [1]}\n'
    assert replay_mod.replay(runner, io.StringIO(text), str(tmp_path), report) == 0
    assert report.getvalue().split() == ["done", "3", "done", "4"] and os.listdir(tmp_path) == ["4.f32"]
