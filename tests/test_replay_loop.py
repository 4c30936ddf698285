"""The replay loop itself (what ``bin/trace_run`` runs after loading the model), on the
CPU with the stand-in runner: which files it writes, in which order the rows lie, when
requests are admitted and given back, what it prints."""

from __future__ import annotations

import io
import json

import numpy as np
from fake_runner import FakeRunner, next_token

from miniserve_amd.config import EngineConfig
from miniserve_amd.engine.replay import replay

VOCAB = 97


def make_runner(blocks=16):
    return FakeRunner(EngineConfig(dtype="float32", kv_block_size=4, num_kv_blocks=blocks, max_num_seqs=4, max_model_len=128),
                      vocab_size=VOCAB)


def line(step, entries, end=()):
    return json.dumps({"step": step, "entries": [{"id": i, "tokens": t, "want": w} for i, t, w in entries], "end": list(end)})


def test_replay_writes_the_wanted_rows_in_order_and_gives_pages_back(tmp_path):
    a, b = [5, 17, 3, 9, 9, 2], [40, 41, 42]
    lines = [
        line(0, [("a", a[:3], [0, 2])]),                                    # a portion of a prompt, two places wanted
        "",                                                                 # blank lines are skipped
        line(1, [("b", b, []), ("a", a[3:5], [1])]),                        # b whole with nothing wanted, beside a's next portion
        line(2, [("a", a[5:], [0])], end=["b"]),                            # b is left out and ends; a goes on with one token
        line(7, [], end=["a"]),                                             # a step that only ends a request
        line(8, [("b", b[:2], [1])], end=["b", "never_seen"]),              # the name again: a new request; unknown names are ignored
    ]
    runner = make_runner()
    report = io.StringIO()
    assert replay(runner, lines, tmp_path / "out", report=report) == 5
    assert report.getvalue().split() == ["done", "0", "done", "1", "done", "2", "done", "7", "done", "8"]
    assert sorted(p.name for p in (tmp_path / "out").iterdir()) == ["0.f32", "1.f32", "2.f32", "8.f32"]   # step 7 wanted nothing

    def rows(step):
        raw = (tmp_path / "out" / f"{step}.f32").read_bytes()
        return np.frombuffer(raw, dtype="<f4").reshape(-1, VOCAB)

    # the stand-in's logits are 1 at the token that the request's tokens so far determine
    assert [int(r.argmax()) for r in rows(0)] == [next_token(tuple(a[:1]), VOCAB), next_token(tuple(a[:3]), VOCAB)]
    assert [int(r.argmax()) for r in rows(1)] == [next_token(tuple(a[:5]), VOCAB)]
    assert [int(r.argmax()) for r in rows(2)] == [next_token(tuple(a), VOCAB)]
    assert [int(r.argmax()) for r in rows(8)] == [next_token(tuple(b[:2]), VOCAB)]          # from its own beginning
    # the steps ran exactly the tokens they brought, from where each request stood
    assert runner.steps == [[("a", 0, 3)], [("b", 0, 3), ("a", 3, 5)], [("a", 5, 6)], [("b", 0, 2)]]
    assert runner.cache.live_requests() == () and runner.cache.capacity().free_blocks == (16,)
    runner.cache.assert_invariants()


def test_replay_reuses_pages_of_requests_that_ended(tmp_path):
    """A pool for 16 tokens serves a chain of requests of 12: each must end before the next fits."""

    runner = make_runner(blocks=4)
    lines = []
    for index in range(5):
        tokens = [(7 * index + j) % VOCAB for j in range(12)]
        lines.append(line(2 * index, [(f"r{index}", tokens[:10], [9])]))
        lines.append(line(2 * index + 1, [(f"r{index}", tokens[10:], [0, 1])], end=[f"r{index}"]))
    assert replay(runner, lines, tmp_path / "out", report=io.StringIO()) == 10
    assert len(list((tmp_path / "out").iterdir())) == 10
    assert runner.cache.capacity().free_blocks == (4,)
