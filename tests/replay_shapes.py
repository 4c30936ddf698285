"""Traces for replay tests: the same requests whole, with the last tokens decoded
one by one, in portions of changing size, and mixed with other requests."""

from __future__ import annotations

import json
import random
from pathlib import Path

import numpy as np
import torch


def whole(requests: dict[str, list[int]]) -> list[dict]:
    """Each request alone and whole: one step holds all its tokens."""

    steps = []
    for name, tokens in requests.items():
        steps.append({"step": len(steps), "entries": [{"id": name, "tokens": tokens, "want": list(range(len(tokens)))}],
                      "end": [name]})
    return steps


def prefill_then_decode(requests: dict[str, list[int]], tail: int = 32) -> list[dict]:
    """Most of a request in one step, the last ``tail`` tokens one by one."""

    steps = []
    for name, tokens in requests.items():
        head = max(len(tokens) - tail, 1)
        steps.append({"step": len(steps), "entries": [{"id": name, "tokens": tokens[:head], "want": list(range(head))}],
                      "end": []})
        for position in range(head, len(tokens)):
            steps.append({"step": len(steps), "entries": [{"id": name, "tokens": [tokens[position]], "want": [0]}],
                          "end": [name] if position == len(tokens) - 1 else []})
        if head == len(tokens):
            steps[-1]["end"] = [name]
    return steps


PORTIONS = (7, 2, 13, 2, 5, 3, 16, 1, 15, 2, 17, 2, 8, 31, 2, 33, 4)


def portions(requests: dict[str, list[int]], sizes=PORTIONS) -> list[dict]:
    """Portions of changing size, down to two tokens (and one), ending on, one
    before and one after page edges of 8 and 16."""

    steps = []
    for name, tokens in requests.items():
        position, index = 0, 0
        while position < len(tokens):
            size = min(sizes[index % len(sizes)], len(tokens) - position)
            part = tokens[position : position + size]
            position += size
            index += 1
            steps.append({"step": len(steps), "entries": [{"id": name, "tokens": part, "want": list(range(size))}],
                          "end": [name] if position == len(tokens) else []})
    return steps


def mixed(requests: dict[str, list[int]], *, seed: int, live_limit: int = 4, tail: int = 12) -> list[dict]:
    """Up to ``live_limit`` live requests; portions of some beside single decoded
    tokens of others in one step; a request may sit a step out; when one ends the
    next begins, so pages are used again."""

    rng = random.Random(seed)
    waiting = list(requests)
    live: dict[str, int] = {}
    steps = []
    while waiting or live:
        while waiting and len(live) < live_limit and (not live or rng.random() < 0.6):
            live[waiting.pop(0)] = 0
        entries, ended = [], []
        for name in list(live):
            tokens, position = requests[name], live[name]
            if len(live) > 1 and rng.random() < 0.2:
                continue                                    # left out of this step, goes on later
            decode_from = max(len(tokens) - tail, 1)
            size = 1 if position >= decode_from else min(rng.choice((2, 3, 5, 8, 9, 16, 21)), decode_from - position)
            part = tokens[position : position + size]
            entries.append({"id": name, "tokens": part, "want": list(range(len(part)))})
            live[name] = position + len(part)
            if live[name] == len(tokens):
                ended.append(name)
                del live[name]
        if entries:
            steps.append({"step": len(steps), "entries": entries, "end": ended})
    return steps


def max_live_tokens(steps: list[dict], block: int = 64) -> int:
    """The most tokens live requests hold at any time, each rounded up to ``block``."""

    held: dict[str, int] = {}
    most = 0
    for step in steps:
        for entry in step["entries"]:
            held[entry["id"]] = held.get(entry["id"], 0) + len(entry["tokens"])
        most = max(most, sum(-(-n // block) * block for n in held.values()))
        for name in step["end"]:
            held.pop(name, None)
    return most


def to_lines(steps: list[dict]) -> list[str]:
    return [json.dumps(step) for step in steps]


def collect(steps: list[dict], out_dir: Path, vocab: int) -> dict[tuple[str, int], torch.Tensor]:
    """Logits by (request, position) from the files a replay wrote."""

    position: dict[str, int] = {}
    result = {}
    for step in steps:
        wanted = [(e["id"], position.get(e["id"], 0) + w) for e in step["entries"] for w in e["want"]]
        for entry in step["entries"]:
            position[entry["id"]] = position.get(entry["id"], 0) + len(entry["tokens"])
        for name in step["end"]:
            position.pop(name, None)
        if not wanted:
            continue
        data = np.fromfile(out_dir / f"{step['step']}.f32", dtype="<f4").reshape(len(wanted), vocab)
        for row, key in enumerate(wanted):
            result[key] = torch.from_numpy(data[row].copy())
    return result
