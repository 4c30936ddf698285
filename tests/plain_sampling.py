"""Plain sampling from the reference's formulas (miniserve/model/sampling.py:34-79),
with the final draw as the inverse CDF, in token order, of a given uniform number
(the reference draws with ``torch.multinomial``, whose stream no other
implementation can reproduce)."""

from __future__ import annotations

import torch


def filter_top_k(logits: torch.Tensor, top_k: int) -> torch.Tensor:
    """Keep the k largest, the rest to -inf; scatter by index so ties keep exactly k
    (reference: sampling.py:34-43)."""

    if top_k == 0:
        return logits
    values, indices = torch.topk(logits, top_k, dim=-1)
    return torch.full_like(logits, float("-inf")).scatter(-1, indices, values)


def filter_top_p(logits: torch.Tensor, top_p: float) -> torch.Tensor:
    """Sort descending, softmax, remove where the cumulative mass exceeds top_p,
    shifted right by one so the crossing token stays; the first always stays
    (reference: sampling.py:46-58)."""

    if top_p == 1.0:
        return logits
    sorted_logits, sorted_indices = torch.sort(logits, descending=True, dim=-1)
    sorted_probs = torch.softmax(sorted_logits, dim=-1, dtype=torch.float64)
    remove = torch.cumsum(sorted_probs, dim=-1) > top_p
    remove[..., 1:] = remove[..., :-1].clone()
    remove[..., 0] = False
    sorted_logits = sorted_logits.masked_fill(remove, float("-inf"))
    return torch.empty_like(sorted_logits).scatter(-1, sorted_indices, sorted_logits)


def running_sums(logits: torch.Tensor, temperature: float, top_k: int, top_p: float) -> torch.Tensor:
    """The running probability sums (float64, token order) that the draw is made from."""

    filtered = logits.to(torch.float32) / temperature
    filtered = filter_top_p(filter_top_k(filtered, top_k), top_p)
    return torch.cumsum(torch.softmax(filtered.to(torch.float64), dim=-1), dim=-1)


def edge_distance(logits: torch.Tensor, temperature: float, top_k: int, top_p: float, uniform: float) -> float:
    """How close ``uniform`` lies to an edge between two tokens' shares: a draw closer
    than an implementation's rounding of its sums may fall to either neighbour."""

    running = running_sums(logits, temperature, top_k, top_p)
    return float((running / running[-1] - uniform).abs().min())


def sample_row(logits: torch.Tensor, temperature: float, top_k: int, top_p: float, uniform: float) -> int:
    """temperature == 0: argmax.  Else temperature, top-k, top-p, softmax
    (reference: sampling.py:69-79), then the first index whose running
    probability sum exceeds ``uniform``."""

    if temperature == 0:
        return int(torch.argmax(logits))
    filtered = logits.to(torch.float32) / temperature
    filtered = filter_top_k(filtered, top_k)
    filtered = filter_top_p(filtered, top_p)
    probabilities = torch.softmax(filtered.to(torch.float64), dim=-1)
    running = torch.cumsum(probabilities, dim=-1)
    index = int(torch.searchsorted(running, torch.tensor(uniform * float(running[-1]), dtype=torch.float64), right=True))
    kept = torch.nonzero(probabilities > 0).flatten()
    return min(index, int(kept[-1]))
