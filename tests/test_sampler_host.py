"""The sampler's host side on the CPU: what it hands to the device kernel (one number of
each kind per row, the uniform number from the request's own stream), staging and
commit of the streams, and that the tokens are those of the plain implementation when
the kernel is replaced by it."""

from __future__ import annotations

import plain_sampling
import pytest
import torch

from miniserve_amd.engine import SamplingParams
from miniserve_amd.sampling import NonFiniteLogitsError, Sampler


@pytest.fixture
def kernel(monkeypatch):
    """``ops.sample_rows`` replaced by the plain implementation; records its arguments."""

    from miniserve_amd import ops

    calls = []

    def sample_rows(logits, temperature=None, top_p=None, uniform=None, top_k=None, top_p_alone=False):
        calls.append(dict(temperature=temperature, top_p=top_p, uniform=uniform, top_k=top_k, top_p_alone=top_p_alone))
        tokens = []
        for row in range(logits.shape[0]):
            if not bool(torch.isfinite(logits[row]).all()):
                tokens.append(-1)
            elif temperature is None:
                tokens.append(int(torch.argmax(logits[row])))
            else:
                tokens.append(plain_sampling.sample_row(
                    logits[row], float(temperature[row]), int(top_k[row]), float(top_p[row]), float(uniform[row])))
        return torch.tensor(tokens, dtype=torch.int32)

    monkeypatch.setattr(ops, "sample_rows", sample_rows)
    return calls


def rows(count, vocab=40, seed=0):
    return torch.randn(count, vocab, generator=torch.Generator().manual_seed(seed)) * 3


def test_rows_carry_their_own_numbers_and_greedy_rows_none(kernel):
    sampler = Sampler()
    requests = [("g", SamplingParams()), ("a", SamplingParams(temperature=0.8, top_k=5, top_p=0.9, seed=3)),
                ("b", SamplingParams(temperature=1.5, seed=4))]
    logits = rows(3)
    staged = sampler.stage(logits, requests)
    sent = kernel[-1]
    assert sent["temperature"].tolist() == pytest.approx([0.0, 0.8, 1.5]) and sent["top_p"].tolist() == pytest.approx([1.0, 0.9, 1.0])
    assert sent["top_k"].dtype == torch.int32 and sent["top_k"].tolist() == [0, 5, 0]
    assert not sent["top_p_alone"]                                        # a's top-p comes with a top-k
    uniforms = sent["uniform"].tolist()
    assert uniforms[0] == 0.0 and all(0 <= u < 1 for u in uniforms)
    # the uniform number of a row is the first of its request's seeded stream
    for row, seed in ((1, 3), (2, 4)):
        expected = float(torch.rand((), generator=torch.Generator().manual_seed(seed), dtype=torch.float64))
        assert uniforms[row] == pytest.approx(expected, abs=1e-7)
    assert staged[0].token_id == int(torch.argmax(logits[0])) and staged[0].generator_state is None
    for row in (1, 2):
        _, params = requests[row]
        assert staged[row].token_id == plain_sampling.sample_row(
            logits[row], params.temperature, params.top_k, params.top_p, uniforms[row])
    # all greedy: the kernel is asked for the largest alone
    sampler.stage(logits[:1], requests[:1])
    assert kernel[-1]["temperature"] is None
    # top-p without a top-k (or with one that cuts nothing) takes the search over the whole row
    sampler.stage(logits[:1], [("c", SamplingParams(temperature=1.0, top_p=0.5))])
    assert kernel[-1]["top_p_alone"]
    sampler.stage(logits[:1], [("c", SamplingParams(temperature=1.0, top_p=0.5, top_k=40))])
    assert kernel[-1]["top_p_alone"]


def test_a_stream_advances_at_commit_only(kernel):
    sampler = Sampler()
    request = [("r", SamplingParams(temperature=1.0, seed=9))]
    logits = rows(1, seed=5)
    first = sampler.stage(logits, request)
    again = sampler.stage(logits, request)
    assert first[0].token_id == again[0].token_id and sampler.active_request_ids == ()      # staged twice: the same draw
    first_uniform = float(kernel[-1]["uniform"][0])
    sampler.commit(first)
    assert sampler.active_request_ids == ("r",)
    sampler.stage(logits, request)
    second_uniform = float(kernel[-1]["uniform"][0])
    assert second_uniform != first_uniform
    stream = torch.Generator().manual_seed(9)
    expected = [float(torch.rand((), generator=stream, dtype=torch.float64)) for _ in range(2)]
    assert [first_uniform, second_uniform] == pytest.approx(expected, abs=1e-7)            # the request's stream, in order
    # a released request starts its stream again; an unseeded one draws from the system's randomness
    sampler.release("r")
    assert sampler.active_request_ids == ()
    sampler.stage(logits, request)
    assert float(kernel[-1]["uniform"][0]) == pytest.approx(first_uniform, abs=1e-7)
    sampler.stage(logits, [("u", SamplingParams(temperature=1.0))])
    one = float(kernel[-1]["uniform"][0])
    sampler.stage(logits, [("u", SamplingParams(temperature=1.0))])
    assert float(kernel[-1]["uniform"][0]) != one
    # sample() is stage and commit
    tokens = sampler.sample(logits, request)
    assert tokens == [first[0].token_id] and sampler.active_request_ids == ("r",)


def test_what_the_sampler_refuses(kernel):
    sampler = Sampler()
    logits = rows(2)
    with pytest.raises(ValueError, match="need logits"):
        sampler.stage(logits, [("a", SamplingParams())])
    with pytest.raises(ValueError, match="need logits"):
        sampler.stage(logits[0], [("a", SamplingParams())])
    with pytest.raises(TypeError, match="floating-point"):
        sampler.stage(torch.zeros(1, 4, dtype=torch.int64), [("a", SamplingParams())])
    with pytest.raises(ValueError, match="vocabulary"):
        sampler.stage(logits, [("a", SamplingParams()), ("b", SamplingParams(temperature=1.0, top_k=41))])
    bad = logits.clone()
    bad[1, 3] = float("nan")
    with pytest.raises(NonFiniteLogitsError, match="finite"):
        sampler.stage(bad, [("a", SamplingParams()), ("b", SamplingParams())])
    assert sampler.active_request_ids == ()
