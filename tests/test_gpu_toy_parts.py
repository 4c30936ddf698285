"""(c)'s generality: a toy mixer with state of its own and a toy architecture that
uses it beside attention layers - one of them with a window, one named twice, one
reading another call's cache - are defined HERE, registered, built from a model
folder with random weights and stepped, without a change to the framework's files.
They are no model of anyone's."""

from __future__ import annotations

import io
from dataclasses import dataclass
from typing import Any, Mapping

import plain_qwen3 as plain
import pytest
import replay_shapes as shapes
import torch
from helpers import random_tokens, read_config, read_weights, tiny_a

pytestmark = pytest.mark.gpu

WINDOW = 6
KINDS = ("attention", "running_mean", "window_attention")
ORDER = ((0, None), (1, None), (2, None), (0, 0), (2, None), (1, None))    # (layer, cache_from)


def define_toy():
    from miniserve_amd import ops
    from miniserve_amd.config import LayerCall, LayerSpec, ModelSpec, PartSpec, Qwen3Config, register_architecture
    from miniserve_amd.parts import Part, StateNeed, StateView, WeightSpec, register_part

    class RunningMean(Part):
        """out_t = W * mean(x_0 .. x_t).  Its state per request: the running sum and
        the count, ``[hidden + 1]`` floats in the request's state slot."""

        def __init__(self, spec, dtype):
            self.hidden = spec.params["hidden_size"]
            self.name = spec.prefix + "proj.weight"
            self.dtype = dtype

        def weight_specs(self):
            return [WeightSpec(self.name, (self.hidden, self.hidden))]

        def load_weights(self, tensors):
            self.weight = tensors[self.name]

        def cache_need(self):
            return StateNeed((self.hidden + 1,), torch.float32)

        def forward(self, x, ctx, cache):
            assert isinstance(cache, StateView)
            means = torch.empty_like(x, dtype=torch.float32)
            for index in range(ctx.num_seqs):
                begin, end = ctx.query_start_host[index], ctx.query_start_host[index + 1]
                slot = ctx.state_slots_host[index]
                state = cache.tensor[slot]
                assert float(state[-1]) == ctx.first_positions_host[index]          # the state is this request's
                sums = state[:-1] + torch.cumsum(x[begin:end].float(), dim=0)
                counts = state[-1] + torch.arange(1, end - begin + 1, device=x.device, dtype=torch.float32)
                means[begin:end] = sums / counts[:, None]
                state[:-1] = sums[-1]
                state[-1] = counts[-1]
            return ops.linear(means.to(self.dtype).contiguous(), self.weight)

    @dataclass(frozen=True)
    class ToyConfig:
        base: Qwen3Config
        architecture = "ToyMixedForCausalLM"

        @classmethod
        def from_dict(cls, data: Mapping[str, Any]):
            inner = dict(data)
            inner["architectures"] = ["Qwen3ForCausalLM"]
            inner["model_type"] = "qwen3"
            return cls(Qwen3Config.from_dict(inner))

        def to_dict(self):
            data = self.base.to_dict()
            data["architectures"] = [self.architecture]
            data["model_type"] = "toy_mixed"
            return data

        def model_spec(self):
            spec = self.base.model_spec()
            layers = []
            for index, kind in enumerate(KINDS):
                layer = spec.layers[index]
                if kind == "running_mean":
                    mixer = PartSpec("test_running_mean", {"hidden_size": spec.hidden_size}, f"model.layers.{index}.mixer.")
                elif kind == "window_attention":
                    mixer = PartSpec("attention", {**layer.mixer.params, "window": WINDOW}, layer.mixer.prefix)
                else:
                    mixer = layer.mixer
                layers.append(LayerSpec(layer.block, mixer, layer.feed_forward, layer.norms))
            return ModelSpec(
                architecture=self.architecture, hidden_size=spec.hidden_size, vocab_size=spec.vocab_size,
                max_positions=spec.max_positions, embedding=spec.embedding, layers=tuple(layers),
                order=tuple(LayerCall(layer, source) for layer, source in ORDER), final_norm=spec.final_norm, head=spec.head,
            )

    register_part("mixer", "test_running_mean", RunningMean)
    register_architecture(ToyConfig.architecture, ToyConfig)
    return ToyConfig


def toy_logits(weights, config, tokens):
    """The toy architecture, plainly: whole sequence, no cache."""

    w = {name: tensor.double() for name, tensor in weights.items()}
    length = len(tokens)
    positions = torch.arange(length)
    eps = config["rms_norm_eps"]
    h = w["model.embed_tokens.weight"][torch.tensor(tokens)]
    kept = {}
    for call, (layer, source) in enumerate(ORDER):
        base = f"model.layers.{layer}."
        x = plain.rms_norm(h, w[base + "input_layernorm.weight"], eps)
        if KINDS[layer] == "running_mean":
            mean = torch.cumsum(x, dim=0) / torch.arange(1, length + 1, dtype=torch.float64)[:, None]
            mixed = mean @ w[base + "mixer.proj.weight"].T
        else:
            window = WINDOW if KINDS[layer] == "window_attention" else None
            mixed, kept[call] = plain.attention_block(
                x, w, base + "self_attn.", config, positions, None if source is None else kept[source], window
            )
        h = h + mixed
        h = h + plain.swiglu(plain.rms_norm(h, w[base + "post_attention_layernorm.weight"], eps), w, base + "mlp.")
    return plain.rms_norm(h, w["model.norm.weight"], eps) @ w["model.embed_tokens.weight"].T


@pytest.fixture(scope="module")
def toy(tmp_path_factory):
    from miniserve_amd.config import load_config
    from miniserve_amd.parts import unregister_part
    from miniserve_amd.weights import write_random_model

    toy_config = define_toy()
    data = tiny_a()
    data["num_hidden_layers"] = 3
    data["architectures"] = [toy_config.architecture]
    folder = write_random_model(toy_config.from_dict(data), tmp_path_factory.mktemp("toy") / "model", seed=8)
    assert type(load_config(folder)).__name__ == "ToyConfig"            # chosen by config.json through the registry
    yield folder
    unregister_part("mixer", "test_running_mean")


def test_the_toy_model_is_built_from_its_folder(toy):
    from miniserve_amd.cache import CacheLayout
    from miniserve_amd.config import load_config
    from miniserve_amd.parts import DecoderModel

    weights = read_weights(toy)
    assert "model.layers.1.mixer.proj.weight" in weights and "model.layers.1.self_attn.q_proj.weight" not in weights
    model = DecoderModel(load_config(toy).model_spec(), "float32")
    layout = CacheLayout.from_needs(model.cache_needs())
    # full attention: one cache (call 0, read again by call 3); window: two caches (calls 2, 4); two states (calls 1, 5)
    assert [(g.need.window, g.calls) for g in layout.groups] == [(None, [0]), (WINDOW, [2, 4])]
    assert len(layout.states) == 2
    assert [p.kind for p in layout.placements] == ["kv", "state", "kv", "kv", "kv", "state"]
    assert layout.placements[3].write is False and layout.placements[3].index == 0


@pytest.mark.parametrize("shape", ["whole", "portions", "mixed"])
def test_the_toy_model_steps_like_its_plain_form(toy, shape, tmp_path):
    from miniserve_amd.config import EngineConfig
    from miniserve_amd.engine import ModelRunner
    from miniserve_amd.engine.replay import replay

    config, weights = read_config(toy), read_weights(toy)
    requests = {f"r{i}": random_tokens(n, config["vocab_size"], 60 + i) for i, n in enumerate((37, 52, 19, 44, 30, 26))}
    steps = getattr(shapes, shape)(requests, **({"seed": 2} if shape == "mixed" else {}))
    pages_full = -(-shapes.max_live_tokens(steps) // 16)
    window_pages = 4 * (-(-(WINDOW + 21) // 16) + 1)
    runner = ModelRunner.from_folder(
        toy, EngineConfig(dtype="float32", kv_block_size=16, num_kv_blocks=max(pages_full, window_pages), max_num_seqs=4,
                          enable_chunked_prefill=True, decode_graphs=False),
    )
    replay(runner, shapes.to_lines(steps), tmp_path, report=io.StringIO())
    got = shapes.collect(steps, tmp_path, config["vocab_size"])
    assert len(got) == sum(len(t) for t in requests.values())
    for rid, tokens in requests.items():
        expected = toy_logits(weights, config, tokens).float()
        for position in range(len(tokens)):
            error = float((got[(rid, position)] - expected[position]).abs().max())
            assert error <= 2e-5, f"{shape}: {rid} position {position}: {error:.3e}"
    assert runner.cache.live_requests() == ()
    runner.cache.assert_invariants()


def test_a_window_group_holds_few_pages_for_a_long_request(toy):
    from miniserve_amd.config import EngineConfig
    from miniserve_amd.engine import ModelRunner, StepEntry

    config = read_config(toy)
    runner = ModelRunner.from_folder(
        toy, EngineConfig(dtype="float32", kv_block_size=4, num_kv_blocks=40, max_num_seqs=2, enable_chunked_prefill=True,
                          decode_graphs=False),
    )
    tokens = random_tokens(120, config["vocab_size"], 1)
    runner.admit("long")
    position = 0
    for size in (9, 3, 1, 1, 20, 1, 1, 1, 30, 2, 1, 50):
        runner.step([StepEntry("long", tuple(tokens[position : position + size]), ())])
        position += size
        free_full, free_window = runner.cache.capacity().free_blocks
        assert free_full == 40 - -(-position // 4)
        assert 40 - free_window <= -(-WINDOW // 4) + 1                  # the window's pages, not the history's
    runner.release("long")
    assert runner.cache.capacity().free_blocks == (40, 40)
