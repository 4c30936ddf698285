"""What a part may ask of the cache manager and of the step, shown with toy parts
that are defined HERE and registered from outside the package: a mixer whose pages
hold one latent vector a token and nothing else (a plane of its own instead of keys
and values), a mixer that needs pages AND a state row, an embedding that reads the
step's positions, and a table that a mixer has the step builder make on the host -
also in recorded steps.  They are no model of anyone's."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping

import plain_qwen3 as plain
import pytest
import torch
from helpers import random_tokens, read_config, read_weights, tiny_a

pytestmark = pytest.mark.gpu

LATENT = 24
KINDS = ("latent_attention", "latent_memory", "attention")


def define_toy():
    from miniserve_amd import ops
    from miniserve_amd.config import LayerCall, LayerSpec, ModelSpec, PartSpec, Qwen3Config, register_architecture
    from miniserve_amd.parts import (PAGE_TOKENS, KVCacheNeed, KVCacheView, PagePlane, Part, StateNeed, StateView,
                                     WeightSpec, register_part)

    class PositionalEmbedding(Part):
        """``h[t] = E[token[t]] + P[position[t]]``: the second term needs the step's context."""

        def __init__(self, spec, dtype):
            self.vocab, self.hidden, self.positions = spec.params["vocab_size"], spec.params["hidden_size"], spec.params["max_positions"]
            self.prefix = spec.prefix

        def weight_specs(self):
            return [WeightSpec(self.prefix + "weight", (self.vocab, self.hidden)),
                    WeightSpec("model.embed_positions.weight", (self.positions, self.hidden))]

        def load_weights(self, tensors):
            self.weight, self.position_weight = tensors[self.prefix + "weight"], tensors["model.embed_positions.weight"]

        def forward(self, token_ids, ctx):
            return ops.embedding_gather(token_ids, self.weight) + ops.embedding_gather(ctx.positions, self.position_weight)

    class LatentAttention(Part):
        """Every token leaves one latent vector ``c = Wc x`` in its page (the only plane);
        ``out_t = Wo softmax_j(q_t . c_j / sqrt(L)) c_j`` over ``j <= t``.  With
        ``memory`` the mean of all latents so far is added before ``Wo``; its running sum
        and count are a state row, so the mixer needs pages and state at once."""

        step_tables_key = "toy_latent"

        def __init__(self, spec, dtype):
            self.hidden, self.latent, self.memory = spec.params["hidden_size"], spec.params["latent"], spec.params["memory"]
            self.prefix, self.dtype = spec.prefix, dtype

        def weight_specs(self):
            return [WeightSpec(self.prefix + "c.weight", (self.latent, self.hidden)),
                    WeightSpec(self.prefix + "q.weight", (self.latent, self.hidden)),
                    WeightSpec(self.prefix + "o.weight", (self.hidden, self.latent))]

        def load_weights(self, tensors):
            self.w_c, self.w_q, self.w_o = (tensors[self.prefix + name + ".weight"] for name in "cqo")

        def cache_need(self):
            pages = KVCacheNeed(num_kv_heads=1, head_dim=self.latent, planes=(PagePlane("latent", (PAGE_TOKENS, self.latent)),))
            return (pages, StateNeed((self.latent + 1,), torch.float32)) if self.memory else pages

        @staticmethod
        def step_tables(batch):
            """The index of every sequence's last token in the batch: made on the host,
            once for all replays of a recorded step."""

            return {"toy_latent.last": [batch.query_start[index + 1] - 1 for index in range(len(batch.query_lens))]}

        def forward(self, x, ctx, cache):
            pages, state = cache if self.memory else (cache, None)
            assert isinstance(pages, KVCacheView) and pages.key is None and set(pages.planes) == {"latent"}
            pool = pages.planes["latent"]                             # [pages, page tokens, latent]
            assert pool.shape[1:] == (pages.block_size, self.latent)
            group = ctx.groups[pages.group]
            latent = ops.linear(x, self.w_c)
            query = ops.linear(x, self.w_q)
            flat = pool.view(-1, self.latent)
            flat[group.slot_mapping.long()] = latent
            table, size = group.block_table.long(), pages.block_size
            place = torch.arange(table.shape[1] * size, device=x.device)
            slots = table[:, place // size] * size + place % size     # [S, places]
            seq = ctx.seq_of_token.long()
            seen = place[None, :] <= ctx.positions.long()[:, None]    # [N, places]
            kept = torch.where(seen[:, :, None], flat[slots[seq]].float(), 0.0)
            scores = (kept @ query.float()[:, :, None]).squeeze(-1) / self.latent**0.5
            weights = torch.softmax(scores.masked_fill(~seen, float("-inf")), dim=-1)
            mixed = (weights[:, None, :] @ kept).squeeze(1)
            if self.memory:
                assert isinstance(state, StateView)
                starts, rows = ctx.query_start.long(), ctx.state_slots.long()
                running = torch.cumsum(latent.double(), dim=0)
                first = starts[seq]
                before = running[(first - 1).clamp(min=0)] * (first > 0)[:, None]
                held = state.tensor[rows[seq]]
                sums = held[:, :-1] + (running - before).float()
                counts = held[:, -1] + (torch.arange(x.shape[0], device=x.device) - first + 1).float()
                last = ctx.tables["toy_latent.last"].long()          # from the host, also in a recorded step
                state.tensor[rows] = torch.cat([sums[last], counts[last, None]], dim=1)
                mixed = mixed + sums / counts[:, None]
            return ops.linear(mixed.to(self.dtype).contiguous(), self.w_o)

    @dataclass(frozen=True)
    class ToyLatentConfig:
        base: Qwen3Config
        architecture = "ToyLatentForCausalLM"

        @classmethod
        def from_dict(cls, data: Mapping[str, Any]):
            inner = dict(data)
            inner["architectures"] = ["Qwen3ForCausalLM"]
            inner["model_type"] = "qwen3"
            return cls(Qwen3Config.from_dict(inner))

        def to_dict(self):
            data = self.base.to_dict()
            data["architectures"] = [self.architecture]
            data["model_type"] = "toy_latent"
            return data

        def model_spec(self):
            spec = self.base.model_spec()
            layers = []
            for index, kind in enumerate(KINDS):
                layer = spec.layers[index]
                mixer = layer.mixer
                if kind != "attention":
                    mixer = PartSpec("test_latent_attention", {"hidden_size": spec.hidden_size, "latent": LATENT,
                                                               "memory": kind == "latent_memory"}, f"model.layers.{index}.latent.")
                layers.append(LayerSpec(layer.block, mixer, layer.feed_forward, layer.norms))
            embedding = PartSpec("test_positional_embedding", {**spec.embedding.params, "max_positions": spec.max_positions},
                                 spec.embedding.prefix)
            return ModelSpec(
                architecture=self.architecture, hidden_size=spec.hidden_size, vocab_size=spec.vocab_size,
                max_positions=spec.max_positions, embedding=embedding, layers=tuple(layers),
                order=tuple(LayerCall(index) for index in range(len(KINDS))), final_norm=spec.final_norm, head=spec.head,
            )

    register_part("embedding", "test_positional_embedding", PositionalEmbedding)
    register_part("mixer", "test_latent_attention", LatentAttention)
    register_architecture(ToyLatentConfig.architecture, ToyLatentConfig)
    return ToyLatentConfig


def toy_logits(weights, config, tokens):
    """The toy architecture, plainly: whole sequence, no cache."""

    w = {name: tensor.double() for name, tensor in weights.items()}
    length = len(tokens)
    positions = torch.arange(length)
    eps = config["rms_norm_eps"]
    h = w["model.embed_tokens.weight"][torch.tensor(tokens)] + w["model.embed_positions.weight"][positions]
    causal = positions[None, :] <= positions[:, None]
    for layer, kind in enumerate(KINDS):
        base = f"model.layers.{layer}."
        x = plain.rms_norm(h, w[base + "input_layernorm.weight"], eps)
        if kind == "attention":
            mixed, _ = plain.attention_block(x, w, base + "self_attn.", config, positions, None, None)
        else:
            latent, query = x @ w[base + "latent.c.weight"].T, x @ w[base + "latent.q.weight"].T
            scores = (query @ latent.T / LATENT**0.5).masked_fill(~causal, float("-inf"))
            mixed = torch.softmax(scores, dim=-1) @ latent
            if kind == "latent_memory":
                mixed = mixed + torch.cumsum(latent, dim=0) / torch.arange(1, length + 1, dtype=torch.float64)[:, None]
            mixed = mixed @ w[base + "latent.o.weight"].T
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
    data["num_hidden_layers"] = len(KINDS)
    data["architectures"] = [toy_config.architecture]
    folder = write_random_model(toy_config.from_dict(data), tmp_path_factory.mktemp("toy_latent") / "model", seed=21)
    assert type(load_config(folder)).__name__ == "ToyLatentConfig"
    yield folder
    unregister_part("embedding", "test_positional_embedding")
    unregister_part("mixer", "test_latent_attention")


def test_the_cache_is_laid_out_as_the_mixers_say(toy):
    from miniserve_amd.cache import CacheLayout, CacheManager
    from miniserve_amd.config import load_config
    from miniserve_amd.parts import DecoderModel, KVCacheView, StateView

    model = DecoderModel(load_config(toy).model_spec(), "float32")
    layout = CacheLayout.from_needs(model.cache_needs())
    # the two latent mixers share a group (one plane, one vector a token); the attention layer has keys and values
    assert [[plane.name for plane in group.need.page_planes()] for group in layout.groups] == [["latent"], ["key", "value"]]
    assert [group.calls for group in layout.groups] == [[0, 1], [2]]
    assert [placement.kind for placement in layout.placements] == ["kv", "many", "kv"]
    assert [part.kind for part in layout.placements[1].parts] == ["kv", "state"] and len(layout.states) == 1
    config = read_config(toy)
    heads, dim = config["num_key_value_heads"], config["head_dim"]
    assert layout.bytes_per_token(4) == 4 * (2 * LATENT + 2 * heads * dim)
    manager = CacheManager(layout, block_size=8, num_blocks=5, max_num_seqs=3, max_model_len=64)
    manager.allocate_storage(torch.float32, "cuda:0")
    assert manager.pools[0]["latent"].shape == (2, 6, 8, LATENT)
    assert manager.key_pools[0].shape == (1, 6, heads, 8, dim) and len(manager.page_pools()) == 3
    first, second, third = manager.call_views()
    assert isinstance(first, KVCacheView) and first.key is None and first.planes["latent"].shape == (6, 8, LATENT)
    assert isinstance(second, tuple) and isinstance(second[0], KVCacheView) and isinstance(second[1], StateView)
    assert second[1].tensor.shape == (4, LATENT + 1)
    assert third.key is not None and set(third.planes) == {"key", "value"}


@pytest.mark.parametrize("graphs", [False, True])
def test_the_toy_model_steps_like_its_plain_form(toy, graphs):
    """Prompts in portions beside decoded tokens, then single tokens: with ``graphs`` those
    come from recordings (rows of 1, 2 and 4; a spare row fills the step of four up),
    where the mixer's host-made table and both of its caches must be in place."""

    from miniserve_amd.config import EngineConfig
    from miniserve_amd.engine import ModelRunner, StepEntry

    config, weights = read_config(toy), read_weights(toy)
    runner = ModelRunner.from_folder(toy, EngineConfig(dtype="float32", kv_block_size=16, num_kv_blocks=14, max_num_seqs=4,
                                                      enable_chunked_prefill=True, decode_graphs=graphs))
    for pool in runner.cache.page_pools():
        pool.fill_(float("nan"))
    requests = {f"r{i}": random_tokens(n, config["vocab_size"], 40 + i) for i, n in enumerate((45, 70, 50))}
    expected = {rid: toy_logits(weights, config, tokens).float() for rid, tokens in requests.items()}
    position = {rid: 0 for rid in requests}

    def step(sizes):
        entries = []
        for rid, size in sizes.items():
            if not runner.cache.is_live(rid):
                runner.admit(rid)
            entries.append(StepEntry(rid, tuple(requests[rid][position[rid] : position[rid] + size]), tuple(range(size))))
        logits = runner.step(entries).cpu()
        row = 0
        for rid, size in sizes.items():
            for offset in range(size):
                error = float((logits[row] - expected[rid][position[rid] + offset]).abs().max())
                assert error <= 2e-5, f"{rid} at {position[rid] + offset} in a step of {sizes}: {error:.3e}"
                row += 1
            position[rid] += size

    step({"r0": 17})
    step({"r0": 1, "r1": 33})                       # a decoded token beside a portion that crosses a page edge
    step({"r0": 1, "r1": 2, "r2": 16})
    for _ in range(20):
        step({"r0": 1, "r1": 1, "r2": 1})           # recorded: three rows in the step of four
    runner.release("r0")                            # its pages and its state slot go back
    for _ in range(12):
        step({"r1": 1, "r2": 1})
    step({"r2": 1})
    for rid in ("r1", "r2"):
        runner.release(rid)
    assert runner.graph_steps == (33 if graphs else 0)
    assert runner.cache.live_requests() == ()
    runner.cache.assert_invariants()
