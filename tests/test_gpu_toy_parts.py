"""(c)'s generality: a toy mixer with state of its own, a toy feed-forward with
routing, a toy position encoding, a toy norm, a toy arrangement of a layer's parts and
a toy architecture that uses them beside attention layers - one of them with a window,
one named twice, one reading another call's cache - are defined HERE, registered, built
from a model folder with random weights and stepped, without a change to the
framework's files.  They are no model of anyone's."""

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
WINDOW_PAGE = 32        # the window layers keep pages of their own size (the engine's are 16 or 4 below)
EXPERTS, EXPERT_WIDTH = 3, 40
# the mixers; layer 1 also has the routed feed-forward, layer 2 the rotation of neighbouring pairs, layer 3 its
# norms after the sums (the first of them a norm that subtracts the mean)
KINDS = ("attention", "running_mean", "window_attention", "post_norm_attention")
ORDER = ((0, None), (1, None), (2, None), (0, 0), (3, None), (2, None), (1, None))    # (layer, cache_from)


def define_toy():
    from miniserve_amd import ops
    from miniserve_amd.config import LayerCall, LayerSpec, ModelSpec, PartSpec, Qwen3Config, register_architecture
    from miniserve_amd.parts import Part, StateNeed, StateView, WeightSpec, build_part, register_part

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
            """Everything on the device, from the context's device tensors alone: a
            recorded step gives no per-request numbers on the host."""

            assert isinstance(cache, StateView)
            state = cache.tensor
            seq, starts, slots = ctx.seq_of_token.long(), ctx.query_start.long(), ctx.state_slots.long()
            running = torch.cumsum(x.double(), dim=0)
            first = starts[seq]                                   # index of the first token of each token's sequence
            before = running[(first - 1).clamp(min=0)] * (first > 0)[:, None]
            kept = state[slots[seq]]
            sums = kept[:, :-1] + (running - before).float()
            place = torch.arange(x.shape[0], device=x.device)
            counts = kept[:, -1] + (place - first + 1).float()
            last = starts[1:] - 1
            state[slots] = torch.cat([sums[last], counts[last, None]], dim=1)
            return ops.linear((sums / counts[:, None]).to(self.dtype).contiguous(), self.weight)

    class RoutedExperts(Part):
        """A feed-forward with routing: router logits in 32-bit, the best of EXPERTS
        experts per token, ``y = p_best * down_best(relu(up_best(x)))`` with p the softmax
        of the router logits.  A toy: every expert runs on every row and the rows pick."""

        def __init__(self, spec, dtype):
            self.hidden, self.width, self.count = spec.params["hidden_size"], spec.params["width"], spec.params["experts"]
            self.prefix, self.dtype = spec.prefix, dtype

        def weight_specs(self):
            decisive = lambda shape, generator, device: torch.randn(shape, generator=generator, dtype=torch.float32, device=device)
            specs = [WeightSpec(self.prefix + "router.weight", (self.count, self.hidden), init=decisive, keep="float32")]
            for expert in range(self.count):
                specs.append(WeightSpec(f"{self.prefix}experts.{expert}.up.weight", (self.width, self.hidden)))
                specs.append(WeightSpec(f"{self.prefix}experts.{expert}.down.weight", (self.hidden, self.width)))
            return specs

        def load_weights(self, tensors):
            self.router = tensors[self.prefix + "router.weight"]
            assert self.router.dtype == torch.float32                      # kept in 32-bit whatever the engine's dtype
            self.up = [tensors[f"{self.prefix}experts.{e}.up.weight"] for e in range(self.count)]
            self.down = [tensors[f"{self.prefix}experts.{e}.down.weight"] for e in range(self.count)]

        def forward(self, x, ctx=None):
            logits = ops.linear(x.float().contiguous(), self.router)      # [N, experts], true 32-bit
            weight, chosen = torch.softmax(logits, dim=-1).max(dim=-1)
            out = torch.zeros((x.shape[0], self.hidden), dtype=torch.float32, device=x.device)
            for expert in range(self.count):
                hidden = torch.relu(ops.linear(x, self.up[expert]))
                out += (chosen == expert)[:, None] * ops.linear(hidden.contiguous(), self.down[expert]).float()
            return (weight[:, None] * out).to(self.dtype)

    class RotaryPairs(Part):
        """Another position encoding: neighbouring pairs (2i, 2i + 1) are rotated by
        ``position * theta^(-2i/dim)``."""

        def __init__(self, spec, dtype):
            self.dim, self.theta = spec.params["dim"], spec.params["theta"]

        def apply(self, x, positions):
            inv = 1.0 / (self.theta ** (torch.arange(0, self.dim, 2, device=x.device, dtype=torch.float32) / self.dim))
            angle = positions.float()[:, None] * inv
            cos, sin = angle.cos()[:, None, :], angle.sin()[:, None, :]
            even, odd = x[..., 0::2].float(), x[..., 1::2].float()
            return torch.stack([even * cos - odd * sin, odd * cos + even * sin], dim=-1).reshape(x.shape).to(x.dtype)

    class CenterNorm(Part):
        """Another norm: ``y = w * (x - mean(x)) * rsqrt(var(x) + eps)``, statistics in 32-bit."""

        def __init__(self, spec, dtype):
            self.dim, self.eps, self.dtype = spec.params["dim"], spec.params["eps"], dtype
            self.name = spec.prefix + "weight"

        def weight_specs(self):
            return [WeightSpec(self.name, (self.dim,), init="norm")]

        def load_weights(self, tensors):
            self.weight = tensors[self.name]

        def forward(self, x):
            centred = x.float() - x.float().mean(dim=-1, keepdim=True)
            scaled = centred * torch.rsqrt(centred.pow(2).mean(dim=-1, keepdim=True) + self.eps)
            return (scaled * self.weight.float()).to(self.dtype)

        def add_forward(self, residual, delta, *, rows=None, write_back=True):
            total = residual if delta is None else residual + delta.float()
            if delta is not None and write_back and rows is None:
                residual.copy_(total)
            return self.forward(total if rows is None else total[rows.long()])

    class PostNormBlock(Part):
        """Another arrangement: ``h <- norm(h + mixer(h)); h <- norm(h + feed_forward(h))``.
        The stream it hands on is the second norm's output; nothing is left to be added."""

        def __init__(self, layer, dtype):
            self.mixer = build_part("mixer", layer.mixer, dtype)
            self.post_mixer = build_part("norm", layer.norms["post_mixer"], dtype)
            self.feed_forward = build_part("feed_forward", layer.feed_forward, dtype)
            self.post_feed_forward = build_part("norm", layer.norms["post_feed_forward"], dtype)
            self.dtype = dtype

        def sub_parts(self):
            return [self.mixer, self.post_mixer, self.feed_forward, self.post_feed_forward]

        def forward(self, residual, delta, ctx, cache):
            if delta is not None:
                ops.residual_add(residual, delta)
            mixed = self.mixer.forward(residual.to(self.dtype), ctx, cache)
            stream = self.post_mixer.add_forward(residual, mixed)
            out = self.feed_forward.forward(stream, ctx)
            stream = self.post_feed_forward.add_forward(stream.float(), out)
            return stream.float(), None

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
                    position = PartSpec("test_rotary_pairs", dict(layer.mixer.params["position"].params))
                    mixer = PartSpec("attention", {**layer.mixer.params, "window": WINDOW, "position": position,
                                                   "block_size": WINDOW_PAGE}, layer.mixer.prefix)
                else:
                    mixer = layer.mixer
                feed_forward = layer.feed_forward
                if kind == "running_mean":
                    feed_forward = PartSpec("test_routed_experts", {"hidden_size": spec.hidden_size, "width": EXPERT_WIDTH,
                                                                    "experts": EXPERTS}, f"model.layers.{index}.moe.")
                block, norms = layer.block, layer.norms
                if kind == "post_norm_attention":
                    first = layer.norms["pre_mixer"]
                    block = "test_post_norm"
                    norms = {"post_mixer": PartSpec("test_center_norm", dict(first.params), first.prefix),
                             "post_feed_forward": layer.norms["pre_feed_forward"]}
                layers.append(LayerSpec(block, mixer, feed_forward, norms))
            return ModelSpec(
                architecture=self.architecture, hidden_size=spec.hidden_size, vocab_size=spec.vocab_size,
                max_positions=spec.max_positions, embedding=spec.embedding, layers=tuple(layers),
                order=tuple(LayerCall(layer, source) for layer, source in ORDER), final_norm=spec.final_norm, head=spec.head,
            )

    register_part("mixer", "test_running_mean", RunningMean)
    register_part("feed_forward", "test_routed_experts", RoutedExperts)
    register_part("position", "test_rotary_pairs", RotaryPairs)
    register_part("norm", "test_center_norm", CenterNorm)
    register_part("block", "test_post_norm", PostNormBlock)
    register_architecture(ToyConfig.architecture, ToyConfig)
    return ToyConfig


def pairs_attention(x, w, prefix, config, positions, window):
    """Attention with the rotation of neighbouring pairs, from the plain parts."""

    length, dim, eps = x.shape[0], config["head_dim"], config["rms_norm_eps"]
    inv = 1.0 / (config["rope_theta"] ** (torch.arange(0, dim, 2, dtype=torch.float32) / dim))
    angle = (positions.float()[:, None] * inv).double()

    def rotate(t):          # [T, heads, dim]
        even, odd = t[..., 0::2], t[..., 1::2]
        cos, sin = angle.cos()[:, None, :], angle.sin()[:, None, :]
        return torch.stack([even * cos - odd * sin, odd * cos + even * sin], dim=-1).reshape(t.shape)

    q = (x @ w[prefix + "q_proj.weight"].T).view(length, -1, dim)
    k = (x @ w[prefix + "k_proj.weight"].T).view(length, -1, dim)
    v = (x @ w[prefix + "v_proj.weight"].T).view(length, -1, dim)
    q = rotate(plain.rms_norm(q, w[prefix + "q_norm.weight"], eps)).transpose(0, 1)
    k = rotate(plain.rms_norm(k, w[prefix + "k_norm.weight"], eps)).transpose(0, 1)
    attended = plain.causal_attention(q, k, v.transpose(0, 1), dim**-0.5, window)
    return attended.transpose(0, 1).reshape(length, -1) @ w[prefix + "o_proj.weight"].T


def routed_experts(x, w, prefix):
    logits = (x.float() @ w[prefix + "router.weight"].float().T).double()      # the router's logits are 32-bit sums
    weight, chosen = torch.softmax(logits, dim=-1).max(dim=-1)
    out = torch.zeros_like(x)
    for expert in range(EXPERTS):
        y = torch.relu(x @ w[f"{prefix}experts.{expert}.up.weight"].T) @ w[f"{prefix}experts.{expert}.down.weight"].T
        out = out + (chosen == expert)[:, None] * y
    return weight[:, None] * out


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
        if KINDS[layer] == "post_norm_attention":
            mixed, kept[call] = plain.attention_block(h, w, base + "self_attn.", config, positions, None, None)
            centred = (h + mixed) - (h + mixed).mean(dim=-1, keepdim=True)
            h = w[base + "input_layernorm.weight"] * centred * torch.rsqrt(centred.pow(2).mean(dim=-1, keepdim=True) + eps)
            h = plain.rms_norm(h + plain.swiglu(h, w, base + "mlp."), w[base + "post_attention_layernorm.weight"], eps)
            continue
        x = plain.rms_norm(h, w[base + "input_layernorm.weight"], eps)
        if KINDS[layer] == "running_mean":
            mean = torch.cumsum(x, dim=0) / torch.arange(1, length + 1, dtype=torch.float64)[:, None]
            mixed = mean @ w[base + "mixer.proj.weight"].T
        elif KINDS[layer] == "window_attention":
            mixed = pairs_attention(x, w, base + "self_attn.", config, positions, WINDOW)
        else:
            mixed, kept[call] = plain.attention_block(
                x, w, base + "self_attn.", config, positions, None if source is None else kept[source], None
            )
        h = h + mixed
        x = plain.rms_norm(h, w[base + "post_attention_layernorm.weight"], eps)
        h = h + (routed_experts(x, w, base + "moe.") if KINDS[layer] == "running_mean" else plain.swiglu(x, w, base + "mlp."))
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
    folder = write_random_model(toy_config.from_dict(data), tmp_path_factory.mktemp("toy") / "model", seed=8)
    assert type(load_config(folder)).__name__ == "ToyConfig"            # chosen by config.json through the registry
    yield folder
    unregister_part("mixer", "test_running_mean")
    unregister_part("feed_forward", "test_routed_experts")
    unregister_part("position", "test_rotary_pairs")
    unregister_part("norm", "test_center_norm")
    unregister_part("block", "test_post_norm")


def test_the_toy_model_is_built_from_its_folder(toy):
    from miniserve_amd.cache import CacheLayout
    from miniserve_amd.config import load_config
    from miniserve_amd.parts import DecoderModel

    weights = read_weights(toy)
    assert "model.layers.1.mixer.proj.weight" in weights and "model.layers.1.self_attn.q_proj.weight" not in weights
    assert "model.layers.1.moe.router.weight" in weights and "model.layers.1.mlp.gate_proj.weight" not in weights
    assert float(weights["model.layers.1.moe.router.weight"].std()) > 0.5         # drawn by the part's own rule
    model = DecoderModel(load_config(toy).model_spec(), "float32")
    layout = CacheLayout.from_needs(model.cache_needs())
    # full attention: two caches (call 0, read again by call 3, and call 4); window: two caches (calls 2, 5); two
    # states (calls 1, 6)
    assert [(g.need.window, g.need.block_size, g.calls) for g in layout.groups] == [(None, None, [0, 4]), (WINDOW, WINDOW_PAGE, [2, 5])]
    assert len(layout.states) == 2
    assert [p.kind for p in layout.placements] == ["kv", "state", "kv", "kv", "kv", "kv", "state"]
    assert layout.placements[3].write is False and layout.placements[3].index == 0
    assert type(model.layers[3]).__name__ == "PostNormBlock" and type(model.layers[3].post_mixer).__name__ == "CenterNorm"


@pytest.mark.parametrize("shape", ["whole", "portions", "mixed"])
def test_the_toy_model_steps_like_its_plain_form(toy, shape, tmp_path):
    from miniserve_amd.config import EngineConfig
    from miniserve_amd.engine import ModelRunner
    from miniserve_amd.engine.replay import replay

    config, weights = read_config(toy), read_weights(toy)
    requests = {f"r{i}": random_tokens(n, config["vocab_size"], 60 + i) for i, n in enumerate((37, 52, 19, 44, 30, 26))}
    steps = getattr(shapes, shape)(requests, **({"seed": 2} if shape == "mixed" else {}))
    pages_full = -(-shapes.max_live_tokens(steps) // 16)
    window_pages = 4 * 2 * (WINDOW_PAGE // 16)         # four live requests, two of the window layers' own pages each
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
    window_pool = 40 * 4 // WINDOW_PAGE            # as many tokens as the engine's 40 pages of 4, in pages of its own size
    assert runner.cache.num_blocks == (40, window_pool) and runner.cache.block_sizes == (4, WINDOW_PAGE)
    tokens = random_tokens(120, config["vocab_size"], 1)
    runner.admit("long")
    position = 0
    for size in (9, 3, 1, 1, 20, 1, 1, 1, 30, 2, 1, 50):
        runner.step([StepEntry("long", tuple(tokens[position : position + size]), ())])
        position += size
        free_full, free_window = runner.cache.capacity().free_blocks
        assert free_full == 40 - -(-position // 4)
        assert window_pool - free_window <= -(-WINDOW // WINDOW_PAGE) + 1        # the window's pages, not the history's
    runner.release("long")
    assert runner.cache.capacity().free_blocks == (40, window_pool)


# ---- state inside recorded steps, aborted steps and preemption ------------------------------------


def toy_runner(toy, *, graphs, pages=24, seqs=4, block=16):
    from miniserve_amd.config import EngineConfig
    from miniserve_amd.engine import ModelRunner

    return ModelRunner.from_folder(
        toy, EngineConfig(dtype="float32", kv_block_size=block, num_kv_blocks=pages, max_num_seqs=seqs,
                          enable_chunked_prefill=True, decode_graphs=graphs),
    )


def test_state_in_recorded_steps(toy):
    """Single-token steps go through recorded graphs: the first step of each recorded
    size runs eagerly and is then replayed, rows that fill a recording up use the spare
    state slot.  Every step's logits equal the plain form's, so no state is updated
    twice and none is mixed up."""

    from miniserve_amd.engine import StepEntry

    config, weights = read_config(toy), read_weights(toy)
    requests = {f"r{i}": random_tokens(n, config["vocab_size"], 90 + i) for i, n in enumerate((21, 33, 27))}
    expected = {rid: toy_logits(weights, config, tokens).float() for rid, tokens in requests.items()}
    runner = toy_runner(toy, graphs=True)
    heads = {"r0": 9, "r1": 14, "r2": 5}
    for rid, tokens in requests.items():
        runner.admit(rid)
        logits = runner.step([StepEntry(rid, tuple(tokens[: heads[rid]]), (heads[rid] - 1,))])
        assert float((logits[0].cpu() - expected[rid][heads[rid] - 1]).abs().max()) <= 2e-5
    position = dict(heads)
    live = list(requests)
    steps = 0
    while live:
        entries = [StepEntry(rid, (requests[rid][position[rid]],), (0,)) for rid in live]
        logits = runner.step(entries).cpu()
        for row, rid in enumerate(live):
            error = float((logits[row] - expected[rid][position[rid]]).abs().max())
            assert error <= 2e-5, f"step {steps}, {rid} at {position[rid]}: {error:.3e}"
            position[rid] += 1
        for rid in [rid for rid in live if position[rid] == len(requests[rid])]:
            runner.release(rid)
            live.remove(rid)
        steps += 1
    assert runner.graph_steps == steps and sorted(runner._decode_graphs) == [(1, 256), (2, 256), (4, 256)]      # three, two, one request


def test_an_aborted_step_puts_the_state_back(toy):
    """A step that fails after its mixers have written their state leaves no trace:
    the same step, run again, gives the plain form's logits."""

    from miniserve_amd.engine import StepEntry

    config, weights = read_config(toy), read_weights(toy)
    tokens = random_tokens(40, config["vocab_size"], 17)
    expected = toy_logits(weights, config, tokens).float()
    for graphs in (False, True):
        runner = toy_runner(toy, graphs=graphs)
        runner.admit("r")
        runner.step([StepEntry("r", tuple(tokens[:12]), ())])
        states_before = [tensor.clone() for tensor in runner.cache.state_tensors]
        head_forward = runner.model.head.forward

        def failing(x):
            raise RuntimeError("the head fails")

        runner.model.head.forward = failing
        for entry in (StepEntry("r", tuple(tokens[12:20]), (7,)), StepEntry("r", (tokens[12],), (0,))):
            with pytest.raises(RuntimeError, match="the head fails"):
                runner.step([entry])
            assert runner.cache.committed_tokens("r") == 12
            for kept, tensor in zip(states_before, runner.cache.state_tensors):
                assert torch.equal(kept, tensor)
        runner.model.head.forward = head_forward
        logits = runner.step([StepEntry("r", tuple(tokens[12:20]), (0, 7))]).cpu()
        assert float((logits - expected[[12, 19]]).abs().max()) <= 2e-5
        for place in range(20, 24):                      # single tokens: recorded steps when graphs are on
            logits = runner.step([StepEntry("r", (tokens[place],), (0,))]).cpu()
            assert float((logits[0] - expected[place]).abs().max()) <= 2e-5
        runner.release("r")
        runner.cache.assert_invariants()


def test_a_preempted_request_builds_its_state_again(toy):
    """With too few pages the youngest request loses its pages and its state slot and
    is run again from its first token: the tokens are those of a roomy engine."""

    from miniserve_amd.engine import SamplingParams
    from miniserve_amd.entrypoint import LLM

    config = read_config(toy)
    prompts = [random_tokens(n, config["vocab_size"], 500 + n) for n in (30, 41, 18, 25)]
    params = SamplingParams(max_new_tokens=24)
    roomy = LLM(str(toy), dtype="float32", kv_block_size=16, num_kv_blocks=32, max_num_seqs=4)
    expected = roomy.generate(prompts, params)
    weights = read_weights(toy)
    for prompt, tokens in zip(prompts[:2], expected[:2]):       # the roomy engine itself against the plain form
        sequence = list(prompt)
        for token in tokens[:6]:
            top = torch.topk(toy_logits(weights, config, sequence)[-1], 2)
            assert int(top.indices[0]) == token or float(top.values[0] - top.values[1]) < 1e-4
            sequence.append(token)
    tight = LLM(str(toy), dtype="float32", kv_block_size=16, num_kv_blocks=9, max_num_seqs=4, enable_chunked_prefill=True)
    assert tight.generate(prompts, params) == expected
    assert tight.engine.counters["preemptions"] > 0
    tight.runner.cache.assert_invariants()


def test_a_chained_step_that_is_thrown_away_puts_the_state_back(toy):
    """Recorded steps are launched before the host has read the tokens they run.  When a
    stop token ends a request, the step that runs already is thrown away, and with it what
    its mixers wrote into the state rows of the OTHER requests: their tokens are those of
    a run without stop tokens, which the plain form and the plain sampler confirm on the way
    (temperature 1 from a seed a request, so that the tokens vary)."""

    import plain_sampling

    from miniserve_amd.engine import SamplingParams
    from miniserve_amd.entrypoint import LLM
    from miniserve_amd.sampling import Sampler

    config, weights = read_config(toy), read_weights(toy)
    prompts = [random_tokens(n, config["vocab_size"], 700 + n) for n in (9, 22, 15)]
    options = dict(dtype="float32", kv_block_size=16, num_kv_blocks=24, max_num_seqs=4)
    sampling = lambda index, **more: SamplingParams(max_new_tokens=30, temperature=1.0, seed=40 + index, **more)
    free_engine = LLM(str(toy), **options)
    free = free_engine.generate(prompts, [sampling(index) for index in range(3)])
    assert free_engine.runner.chained_steps > 10 and free_engine.runner.voided_chained_steps == 0
    for index, (prompt, tokens) in enumerate(zip(prompts, free)):         # against the plain form and the plain sampler
        logits = toy_logits(weights, config, list(prompt) + tokens[:-1])[len(prompt) - 1 :].float()
        stream = torch.Generator().manual_seed(40 + index)
        for place, token in enumerate(tokens):
            uniform = Sampler.draw_uniform(stream)
            if plain_sampling.edge_distance(logits[place], 1.0, 0, 1.0, uniform) > 1e-4:      # a draw on an edge may fall either way
                assert token == plain_sampling.sample_row(logits[place], 1.0, 0, 1.0, uniform), (index, place)
    # request 1 stops at the first token that it produces for the first time at its 7th place or later
    at = next(p for p in range(6, 30) if free[1][p] not in free[1][:p])
    stopped_engine = LLM(str(toy), **options)
    stopped = stopped_engine.generate(prompts, [sampling(0), sampling(1, stop_token_ids=(free[1][at],)), sampling(2)])
    assert stopped == [free[0], free[1][: at + 1], free[2]]
    assert stopped_engine.runner.voided_chained_steps == 1
    stopped_engine.runner.cache.assert_invariants()
