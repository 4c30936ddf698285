"""Stand-ins for the library's kernels, written with torch on CPU tensors, for tests of
everything *around* the kernels (parts, step function, cache, batch builder, engine)
where no GPU is visible.  They are test doubles with the kernels' interfaces, not a
path of the product: the product has no CPU path and fails loudly without its library.

Each follows the kernel's contract as ``miniserve_amd/ops/__init__.py`` states it, in
32-bit arithmetic; outputs take the dtype the kernel gives them."""

from __future__ import annotations

import plain_sampling
import torch


def embedding_gather(token_ids, table):
    return table[token_ids.long()].float()


def rmsnorm(x, weight, eps, *, delta=None, rows=None, write_back=False):
    value = x.float() if delta is None else x.float() + delta.float()
    if delta is not None and write_back:
        x.copy_(value)
    if rows is not None:
        value = value[rows.long()]
    normed = value * torch.rsqrt(value.pow(2).mean(-1, keepdim=True) + eps)
    return normed.to(weight.dtype) * weight


def residual_add(h, delta):
    h += delta.float()


def rope_table(positions, inv_freq):
    angles = positions.float()[:, None] * inv_freq[None, :]
    return torch.cos(angles), torch.sin(angles)


def _head_norm(x, weight, eps):
    if weight is None:
        return x
    return (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)) * weight.float()


def _rotate(x, rope):
    if rope is None:
        return x
    cos, sin = (t[:, None, :] for t in rope)
    half = x.shape[-1] // 2
    first, second = x[..., :half], x[..., half:]
    return torch.cat([first * cos - second * sin, second * cos + first * sin], dim=-1)


def qk_norm_rope_append(packed, *, num_q_heads, num_kv_heads, head_dim, q_weight, k_weight, eps, rope,
                        slot_mapping=None, key_pool=None, value_pool=None):
    n = packed.shape[0]
    heads = packed.float().reshape(n, num_q_heads + 2 * num_kv_heads, head_dim)
    q = _rotate(_head_norm(heads[:, :num_q_heads], q_weight, eps), rope)
    if num_kv_heads:
        k = _rotate(_head_norm(heads[:, num_q_heads : num_q_heads + num_kv_heads], k_weight, eps), rope)
        v = heads[:, num_q_heads + num_kv_heads :]
        block_size = key_pool.shape[2]
        page, offset = slot_mapping.long() // block_size, slot_mapping.long() % block_size
        key_pool[page, :, offset, :] = k.to(key_pool.dtype)
        value_pool[page, :, :, offset] = v.to(value_pool.dtype)
    return q.to(packed.dtype) if num_q_heads else None


def attention(q, key_pool, value_pool, *, block_table, seq_of_token, positions, scale, window=None, decode_prefix=0,
              tiles=None, max_context=None, splits=None):
    n, heads, head_dim = q.shape
    kv_heads, block_size = key_pool.shape[1], key_pool.shape[2]
    group = heads // kv_heads
    out = torch.empty((n, heads, head_dim), dtype=torch.float32)
    for token in range(n):
        row, position = int(seq_of_token[token]), int(positions[token])
        low = 0 if window is None else max(0, position - window + 1)
        seen = torch.arange(low, position + 1)
        pages = block_table[row, seen // block_size].long()
        keys = key_pool[pages, :, seen % block_size, :].float()                      # [L, kv_heads, D]
        values = value_pool[pages, :, :, seen % block_size].float()                  # [L, kv_heads, D]
        keys = keys.repeat_interleave(group, dim=1)
        values = values.repeat_interleave(group, dim=1)
        scores = torch.einsum("hd,lhd->hl", q[token].float(), keys) * scale
        out[token] = torch.einsum("hl,lhd->hd", torch.softmax(scores, dim=-1), values)
    return out.to(q.dtype)


def linear(x, weight, *, accumulate_into=None, out_float32=False):
    product = x.float() @ weight.float().T
    if accumulate_into is not None:
        accumulate_into += product
        return accumulate_into
    return product if out_float32 else product.to(x.dtype)


def silu_mul(gate_up):
    half = gate_up.shape[1] // 2
    gate, up = gate_up[:, :half].float(), gate_up[:, half:].float()
    return (torch.nn.functional.silu(gate) * up).to(gate_up.dtype)


def linear_silu_mul(x, weight):
    return silu_mul(linear(x, weight))


def linear_normed(residual, norm_weight, eps, weight, *, gated=False):
    """The norm as the product's prologue: weight x value is rounded once, the sums are scaled."""

    scale = torch.rsqrt(residual.float().pow(2).mean(-1, keepdim=True) + eps)
    product = ((norm_weight.float() * residual.float()).to(weight.dtype).float() @ weight.float().T) * scale
    product = product.to(weight.dtype)
    return silu_mul(product) if gated else product


def linear_norm_ahead(x, weight, residual, norm_weight):
    """``residual += x W^T``; what the norm behind it needs: weight x value, and the squares
    in two partial sums a row (as if two workgroups had shared the columns)."""

    residual += x.float() @ weight.float().T
    half = residual.shape[1] // 2
    squares = torch.stack([residual[:, :half].pow(2).sum(-1), residual[:, half:].pow(2).sum(-1)])
    return (norm_weight.float() * residual).to(weight.dtype), squares


def linear_prepared(weighted, squares, eps, weight, *, gated=False):
    scale = torch.rsqrt(squares.sum(0) / weighted.shape[1] + eps)[:, None]
    product = ((weighted.float() @ weight.float().T) * scale).to(weight.dtype)
    return silu_mul(product) if gated else product


def sample_rows(logits, *, temperature=None, top_k=None, top_p=None, uniform=None, top_p_alone=True):
    tokens = []
    for row in range(logits.shape[0]):
        if not bool(torch.isfinite(logits[row]).all()):
            tokens.append(-1)
        elif temperature is None or float(temperature[row]) == 0:
            tokens.append(int(torch.argmax(logits[row])))
        else:
            tokens.append(plain_sampling.sample_row(
                logits[row], float(temperature[row]), 0 if top_k is None else int(top_k[row]),
                1.0 if top_p is None else float(top_p[row]), float(uniform[row])))
    return torch.tensor(tokens, dtype=torch.int32)


class OnDevice(torch.Tensor):
    """A CPU tensor that says it lives on the device: what the sampling stand-in returns
    where recorded steps are played, so that the engine feeds it to the next step "on the
    device" as it does with the kernel's output."""

    @property
    def is_cuda(self):
        return True


class Recording:
    """Stands for ``torch.cuda.graph(graph, pool=...)``: while it is open, a model's forward
    pass is not run but noted in ``graph``, with an output tensor of its own."""

    current = None

    def __init__(self, graph, pool=None):
        self.graph = graph

    def __enter__(self):
        Recording.current = self.graph

    def __exit__(self, *exc):
        Recording.current = None


class RecordedGraph:
    """Stands for ``torch.cuda.CUDAGraph``: ``replay`` runs what was noted, on what the
    step's tensors hold at that moment, into the same output tensors."""

    def __init__(self):
        self.calls = []

    def replay(self):
        for call in self.calls:
            call()


class PassedEvent:
    def record(self):
        pass

    def synchronize(self):
        pass


def install(monkeypatch, *, fused: str | None = None, recordings: bool = False):
    """Puts the stand-ins in the kernels' places for one test and lets a runner stand on
    the CPU.  ``fused``: None, the parts take the plain calls; ``"prologue"``, every norm
    before a product is that product's prologue; ``"prepared"``, every norm behind a
    product that adds into the residual stream is prepared by it.  ``recordings``: the
    runner may record decode steps; a recording is a note of the model's forward pass that
    ``replay`` runs again (so everything around the recordings is the product's own: the
    numbers of a step, block tables at their fixed widths, spare rows, the two host
    buffers, steps launched behind the sampling "on the device")."""

    import miniserve_amd.engine.runner as runner_module
    import miniserve_amd.parts.mlp as mlp_module
    from miniserve_amd import ops

    for name in ("embedding_gather", "rmsnorm", "residual_add", "rope_table", "qk_norm_rope_append", "attention", "linear",
                 "silu_mul", "linear_silu_mul", "sample_rows"):
        monkeypatch.setattr(ops, name, globals()[name])
    for name in ("linear_normed", "linear_norm_ahead", "linear_prepared"):
        monkeypatch.setattr(ops, name, globals()[name])
    monkeypatch.setattr(ops, "can_fuse_norm", lambda *args, **kwargs: fused == "prologue")
    monkeypatch.setattr(ops, "can_prepare_norm", lambda *args, **kwargs: fused == "prepared")
    monkeypatch.setattr(ops, "can_use_prepared_norm", lambda *args, **kwargs: fused == "prepared")
    monkeypatch.setattr(ops, "can_accumulate", lambda rows, weight: True)
    monkeypatch.setattr(ops, "load", lambda: None)
    monkeypatch.setattr(ops, "prepare_products", lambda device: None)
    monkeypatch.setattr(runner_module, "_require_gpu", lambda device: None)
    # (the feed-forward keeps its activation's two kernels by name)
    monkeypatch.setitem(mlp_module._ACTIVATIONS, "silu", (silu_mul, linear_silu_mul))
    if not recordings:
        return
    from miniserve_amd.parts import DecoderModel
    from miniserve_amd.sampling import Sampler

    forward = DecoderModel.forward

    def noted_forward(self, ctx, caches, logit_rows):
        graph = Recording.current
        if graph is None:
            return forward(self, ctx, caches, logit_rows)
        output = torch.zeros((logit_rows.numel(), self.spec.vocab_size), dtype=torch.float32)

        def again():
            ctx.scratch.clear()             # what a step shares between layers is made again in every replay
            output.copy_(forward(self, ctx, caches, logit_rows))

        graph.calls.append(again)
        return output

    monkeypatch.setattr(DecoderModel, "forward", noted_forward)
    monkeypatch.setattr(torch.cuda, "CUDAGraph", RecordedGraph)
    monkeypatch.setattr(torch.cuda, "graph", Recording)
    monkeypatch.setattr(torch.cuda, "graph_pool_handle", lambda: None)
    monkeypatch.setattr(torch.cuda, "synchronize", lambda device=None: None)
    monkeypatch.setattr(torch.cuda, "Event", PassedEvent)
    monkeypatch.setattr(torch.Tensor, "pin_memory", lambda self: self)
    monkeypatch.setattr(Sampler, "_token_buffer", lambda self, rows: torch.empty(rows, dtype=torch.int32))
    monkeypatch.setattr(ops, "sample_rows", lambda *args, **kwargs: sample_rows(*args, **kwargs).as_subclass(OnDevice))
