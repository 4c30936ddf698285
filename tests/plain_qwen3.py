"""A plain, slow Qwen3 dense decoder: whole sequences, no cache, one function per
part, written from the reference's formulas.  It shares no code with the engine
(it imports nothing from the package) and is the oracle of every comparison.

Weights are a dict of tensors under their checkpoint names; ``config`` is the
``config.json`` mapping.  ``dtype`` is the arithmetic type (float64 by default,
so that differences to an engine in float32 are the engine's rounding alone).
"""

from __future__ import annotations


import torch

# ``rd``: a storage type (torch.bfloat16) to which every intermediate result is rounded
# at the places where the reference, computing in its model dtype, rounds.  None: no
# rounding.  It serves as a yardstick: how far the reference's own reduced-precision
# arithmetic lies from exact arithmetic on a given model and input.


def _r(x: torch.Tensor, rd) -> torch.Tensor:
    return x if rd is None else x.to(rd).to(x.dtype)


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float, rd=None) -> torch.Tensor:
    """``w * (x * rsqrt(mean(x^2) + eps))`` over the last dimension: no mean
    subtraction, no bias, plain ``w`` (reference: miniserve/model/layers.py:30-34)."""

    variance = x.pow(2).mean(dim=-1, keepdim=True)
    return _r(weight * _r(x * torch.rsqrt(variance + eps), rd), rd)


def rope_angles(positions: torch.Tensor, head_dim: int, theta: float) -> tuple[torch.Tensor, torch.Tensor]:
    """cos and sin ``[T, head_dim]`` for absolute positions: ``inv_freq[i] =
    1 / theta^(2i/D)``, ``angle = pos * inv_freq``, the half-table repeated twice.
    The table is made in float32 as the reference does (miniserve/model/rope.py:24-29)."""

    frequencies = torch.arange(0, head_dim, 2, dtype=torch.float32)
    inverse_frequency = 1.0 / (theta ** (frequencies / head_dim))
    angles = positions.to(torch.float32).unsqueeze(-1) * inverse_frequency
    embedding = torch.cat((angles, angles), dim=-1)
    return embedding.cos(), embedding.sin()


def rotate_half(x: torch.Tensor) -> torch.Tensor:
    """``cat(-x[D/2:], x[:D/2])`` (reference: miniserve/model/rope.py:32-34)."""

    first, second = x.chunk(2, dim=-1)
    return torch.cat((-second, first), dim=-1)


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, rd=None) -> torch.Tensor:
    """``x * cos + rotate_half(x) * sin`` for ``x [heads, T, D]`` and tables
    ``[T, D]`` shared by all heads (reference: miniserve/model/rope.py:47-52)."""

    cos = _r(cos.to(x.dtype), rd).unsqueeze(0)
    sin = _r(sin.to(x.dtype), rd).unsqueeze(0)
    return _r(_r(x * cos, rd) + _r(rotate_half(x) * sin, rd), rd)


def repeat_kv(x: torch.Tensor, repeats: int) -> torch.Tensor:
    """Each kv head serves ``repeats`` consecutive query heads: ``[kv0 x G, kv1 x G, ...]``
    (reference: miniserve/model/qwen3.py:20-27)."""

    heads, length, dim = x.shape
    return x[:, None, :, :].expand(heads, repeats, length, dim).reshape(heads * repeats, length, dim)


def causal_attention(
    q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, window: int | None = None, rd=None
) -> torch.Tensor:
    """``softmax(q k^T * scale + mask) v`` for ``q [Hq, T, D]``, ``k, v [Hkv, T, D]``;
    the scale is applied after the product; key j is visible to query t iff
    ``j <= t`` (reference: miniserve/model/qwen3.py:132-138, 243-249), and, with a
    window, iff also ``j > t - window``."""

    groups = q.shape[0] // k.shape[0]
    k = repeat_kv(k, groups)
    v = repeat_kv(v, groups)
    length = q.shape[1]
    scores = _r(_r(torch.matmul(q, k.transpose(1, 2)), rd) * scale, rd)
    index = torch.arange(length)
    allowed = index.view(1, length) <= index.view(length, 1)
    if window is not None:
        allowed = allowed & (index.view(1, length) > index.view(length, 1) - window)
    scores = scores.masked_fill(~allowed.unsqueeze(0), float("-inf"))
    return _r(torch.matmul(_r(torch.softmax(scores, dim=-1), rd), v), rd)


def attention_block(
    x: torch.Tensor, weights: dict, prefix: str, config: dict, positions: torch.Tensor,
    shared_kv: tuple[torch.Tensor, torch.Tensor] | None = None, window: int | None = None, rd=None,
) -> tuple[torch.Tensor, tuple[torch.Tensor, torch.Tensor]]:
    """Project, norm q and k per head over ``D`` (before the rotation), rotate q and
    k, attend, project back (reference: miniserve/model/qwen3.py:113-138).  Returns the
    output and the (k, v) it attended over, which another layer may share."""

    length = x.shape[0]
    heads, kv_heads, dim = config["num_attention_heads"], config["num_key_value_heads"], config["head_dim"]
    eps = config["rms_norm_eps"]
    cos, sin = rope_angles(positions, dim, config["rope_theta"])
    q = _r(x @ weights[prefix + "q_proj.weight"].T, rd).view(length, heads, dim)
    q = rms_norm(q, weights[prefix + "q_norm.weight"], eps, rd).transpose(0, 1)
    q = apply_rope(q, cos, sin, rd)
    if shared_kv is None:
        k = _r(x @ weights[prefix + "k_proj.weight"].T, rd).view(length, kv_heads, dim)
        v = _r(x @ weights[prefix + "v_proj.weight"].T, rd).view(length, kv_heads, dim)
        k = rms_norm(k, weights[prefix + "k_norm.weight"], eps, rd).transpose(0, 1)
        k = apply_rope(k, cos, sin, rd)
        v = v.transpose(0, 1)
    else:
        k, v = shared_kv
    attended = causal_attention(q, k, v, dim**-0.5, window, rd)
    attended = attended.transpose(0, 1).reshape(length, heads * dim)
    return _r(attended @ weights[prefix + "o_proj.weight"].T, rd), (k, v)


def swiglu(x: torch.Tensor, weights: dict, prefix: str, rd=None) -> torch.Tensor:
    """``down(silu(gate(x)) * up(x))`` without biases (reference: miniserve/model/layers.py:86-87)."""

    gate = _r(x @ weights[prefix + "gate_proj.weight"].T, rd)
    up = _r(x @ weights[prefix + "up_proj.weight"].T, rd)
    return _r(_r(_r(torch.nn.functional.silu(gate), rd) * up, rd) @ weights[prefix + "down_proj.weight"].T, rd)


def decoder_layer(h, weights, index, config, positions, shared_kv=None, window=None, rd=None):
    """Pre-norm residual block: ``h += attn(norm(h)); h += mlp(norm(h))``
    (reference: miniserve/model/qwen3.py:342-347)."""

    base = f"model.layers.{index}."
    eps = config["rms_norm_eps"]
    attended, kv = attention_block(
        rms_norm(h, weights[base + "input_layernorm.weight"], eps, rd), weights, base + "self_attn.", config,
        positions, shared_kv, window, rd,
    )
    h = _r(h + attended, rd)
    h = _r(
        h + swiglu(rms_norm(h, weights[base + "post_attention_layernorm.weight"], eps, rd), weights, base + "mlp.", rd),
        rd,
    )
    return h, kv


def forward_logits(
    weights: dict, config: dict, token_ids, *, dtype: torch.dtype = torch.float64,
    order=None, windows=None, first_position: int = 0, rd=None, rows=None,
) -> torch.Tensor:
    """Logits ``[T, V]`` for one whole sequence: embed, layers, final norm, head
    (reference: miniserve/model/qwen3.py:436-448, 547-558).  The head is the
    embedding when ``tie_word_embeddings`` (qwen3.py:537-540), else ``lm_head.weight``.

    ``order``: list of ``(layer, cache_from)`` (default: every layer once);
    ``windows``: per call, a window or None; ``first_position``: absolute position
    of the first token (for the shift invariant); ``rows``: the positions whose
    logits are returned (default: all), for vocabularies too large to keep whole."""

    weights = {name: tensor.to(dtype) for name, tensor in weights.items()}
    tokens = torch.as_tensor(token_ids, dtype=torch.long)
    positions = torch.arange(first_position, first_position + tokens.numel())
    h = weights["model.embed_tokens.weight"][tokens]
    if order is None:
        order = [(index, None) for index in range(config["num_hidden_layers"])]
    kept: list = []
    for call, (layer, cache_from) in enumerate(order):
        window = None if windows is None else windows[call]
        shared = None if cache_from is None else kept[cache_from]
        h, kv = decoder_layer(h, weights, layer, config, positions, shared, window, rd)
        kept.append(kv)
    if rows is not None:
        h = h[torch.as_tensor(rows, dtype=torch.long)]
    h = rms_norm(h, weights["model.norm.weight"], config["rms_norm_eps"], rd)
    head = weights["model.embed_tokens.weight"] if config.get("tie_word_embeddings") else weights["lm_head.weight"]
    return _r(h @ head.T, rd)


def greedy_generate(weights: dict, config: dict, prompt, max_new_tokens: int, *, dtype=torch.float64):
    """Greedy continuation by recomputing the whole sequence for every token.
    Also returns, per generated token, the gap between the two largest logits, so
    a caller can tell a real mismatch from a near tie."""

    tokens = list(prompt)
    generated, margins = [], []
    for _ in range(max_new_tokens):
        logits = forward_logits(weights, config, tokens, dtype=dtype)[-1]
        top = torch.topk(logits, 2)
        generated.append(int(top.indices[0]))
        margins.append(float(top.values[0] - top.values[1]))
        tokens.append(generated[-1])
    return generated, margins
