"""Random-weights mode: a model folder (``config.json`` + ``model.safetensors``)
from a configuration and a seed.  The reference has no such mode (its model is
filled from safetensors only, miniserve/api/bootstrap.py:113-115).

Matrices and embeddings ~ N(0, 0.02), norm weights ~ 1 + N(0, 0.1), drawn in
float32 from one CPU generator in the model's fixed tensor order, so a seed
names one model everywhere.
"""

from __future__ import annotations

import json
from pathlib import Path
from typing import Callable, Sequence

import torch

from ..parts.base import WeightSpec

MATRIX_STD = 0.02
NORM_STD = 0.1
STORE_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}


# name -> rule(shape, generator, device) -> float32 tensor.  Parts name a rule in their
# ``WeightSpec.init`` or bring a callable of the same form; ``register_init`` adds a name.
InitRule = Callable[[tuple, torch.Generator, "torch.device | str"], torch.Tensor]
_INIT_RULES: dict[str, InitRule] = {
    "matrix": lambda shape, generator, device: torch.randn(shape, generator=generator, dtype=torch.float32, device=device) * MATRIX_STD,
    "norm": lambda shape, generator, device: 1.0 + torch.randn(shape, generator=generator, dtype=torch.float32, device=device) * NORM_STD,
    "zeros": lambda shape, generator, device: torch.zeros(shape, dtype=torch.float32, device=device),
}


def register_init(name: str, rule: InitRule) -> None:
    """Adds a named rule for ``WeightSpec.init``."""

    if not callable(rule):
        raise TypeError("an init rule is a callable (shape, generator, device) -> float32 tensor.")
    _INIT_RULES[name] = rule


def draw_tensor(spec: WeightSpec, generator: torch.Generator, device: torch.device | str = "cpu") -> torch.Tensor:
    if spec.keep == "int32":
        return torch.zeros(spec.shape, dtype=torch.int32, device=device)
    rule = spec.init if callable(spec.init) else _INIT_RULES.get(spec.init)
    if rule is None:
        raise ValueError(f"{spec.name}: unknown init rule {spec.init!r} (known: {sorted(_INIT_RULES)}).")
    tensor = rule(tuple(spec.shape), generator, device)
    if tuple(tensor.shape) != tuple(spec.shape) or tensor.dtype != torch.float32:
        raise ValueError(f"{spec.name}: its init rule must give a float32 tensor of shape {tuple(spec.shape)}.")
    return tensor


def random_tensors(specs: Sequence[WeightSpec], seed: int) -> dict[str, torch.Tensor]:
    """Float32 CPU tensors for every non-tied spec, in spec order."""

    generator = torch.Generator(device="cpu").manual_seed(seed)
    return {spec.name: draw_tensor(spec, generator) for spec in specs if spec.same_as is None}


def write_random_model(config, folder: str | Path, *, seed: int, store_dtype: str = "float32") -> Path:
    """Write ``config.json`` and ``model.safetensors`` for ``config`` (any
    registered architecture's configuration object) into ``folder``."""

    from safetensors.torch import save_file

    from ..parts.model import DecoderModel

    if store_dtype not in STORE_DTYPES:
        raise ValueError(f"store_dtype must be one of {sorted(STORE_DTYPES)}.")
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    specs = DecoderModel(config.model_spec(), "float32").weight_specs()
    tensors = {}
    for name, tensor in random_tensors(specs, seed).items():
        if tensor.is_floating_point():
            tensor = tensor.to(STORE_DTYPES[store_dtype])
        tensors[name] = tensor.contiguous()
    data = config.to_dict()
    data["torch_dtype"] = store_dtype
    (folder / "config.json").write_text(json.dumps(data, indent=2) + "\n", encoding="utf-8")
    save_file(tensors, str(folder / "model.safetensors"))
    return folder


# Up to this many float32 bytes a random model is drawn by the CPU generator, so that a
# seed names the model that ``write_random_model`` writes; larger ones are drawn on the device.
HOST_DRAW_BYTES = 1 << 30


def random_model_tensors(
    specs: Sequence[WeightSpec], *, seed: int, dtype: torch.dtype, device: torch.device | str
) -> dict[str, torch.Tensor]:
    """Random weights on ``device`` in the engine's types.  A model of up to
    ``HOST_DRAW_BYTES`` is drawn by :func:`random_tensors` (the CPU generator: the same
    values as a folder written by :func:`write_random_model` with this seed holds); a
    larger one by :func:`random_device_tensors`, whose values differ."""

    drawn = [spec for spec in specs if spec.same_as is None]
    size = sum(4 * int(torch.Size(spec.shape).numel()) for spec in drawn)
    if size > HOST_DRAW_BYTES:
        return random_device_tensors(specs, seed=seed, dtype=dtype, device=device)
    tensors = {}
    for spec, (name, tensor) in zip(drawn, random_tensors(specs, seed).items()):
        if tensor.is_floating_point() and spec.keep == "compute":
            tensor = tensor.to(dtype)
        tensors[name] = tensor.to(device)
    return tensors


def random_device_tensors(
    specs: Sequence[WeightSpec], *, seed: int, dtype: torch.dtype, device: torch.device | str
) -> dict[str, torch.Tensor]:
    """The same distributions drawn tensor by tensor on the device, for models too
    large to pass through a file or host memory (benchmarks).  The values differ
    from :func:`random_tensors` with the same seed."""

    generator = torch.Generator(device=device).manual_seed(seed)
    tensors = {}
    for spec in specs:
        if spec.same_as is not None:
            continue
        tensor = draw_tensor(spec, generator, device)
        if tensor.is_floating_point() and spec.keep == "compute":
            tensor = tensor.to(dtype)
        tensors[spec.name] = tensor
    return tensors
