"""Weights from safetensors, by tensor name, with one strict check up front.

File discovery and strictness follow the reference (miniserve/model/loader.py:105-129,
155-217): an index file names the shards, else every ``*.safetensors`` of the
folder is read; a name in two shards is an error; the set of names must equal
what the model wants; every shape must match; a tied head stored in the file
must equal the embedding bit for bit.  All findings are reported in ONE error.
"""

from __future__ import annotations

import json
import re
from dataclasses import dataclass, field
from pathlib import Path
from typing import Sequence

import torch

from ..parts.base import WeightSpec


class WeightLoadError(RuntimeError):
    """The checkpoint does not fit the model.  ``missing``, ``unexpected``,
    ``wrong_shape`` and ``other`` hold the findings that the message lists."""

    def __init__(self, missing, unexpected, wrong_shape, other) -> None:
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        self.other = list(other)
        lines = ["checkpoint does not match the model:"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): {self.missing}")
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): {self.unexpected}")
        for name, found, wanted in self.wrong_shape:
            lines.append(f"  wrong shape: {name} is {found}, the model wants {wanted}")
        lines.extend(f"  {message}" for message in self.other)
        super().__init__("\n".join(lines))


@dataclass
class WeightLoadReport:
    """What was loaded (reference: loader.py:19-26)."""

    model_dir: str
    loaded_tensors: int = 0
    source_bytes: int = 0
    source_dtype_counts: dict[str, int] = field(default_factory=dict)
    target_dtype: str = ""
    target_device: str = ""


_STORED_FLOATS = (torch.float32, torch.bfloat16, torch.float16, torch.float64)


def weight_files(model_dir: Path) -> tuple[Path, ...]:
    index_files = sorted(model_dir.glob("*.safetensors.index.json"))
    if len(index_files) > 1:
        raise RuntimeError("Expected at most one safetensors index.")
    if index_files:
        index = json.loads(index_files[0].read_text(encoding="utf-8"))
        weight_map = index.get("weight_map")
        if not isinstance(weight_map, dict) or not weight_map:
            raise ValueError("Safetensors index has no non-empty weight_map.")
        if any(not isinstance(k, str) or not isinstance(v, str) for k, v in weight_map.items()):
            raise ValueError("Safetensors index weight_map must contain string keys and values.")
        files = []
        for name in sorted(set(weight_map.values())):
            path = (model_dir / name).resolve()
            if model_dir.resolve() not in path.parents:
                raise ValueError(f"shard {name!r} lies outside the model folder.")
            files.append(path)
    else:
        files = sorted(model_dir.glob("*.safetensors"))
    if not files or any(not path.is_file() for path in files):
        raise FileNotFoundError(f"{model_dir} holds no safetensors shards (or some named by the index are missing).")
    return tuple(files)


def _target_dtype(spec: WeightSpec, compute_dtype: torch.dtype) -> torch.dtype:
    if spec.keep == "compute":
        return compute_dtype
    if spec.keep == "float32":
        return torch.float32
    if spec.keep == "int32":
        return torch.int32
    raise ValueError(f"{spec.name}: unknown keep rule {spec.keep!r}.")


def load_weights(
    model_dir: str | Path,
    specs: Sequence[WeightSpec],
    *,
    dtype: torch.dtype,
    device: torch.device | str,
) -> tuple[dict[str, torch.Tensor], WeightLoadReport]:
    """Read the tensors that ``specs`` name from ``model_dir`` onto ``device``.

    Names and shapes of the whole checkpoint are checked before a single tensor
    is read, so a forward pass never sees a half-loaded model."""

    from safetensors import safe_open

    model_dir = Path(model_dir)
    files = weight_files(model_dir)
    report = WeightLoadReport(model_dir=str(model_dir), target_dtype=str(dtype), target_device=str(device))

    locations: dict[str, Path] = {}
    shapes: dict[str, tuple[int, ...]] = {}
    other: list[str] = []
    for path in files:
        report.source_bytes += path.stat().st_size
        with safe_open(path, framework="pt", device="cpu") as handle:
            for key in handle.keys():
                if key in locations:
                    other.append(f"duplicate tensor across shards: {key}")
                    continue
                locations[key] = path
                shapes[key] = tuple(handle.get_slice(key).get_shape())

    wanted = {spec.name: spec for spec in specs}
    missing = sorted(name for name, spec in wanted.items() if name not in locations and not spec.optional)
    unexpected = sorted(name for name in locations if name not in wanted)
    wrong_shape = sorted(
        (name, shapes[name], tuple(spec.shape))
        for name, spec in wanted.items()
        if name in shapes and shapes[name] != tuple(spec.shape)
    )
    # An unexpected tensor of a layer that the model does not have most often means a
    # checkpoint of a deeper model; it gets a line of its own (reference: weight_map.py:49-59).
    layer_of = re.compile(r"(?:^|\.)layers\.(\d+)\.")
    depth = 1 + max((int(found.group(1)) for found in map(layer_of.search, wanted) if found), default=-1)
    beyond = sorted({int(found.group(1)) for found in map(layer_of.search, unexpected) if found and int(found.group(1)) >= depth})
    if depth > 0 and beyond:
        other.append(f"tensors of layers {beyond} are stored, the model has layers 0..{depth - 1}")
    if missing or unexpected or wrong_shape or other:
        raise WeightLoadError(missing, unexpected, wrong_shape, other)

    tensors: dict[str, torch.Tensor] = {}
    handles = {path: safe_open(path, framework="pt", device="cpu") for path in set(locations.values())}
    try:
        for spec in specs:
            if spec.name not in locations:
                continue
            source = handles[locations[spec.name]].get_tensor(spec.name)
            report.source_dtype_counts[str(source.dtype)] = report.source_dtype_counts.get(str(source.dtype), 0) + 1
            target = _target_dtype(spec, dtype)
            if target.is_floating_point and source.dtype not in _STORED_FLOATS:
                other.append(f"{spec.name} is stored as {source.dtype}, a floating type is wanted")
                continue
            if not target.is_floating_point and source.dtype.is_floating_point:
                other.append(f"{spec.name} is stored as {source.dtype}, an integer table is wanted")
                continue
            if spec.same_as is not None:
                # A tied tensor that the file stores must equal its source bit for
                # bit; it is then dropped, the source tensor stands for both.
                twin = handles[locations[spec.same_as]].get_tensor(spec.same_as)
                if twin.dtype != source.dtype or not torch.equal(twin, source):
                    other.append(f"{spec.name} is tied to {spec.same_as} but their values differ")
                continue
            tensors[spec.name] = source.to(device=device, dtype=target).contiguous()
            report.loaded_tensors += 1
    finally:
        handles.clear()
    if other:
        raise WeightLoadError([], [], [], other)
    return tensors, report
