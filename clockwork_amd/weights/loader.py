"""Fill a model's parameters from a checkpoint, by tensor name.

One pass checks names and shapes of the whole plan and raises a single error
that lists every missing tensor, every tensor the model has no use for and every
wrong shape (the reference raises on missing/unexpected keys,
clockwork/engine/loader.py:57-64). Then tensors are read one by one, cast and
moved to the device; fused projections are written into slices of one buffer.
"""

from __future__ import annotations

import json
from pathlib import Path

from clockwork_amd.config.spec import ParamSpec, WeightTarget
from clockwork_amd.weights.checkpoint import CheckpointIndex, WeightMismatchError
from clockwork_amd.weights.transforms import apply_transform, transformed_shape


def read_config_json(model: str | Path) -> dict:
    """The architecture's configuration: ``model`` is a folder that holds a config.json, or (for
    a model that needs no checkpoint: random weights) such a file itself."""
    path = Path(model)
    if path.is_dir():
        path = path / "config.json"
    if not path.is_file():
        raise FileNotFoundError(f"no config.json in {model}")
    return json.loads(path.read_text(encoding="utf-8"))


def check_plan(
    available: dict[str, tuple[int, ...]], plan: list[WeightTarget]
) -> tuple[list[str], list[str], list[str]]:
    """Names and shapes only: (missing, unexpected, wrong_shape)."""
    missing: list[str] = []
    wrong: list[str] = []
    used: set[str] = set()
    for target in plan:
        for name, shape in zip(target.sources, target.source_shapes):
            if name not in available:
                if not target.optional:
                    missing.append(name)
                continue
            used.add(name)
            if tuple(available[name]) != tuple(shape):
                wrong.append(f"{name}: checkpoint {tuple(available[name])}, model {tuple(shape)}")
    unexpected = [name for name in available if name not in used]
    return missing, unexpected, wrong


def _target_dtype(spec: ParamSpec, stored: list[str], compute_dtype):
    import torch

    if spec.precision == "float32":
        return torch.float32
    if spec.precision == "int32":
        return torch.int32
    if spec.precision == "stored" and all(tag in ("F32", "F64") for tag in stored):
        return torch.float32
    return compute_dtype


def load_parameters(
    model_dir: str | Path,
    plan: list[WeightTarget],
    param_specs: dict[str, ParamSpec],
    compute_dtype,
    device,
    source=None,
) -> dict:
    """Returns ``{param name: device tensor}`` for every entry of ``param_specs``.

    ``source`` replaces the folder's safetensors files by any object with
    ``entries`` (name -> shape/dtype) and ``read(name)``; the random-weights
    generator is one. An optional target whose tensors are absent is left out of
    the result: the model decides what stands in for it (a tied head).
    """
    import torch

    index = source if source is not None else CheckpointIndex(model_dir)
    available = {name: entry.shape for name, entry in index.entries.items()}
    missing, unexpected, wrong = check_plan(available, plan)
    if missing or unexpected or wrong:
        raise WeightMismatchError(missing, unexpected, wrong)
    planned = {t.param for t in plan}
    unplanned = sorted(set(param_specs) - planned)
    if unplanned:
        raise RuntimeError(f"the weight plan fills no tensor into parameters {unplanned}")

    params: dict = {}
    for target in plan:
        present = [name in index.entries for name in target.sources]
        if not all(present):
            continue  # optional and absent
        spec = param_specs[target.param]
        # the sources as they are after the target's transform (a transpose, a slice of rows): these
        # are what is stacked along dim 0
        shapes = [transformed_shape(target.transform, shape) for shape in target.source_shapes]
        rows = sum(shape[0] for shape in shapes)
        full_shape = (rows, *shapes[0][1:])
        if any(shape[1:] != shapes[0][1:] for shape in shapes):
            raise RuntimeError(f"weight plan for {target.param} stacks sources whose rows differ: {shapes}")
        if tuple(spec.shape) != full_shape:
            raise RuntimeError(
                f"weight plan for {target.param} yields {full_shape}, the part declares {spec.shape}"
            )
        stored = [index.entries[name].dtype for name in target.sources]
        if spec.precision == "int32" and not all(tag[0] in "IU" for tag in stored):
            raise WeightMismatchError([], [], [f"{target.param}: expected an integer table, got {stored}"])
        dtype = _target_dtype(spec, stored, compute_dtype)
        out = torch.empty(full_shape, dtype=dtype, device=device)
        row = 0
        for name, shape in zip(target.sources, shapes):
            out[row : row + shape[0]].copy_(apply_transform(target.transform, index.read(name)))
            row += shape[0]
        params[target.param] = out
    if hasattr(index, "close"):
        index.close()
    return params
