"""Random weights from a configuration and a seed, as checkpoint tensors or as a model folder.

Distributions: matrices and embeddings N(0, 0.02), q/k/v biases N(0, 0.02), norm
weights 1 + U(-0.1, 0.1). Each checkpoint tensor has a generator of its own,
seeded from the seed and the tensor's position in the sorted list of names, so a
tensor's values depend on neither the others nor the order of generation.
"""

from __future__ import annotations

import json
from dataclasses import dataclass
from pathlib import Path

from clockwork_amd.config.spec import ParamSpec, WeightTarget
from clockwork_amd.registry import resolve_architecture


@dataclass(frozen=True)
class _Entry:
    shape: tuple[int, ...]
    dtype: str


class RandomSource:
    """Stands in for a :class:`CheckpointIndex`: the same names and shapes, values drawn on demand."""

    def __init__(self, plan: list[WeightTarget], param_specs: dict[str, ParamSpec], seed: int,
                 device="cpu", skip_optional: bool = True, dtype: str = "bfloat16") -> None:
        if dtype not in ("bfloat16", "float32"):
            raise ValueError(f"random weights come as bfloat16 or float32, not {dtype!r}")
        self.seed = int(seed)
        self.device = device
        self.dtype = dtype
        self._init: dict[str, tuple] = {}
        shapes: dict[str, tuple[int, ...]] = {}
        for target in plan:
            if target.optional and skip_optional:
                continue
            for name, shape in zip(target.sources, target.source_shapes):
                shapes[name] = tuple(shape)
                self._init[name] = param_specs[target.param].init
        self._order = {name: i for i, name in enumerate(sorted(shapes))}
        tag = "BF16" if dtype == "bfloat16" else "F32"
        self.entries = {name: _Entry(shape, tag) for name, shape in shapes.items()}

    def read(self, name: str):
        import torch

        shape = self.entries[name].shape
        init = self._init[name]
        gen = torch.Generator(device=self.device)
        gen.manual_seed(self.seed * 1_000_003 + self._order[name])
        if init[0] == "normal":
            t = torch.empty(shape, dtype=torch.float32, device=self.device)
            t.normal_(0.0, float(init[1]), generator=gen)
        elif init[0] == "one_plus_uniform":
            t = torch.empty(shape, dtype=torch.float32, device=self.device)
            t.uniform_(-float(init[1]), float(init[1]), generator=gen).add_(1.0)
        elif init[0] == "zeros":
            t = torch.zeros(shape, dtype=torch.float32, device=self.device)
        else:
            raise ValueError(f"unknown init {init!r}")
        # float32: the values as drawn, with full mantissas (no bfloat16 number among them but by chance)
        return t if self.dtype == "float32" else t.to(torch.bfloat16)


def _describe(config: dict):
    from clockwork_amd.parts.model import model_param_specs

    arch = resolve_architecture(config)
    cfg = arch.parse_config(config)
    spec = arch.build_spec(cfg)
    return arch, cfg, spec, arch.weight_plan(cfg, spec), model_param_specs(spec)


def random_checkpoint_tensors(config: dict, seed: int, device="cpu", dtype: str = "bfloat16") -> dict:
    """``{checkpoint tensor name: tensor}`` for the architecture that ``config`` names, bfloat16
    or (``dtype="float32"``) float32 values that bfloat16 cannot hold."""
    _, _, _, plan, specs = _describe(config)
    source = RandomSource(plan, specs, seed, device=device, dtype=dtype)
    return {name: source.read(name) for name in sorted(source.entries)}


def write_random_model(out_dir: str | Path, config: dict, seed: int, dtype: str = "bfloat16") -> Path:
    """Write ``config.json`` and ``model.safetensors`` (bfloat16, or float32 tensors with full
    mantissas for ``dtype="float32"``) into ``out_dir``."""
    from safetensors.torch import save_file

    out = Path(out_dir)
    out.mkdir(parents=True, exist_ok=True)
    config = dict(config)
    arch, _, _, _, _ = _describe(config)
    config.setdefault("architectures", [arch.name])
    config.setdefault("torch_dtype", dtype)
    tensors = random_checkpoint_tensors(config, seed, dtype=dtype)
    (out / "config.json").write_text(json.dumps(config, indent=2) + "\n", encoding="utf-8")
    save_file({k: v.contiguous() for k, v in tensors.items()}, str(out / "model.safetensors"))
    return out
