"""Engine configuration: model, cache and scheduler sections, YAML and key=value overrides.

Same sections and field names as the reference (clockwork/config.py:17-87); the
reference's ``attention_backend`` is gone (there is one backend: the HIP kernels)
and the scheduler gains the chunked-prefill knobs.
"""

from __future__ import annotations

from dataclasses import dataclass, field, fields
from pathlib import Path

import yaml


WEIGHT_MODES = ("checkpoint", "random", "random_device")


@dataclass
class ModelConfig:
    """Which model folder to serve and how (clockwork/config.py:17-31)."""

    model: str
    dtype: str = "float32"
    device: str = "cuda"
    max_model_len: int = 4096
    seed: int = 0
    trust_remote_code: bool = False
    # at start-up, let the matrix library time its kernels for the products of a full prefill
    # portion and of the wide decode batches and keep the fastest (bfloat16 only)
    tune_products: bool = False
    # run the large bfloat16 products on this package's own tiled kernel instead of the matrix
    # library (slower; for runs that must not depend on the library)
    hip_products: bool = False
    # where the weights come from: "checkpoint" (the safetensors files of the folder ``model``),
    # "random" (drawn from ``weight_seed`` on the host, the very values that ``make-random`` writes
    # into a folder; ``model`` may then name a bare config.json) or "random_device" (drawn by the
    # GPU's generator: other values, made in seconds for the largest shapes)
    weights: str = "checkpoint"
    weight_seed: int = 0

    def __post_init__(self):
        if self.weights not in WEIGHT_MODES:
            raise ValueError(f"weights {self.weights!r}: expected one of {WEIGHT_MODES}")

    def torch_dtype(self):
        """The torch dtype of ``dtype``; the reference's float16 is named so that a user of it
        knows why it is refused (clockwork/config.py:26-31)."""
        import torch

        names = {"float32": torch.float32, "bfloat16": torch.bfloat16}
        if self.dtype == "float16":
            raise ValueError("dtype 'float16' is not built in this engine; use 'bfloat16' or 'float32'")
        try:
            return names[self.dtype]
        except KeyError:
            raise ValueError(f"unknown dtype {self.dtype!r}, expected one of {tuple(names)}") from None


@dataclass
class CacheConfig:
    """Paged cache sizing (clockwork/config.py:34-39). ``num_blocks`` is pages per layer group;
    0 leaves it to the engine: ``memory_fraction`` of the device memory that is free once the
    weights are loaded, capped at twice what ``max_num_seqs`` requests of ``max_model_len``
    tokens can hold (the second half is room for cached prefixes)."""

    block_size: int = 16
    num_blocks: int = 512
    memory_fraction: float = 0.8
    enable_prefix_cache: bool = True
    watermark: float = 0.01


@dataclass
class SchedulerConfig:
    """Batching limits (clockwork/config.py:42-47) plus chunked prefill.

    ``max_prefill_chunk`` caps the tokens one request contributes to a step
    (only with chunked prefill on); 0 means "as many as the token budget allows". With
    ``enable_chunked_prefill`` off a prompt is admitted only whole, as in the
    reference (clockwork/scheduler/scheduler.py:120-146).
    """

    max_num_seqs: int = 64
    max_num_batched_tokens: int = 2048
    max_model_len: int = 4096
    preemption_mode: str = "recompute"
    enable_chunked_prefill: bool = True
    max_prefill_chunk: int = 0
    # decide a decode-only step while the step before it still runs on the GPU
    lookahead: bool = True


@dataclass
class EngineConfig:
    model: ModelConfig
    cache: CacheConfig = field(default_factory=CacheConfig)
    scheduler: SchedulerConfig = field(default_factory=SchedulerConfig)

    def sections(self) -> dict:
        """Section name -> its dataclass instance, in the order a key is looked up."""
        return {"model": self.model, "cache": self.cache, "scheduler": self.scheduler}

    @classmethod
    def from_yaml(cls, path: str | Path) -> "EngineConfig":
        """A file with the sections ``model:`` (which must name the model), ``cache:`` and
        ``scheduler:`` (clockwork/config.py:57-68). The reference's top-level
        ``attention_backend`` key is accepted and ignored."""
        loaded = yaml.safe_load(Path(path).read_text(encoding="utf-8"))
        loaded = {} if loaded is None else dict(loaded)
        loaded.pop("attention_backend", None)
        model_section = loaded.pop("model", None)
        if not (isinstance(model_section, dict) and "model" in model_section):
            raise ValueError(f"{path}: expected a top-level 'model' section naming the model")
        kinds = {"cache": CacheConfig, "scheduler": SchedulerConfig}
        strangers = sorted(set(loaded) - set(kinds))
        if strangers:
            raise ValueError(f"{path}: unknown top-level sections {strangers}")
        rest = {name: kind(**(loaded.get(name) or {})) for name, kind in kinds.items()}
        return cls(model=ModelConfig(**model_section), **rest)

    @classmethod
    def defaults(cls, model: str, **overrides) -> "EngineConfig":
        """Defaults plus keyword overrides routed by field name (clockwork/config.py:70-87)."""
        cfg = cls(model=ModelConfig(model=model))
        for key, value in overrides.items():
            cfg.set(key, value)
        return cfg

    def set(self, key: str, value) -> None:
        """Set ``key`` in every section that has a field of that name; a key that no section has
        is an error. ``max_model_len`` is a field of the model and of the scheduler section and
        changes in both, as in the reference (clockwork/config.py:76-86)."""
        hits = 0
        for section in self.sections().values():
            if any(f.name == key for f in fields(section)):
                previous = getattr(section, key)
                setattr(section, key, value)
                check = getattr(section, "__post_init__", None)
                if check is not None:
                    try:
                        check()
                    except ValueError:
                        setattr(section, key, previous)
                        raise
                hits += 1
        if hits == 0:
            raise ValueError(f"unknown config override {key!r}")

    def apply_overrides(self, pairs: list[str]) -> None:
        """``KEY=VALUE`` strings, the value read as YAML (scripts/serve.py:13-30)."""
        for pair in pairs:
            key, sep, raw = pair.partition("=")
            if not sep:
                raise ValueError(f"override {pair!r} is not KEY=VALUE")
            self.set(key, yaml.safe_load(raw))
