"""Index of a model folder's safetensors files: tensor name -> file, shape, stored dtype.

Every ``*.safetensors`` file of the folder is read, sorted by name, as the
reference does (clockwork/engine/loader.py:47-54); no index file is consulted.
Only headers are parsed here; tensors are read one at a time by the loader.
"""

from __future__ import annotations

import json
import struct
from dataclasses import dataclass
from pathlib import Path


class WeightMismatchError(RuntimeError):
    """The checkpoint does not hold exactly the tensors the model needs."""

    def __init__(self, missing, unexpected, wrong_shape):
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        super().__init__(
            "state dict mismatch: "
            f"missing={self.missing} unexpected={self.unexpected} wrong_shape={self.wrong_shape}"
        )


@dataclass(frozen=True)
class TensorEntry:
    file: Path
    shape: tuple[int, ...]
    dtype: str  # safetensors dtype tag: "BF16", "F32", "I64", ...


def _read_header(path: Path) -> dict:
    with open(path, "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        return json.loads(f.read(n))


class CheckpointIndex:
    def __init__(self, model_dir: str | Path) -> None:
        self.model_dir = Path(model_dir)
        files = sorted(self.model_dir.glob("*.safetensors"))
        if not files:
            raise FileNotFoundError(f"no .safetensors files in {self.model_dir}")
        self.entries: dict[str, TensorEntry] = {}
        for file in files:
            for name, meta in _read_header(file).items():
                if name == "__metadata__":
                    continue
                self.entries[name] = TensorEntry(file, tuple(meta["shape"]), meta["dtype"])
        self._open: dict[Path, object] = {}

    def names(self) -> list[str]:
        return list(self.entries)

    def __contains__(self, name: str) -> bool:
        return name in self.entries

    def read(self, name: str):
        """One tensor, on the CPU, in its stored dtype."""
        from safetensors import safe_open

        entry = self.entries[name]
        handle = self._open.get(entry.file)
        if handle is None:
            handle = safe_open(str(entry.file), framework="pt", device="cpu")
            self._open[entry.file] = handle
        return handle.get_tensor(name)

    def close(self) -> None:
        self._open.clear()
