"""What can be done to a checkpoint tensor between the file and the parameter it fills.

A :class:`WeightTarget` names its steps as tuples, ``("transpose",)`` or ``("split_rows", i, n)``;
this registry maps the names to functions ``fn(tensor, *args) -> tensor``. A function must work
on a tensor of any device, the "meta" device included: the loader runs it on an empty meta tensor
to learn the shape it yields before anything is read.
"""

from __future__ import annotations

from typing import Callable, Optional

_TRANSFORMS: dict[str, Callable] = {}


def register_transform(name: str, fn: Callable) -> None:
    """``fn(tensor, *args) -> tensor`` under ``name``; an architecture's module may add its own
    (a de-interleave of rotary pairs, say) without touching the loader."""
    _TRANSFORMS[name] = fn


def _transpose(t):
    if t.dim() != 2:
        raise ValueError(f"'transpose' takes a matrix, got a tensor of shape {tuple(t.shape)}")
    return t.t()


def _split_rows(t, index: int, parts: int):
    if parts < 1 or not 0 <= index < parts or t.shape[0] % parts:
        raise ValueError(f"'split_rows' {index} of {parts} does not divide {t.shape[0]} rows")
    rows = t.shape[0] // parts
    return t[index * rows : (index + 1) * rows]


register_transform("transpose", _transpose)
register_transform("split_rows", _split_rows)


def steps_of(transform: Optional[tuple]) -> tuple:
    """A target's ``transform`` as a tuple of steps: one step (its first element is a name) or several."""
    if not transform:
        return ()
    if isinstance(transform[0], str):
        return (tuple(transform),)
    return tuple(tuple(step) for step in transform)


def apply_transform(transform: Optional[tuple], tensor):
    for name, *args in steps_of(transform):
        fn = _TRANSFORMS.get(name)
        if fn is None:
            raise KeyError(f"no weight transform is registered under {name!r} (known: {sorted(_TRANSFORMS)})")
        tensor = fn(tensor, *args)
    return tensor


def transformed_shape(transform: Optional[tuple], shape) -> tuple:
    """The shape that a checkpoint tensor of ``shape`` has after ``transform``."""
    if not transform:
        return tuple(shape)
    import torch

    return tuple(apply_transform(transform, torch.empty(tuple(shape), device="meta")).shape)
