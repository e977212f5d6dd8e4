"""The HIP libraries: no execution path without them, and clear errors on the way to them."""

import pytest

from clockwork_amd import ops
from clockwork_amd.csrc import build


def test_head_sizes_outside_the_kernels_range_are_refused_by_name():
    for hd in (8, 24, 272):
        with pytest.raises(ValueError, match="head sizes in steps of 16"):
            build.library_path("attention", hd)
    with pytest.raises(KeyError):
        build.library_path("no_such_library")


def test_a_library_that_cannot_be_built_is_an_error_not_a_fallback(monkeypatch):
    """Nothing is built and there is no compiler: the first op that needs a library raises."""
    monkeypatch.setattr(build, "_find_built", lambda name, head_dim: None)
    monkeypatch.setenv("HIPCC", "/nonexistent/hipcc")
    monkeypatch.setattr(build.shutil, "which", lambda name: None)
    monkeypatch.setattr(build.Path, "exists", lambda self: False)
    monkeypatch.setattr(ops, "_libs", {})
    with pytest.raises(RuntimeError, match="hipcc was not found"):
        ops._load("core")


def test_a_library_that_does_not_load_is_an_error(monkeypatch, tmp_path):
    broken = tmp_path / "core-broken.so"
    broken.write_bytes(b"not a shared object")
    monkeypatch.setattr(build, "ensure_built", lambda name, head_dim=None: broken)
    monkeypatch.setattr(ops, "_libs", {})
    with pytest.raises(ops.KernelError, match="cannot load the HIP library"):
        ops._load("core")


def test_the_digest_follows_the_source_and_the_flags(monkeypatch):
    before = build.library_path("core").name
    monkeypatch.setattr(build, "FLAGS", build.FLAGS + ["-DSOMETHING_ELSE"])
    assert build.library_path("core").name != before


def test_the_target_rules_xnack_out_unless_told_otherwise(monkeypatch):
    monkeypatch.delenv("CLOCKWORK_AMD_ARCH", raising=False)
    assert build.target_arch() in ("gfx950:xnack-", "gfx950")  # the latter only on a card with XNACK on
    monkeypatch.setenv("CLOCKWORK_AMD_ARCH", "gfx950")
    assert build.target_arch() == "gfx950"
    assert "--offload-arch" not in " ".join(build.FLAGS)  # the target is added per compile
