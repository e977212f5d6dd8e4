"""Compile the HIP sources for gfx950 into shared libraries, in-tree, on demand.

Each source becomes one library ``_build/<name>-<hash>.so``; the hash covers the
source text, the headers beside it and the compiler flags, so a changed source is
never served by a stale library. The attention source is built once per head
size (``-DCW_HD=<n>``): a model compiles only the size it needs. Libraries are
plain C ABI (no Python or torch headers), loaded with ctypes.

``ensure_built`` compiles only what is missing and prints a line now and then
while hipcc runs; ``build_all`` recompiles everything (the build check).
"""

from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

CSRC = Path(__file__).resolve().parent
ARCH = "gfx950"


def target_arch() -> str:
    """The offload target: gfx950 with XNACK (page-fault replay) ruled out, which is how these
    cards run and lets the compiler schedule loads more freely; plain gfx950 (code that runs
    either way) only where the card at hand says it has XNACK on. ``CLOCKWORK_AMD_ARCH`` overrides."""
    override = os.environ.get("CLOCKWORK_AMD_ARCH")
    if override:
        return override
    torch = sys.modules.get("torch")
    try:
        if torch is not None and torch.cuda.is_available():
            name = torch.cuda.get_device_properties(torch.cuda.current_device()).gcnArchName
            if "xnack+" in name:
                return ARCH
    except Exception:  # no usable card here: cross-compiling
        pass
    return f"{ARCH}:xnack-"


FLAGS = [
    "-O3",
    "-std=c++17",
    "-shared",
    "-fPIC",
    "-fvisibility=hidden",
    # hipcc -O3 forms packed float32 instructions by itself; they are kept out of these kernels
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # the first kernel arguments arrive in scalar registers with the wave instead of by a load
    # from the argument buffer: a short kernel's first addresses are ready that much sooner
    "-mllvm", "-amdgpu-kernarg-preload-count=16",
]
PLAIN_SOURCES = {"core": "core.hip", "gemm": "gemm.hip", "gemm_tile": "gemm_tile.hip", "sampling": "sampling.hip"}
ATTENTION_SOURCE = "attention.hip"
# head sizes compiled by build_all: the tests' models, the kernel tests and the benchmark's
DEFAULT_HEAD_DIMS = (16, 32, 48, 64, 96, 128, 160, 224, 256)


def _log(msg: str) -> None:
    print(f"[clockwork_amd] {msg}", file=sys.stderr, flush=True)


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and Path(cand).exists():
            return cand
    raise RuntimeError(
        "hipcc was not found (looked at $HIPCC, PATH and /opt/rocm/bin): the HIP kernels "
        "cannot be compiled and there is no other execution path"
    )


def build_dir() -> Path:
    """In-tree ``_build`` when it can be written, else a per-user folder under the temp dir."""
    override = os.environ.get("CLOCKWORK_AMD_BUILD_DIR")
    cands = [Path(override)] if override else []
    cands.append(CSRC / "_build")
    cands.append(Path(tempfile.gettempdir()) / f"clockwork_amd_build_{os.getuid()}")
    for d in cands:
        try:
            d.mkdir(parents=True, exist_ok=True)
            probe = d / f".probe_{os.getpid()}"
            probe.write_text("")
            probe.unlink()
            return d
        except OSError:
            continue
    raise RuntimeError(f"no writable build folder among {[str(c) for c in cands]}")


def _spec(name: str, head_dim: int | None) -> tuple[str, Path, list[str]]:
    if name == "attention":
        if head_dim is None or head_dim % 16 or not 16 <= head_dim <= 256:
            raise ValueError(
                f"attention kernels take head sizes in steps of 16 from 16 to 256, got {head_dim}"
            )
        return f"attention_hd{head_dim}", CSRC / ATTENTION_SOURCE, [f"-DCW_HD={head_dim}"]
    if name not in PLAIN_SOURCES:
        raise KeyError(f"unknown kernel library {name!r}")
    return name, CSRC / PLAIN_SOURCES[name], []


def _digest(src: Path, defines: list[str]) -> str:
    h = hashlib.sha256()
    h.update(src.read_bytes())
    for header in sorted(CSRC.glob("*.h")):
        h.update(header.read_bytes())
    h.update(" ".join([f"--offload-arch={target_arch()}"] + FLAGS + defines).encode())
    return h.hexdigest()[:12]


def library_path(name: str, head_dim: int | None = None, directory: Path | None = None) -> Path:
    stem, src, defines = _spec(name, head_dim)
    return (directory or build_dir()) / f"{stem}-{_digest(src, defines)}.so"


def _find_built(name: str, head_dim: int | None) -> Path | None:
    """A current library in the in-tree folder or the fallback folder, if either holds one."""
    stem, src, defines = _spec(name, head_dim)
    fname = f"{stem}-{_digest(src, defines)}.so"
    for d in (CSRC / "_build", Path(tempfile.gettempdir()) / f"clockwork_amd_build_{os.getuid()}"):
        if (d / fname).is_file():
            return d / fname
    override = os.environ.get("CLOCKWORK_AMD_BUILD_DIR")
    if override and (Path(override) / fname).is_file():
        return Path(override) / fname
    return None


def _compile(name: str, head_dim: int | None, out: Path) -> Path:
    stem, src, defines = _spec(name, head_dim)
    tmp = out.with_suffix(f".tmp{os.getpid()}.so")
    cmd = [_hipcc(), f"--offload-arch={target_arch()}", *FLAGS, *defines, "-I", str(CSRC), "-o", str(tmp), str(src)]
    t0 = time.time()
    _log(f"compiling {stem} for {target_arch()} ...")
    env = dict(os.environ)
    env.setdefault("HOME", tempfile.gettempdir())
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env)
    while True:
        try:
            output, _ = proc.communicate(timeout=15)
            break
        except subprocess.TimeoutExpired:
            _log(f"still compiling {stem} ({time.time() - t0:.0f} s)")
    if proc.returncode != 0:
        tmp.unlink(missing_ok=True)
        raise RuntimeError(f"hipcc failed for {src.name} ({' '.join(cmd)}):\n{output}")
    os.replace(tmp, out)
    # older builds of the same library are of no use any more
    for old in out.parent.glob(f"{stem}-*.so"):
        if old != out and ".tmp" not in old.name:
            old.unlink(missing_ok=True)
    _log(f"compiled {stem} in {time.time() - t0:.0f} s -> {out}")
    return out


def ensure_built(name: str, head_dim: int | None = None) -> Path:
    """Path of a current library, compiling it first if none is there."""
    found = _find_built(name, head_dim)
    if found is not None:
        return found
    return _compile(name, head_dim, library_path(name, head_dim))


def ensure_many(jobs: list[tuple[str, int | None]]) -> dict[tuple[str, int | None], Path]:
    """Like ``ensure_built`` for several libraries, missing ones compiled side by side."""
    jobs = list(dict.fromkeys(jobs))
    missing = [j for j in jobs if _find_built(*j) is None]
    if missing:
        directory = build_dir()
        with ThreadPoolExecutor(max_workers=min(len(missing), 8)) as pool:
            list(pool.map(lambda j: _compile(j[0], j[1], library_path(j[0], j[1], directory)), missing))
    return {j: _find_built(*j) for j in jobs}


def build_all(head_dims=DEFAULT_HEAD_DIMS) -> list[Path]:
    """Compile every library anew (also where a built one is there)."""
    directory = build_dir()
    jobs: list[tuple[str, int | None]] = [(n, None) for n in PLAIN_SOURCES]
    jobs += [("attention", hd) for hd in head_dims]
    with ThreadPoolExecutor(max_workers=min(len(jobs), 8)) as pool:
        return list(pool.map(lambda j: _compile(j[0], j[1], library_path(j[0], j[1], directory)), jobs))


if __name__ == "__main__":
    for path in build_all():
        print(path)
