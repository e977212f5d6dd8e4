"""Python face of the HIP libraries: shape and type checks on the host, then one C call.

Every function takes torch tensors that live on the GPU, checks what the kernel
and its grid assume (so a wrong shape is an exception here, never an
out-of-bounds access there) and launches on torch's current stream. There is no
other implementation behind these functions: if a library cannot be built or
loaded the call raises.
"""

from __future__ import annotations

import contextlib
import ctypes
import gc
import hashlib
import json
import os
import tempfile
from ctypes import c_float, c_int, c_int64, c_void_p

import torch

from clockwork_amd.csrc import build

F32, BF16 = 0, 1
_ERRORS = {
    -1: "an argument the kernel does not take",
    -2: "an element type the kernel is not built for",
    -3: "the HIP runtime refused the launch",
    -4: "a size beyond the kernel's stated maximum",
}


class KernelError(RuntimeError):
    pass


def _check(code: int, what: str) -> None:
    if code != 0:
        raise KernelError(f"{what}: {_ERRORS.get(code, f'error {code}')}")


def dtype_code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return F32
    if dtype == torch.bfloat16:
        return BF16
    raise KernelError(f"the kernels take float32 and bfloat16 tensors, not {dtype}")


_libs: dict = {}


def _load(name: str, head_dim: int | None = None) -> ctypes.CDLL:
    key = (name, head_dim)
    lib = _libs.get(key)
    if lib is None:
        path = build.ensure_built(name, head_dim)
        try:
            lib = ctypes.CDLL(str(path))
        except OSError as e:
            raise KernelError(f"cannot load the HIP library {path}: {e}") from e
        _declare(name, lib)
        _libs[key] = lib
    return lib


def preload(libraries=(), tiled_products: bool = False, sampling: bool = False) -> None:
    """Build (side by side, if several are missing) and load what a model runs: the common
    kernels, the products and the ``libraries`` its parts name, as (name, head size or None)
    pairs, e.g. ("attention", 128); the tiled products (a bfloat16 model's gate/up product of a
    long portion, and every large product with ``hip_products``) and the sampling kernels only for
    a caller that uses them."""
    jobs = [("core", None), ("gemm", None)]
    if tiled_products:
        jobs.append(("gemm_tile", None))
    if sampling:
        jobs.append(("sampling", None))
    for name, head_dim in libraries:
        job = (str(name), None if head_dim is None else int(head_dim))
        if job not in jobs:
            jobs.append(job)
    build.ensure_many(jobs)
    for name, hd in jobs:
        _load(name, hd)


def loaded_libraries() -> list[str]:
    return sorted(str(lib._name) for lib in _libs.values())


def _declare(name: str, lib: ctypes.CDLL) -> None:
    P, I, L, F = c_void_p, c_int, c_int64, c_float
    sigs = {
        "core": {
            "cw_embedding": [P, I, P, P, I, I, I, P],
            "cw_add_rmsnorm": [P, P, P, I, I, P, I, F, P, I, P, I, I, P],
            "cw_rope_kv_write": [P, I, P, I, P, P, P, I, I, I, I, I, P, P, L, P],
            "cw_silu_mul": [P, P, I, I, I, P],
            "cw_copy_pages": [P, I, L, L, P, I, P],
            "cw_fresh_state_rows": [P, I, I, I, I, L, P, P, I, P],
            "cw_bf16_to_f32": [P, P, L, P],
        },
        "gemm": {
            "cw_gemm_f32": [P, L, P, P, P, L, I, I, I, P, L, P],
            "cw_gemm_f32_workspace_floats": [I, I, I],
            "cw_gemm_bf16_skinny": [I, P, L, P, P, L, I, I, I, I, P],
            "cw_gemm_bf16_skinny_ksplits": [I, I, I],
            "cw_gemm_bf16_skinny_fast": [I, I, I, I],
            "cw_gemm_bf16_swiglu_normed_ok": [I, I, I],
            "cw_gemm_bf16_swiglu_normed": [P, P, P, I, F, P, P, L, I, I, I, P],
            "cw_gemm_qkv_rope_bf16": [P, L, P, P, I, P, P, P, P, P, P, L, I, I, I, I, I, P],
        },
        "gemm_tile": {
            "cw_gemm_bf16_tiled": [I, P, L, P, P, I, P, L, I, I, I, P],
            "cw_gemm_bf16_wide_tiles": [I, I, I, I, L],
            "cw_gemm_bf16_wide": [I, P, L, P, P, I, P, L, I, I, I, I, P],
            "cw_gemm_bf16_wide_partial_ok": [I, I, I, L, I],
            "cw_gemm_bf16_wide_partial": [P, L, P, P, L, I, I, I, I, I, P],
        },
        "sampling": {
            "cw_argmax_chunks": [I],
            "cw_argmax": [P, L, I, I, P, P, L, P],
            "cw_argmax_static_init": [],
            "cw_argmax_static": [P, L, I, I, P, P],
            "cw_sample": [P, L, I, I, P, P, P, P, P, P, P, L, I, P],
            "cw_sample_workspace_bytes": [I, I],
        },
        "attention": {
            "cw_attention_head_dim": [],
            "cw_attention_workspace_floats": [I, I, I, I, I],
            "cw_attention": [I, I, P, L, P, L, P, P, P, I, P, P, P, I, I, I, I, I, I, I, F, P, L, P],
            "cw_attention_prefill_supported": [],
            "cw_attention_prefill_bf16": [P, L, P, L, P, P, P, I, P, P, P, I, I, I, I, I, F, P, I, I, P, L, P],
            "cw_attention_prefill_workspace_floats": [I, I, I, I],
            "cw_attention_prefill_row_blocks_ok": [I],
            "cw_attention_decode_supported": [],
            "cw_attention_decode_gh": [I],
            "cw_attention_decode_max_splits": [],
            "cw_attention_decode_workspace_floats": [I, I, I, I],
            "cw_attention_decode_bf16": [P, L, P, L, P, P, P, I, P, P, P, I, I, I, I, I, I, F, P, L, P, I, I, I, P],
        },
    }[name]
    for fn, argtypes in sigs.items():
        f = getattr(lib, fn)
        f.argtypes = argtypes
        f.restype = c_int64 if fn.endswith(("workspace_floats", "workspace_bytes")) else c_int


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> int:
    """The current HIP stream's handle (also the capture stream inside a graph capture). Asked
    for at every launch, so through torch's raw accessor where there is one: a tenth of the cost
    of building a Stream object."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _ptr(t) -> int | None:
    return None if t is None else t.data_ptr()


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise KernelError(msg)


def _gpu(*tensors) -> None:
    for t in tensors:
        if t is not None and not (t.is_cuda and t.is_contiguous()):
            raise KernelError("kernel arguments must live on the GPU and be contiguous")


def _i32(t, n: int | None, what: str) -> None:
    if not (t.dtype == torch.int32 and t.dim() == 1):
        raise KernelError(f"{what} must be a 1-d int32 tensor")
    if n is not None:
        if not (t.numel() >= n):
            raise KernelError(f"{what} holds {t.numel()} entries, {n} needed")


# ---------------------------------------------------------------------------------------------
def embedding(table: torch.Tensor, ids: torch.Tensor, out_resid: torch.Tensor) -> torch.Tensor:
    """out_resid[t] = float32(table[ids[t]]); out_resid is [T, H] float32."""
    _gpu(table, ids, out_resid)
    T = ids.numel()
    V, H = table.shape
    _i32(ids, T, "ids")
    if not (out_resid.dtype == torch.float32 and tuple(out_resid.shape) == (T, H)):
        raise KernelError("residual must be [T, H] float32")
    _check(
        _load("core").cw_embedding(_ptr(table), dtype_code(table.dtype), _ptr(ids), _ptr(out_resid), T, H, V, _stream()),
        "embedding",
    )
    return out_resid


class PartialSums:
    """A product whose K loop was split over workgroups: ``parts`` is float32 [splits, M, N] and the
    value is their sum, taken in order by whoever reads it next (``add_rmsnorm`` does)."""

    __slots__ = ("parts",)

    def __init__(self, parts: torch.Tensor) -> None:
        self.parts = parts

    @property
    def shape(self):
        return self.parts.shape[1:]

    def sum(self, dtype=None) -> torch.Tensor:
        total = self.parts[0].clone()
        for i in range(1, self.parts.shape[0]):
            total += self.parts[i]
        return total if dtype is None else total.to(dtype)


_row_indices: dict = {}


def _all_rows(n: int, device) -> torch.Tensor:
    """int32 [0, n) on ``device`` (kept: a HIP graph may hold its address)."""
    t = _row_indices.get((n, device))
    if t is None:
        t = _row_indices[(n, device)] = torch.arange(n, dtype=torch.int32, device=device)
    return t


class PendingPair:
    """Two branch outputs that are both still to be added to the residual stream, ``first``
    before ``second``: what a block hands on when its second norm ran inside the feed-forward's
    product kernel (which writes no residual). ``first`` is a tensor in the activation type,
    ``second`` a tensor or :class:`PartialSums`."""

    __slots__ = ("first", "second")

    def __init__(self, first, second) -> None:
        self.first = first
        self.second = second


class LazyAddNorm:
    """rmsnorm(resid + delta) * weight, not computed yet: a consumer that can make it inside its
    own kernel takes the pieces, any other calls :meth:`value`. The residual is not updated
    either way: ``delta`` stays pending."""

    __slots__ = ("resid", "delta", "weight", "eps", "dtype")

    def __init__(self, resid, delta, weight, eps: float, dtype) -> None:
        self.resid, self.delta, self.weight, self.eps, self.dtype = resid, delta, weight, eps, dtype

    @property
    def shape(self):
        return self.resid.shape

    def value(self) -> torch.Tensor:
        out = torch.empty(tuple(self.resid.shape), dtype=self.dtype, device=self.resid.device)
        return add_rmsnorm(self.resid, self.delta, self.weight, self.eps, out, write_back=False)


def add_rmsnorm(resid, delta, weight, eps: float, out, rows=None, write_back: bool = True) -> torch.Tensor:
    """resid += delta (when given), out = rmsnorm(resid) * weight; with ``rows`` only those rows
    are normed into out[i] and resid is left alone, as it is with ``write_back`` off. resid
    float32 [T, H]; delta/out in the activation type, or delta a :class:`PartialSums` of that
    shape, or a :class:`PendingPair` (both are added, ``first`` first)."""
    delta0 = None
    if isinstance(delta, PendingPair):
        delta0, delta = delta.first, delta.second
    if not write_back and rows is None:
        rows = _all_rows(resid.shape[0], resid.device)
    parts = 0
    if isinstance(delta, PartialSums):
        parts = delta.parts.shape[0]
        delta = delta.parts
    _gpu(resid, delta, delta0, weight, out, rows)
    T, H = resid.shape
    if not (resid.dtype == torch.float32):
        raise KernelError("the residual stream is float32")
    if delta0 is not None:
        if not (tuple(delta0.shape) == (T, H) and delta0.dtype == out.dtype):
            raise KernelError("the first pending delta must be [T, H] in the activation type")
    n = T if rows is None else rows.numel()
    if rows is not None:
        _i32(rows, n, "rows")
    if not (tuple(out.shape) == (n, H)):
        raise KernelError(f"out must be [{n}, {H}]")
    if not (weight.numel() == H):
        raise KernelError("norm weight has the wrong size")
    if parts:
        if not (tuple(delta.shape) == (parts, T, H) and delta.dtype == torch.float32):
            raise KernelError("partial sums must be float32 [parts, T, H]")
    elif delta is not None:
        if not (tuple(delta.shape) == (T, H) and delta.dtype == out.dtype):
            raise KernelError("delta must be [T, H] in the activation type")
    _check(
        _load("core").cw_add_rmsnorm(
            _ptr(resid), _ptr(delta0), _ptr(delta), parts, T, _ptr(weight), dtype_code(weight.dtype), float(eps), _ptr(out),
            dtype_code(out.dtype), _ptr(rows), n, H, _stream()),
        "add_rmsnorm",
    )
    return out


def rope_kv_write(qkv, bias, positions, slots, inv_freq, rotary_dim: int, nh: int, nkv: int, hd: int,
                  k_cache, v_cache) -> None:
    """Add the bias, rotate q (in place) and k, write k and v rows to the cache at ``slots``.

    qkv [T, (nh + 2 nkv) hd]; k_cache/v_cache [rows, nkv, hd] flat over pages; slots int32 [T]
    (None: nothing is cached, for a mixer that reads another's cache: then nkv must be 0)."""
    _gpu(qkv, bias, positions, slots, inv_freq, k_cache, v_cache)
    T = qkv.shape[0]
    width = (nh + 2 * nkv) * hd
    if not (qkv.dim() == 2 and qkv.shape[1] == width):
        raise KernelError(f"qkv must be [T, {width}]")
    _i32(positions, T, "positions")
    cache_rows = 0
    if slots is not None:
        _i32(slots, T, "slots")
        if not (k_cache is not None and v_cache is not None):
            raise KernelError("slots without a cache")
        if not (k_cache.dtype == qkv.dtype and v_cache.dtype == qkv.dtype):
            raise KernelError("cache and activations differ in type")
        if not (tuple(k_cache.shape[-2:]) == (nkv, hd) and k_cache.shape == v_cache.shape):
            raise KernelError("cache must be [..., nkv, hd]")
        cache_rows = k_cache.numel() // (nkv * hd)
    else:
        if not (nkv == 0):
            raise KernelError("keys and values need slots to be written to")
    if bias is not None:
        if not (bias.numel() == width):
            raise KernelError("qkv bias has the wrong size")
    if inv_freq is not None:
        if not (inv_freq.dtype == torch.float32 and inv_freq.numel() == rotary_dim // 2):
            raise KernelError("inv_freq must be float32 [rotary_dim / 2]")
    else:
        rotary_dim = 0
    _check(
        _load("core").cw_rope_kv_write(
            _ptr(qkv), dtype_code(qkv.dtype), _ptr(bias), dtype_code(bias.dtype) if bias is not None else 0,
            _ptr(positions), _ptr(slots), _ptr(inv_freq), int(rotary_dim), T, nh, nkv, hd,
            _ptr(k_cache), _ptr(v_cache), cache_rows, _stream()),
        "rope_kv_write",
    )


def silu_mul(gate_up: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[t, i] = silu(gate_up[t, i]) * gate_up[t, I + i]."""
    _gpu(gate_up, out)
    T, two_i = gate_up.shape
    if not (two_i % 2 == 0 and tuple(out.shape) == (T, two_i // 2) and out.dtype == gate_up.dtype):
        raise KernelError("silu_mul shapes")
    _check(_load("core").cw_silu_mul(_ptr(gate_up), _ptr(out), dtype_code(out.dtype), T, two_i // 2, _stream()), "silu_mul")
    return out


def copy_pages(pool: torch.Tensor, pairs: torch.Tensor) -> None:
    """pool [planes, num_blocks, ...]: for each (src, dst) row of ``pairs`` copy page src to dst in every plane."""
    _gpu(pool, pairs)
    planes, num_blocks = pool.shape[0], pool.shape[1]
    block_bytes = pool[0, 0].numel() * pool.element_size()
    if not (pairs.dtype == torch.int32 and pairs.dim() == 2 and pairs.shape[1] == 2):
        raise KernelError("pairs must be int32 [n, 2]")
    _check(_load("core").cw_copy_pages(_ptr(pool), planes, num_blocks, block_bytes, _ptr(pairs), pairs.shape[0], _stream()), "copy_pages")


def fresh_state_rows(pool: torch.Tensor, slots: torch.Tensor, starts: torch.Tensor, n: int) -> None:
    """pool [entries, slots, ...], its last slot the template of a fresh state: for each of the
    first ``n`` requests of a step that starts at position 0 (``starts[r] == 0``), set row
    ``slots[r]`` to the template in every entry; a slot outside [0, slots - 1) writes nothing. A
    kernel, so a captured step may hold it."""
    _gpu(pool, slots, starts)
    _i32(slots, n, "slots")
    _i32(starts, n, "starts")
    if pool.dim() < 2 or pool.shape[1] < 2:
        raise KernelError("a state pool is [entries, slots, ...] with the template as its last slot")
    row_bytes = (pool[0, 0].numel() if pool.dim() > 2 else 1) * pool.element_size()
    pool_slots = pool.shape[1]
    _check(_load("core").cw_fresh_state_rows(_ptr(pool), pool.shape[0], pool_slots, pool_slots - 1, pool_slots - 1,
                                             row_bytes, _ptr(slots), _ptr(starts), int(n), _stream()), "fresh_state_rows")


def linear(x: torch.Tensor, weight: torch.Tensor, bias=None, out_dtype=None, partial_ok: bool = False,
           policy: "ProductPolicy | None" = None):
    """y = x @ weight.T (+ bias). float32: the true-float32 HIP product. bfloat16: few rows go
    through the weight-streaming kernel, many through the library product (as the reference's
    engine uses one) or, where ``policy`` (the calling engine's :class:`ProductPolicy`) says so,
    through this package's tiled kernels; float32 accumulation either way. With ``partial_ok``
    the result may come back as :class:`PartialSums` (a narrow output with a long K, few rows):
    only for a result that goes straight into ``add_rmsnorm``."""
    policy = policy if policy is not None else DEFAULT_POLICY
    _gpu(x, weight, bias)
    M, K = x.shape
    N = weight.shape[0]
    if not (weight.shape[1] == K):
        raise KernelError(f"weight is {tuple(weight.shape)}, input has {K} columns")
    if x.dtype == torch.float32:
        if not (weight.dtype == torch.float32):
            raise KernelError("a float32 product needs float32 weights")
        out = torch.empty((M, N), dtype=torch.float32, device=x.device)
        if bias is not None:
            if not (bias.dtype == torch.float32 and bias.numel() == N):
                raise KernelError("bias must be float32 [N]")
        lib = _load("gemm")
        # a narrow output with a long K is summed in parts over K (the same parts whatever M is)
        need = lib.cw_gemm_f32_workspace_floats(M, N, K)
        parts = torch.empty(need, dtype=torch.float32, device=x.device) if need else None
        _check(lib.cw_gemm_f32(_ptr(x), K, _ptr(weight), _ptr(bias), _ptr(out), N, M, N, K, _ptr(parts), need, _stream()),
               "gemm_f32")
        return out
    if not (x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16):
        raise KernelError("a bfloat16 product needs bfloat16 operands")
    if M <= STREAM_MAX_ROWS and K % 8 == 0 and bias is None:
        lib = _load("gemm")
        if partial_ok and out_dtype is None:
            splits = lib.cw_gemm_bf16_skinny_ksplits(M, N, K)
            chosen = 0
            if splits > 1 and M <= SKINNY_MAX_ROWS:
                # a tuning start-up has timed the split counts for this shape, or does so now
                if policy.tuning and (N, K) not in policy.k_split_choices and policy.recall("k_split_choices", (N, K)) is None:
                    policy.k_split_choices[(N, K)] = _measure_k_splits(x, weight, splits)
                chosen = policy.k_split_choices.get((N, K), 0)
                splits = chosen or splits
            if splits > 1:
                parts = torch.empty((splits, M, N), dtype=torch.float32, device=x.device)
                _check(lib.cw_gemm_bf16_skinny(3, _ptr(x), K, _ptr(weight), _ptr(parts), N, M, N, K, chosen, _stream()),
                       "gemm_bf16_skinny(partial)")
                return PartialSums(parts)
        want_f32 = out_dtype == torch.float32
        if lib.cw_gemm_bf16_skinny_fast(1 if want_f32 else 0, M, N, K):
            out = torch.empty((M, N), dtype=torch.float32 if want_f32 else torch.bfloat16, device=x.device)
            _check(lib.cw_gemm_bf16_skinny(1 if want_f32 else 0, _ptr(x), K, _ptr(weight), _ptr(out), N, M, N, K, 0, _stream()),
                   "gemm_bf16_skinny")
            return out
    if partial_ok and out_dtype is None and bias is None and M >= WIDE_PRODUCT_MIN_ROWS and x.is_contiguous():
        splits = _wide_partial_chosen(x, weight, policy)
        if splits:
            return linear_wide_partial(x, weight, splits)
    if policy.hip_products and K % 8 == 0 and x.is_contiguous():
        y = linear_tiled(x, weight, bias)
    elif _wide_product_chosen(x, weight, bias, policy):
        y = linear_tiled(x, weight, bias, wide=True)
    else:
        y = _library_product(x, weight, bias)
    if out_dtype == torch.float32:
        out = torch.empty((M, N), dtype=torch.float32, device=x.device)
        _check(_load("core").cw_bf16_to_f32(_ptr(y), _ptr(out), M * N, _stream()), "bf16_to_f32")
        return out
    return y


class ProductPolicy:
    """How one engine runs its products of many bfloat16 rows. Every runner has one of its own and
    hands it to the parts through the step context, so two engines in a process (other options,
    other weights) never see each other's choices.

    ``hip_products``: such products go through this package's own LDS-tiled kernels instead of the
    library (about half as fast on an MI355X; for a run that must not depend on the library).
    ``swiglu_choices`` / ``product_choices``: for a weight shape that a tuning start-up has timed
    both ways, whether the wide-tile kernel was the faster one ((rows of [gate; up], K) and
    (N, K, with bias)); shapes never timed follow the fixed rules. ``k_split_choices``: for an
    (N, K) whose product of few rows is summed in parts over K (a narrow output with a long K),
    the number of parts that start-up found the fastest, the same for every step of up to 16 rows.
    ``wide_partial_choices``: for an (N, K) of a long portion's product with a narrow output and a
    long K, into how many runs of K the wide-tile kernel sums it (0: the library's product stays).
    ``tuning``: such a start-up is under way (``library_tuning``)."""

    __slots__ = ("hip_products", "swiglu_choices", "product_choices", "k_split_choices", "wide_partial_choices", "tuning",
                 "_remembered")

    TABLES = ("swiglu_choices", "product_choices", "k_split_choices", "wide_partial_choices")

    def __init__(self, hip_products: bool = False) -> None:
        self.hip_products = bool(hip_products)
        self.swiglu_choices: dict = {}
        self.product_choices: dict = {}
        self.k_split_choices: dict = {}
        self.wide_partial_choices: dict = {}
        self.tuning = False
        self._remembered: dict = {name: {} for name in self.TABLES}

    def read_choices(self, path: str) -> int:
        """Remember what earlier start-ups on this card and kernel build measured and left in
        ``path``: a shape's entry comes into use when this engine's own start-up asks for that
        shape (``recall``), in place of measuring it again; other models' shapes stay aside. A file
        that is missing, unreadable or from another card or build is passed over. Returns the number
        of entries remembered."""
        try:
            with open(path) as f:
                record = json.load(f)
            if record.get("made_for") != _choices_made_for():
                return 0
            taken = 0
            for name in self.TABLES:
                for key, value in record.get(name, []):
                    self._remembered[name][tuple(key)] = value
                    taken += 1
            return taken
        except (OSError, ValueError, TypeError, AttributeError):
            return 0

    def recall(self, table: str, key):
        """What an earlier start-up measured for ``key`` of ``table``, put into use; None if
        nothing is remembered (or this policy holds a choice of its own already)."""
        active = getattr(self, table)
        if key in active or key not in self._remembered[table]:
            return None
        active[key] = self._remembered[table][key]
        return active[key]

    def write_choices(self, path: str) -> None:
        """Leave what is remembered and this policy's own choices (which win) in ``path``, written
        beside it and moved over it, so a reader never sees half a file; where the folder cannot be
        written nothing is kept."""
        record = {"made_for": _choices_made_for()}
        for name in self.TABLES:
            merged = {**self._remembered[name], **getattr(self, name)}
            record[name] = [[list(key), value] for key, value in merged.items()]
        try:
            fd, tmp = tempfile.mkstemp(dir=os.path.dirname(path) or ".", prefix=".choices-")
            with os.fdopen(fd, "w") as f:
                json.dump(record, f)
            os.replace(tmp, path)
        except OSError:
            pass


def choices_file() -> str:
    """Where a tuning start-up keeps what it measured for this package's own kernels: a file in
    the temporary folder, one per user and per card and kernel build (so that what one kind of
    card measured is never handed to, or overwritten by, another), or where
    CLOCKWORK_AMD_CHOICES_FILE points."""
    named = os.environ.get("CLOCKWORK_AMD_CHOICES_FILE")
    if named:
        return named
    mark = hashlib.sha256(json.dumps(_choices_made_for()).encode()).hexdigest()[:10]
    return os.path.join(tempfile.gettempdir(), f"clockwork_amd_choices_{os.getuid()}_{mark}.json")


def _choices_made_for() -> list:
    """What measured choices hold for: the card (its architecture, compute units and memory: the
    marketing name is empty under a profiler) and the builds of the kernels that were timed."""
    card = ["none"]
    if torch.cuda.is_available():
        props = torch.cuda.get_device_properties(torch.cuda.current_device())
        card = [str(getattr(props, "gcnArchName", props.name)), int(props.multi_processor_count), int(props.total_memory)]
    return card + [torch.__version__] + [build.library_path(n).name for n in ("gemm", "gemm_tile", "core")]


# what a call without an engine behind it runs by: the library for large products, nothing timed
DEFAULT_POLICY = ProductPolicy()


# up to this many rows every product goes through the weight-streaming kernels
SKINNY_MAX_ROWS = 16
# up to this many rows the shapes that the persistent streaming kernel takes do (the library
# product is faster for the others, measured)
STREAM_MAX_ROWS = 64
# the fused q/k/v kernel takes more than SKINNY_MAX_ROWS rows for weight matrices up to this many elements
FUSED_QKV_MAX_WEIGHTS = 8 << 20


def linear_tiled(x: torch.Tensor, weight: torch.Tensor, bias=None, swiglu: bool = False, wide=None) -> torch.Tensor:
    """y = x @ weight.T (+ bias), or with ``swiglu`` silu(x @ gate.T) * (x @ up.T) for weight =
    [gate; up], through the LDS-tiled matrix-core kernels for many bfloat16 rows (csrc/gemm_tile.hip):
    the one with 256 x 192 tiles where it takes the shape and has tiles enough to fill the GPU, the
    one with 128 x 128 tiles otherwise (``wide``: True or False to say which). The rows of x may
    have a stride (a slice of a wider buffer)."""
    _gpu(weight, bias)
    if not (x.is_cuda and x.dim() == 2):
        raise KernelError("x must be a 2-d tensor on the GPU")
    M, K = x.shape
    N = weight.shape[0]
    if not (x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16):
        raise KernelError("the tiled product is bfloat16")
    if not (weight.shape[1] == K and K % 8 == 0 and x.stride(1) == 1 and x.stride(0) % 8 == 0):
        raise KernelError("rows of 16-byte multiples")
    if not (not swiglu or (N % 2 == 0 and bias is None)):
        raise KernelError("gate_up weight must be [2 I, K], without bias")
    if bias is not None:
        if not (bias.numel() == N and bias.dtype in (torch.bfloat16, torch.float32)):
            raise KernelError("bias must be [N] bfloat16 or float32")
    out = torch.empty((M, N // 2 if swiglu else N), dtype=torch.bfloat16, device=x.device)
    lib = _load("gemm_tile")
    mode = 2 if swiglu else 0
    bias_f32 = int(bias is not None and bias.dtype == torch.float32)
    if wide is None:
        wide = lib.cw_gemm_bf16_wide_tiles(mode, M, N, K, x.stride(0)) >= WIDE_MIN_TILES
    if wide:
        _check(lib.cw_gemm_bf16_wide(mode, _ptr(x), x.stride(0), _ptr(weight), _ptr(bias), bias_f32, _ptr(out), out.shape[1],
                                     M, N, K, _compute_units(x.device), _stream()), "gemm_bf16_wide")
    else:
        _check(lib.cw_gemm_bf16_tiled(mode, _ptr(x), x.stride(0), _ptr(weight), _ptr(bias), bias_f32, _ptr(out), out.shape[1],
                                      M, N, K, _stream()), "gemm_bf16_tiled")
    return out


# the wide-tile kernel runs one workgroup per compute unit: with fewer tiles than this the
# 128 x 128 kernel, whose tiles are a quarter of the size, fills the GPU better
WIDE_MIN_TILES = 64
# The engine takes the wide-tile kernel for the gate/up product by itself (no ``hip_products``)
# where it beats the library product followed by the gate kernel. Measured on an MI355X over the
# Qwen2.5 layer shapes from 0.5B to 72B with 256 to 4096 rows: with 180 tiles or more (seven tenths
# of the compute units busy in the last round) and 1024 rows or more it is 5 to 25 % faster; with
# fewer rows the product is bound by reading W once, which the library does better for the large
# shapes (and 512 rows win only for the small ones). Against the library's TUNED choice it wins for
# the 0.5B, 1.5B, 3B, 14B and 32B shapes (the 1.5B shape's whole prefill step: 8.9 -> 7.9 ms) and
# loses 3 % of the step for the 7B and 72B shapes, so a start-up that tunes (``library_tuning``)
# times both ways on the model's own weights and keeps the faster (``ProductPolicy.swiglu_choices``).
WIDE_SWIGLU_MIN_TILES = 180
WIDE_SWIGLU_MIN_ROWS = 1024
WIDE_SWIGLU_SMALL_WEIGHTS = 64 << 20    # elements of [gate; up] up to which 512 rows are enough

_cu_counts: dict = {}


def _compute_units(device) -> int:
    n = _cu_counts.get(device)
    if n is None:
        n = _cu_counts[device] = int(torch.cuda.get_device_properties(device).multi_processor_count)
    return n


def wide_swiglu_pays(M: int, two_i: int, K: int, ldx: int) -> bool:
    """Is the gate/up product of M rows faster through the wide-tile kernel (with the gate in its
    epilogue) than through the library and the gate kernel?"""
    if M < WIDE_SWIGLU_MIN_ROWS and not (M >= WIDE_SWIGLU_MIN_ROWS // 2 and two_i * K <= WIDE_SWIGLU_SMALL_WEIGHTS):
        return False
    return _load("gemm_tile").cw_gemm_bf16_wide_tiles(2, M, two_i, K, ldx) >= WIDE_SWIGLU_MIN_TILES


@contextlib.contextmanager
def library_tuning(policy: "ProductPolicy | None" = None):
    """While active, a library product of a shape not seen before is timed over the library's
    candidate kernels and the fastest is remembered; afterwards the remembered choices stay in
    use and unseen shapes take the library's own default again. The library keeps its choices in a
    file in the temporary folder (or where PYTORCH_TUNABLEOP_FILENAME points), which later
    processes of the same user read. ``policy``: the engine whose own kernels are timed against the
    library's meanwhile; what it measures is kept in a file beside the library's
    (``choices_file``), so that a later process on the same card and build, a profiled run among
    them, takes the same kernels without timing them again. Not to be left active during
    HIP-graph capture."""
    import torch.cuda.tunable as tunable

    policy = policy if policy is not None else DEFAULT_POLICY
    if not os.environ.get("PYTORCH_TUNABLEOP_FILENAME"):
        tunable.set_filename(os.path.join(tempfile.gettempdir(), f"clockwork_amd_products_{os.getuid()}.csv"), True)
    tunable.enable(True)
    tunable.tuning_enable(True)
    policy.tuning = True
    policy.read_choices(choices_file())
    try:
        yield
    finally:
        policy.tuning = False
        tunable.tuning_enable(False)
        policy.write_choices(choices_file())


# a plain product is timed against the library's only with this many rows and tiles (half the
# compute units busy): below that the library has always been the faster one
WIDE_PRODUCT_MIN_ROWS = 1024
WIDE_PRODUCT_MIN_TILES = 128


def _library_product(x, weight, bias):
    return torch.mm(x, weight.t()) if bias is None else torch.addmm(bias, x, weight.t())


def _wide_product_chosen(x: torch.Tensor, weight: torch.Tensor, bias, policy: ProductPolicy) -> bool:
    """Does a plain product of many bfloat16 rows go through the wide-tile kernel? Only where a
    tuning start-up has timed it against the library's tuned kernel on these very shapes and
    found it faster (measured: the 7B shape's down product, 279 against 351 us)."""
    M, K = x.shape
    if M < WIDE_PRODUCT_MIN_ROWS or not policy.product_choices and not policy.tuning:
        return False
    key = (weight.shape[0], K, bias is not None)
    choice = policy.product_choices.get(key)
    if choice is None and policy.tuning:
        choice = policy.recall("product_choices", key)
    if choice is None and policy.tuning and x.is_contiguous():
        if _load("gemm_tile").cw_gemm_bf16_wide_tiles(0, M, key[0], K, K) >= WIDE_PRODUCT_MIN_TILES:
            library = _timed_us(lambda: _library_product(x, weight, bias))
            own = _timed_us(lambda: linear_tiled(x, weight, bias, wide=True))
            choice = own <= library
        else:
            choice = False
        policy.product_choices[key] = choice
    return bool(choice) and x.is_contiguous()


def _timed_us(fn, repeats: int = 5) -> float:
    """The median time of ``fn`` with its operands out of the caches, as a layer finds its weights
    in a model larger than the last-level cache: 512 MB are written between the runs. (Timed
    back to back, a product whose weights fit that cache looks faster than it is in a step.)"""
    fn()
    flush = torch.empty(512 << 20, dtype=torch.uint8, device="cuda")
    times = []
    for _ in range(repeats):
        flush.zero_()
        begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        begin.record()
        fn()
        end.record()
        end.synchronize()
        times.append(begin.elapsed_time(end) * 1e3)
    return sorted(times)[len(times) // 2]


def _replayed_us(candidates: dict, rounds: int, flush: bool, replays: int = 3) -> dict:
    """The time of each of ``candidates`` (name -> a function of the round's number that launches
    this package's own kernels only) as the kernels take it inside a captured graph of ``rounds``
    rounds, replayed a few times. The operands have to come from memory as they do in a step:
    either the candidate takes other copies of them from round to round, more than the caches
    hold, or (``flush``) 512 MB are written before every round and what a graph of the writes
    alone takes is subtracted. For kernels of a few microseconds, whose differences a timing of
    eager launches blurs (the launches' own time lies on top and overlaps the kernels differently
    from one candidate to the next: two counts of parts over K that differ by 5 us in the decode
    step differed by 2 us timed that way)."""
    wash = torch.empty(512 << 20, dtype=torch.uint8, device="cuda") if flush else None

    def median_replay(fn) -> float:
        def body():
            for i in range(rounds):
                if wash is not None:
                    wash.zero_()
                if fn is not None:
                    fn(i)

        body()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        was_enabled = gc.isenabled()
        gc.disable()  # a collection must not destroy another graph while this capture is open
        try:
            with torch.cuda.graph(graph):
                body()
        finally:
            if was_enabled:
                gc.enable()
        graph.replay()
        torch.cuda.synchronize()
        times = []
        for _ in range(replays):
            begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            begin.record()
            graph.replay()
            end.record()
            end.synchronize()
            times.append(begin.elapsed_time(end) * 1e3)
        del graph
        return sorted(times)[len(times) // 2]

    writes = median_replay(None) if flush else 0.0
    return {name: (median_replay(fn) - writes) / rounds for name, fn in candidates.items()}


# copies of a weight matrix that a timing walks through so that each comes from memory again:
# together more than the memory-side cache holds
_COLD_COPIES_BYTES = 320 << 20


def _cold_copies(weight: torch.Tensor) -> list:
    """``weight`` and as many copies of it as together exceed the caches (16 at most); the matrix
    alone where the memory for them is not there."""
    n = min(16, max(2, -(-_COLD_COPIES_BYTES // (weight.numel() * weight.element_size())) + 1))
    try:
        return [weight] + [weight.clone() for _ in range(n - 1)]
    except torch.OutOfMemoryError:
        return [weight]


def linear_wide_partial(x: torch.Tensor, weight: torch.Tensor, k_splits: int) -> PartialSums:
    """x @ weight.T as ``k_splits`` float32 planes of partial sums over runs of K, through the
    wide-tile kernel (csrc/gemm_tile.hip): for a long portion's product whose output is too narrow
    to fill the card with whole tiles (the down product: 64 tiles of 256 x 192 for 2048 rows of the
    1.5B shape), and whose result goes straight into ``add_rmsnorm``."""
    _gpu(x, weight)
    M, K = x.shape
    N = weight.shape[0]
    lib = _load("gemm_tile")
    if not (x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and weight.shape[1] == K
            and lib.cw_gemm_bf16_wide_partial_ok(M, N, K, x.stride(0), int(k_splits))):
        raise KernelError("the wide-tile kernel does not sum this product in parts")
    parts = torch.empty((int(k_splits), M, N), dtype=torch.float32, device=x.device)
    _check(lib.cw_gemm_bf16_wide_partial(_ptr(x), x.stride(0), _ptr(weight), _ptr(parts), N, M, N, K, int(k_splits),
                                         _compute_units(x.device), _stream()), "gemm_bf16_wide_partial")
    return PartialSums(parts)


# a long portion's product is a candidate for the wide-tile kernel's partial sums when whole tiles
# would leave most compute units idle and K is long enough to cut
WIDE_PARTIAL_MAX_TILES = 128
WIDE_PARTIAL_MIN_K = 1024


def _wide_partial_chosen(x: torch.Tensor, weight: torch.Tensor, policy: ProductPolicy) -> int:
    """Into how many runs of K does the wide-tile kernel sum this product of many rows (0: it
    does not, the library's product runs)? Only what a tuning start-up has measured on these very
    shapes: the kernel's partial sums and the norm that adds them against the library's product and
    the norm of its bfloat16 result."""
    M, K = x.shape
    N = weight.shape[0]
    key = (N, K)
    choice = policy.wide_partial_choices.get(key)
    if choice is None and policy.tuning:
        choice = policy.recall("wide_partial_choices", key)
    if choice is None and policy.tuning:
        lib = _load("gemm_tile")
        tiles = lib.cw_gemm_bf16_wide_tiles(0, M, N, K, K)
        choice = 0
        if 0 < tiles <= WIDE_PARTIAL_MAX_TILES and K >= WIDE_PARTIAL_MIN_K:
            resid = torch.zeros((M, N), dtype=torch.float32, device=x.device)
            norm_weight = torch.ones(N, dtype=torch.bfloat16, device=x.device)
            out = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
            best = _timed_us(lambda: add_rmsnorm(resid, _library_product(x, weight, None), norm_weight, 1e-6, out, write_back=False))
            for splits in (2, 3, 4, 5, 6, 7, 8):
                if not lib.cw_gemm_bf16_wide_partial_ok(M, N, K, K, splits):
                    continue
                t = _timed_us(lambda: add_rmsnorm(resid, linear_wide_partial(x, weight, splits), norm_weight, 1e-6, out, write_back=False))
                if t < 0.97 * best:
                    best, choice = t, splits
        policy.wide_partial_choices[key] = choice
    return int(choice or 0)


def _measure_k_splits(x: torch.Tensor, weight: torch.Tensor, default: int) -> int:
    """Into how many parts over K is the product of these few rows with ``weight`` [N, K] summed
    the fastest, together with the norm kernel that adds the parts up? Which count lets the
    streaming kernel in, fills the card evenly and leaves whole chunks to a wave differs from shape
    to shape (the 7B shape's down product with the norm: 38.4 us with 5 parts, 32.4 with 7; the 32B
    shape's: 64.8 with 7, 59.2 with 6), so the candidates are timed on the model's own weights,
    inside captured graphs that walk through copies of the matrix (each comes from memory again)."""
    M, K = x.shape
    N = weight.shape[0]
    lib = _load("gemm")
    resid = torch.zeros((M, N), dtype=torch.float32, device=x.device)
    norm_weight = torch.ones(N, dtype=torch.bfloat16, device=x.device)
    out = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)

    weights = _cold_copies(weight)

    def run(splits: int, round_no: int):
        w = weights[round_no % len(weights)]
        parts = torch.empty((splits, M, N), dtype=torch.float32, device=x.device)
        _check(lib.cw_gemm_bf16_skinny(3, _ptr(x), K, _ptr(w), _ptr(parts), N, M, N, K, splits, _stream()),
               "gemm_bf16_skinny(partial)")
        add_rmsnorm(resid, PartialSums(parts), norm_weight, 1e-6, out, write_back=False)

    candidates = sorted({default, *(s for s in (2, 3, 4, 5, 6, 7, 8, 10, 12) if K // s >= 256)})
    rounds = len(weights) * -(-12 // len(weights)) if len(weights) > 1 else 6
    times = _replayed_us({splits: (lambda i, splits=splits: run(splits, i)) for splits in candidates},
                         rounds=rounds, flush=len(weights) == 1)
    best = min(times, key=times.get)
    # the fixed rule stays unless something is clearly faster: no flapping between equals
    return best if times[best] < 0.97 * times[default] else default


def _measure_swiglu(x: torch.Tensor, gate_up_weight: torch.Tensor, out: torch.Tensor) -> bool:
    """Time the two ways of a long portion's gate/up product on these operands (the library has
    just chosen its kernel for the shape): is this package's kernel at least as fast as the
    library's product followed by the gate kernel?"""
    library = _timed_us(lambda: silu_mul(_library_product(x, gate_up_weight, None), out))
    own = _timed_us(lambda: linear_tiled(x, gate_up_weight, swiglu=True, wide=True))
    return own <= library


def qkv_rope_fused_supported(x: torch.Tensor, weight: torch.Tensor, rotary_dim: int, hd: int) -> bool:
    """The fused q/k/v product + rotary + cache write takes few bfloat16 rows and a full rotary
    dimension. Beyond 16 rows it serves small weight matrices only: a large one is faster as a
    product and a rotation kernel (measured: 33 MB at 24 rows and more)."""
    rows = x.shape[0]
    return (x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16
            and (rows <= SKINNY_MAX_ROWS or (rows <= STREAM_MAX_ROWS and weight.numel() <= FUSED_QKV_MAX_WEIGHTS))
            and x.shape[1] % 8 == 0 and rotary_dim == hd and hd % 16 == 0)


def qkv_rope_fused(x, weight, bias, positions, slots, inv_freq, nh: int, nkv: int, hd: int, k_cache, v_cache) -> torch.Tensor:
    """q = rope(x @ Wq.T + bq) returned as [M, nh * hd]; rope(x @ Wk.T + bk) and x @ Wv.T + bv written
    to the cache rows ``slots``: one kernel for few bfloat16 rows (see csrc/gemm.hip)."""
    _gpu(x, weight, bias, positions, slots, inv_freq, k_cache, v_cache)
    M, K = x.shape
    if not (qkv_rope_fused_supported(x, weight, hd, hd)):
        raise KernelError("the fused q/k/v kernel does not take these operands")
    if not (tuple(weight.shape) == ((nh + 2 * nkv) * hd, K)):
        raise KernelError("qkv weight must be [(nh + 2 nkv) hd, K]")
    _i32(positions, M, "positions")
    _i32(slots, M, "slots")
    if not (inv_freq.dtype == torch.float32 and inv_freq.numel() == hd // 2):
        raise KernelError("inv_freq must be float32 [hd / 2]")
    _need(k_cache.dtype == torch.bfloat16 and tuple(k_cache.shape[-2:]) == (nkv, hd) and k_cache.shape == v_cache.shape,
          "cache must be bfloat16 [..., nkv, hd]")
    if bias is not None:
        if not (bias.numel() == weight.shape[0] and bias.dtype in (torch.bfloat16, torch.float32)):
            raise KernelError("qkv bias")
    q = torch.empty((M, nh * hd), dtype=torch.bfloat16, device=x.device)
    _check(
        _load("gemm").cw_gemm_qkv_rope_bf16(
            _ptr(x), K, _ptr(weight), _ptr(bias), int(bias is not None and bias.dtype == torch.float32), _ptr(positions),
            _ptr(slots), _ptr(inv_freq), _ptr(q), _ptr(k_cache), _ptr(v_cache), k_cache.numel() // (nkv * hd),
            M, K, nh, nkv, hd, _stream()),
        "gemm_qkv_rope_bf16",
    )
    return q


def swiglu_norm_fusable(M: int, two_i: int, K: int, dtype, gate_up_weight, delta) -> bool:
    """Can the gate/up product make its own input rmsnorm(resid + delta)? Few bfloat16 rows of a
    shape the streaming kernel takes, the pending delta a plain bfloat16 tensor."""
    return (dtype == torch.bfloat16 and gate_up_weight.dtype == torch.bfloat16 and gate_up_weight.shape[1] == K
            and isinstance(delta, torch.Tensor) and delta.dtype == torch.bfloat16 and delta.is_contiguous()
            and bool(_load("gemm").cw_gemm_bf16_swiglu_normed_ok(M, two_i, K)))


def linear_swiglu(x, gate_up_weight: torch.Tensor, policy: "ProductPolicy | None" = None) -> torch.Tensor:
    """silu(x @ gate.T) * (x @ up.T) for gate_up_weight = [gate; up] stacked along dim 0.

    Few bfloat16 rows: one kernel that streams the weights once and applies the gate in its
    epilogue. Otherwise the product followed by the gate kernel, or (``policy``, see ``linear``)
    a tiled kernel with the gate in its epilogue."""
    policy = policy if policy is not None else DEFAULT_POLICY
    if isinstance(x, LazyAddNorm):
        M, K = x.shape
        two_i = gate_up_weight.shape[0]
        if swiglu_norm_fusable(M, two_i, K, x.dtype, gate_up_weight, x.delta):
            _gpu(x.resid, x.delta, x.weight, gate_up_weight)
            out = torch.empty((M, two_i // 2), dtype=x.dtype, device=x.resid.device)
            _check(
                _load("gemm").cw_gemm_bf16_swiglu_normed(
                    _ptr(x.resid), _ptr(x.delta), _ptr(x.weight), int(x.weight.dtype == torch.float32), float(x.eps),
                    _ptr(gate_up_weight), _ptr(out), two_i // 2, M, two_i, K, _stream()),
                "gemm_bf16_swiglu_normed",
            )
            return out
        x = x.value()
    _gpu(x, gate_up_weight)
    M, K = x.shape
    two_i = gate_up_weight.shape[0]
    if not (gate_up_weight.shape[1] == K and two_i % 2 == 0):
        raise KernelError("gate_up weight must be [2 I, K]")
    out = torch.empty((M, two_i // 2), dtype=x.dtype, device=x.device)
    if (x.dtype == torch.bfloat16 and M <= STREAM_MAX_ROWS and K % 8 == 0
            and _load("gemm").cw_gemm_bf16_skinny_fast(2, M, two_i, K)):
        if not (gate_up_weight.dtype == torch.bfloat16):
            raise KernelError("a bfloat16 product needs bfloat16 operands")
        _check(_load("gemm").cw_gemm_bf16_skinny(2, _ptr(x), K, _ptr(gate_up_weight), _ptr(out), two_i // 2, M, two_i, K, 0, _stream()),
               "gemm_bf16_skinny(swiglu)")
        return out
    if x.dtype == torch.bfloat16 and gate_up_weight.dtype == torch.bfloat16 and K % 8 == 0 and x.is_contiguous():
        if policy.hip_products:
            return linear_tiled(x, gate_up_weight, swiglu=True)
        if wide_swiglu_pays(M, two_i, K, K):
            # with enough rows the shape of the weights decides, and a start-up that tunes the
            # library's products has measured it for this model's
            measured = M >= WIDE_SWIGLU_MIN_ROWS
            if (measured and policy.tuning and (two_i, K) not in policy.swiglu_choices
                    and policy.recall("swiglu_choices", (two_i, K)) is None):
                policy.swiglu_choices[(two_i, K)] = _measure_swiglu(x, gate_up_weight, out)
            if not measured or policy.swiglu_choices.get((two_i, K), True):
                return linear_tiled(x, gate_up_weight, swiglu=True, wide=True)
    return silu_mul(linear(x, gate_up_weight, policy=policy), out)


_zero_rows: dict = {}


def _zero_row(device) -> int:
    """Address of 1 KiB of zeros on ``device``: what the attention kernels read masked rows from."""
    t = _zero_rows.get(device)
    if t is None:
        t = _zero_rows[device] = torch.zeros(512, dtype=torch.bfloat16, device=device)
    return t.data_ptr()


def prefill_attention_supported(hd: int, dtype: torch.dtype) -> bool:
    return dtype == torch.bfloat16 and bool(_load("attention", hd).cw_attention_prefill_supported())


def attention_prefill(q, q_stride: int, out, k_cache, v_cache, block_tables, ctx_lens, cu_q, items, n_items: int,
                      nh: int, nkv: int, hd: int, block_size: int, window: int, scale: float,
                      n_tokens: int, n_requests: int, row_blocks: int = 4, workspace=None) -> None:
    """Portions of prompts through the bfloat16 matrix-core kernel; an item holds at most
    ``prefill_tokens_per_item(nh // nkv, row_blocks)`` tokens. ``row_blocks`` 2 instead of 4: smaller
    workgroups for launches with few items (head sizes up to 128). Other arguments as for ``attention``.
    An item's fourth field is ``part | parts << 8``: with parts > 1 the item stands that many times
    in the list, one after the other, and each takes a share of its keys; such a list needs a
    float32 ``workspace`` of ``prefill_attention_workspace_floats`` elements (without one every item
    computes all of its keys)."""
    if not (prefill_row_blocks_ok(hd, row_blocks)):
        raise KernelError(f"the kernel for head size {hd} does not take {row_blocks} row blocks")
    _gpu(out, k_cache, v_cache, block_tables, ctx_lens, cu_q, items, workspace)
    ws_floats = 0
    if workspace is not None:
        need = prefill_attention_workspace_floats(hd, n_items, nh, nkv, row_blocks)
        _need(workspace.dtype == torch.float32 and workspace.numel() >= need,
              f"attention over parts of key ranges needs a float32 workspace of {need} elements")
        ws_floats = workspace.numel()
    if not (q.is_cuda and q.dtype == out.dtype == k_cache.dtype == v_cache.dtype == torch.bfloat16):
        raise KernelError("the kernel is bfloat16")
    if not (out.dim() == 2 and out.shape[0] >= n_tokens and out.shape[1] == nh * hd):
        raise KernelError("attention output must be [T, nh * hd]")
    if not (q_stride >= nh * hd):
        raise KernelError("query rows overlap")
    if not (block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.shape[0] >= n_requests):
        raise KernelError("block_tables must be int32 [R, max_blocks]")
    _i32(ctx_lens, n_requests, "ctx_lens")
    _i32(cu_q, n_requests + 1, "cu_q")
    if not (items.dtype == torch.int32 and items.numel() >= 4 * n_items):
        raise KernelError("items must be int32 [n_items, 4]")
    if not (tuple(k_cache.shape[-2:]) == (nkv, hd) and k_cache.shape == v_cache.shape):
        raise KernelError("cache must be [..., nkv, hd]")
    _check(
        _load("attention", hd).cw_attention_prefill_bf16(
            q.data_ptr(), int(q_stride), _ptr(out), out.shape[1], _ptr(k_cache), _ptr(v_cache), _ptr(block_tables),
            block_tables.shape[1], _ptr(ctx_lens), _ptr(cu_q), _ptr(items), n_items, nh, nkv, block_size,
            window, float(scale), _zero_row(out.device), int(row_blocks), int(workspace is not None), _ptr(workspace),
            ws_floats, _stream()),
        "attention_prefill_bf16",
    )


def prefill_attention_workspace_floats(hd: int, n_items: int, nh: int, nkv: int, row_blocks: int) -> int:
    return int(_load("attention", hd).cw_attention_prefill_workspace_floats(n_items, nh, nkv, int(row_blocks)))


def prefill_row_blocks_ok(hd: int, row_blocks: int) -> bool:
    return bool(_load("attention", hd).cw_attention_prefill_row_blocks_ok(int(row_blocks)))


def prefill_tokens_per_item(group: int, row_blocks: int = 4) -> int:
    """Tokens one work item of ``attention_prefill`` may hold: a row block is 32 rows, a row a
    (token, head of the group) pair."""
    return row_blocks * (32 // min(group, 32))


def decode_attention_supported(hd: int, dtype: torch.dtype) -> bool:
    return dtype == torch.bfloat16 and bool(_load("attention", hd).cw_attention_decode_supported())


# the most splits the bfloat16 decode kernel takes (DEC_MAX_SPLITS in csrc/attention.hip)
DECODE_MAX_SPLITS = 256


def decode_attention_workspace_floats(hd: int, n_items: int, nh: int, nkv: int, n_splits: int) -> int:
    return int(_load("attention", hd).cw_attention_decode_workspace_floats(n_items, nh, nkv, n_splits))


def attention_decode(q, q_stride: int, out, k_cache, v_cache, block_tables, ctx_lens, cu_q, items, n_items: int,
                     nh: int, nkv: int, hd: int, block_size: int, n_splits: int, window: int, scale: float,
                     n_tokens: int, n_requests: int, workspace=None, identity: bool = False,
                     split_keys: int = 0, max_ctx: int = 0) -> None:
    """Single-token items through the bfloat16 decode kernel; arguments as for ``attention``.
    With more than one split it needs a float32 ``workspace``. ``identity``: item i is request i
    with its token in row i (no other items). ``split_keys`` > 0: every split takes that many
    keys at a fixed place; no context may then be longer than ``max_ctx`` <= n_splits * split_keys."""
    _gpu(out, k_cache, v_cache, block_tables, ctx_lens, cu_q, items, workspace)
    if not (q.is_cuda and q.dtype == out.dtype == k_cache.dtype == v_cache.dtype == torch.bfloat16):
        raise KernelError("the decode kernel is bfloat16")
    if not (out.dim() == 2 and out.shape[0] >= n_tokens and out.shape[1] == nh * hd):
        raise KernelError("attention output must be [T, nh * hd]")
    if not (q_stride >= nh * hd):
        raise KernelError("query rows overlap")
    if not (block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.shape[0] >= n_requests):
        raise KernelError("block_tables must be int32 [R, max_blocks]")
    _i32(ctx_lens, n_requests, "ctx_lens")
    _i32(cu_q, n_requests + 1, "cu_q")
    if not (items.dtype == torch.int32 and items.numel() >= 4 * n_items):
        raise KernelError("items must be int32 [n_items, 4]")
    if not (tuple(k_cache.shape[-2:]) == (nkv, hd) and k_cache.shape == v_cache.shape):
        raise KernelError("cache must be [..., nkv, hd]")
    if identity:
        if not (n_items == n_requests == n_tokens):
            raise KernelError("identity items: one single-token item per request, nothing else")
    if split_keys:
        if not (split_keys % 32 == 0 and split_keys * n_splits >= max_ctx > 0):
            raise KernelError("fixed key ranges do not cover the longest context")
    lib = _load("attention", hd)
    need = lib.cw_attention_decode_workspace_floats(n_items, nh, nkv, n_splits)
    ws_floats = 0
    if need > 0:
        _need(workspace is not None and workspace.dtype == torch.float32 and workspace.numel() >= need,
              f"decode attention needs a float32 workspace of {need} elements")
        ws_floats = workspace.numel()
    _check(
        lib.cw_attention_decode_bf16(
            q.data_ptr(), int(q_stride), _ptr(out), out.shape[1], _ptr(k_cache), _ptr(v_cache), _ptr(block_tables),
            block_tables.shape[1], _ptr(ctx_lens), _ptr(cu_q), _ptr(items), n_items, nh, nkv, block_size, n_splits,
            window, float(scale), _ptr(workspace), ws_floats, _zero_row(out.device), int(bool(identity)),
            int(split_keys), int(max_ctx), _stream()),
        "attention_decode_bf16",
    )


def attention(q, q_stride: int, out, k_cache, v_cache, block_tables, ctx_lens, cu_q, items, n_items: int,
              rows: int, nh: int, nkv: int, hd: int, block_size: int, gh: int, n_splits: int, window: int,
              scale: float, n_tokens: int, n_requests: int, workspace=None) -> None:
    """Paged causal attention for ``n_items`` work items (see csrc/attention.hip).

    q: any tensor whose token rows are ``q_stride`` elements apart with head h at column h * hd;
    out [n_tokens, nh * hd]; caches [num_blocks * block_size, nkv, hd]; block_tables int32
    [n_requests, max_blocks]; items int32 [n_items, 4] = (request, first token, tokens, 0)."""
    _gpu(out, k_cache, v_cache, block_tables, ctx_lens, cu_q, items, workspace)
    if not (q.is_cuda and q.dtype == out.dtype == k_cache.dtype == v_cache.dtype):
        raise KernelError("attention operands differ in type or device")
    if not (out.dim() == 2 and out.shape[0] >= n_tokens and out.shape[1] == nh * hd):
        raise KernelError("attention output must be [T, nh * hd]")
    if not (q_stride >= nh * hd):
        raise KernelError("query rows overlap")
    if not (block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.shape[0] >= n_requests):
        raise KernelError("block_tables must be int32 [R, max_blocks]")
    _i32(ctx_lens, n_requests, "ctx_lens")
    _i32(cu_q, n_requests + 1, "cu_q")
    if not (items.dtype == torch.int32 and items.numel() >= 4 * n_items):
        raise KernelError("items must be int32 [n_items, 4]")
    if not (tuple(k_cache.shape[-2:]) == (nkv, hd) and k_cache.shape == v_cache.shape):
        raise KernelError("cache must be [..., nkv, hd]")
    lib = _load("attention", hd)
    group = nh // nkv
    n_chunks = -(-group // gh)
    need = lib.cw_attention_workspace_floats(rows, n_items, nkv, n_chunks, n_splits)
    ws_floats = 0
    if need > 0:
        _need(workspace is not None and workspace.dtype == torch.float32 and workspace.numel() >= need,
              f"attention needs a float32 workspace of {need} elements")
        ws_floats = workspace.numel()
    _check(
        lib.cw_attention(
            rows, dtype_code(out.dtype), q.data_ptr(), int(q_stride), _ptr(out), out.shape[1], _ptr(k_cache), _ptr(v_cache),
            _ptr(block_tables), block_tables.shape[1], _ptr(ctx_lens), _ptr(cu_q), _ptr(items), n_items, nh, nkv,
            block_size, gh, n_splits, window, float(scale), _ptr(workspace), ws_floats, _stream()),
        "attention",
    )


def attention_workspace_floats(hd: int, rows: int, n_items: int, nkv: int, n_chunks: int, n_splits: int) -> int:
    return int(_load("attention", hd).cw_attention_workspace_floats(rows, n_items, nkv, n_chunks, n_splits))


def argmax(logits: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
    """First index of the maximum of every row of float32 ``logits`` [n, V] -> int32 [n]."""
    _gpu(logits, out)
    if not (logits.dtype == torch.float32 and logits.dim() == 2):
        raise KernelError("logits must be float32 [n, V]")
    n, V = logits.shape
    lib = _load("sampling")
    chunks = lib.cw_argmax_chunks(V)
    ws = torch.empty(max(1, n * chunks * 2), dtype=torch.int32, device=logits.device)
    if out is None:
        out = torch.empty(n, dtype=torch.int32, device=logits.device)
    _i32(out, n, "out")
    _check(lib.cw_argmax(_ptr(logits), V, n, V, _ptr(out), _ptr(ws), ws.numel() * 4, _stream()), "argmax")
    return out


def sample(logits, temperature, top_k, top_p, seeds, draws, out=None, any_top_k: bool = True,
           any_top_p: bool = True) -> torch.Tensor:
    """One token per row: rows with temperature 0 take the arg-max, the others are drawn.
    ``any_top_k`` / ``any_top_p`` off: the caller knows that no row has that option, and its
    kernels are not launched."""
    _gpu(logits, temperature, top_k, top_p, seeds, draws, out)
    if not (logits.dtype == torch.float32 and logits.dim() == 2):
        raise KernelError("logits must be float32 [n, V]")
    n, V = logits.shape
    if not (temperature.dtype == torch.float32 and temperature.numel() == n):
        raise KernelError("temperature must be float32 [n]")
    if not (top_p.dtype == torch.float32 and top_p.numel() == n):
        raise KernelError("top_p must be float32 [n]")
    _i32(top_k, n, "top_k")
    if not (seeds.dtype == torch.int64 and seeds.numel() == n):
        raise KernelError("seeds must be int64 [n]")
    if not (draws.dtype == torch.int64 and draws.numel() == n):
        raise KernelError("draws must be int64 [n]")
    if out is None:
        out = torch.empty(n, dtype=torch.int32, device=logits.device)
    _i32(out, n, "out")
    lib = _load("sampling")
    ws = torch.empty(int(lib.cw_sample_workspace_bytes(n, V)), dtype=torch.uint8, device=logits.device)
    _check(
        lib.cw_sample(_ptr(logits), V, n, V, _ptr(temperature), _ptr(top_k), _ptr(top_p), _ptr(seeds), _ptr(draws),
                      _ptr(out), _ptr(ws), ws.numel(), int(bool(any_top_k)) | (int(bool(any_top_p)) << 1), _stream()),
        "sample",
    )
    return out
