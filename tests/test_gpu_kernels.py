"""Each HIP kernel alone against a plain float32 formula, at sizes other than the engine's."""

import math

import pytest
import torch

from tests.plain import qwen2_plain as plain

pytestmark = pytest.mark.gpu

DEV = "cuda"
DTYPES = [torch.float32, torch.bfloat16]


def tol(dtype):
    return dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)


@pytest.fixture(autouse=True)
def _seed():
    torch.manual_seed(1234)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("V,H,T", [(777, 100, 13), (32, 1536, 1)])
def test_embedding(dtype, V, H, T):
    from clockwork_amd import ops

    table = torch.randn(V, H, device=DEV).to(dtype)
    ids = torch.randint(0, V, (T,), device=DEV, dtype=torch.int32)
    ids[0] = V - 1
    out = torch.full((T, H), 7.0, device=DEV)
    ops.embedding(table, ids, out)
    torch.testing.assert_close(out, plain.embedding(table.float().cpu(), ids.long().cpu()).to(DEV), rtol=0, atol=0)


@pytest.mark.parametrize("dtype,wdtype", [(torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16), (torch.bfloat16, torch.float32)])
@pytest.mark.parametrize("T,H,eps", [(5, 100, 1e-5), (3, 1536, 1e-6), (2, 7, 3e-6), (1, 4100, 1e-6), (2, 8192, 1e-6), (1, 8196, 1e-5)])
def test_add_rmsnorm(dtype, wdtype, T, H, eps):
    from clockwork_amd import ops

    resid = torch.randn(T, H, device=DEV) * 3
    delta = torch.randn(T, H, device=DEV).to(dtype)
    weight = (1 + 0.1 * torch.randn(H, device=DEV)).to(wdtype)
    want_resid = resid + delta.float()
    want = plain.rmsnorm(want_resid.cpu(), weight.float().cpu(), eps).to(DEV)
    r = resid.clone()
    out = torch.empty(T, H, device=DEV, dtype=dtype)
    ops.add_rmsnorm(r, delta, weight, eps, out)
    torch.testing.assert_close(r, want_resid, rtol=0, atol=0)
    torch.testing.assert_close(out.float(), want, **tol(dtype))
    # without a delta the stream is left as it is
    r2 = resid.clone()
    ops.add_rmsnorm(r2, None, weight, eps, out)
    torch.testing.assert_close(r2, resid, rtol=0, atol=0)
    torch.testing.assert_close(out.float(), plain.rmsnorm(resid.cpu(), weight.float().cpu(), eps).to(DEV), **tol(dtype))
    # selected rows: normed into a compact output, the stream untouched
    rows = torch.tensor([T - 1, 0], dtype=torch.int32, device=DEV)
    r3 = resid.clone()
    out2 = torch.empty(2, H, device=DEV, dtype=dtype)
    ops.add_rmsnorm(r3, delta, weight, eps, out2, rows)
    torch.testing.assert_close(r3, resid, rtol=0, atol=0)
    torch.testing.assert_close(out2.float(), want[rows.long()], **tol(dtype))


def _norm_cast_orders(v: torch.Tensor, weight: torch.Tensor, eps: float):
    """rmsnorm of float32 rows ``v`` with a bfloat16 ``weight``, rounded the reference's way,
    weight * bfloat16(x / rms) (clockwork/engine/model.py:49: the cast comes before the weight),
    and the other way, bfloat16(weight * x / rms). Both bfloat16."""
    xhat = v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps)
    first = weight.to(torch.bfloat16) * xhat.to(torch.bfloat16)          # a bfloat16 product: rounded once more
    other = (weight.float() * xhat).to(torch.bfloat16)
    return first, other


@pytest.mark.parametrize("T,H", [(6, 1536), (5, 100), (3, 4104), (4, 70)])
@pytest.mark.parametrize("wdtype", [torch.bfloat16, torch.float32])
def test_rmsnorm_rounds_before_the_weight_multiplies(T, H, wdtype):
    """The order of the two roundings of a bfloat16 norm, which a tolerance cannot see: weights far
    from 1 with full mantissas make weight * bfloat16(x) and bfloat16(weight * x) differ in the last
    bit of about a third of the elements. The kernel (both its vector and its scalar form, with a
    delta and with selected rows) must give the first, bit for bit; one element in a thousand is
    allowed to differ, where the float32 statistic's own last bit decides a rounding."""
    from clockwork_amd import ops

    resid = torch.randn(T, H, device=DEV) * 2
    delta = torch.randn(T, H, device=DEV).to(torch.bfloat16)
    weight = (1.37 + 0.41 * torch.randn(H, device=DEV)).to(torch.bfloat16)   # bfloat16 values either way
    first, other = _norm_cast_orders((resid + delta.float()).cpu(), weight.cpu(), 1e-6)
    assert float((first != other).float().mean()) > 0.15, "the inputs do not tell the two orders apart"
    out = torch.empty(T, H, device=DEV, dtype=torch.bfloat16)
    ops.add_rmsnorm(resid.clone(), delta, weight.to(wdtype), 1e-6, out)
    assert float((out.cpu() != first).float().mean()) < 1e-3
    rows = torch.tensor([T - 1, 1], dtype=torch.int32, device=DEV)
    out2 = torch.empty(2, H, device=DEV, dtype=torch.bfloat16)
    ops.add_rmsnorm(resid.clone(), delta, weight.to(wdtype), 1e-6, out2, rows)
    assert float((out2.cpu() != first[rows.long().cpu()]).float().mean()) < 1e-3


@pytest.mark.parametrize("wdtype", [torch.bfloat16, torch.float32])
def test_norm_inside_the_gate_up_product_rounds_before_the_weight_multiplies(wdtype):
    """The same pin for the norm that the gate/up product makes for itself. Its normed row is not
    written anywhere, so the weights are chosen to show it: up row j is the unit vector of element
    j % K and gate row j four times the unit vector of another element, so that (products with 1
    and 4 and sums with zeros being exact) output j is silu(4 n[a]) * n[b] for two elements of the
    normed row n. The expected outputs are made from the row rounded the reference's way and from
    the row rounded the other way; the kernel must follow the first."""
    from clockwork_amd import ops

    M, K, I = 7, 1024, 4096
    resid = torch.randn(M, K, device=DEV) * 2
    delta = torch.randn(M, K, device=DEV).to(torch.bfloat16)
    weight = (1.37 + 0.41 * torch.randn(K, device=DEV)).to(torch.bfloat16)
    j = torch.arange(I)
    gate_at, up_at = (7 * j + 3) % K, j % K
    w = torch.zeros(2 * I, K)
    w[j, gate_at] = 4.0
    w[I + j, up_at] = 1.0
    w = w.to(torch.bfloat16).to(DEV)
    assert ops.swiglu_norm_fusable(M, 2 * I, K, torch.bfloat16, w, delta)
    got = ops.linear_swiglu(ops.LazyAddNorm(resid, delta, weight.to(wdtype), 1e-6, torch.bfloat16), w).cpu()
    first, other = _norm_cast_orders((resid + delta.float()).cpu(), weight.cpu(), 1e-6)

    def outputs(n):
        n = n.double()
        g = 4.0 * n[:, gate_at]
        return (g / (1.0 + torch.exp(-g)) * n[:, up_at]).to(torch.bfloat16)

    want, wrong = outputs(first), outputs(other)
    assert float((want != wrong).float().mean()) > 0.15, "the inputs do not tell the two orders apart"
    # the kernel's float32 exponential may decide a rounding otherwise now and then
    assert float((got != want).float().mean()) < 5e-3
    assert float((got != wrong).float().mean()) > 0.15


@pytest.mark.parametrize("M,N,K", [(1, 1536, 8960), (8, 1536, 8960), (16, 96, 4096), (3, 1000, 5000 * 8)])
def test_split_k_partial_sums_feed_the_norm(M, N, K):
    """A narrow product with a long K comes back as float32 partial sums; the norm kernel adds them
    to the residual stream in order."""
    from clockwork_amd import ops

    x = torch.randn(M, K, device=DEV).to(torch.bfloat16)
    w = (torch.randn(N, K, device=DEV) / K ** 0.5).to(torch.bfloat16)
    got = ops.linear(x, w, partial_ok=True)
    assert isinstance(got, ops.PartialSums) and got.parts.shape[0] > 1 and tuple(got.shape) == (M, N)
    want = x.float() @ w.float().t()
    torch.testing.assert_close(got.sum(), want, rtol=1e-4, atol=1e-4)
    resid = torch.randn(M, N, device=DEV)
    weight = (1 + 0.1 * torch.randn(N, device=DEV)).to(torch.bfloat16)
    out = torch.empty(M, N, device=DEV, dtype=torch.bfloat16)
    r = resid.clone()
    ops.add_rmsnorm(r, got, weight, 1e-6, out)
    torch.testing.assert_close(r, resid + want, rtol=1e-4, atol=1e-4)
    torch.testing.assert_close(out.float().cpu(), plain.rmsnorm((resid + want).cpu(), weight.float().cpu(), 1e-6), **tol(torch.bfloat16))
    rows = torch.tensor([M - 1], dtype=torch.int32, device=DEV)
    out1 = torch.empty(1, N, device=DEV, dtype=torch.bfloat16)
    r2 = resid.clone()
    ops.add_rmsnorm(r2, got, weight, 1e-6, out1, rows)
    assert torch.equal(r2, resid) and torch.equal(out1[0], out[M - 1])
    assert not isinstance(ops.linear(x, w), ops.PartialSums)


def test_rmsnorm_zero_row_and_scale_invariance():
    from clockwork_amd import ops

    H = 96
    x = torch.randn(2, H, device=DEV)
    x[1] = 0
    w = torch.ones(H, device=DEV)
    out = torch.empty(2, H, device=DEV)
    ops.add_rmsnorm(x.clone(), None, w, 1e-6, out)
    assert torch.all(out[1] == 0)
    assert abs(float(out[0].pow(2).mean().sqrt()) - 1.0) < 1e-4
    out2 = torch.empty(2, H, device=DEV)
    ops.add_rmsnorm((x * 37.0).clone(), None, w, 1e-6, out2)
    torch.testing.assert_close(out2[0], out[0], rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,hd,rotary,theta", [(4, 2, 16, 16, 1e4), (6, 1, 32, 32, 1e6), (3, 3, 48, 48, 5e4), (5, 1, 64, 32, 1e4),
                                                    (12, 2, 128, 128, 1e6)])
def test_rope_kv_write(dtype, nh, nkv, hd, rotary, theta):
    from clockwork_amd import ops

    T, rows = 9, 40
    width = (nh + 2 * nkv) * hd
    qkv = torch.randn(T, width, device=DEV).to(dtype)
    bias = (0.5 * torch.randn(width, device=DEV)).to(dtype)
    positions = torch.tensor([0, 1, 2, 3, 4000, 4001, 17, 255, 256], dtype=torch.int32, device=DEV)
    slots = torch.tensor([5, 39, 0, 17, 3, -1, 8, 21, 30], dtype=torch.int32, device=DEV)
    kc = torch.full((rows, nkv, hd), 100.0, device=DEV, dtype=dtype)
    vc = torch.full((rows, nkv, hd), 100.0, device=DEV, dtype=dtype)
    inv_freq = plain.inv_frequencies(rotary, theta).to(DEV)

    x = (qkv.float() + bias.float()).cpu()
    q = x[:, : nh * hd].view(T, nh, hd)
    k = x[:, nh * hd : (nh + nkv) * hd].view(T, nkv, hd)
    v = x[:, (nh + nkv) * hd :].view(T, nkv, hd)
    cos, sin = plain.rope_tables(positions.cpu(), rotary, theta)
    q_ref, k_ref = q.clone(), k.clone()
    q_ref[..., :rotary] = plain.apply_rope(q[..., :rotary], cos, sin)
    k_ref[..., :rotary] = plain.apply_rope(k[..., :rotary], cos, sin)

    work = qkv.clone()
    ops.rope_kv_write(work, bias, positions, slots, inv_freq, rotary, nh, nkv, hd, kc, vc)
    t = dict(rtol=1e-5, atol=2e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(work[:, : nh * hd].float().cpu().view(T, nh, hd), q_ref, **t)
    written = set()
    for i, s in enumerate(slots.tolist()):
        if s < 0:
            continue
        written.add(s)
        torch.testing.assert_close(kc[s].float().cpu(), k_ref[i], **t)
        torch.testing.assert_close(vc[s].float().cpu(), v[i], **t)
    for s in range(rows):
        if s not in written:
            assert torch.all(kc[s] == 100.0) and torch.all(vc[s] == 100.0)


@pytest.mark.parametrize("bias_dtype", [None, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("nh,nkv,hd", [(12, 2, 128), (5, 1, 48), (2, 2, 256)])
def test_rope_kv_write_in_16_byte_pieces_equals_the_kernel_for_any_row(nh, nkv, hd, bias_dtype):
    """bfloat16 rows whose heads are rotated whole go through a kernel that moves 16 bytes at a
    time; rows that do not lie on a 16-byte boundary go through the one that moves single
    elements. The same rows through both: the same bits, in q and in the cache."""
    from clockwork_amd import ops

    T, rows = 37, 64
    width = (nh + 2 * nkv) * hd
    gen = torch.Generator(device="cpu").manual_seed(nh * hd)
    values = torch.randn(T, width, generator=gen).to(torch.bfloat16)
    bias = None if bias_dtype is None else (0.5 * torch.randn(width, generator=gen)).to(bias_dtype).to(DEV)
    positions = torch.randint(0, 30000, (T,), generator=gen).to(torch.int32).to(DEV)
    slots = torch.randperm(rows, generator=gen)[:T].to(torch.int32)
    slots[5] = -1
    slots = slots.to(DEV)
    inv_freq = plain.inv_frequencies(hd, 1e6).to(DEV)
    results = []
    for shift in (0, 4):   # 4 elements: 8 bytes off the boundary
        store = torch.zeros(T * width + 8, dtype=torch.bfloat16, device=DEV)
        work = store[shift : shift + T * width].view(T, width)
        work.copy_(values)
        assert (work.data_ptr() % 16 == 0) == (shift == 0)
        kc = torch.full((rows, nkv, hd), 100.0, device=DEV, dtype=torch.bfloat16)
        vc = torch.full((rows, nkv, hd), 100.0, device=DEV, dtype=torch.bfloat16)
        ops.rope_kv_write(work, bias, positions, slots, inv_freq, hd, nh, nkv, hd, kc, vc)
        results.append((work[:, : nh * hd].clone(), kc, vc))
    for a, b in zip(*results):
        assert torch.equal(a, b)


@pytest.mark.parametrize("M", [1, 8, 16, 17, 33, 64])
@pytest.mark.parametrize("nh,nkv,hd,K,theta,bias_dtype", [(12, 2, 128, 1536, 1e6, torch.bfloat16), (6, 1, 32, 192, 1e6, torch.float32),
                                                         (4, 2, 16, 64, 1e4, torch.bfloat16), (3, 3, 48, 80, 5e4, None)])
def test_fused_qkv_rope_cache_write(M, nh, nkv, hd, K, theta, bias_dtype):
    """The one-kernel q/k/v product + bias + rotary + cache write against product, then rotation."""
    from clockwork_amd import ops

    width = (nh + 2 * nkv) * hd
    x = torch.randn(M, K, device=DEV).to(torch.bfloat16)
    w = (torch.randn(width, K, device=DEV) / K ** 0.5).to(torch.bfloat16)
    bias = None if bias_dtype is None else (0.5 * torch.randn(width, device=DEV)).to(bias_dtype)
    positions = torch.randint(0, 5000, (M,), dtype=torch.int32, device=DEV)
    slots = torch.randperm(80, device=DEV)[:M].to(torch.int32)
    if M > 2:
        slots[1] = -1  # a padding row of a captured decode batch: no cache row
    kc = torch.full((80, nkv, hd), 100.0, device=DEV, dtype=torch.bfloat16)
    vc = torch.full((80, nkv, hd), 100.0, device=DEV, dtype=torch.bfloat16)
    inv_freq = plain.inv_frequencies(hd, theta).to(DEV)
    q = ops.qkv_rope_fused(x, w, bias, positions, slots, inv_freq, nh, nkv, hd, kc, vc)

    y = (x.float() @ w.float().t()).cpu()
    if bias is not None:
        y = y + bias.float().cpu()
    cos, sin = plain.rope_tables(positions.cpu(), hd, theta)
    q_ref = plain.apply_rope(y[:, : nh * hd].view(M, nh, hd), cos, sin)
    k_ref = plain.apply_rope(y[:, nh * hd : (nh + nkv) * hd].view(M, nkv, hd), cos, sin)
    v_ref = y[:, (nh + nkv) * hd :].view(M, nkv, hd)
    t = dict(rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(q.float().cpu().view(M, nh, hd), q_ref, **t)
    written = set()
    for i, sl in enumerate(slots.tolist()):
        if sl < 0:
            continue
        written.add(sl)
        torch.testing.assert_close(kc[sl].float().cpu(), k_ref[i], **t)
        torch.testing.assert_close(vc[sl].float().cpu(), v_ref[i], **t)
    for sl in range(80):
        if sl not in written:
            assert torch.all(kc[sl] == 100.0) and torch.all(vc[sl] == 100.0)


def test_rope_is_relative_and_identity_at_zero():
    """<R_m q, R_n k> depends on m - n only; position 0 rotates nothing; values pass through."""
    from clockwork_amd import ops

    nh, nkv, hd = 1, 1, 32
    inv_freq = plain.inv_frequencies(hd, 1e4).to(DEV)
    base = torch.randn(1, 3 * hd, device=DEV)

    def rotated(pos_q, pos_k):
        out = []
        for pos in (pos_q, pos_k):
            qkv = base.clone()
            kc = torch.zeros(1, 1, hd, device=DEV)
            vc = torch.zeros(1, 1, hd, device=DEV)
            ops.rope_kv_write(qkv, None, torch.tensor([pos], dtype=torch.int32, device=DEV),
                              torch.tensor([0], dtype=torch.int32, device=DEV), inv_freq, hd, nh, nkv, hd, kc, vc)
            out.append((qkv[0, :hd].clone(), kc[0, 0].clone(), vc[0, 0].clone()))
        return out

    (q0, k0, v0), _ = rotated(0, 0)
    torch.testing.assert_close(q0, base[0, :hd], rtol=0, atol=0)
    torch.testing.assert_close(k0, base[0, hd : 2 * hd], rtol=0, atol=0)
    torch.testing.assert_close(v0, base[0, 2 * hd :], rtol=0, atol=0)
    (qa, _, _), (_, kb, _) = rotated(7, 3)
    (qc, _, _), (_, kd, _) = rotated(107, 103)
    assert abs(float(qa @ kb) - float(qc @ kd)) < 1e-4
    assert abs(float(qa @ kb) - float(q0 @ k0)) > 1e-3  # and it does depend on the distance


# the last four are summed in parts over K: 22 parts of 416 of a down product, 6 of 256 that a
# block sums itself (more than 256 rows), parts whose last is short (K = 1000: 3 of 336), a K that
# no part's length divides
@pytest.mark.parametrize("M,N,K", [(1, 100, 176), (7, 64, 33), (64, 130, 64), (130, 17, 1000), (3, 1000, 192),
                                   (8, 1536, 8960), (300, 1536, 1536), (1, 2048, 1000), (9, 70, 777)])
def test_gemm_f32(M, N, K):
    from clockwork_amd import ops

    x = torch.randn(M, K, device=DEV)
    w = torch.randn(N, K, device=DEV)
    b = torch.randn(N, device=DEV)
    want = (x.double() @ w.double().t() + b.double()).float()
    got = ops.linear(x, w, b)
    torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-5 * math.sqrt(K))
    got = ops.linear(x, w)
    torch.testing.assert_close(got, (x.double() @ w.double().t()).float(), rtol=1e-5, atol=1e-5 * math.sqrt(K))


def test_gemm_f32_rows_do_not_depend_on_batch():
    from clockwork_amd import ops

    x = torch.randn(70, 200, device=DEV)
    w = torch.randn(90, 200, device=DEV)
    whole = ops.linear(x, w)
    for i in (0, 33, 69):
        assert torch.equal(ops.linear(x[i : i + 1].contiguous(), w)[0], whole[i])
    # a product that is summed in parts over K, by blocks of their own for few rows and inside a
    # block for many: the same bits for a row alone, among 300 and among 17
    x = torch.randn(300, 1024, device=DEV)
    w = torch.randn(90, 1024, device=DEV)
    b = torch.randn(90, device=DEV)
    assert ops._load("gemm").cw_gemm_f32_workspace_floats(17, 90, 1024) == 4 * 17 * 90
    assert ops._load("gemm").cw_gemm_f32_workspace_floats(300, 90, 1024) == 0
    whole = ops.linear(x, w, b)
    for i in (0, 255, 256, 299):
        assert torch.equal(ops.linear(x[i : i + 1].contiguous(), w, b)[0], whole[i])
    assert torch.equal(ops.linear(x[250:267].contiguous(), w, b), whole[250:267])


@pytest.mark.parametrize("M", [1, 8, 16, 17, 33, 64])
@pytest.mark.parametrize("N,K", [(100, 176), (2048, 1536), (48, 64), (5000, 200)])
def test_skinny_bf16_product(M, N, K):
    """Few rows of x against a streamed weight matrix: bfloat16 and float32 outputs."""
    from clockwork_amd import ops

    x = torch.randn(M, K, device=DEV).to(torch.bfloat16)
    w = (torch.randn(N, K, device=DEV) / K ** 0.5).to(torch.bfloat16)
    want = x.float() @ w.float().t()
    got32 = ops.linear(x, w, out_dtype=torch.float32)
    assert got32.dtype == torch.float32
    if M <= ops.SKINNY_MAX_ROWS:
        torch.testing.assert_close(got32, want, rtol=1e-4, atol=1e-4)  # float32 accumulation of exact products
    else:
        torch.testing.assert_close(got32, want, rtol=1e-2, atol=1e-2)  # the library product rounds to bfloat16
    got = ops.linear(x, w)
    assert got.dtype == torch.bfloat16
    torch.testing.assert_close(got.float(), want, rtol=1e-2, atol=1e-2)
    # a row's result does not depend on the other rows, beyond the rounding of a different split of K
    alone = ops.linear(x[M - 1 :].contiguous(), w, out_dtype=torch.float32)[0]
    if M <= ops.SKINNY_MAX_ROWS:
        torch.testing.assert_close(alone, got32[M - 1], rtol=1e-5, atol=1e-5)
    else:
        torch.testing.assert_close(alone, got32[M - 1], rtol=1e-2, atol=1e-2)
    # and not at all on rows that share its launch shape
    if M > 1:
        other = x.clone()
        other[0] = 0
        assert torch.equal(ops.linear(other, w, out_dtype=torch.float32)[M - 1], got32[M - 1])


@pytest.mark.parametrize("M", [3, 16, 17, 32, 40, 64])
def test_streaming_product_many_row_tiles(M):
    """Shapes that the persistent streaming kernel takes (many row tiles, a short K per wave),
    with up to 64 rows of x: plain, float32, gated and partial-sum outputs. The sizes are no
    multiples of the tiles."""
    from clockwork_amd import ops

    lib = ops._load("gemm")
    N, K = 8192 + 40, 1536
    x = torch.randn(M, K, device=DEV).to(torch.bfloat16)
    w = (torch.randn(N, K, device=DEV) / K ** 0.5).to(torch.bfloat16)
    assert lib.cw_gemm_bf16_skinny_fast(0, M, N, K) == 1
    want = x.float() @ w.float().t()
    got32 = ops.linear(x, w, out_dtype=torch.float32)
    torch.testing.assert_close(got32, want, rtol=1e-4, atol=1e-4)
    got = ops.linear(x, w)
    assert got.dtype == torch.bfloat16
    torch.testing.assert_close(got.float(), want, rtol=1e-2, atol=1e-2)
    alone = ops.linear(x[M - 1 :].contiguous(), w, out_dtype=torch.float32)[0]
    torch.testing.assert_close(alone, got32[M - 1], rtol=1e-5, atol=1e-5)
    # gated: I no multiple of 8
    I = 4100 + 4
    wg = (torch.randn(2 * I, K, device=DEV) / K ** 0.5).to(torch.bfloat16)
    assert lib.cw_gemm_bf16_skinny_fast(2, M, 2 * I, K) == 1
    y = x.float() @ wg.float().t()
    torch.testing.assert_close(ops.linear_swiglu(x, wg).float(), torch.nn.functional.silu(y[:, :I]) * y[:, I:],
                               rtol=2e-2, atol=2e-2)
    # partial sums over a long K: K no multiple of 32 * waves * splits
    N2, K2 = 1536 + 8, 8960 + 8
    x2 = torch.randn(M, K2, device=DEV).to(torch.bfloat16)
    w2 = (torch.randn(N2, K2, device=DEV) / K2 ** 0.5).to(torch.bfloat16)
    parts = ops.linear(x2, w2, partial_ok=True)
    assert isinstance(parts, ops.PartialSums) and parts.parts.shape[0] == lib.cw_gemm_bf16_skinny_ksplits(M, N2, K2) > 1
    torch.testing.assert_close(parts.parts.sum(0), x2.float() @ w2.float().t(), rtol=1e-4, atol=2e-4)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,H", [(3, 176), (9, 1536), (2, 5000)])
def test_add_rmsnorm_two_pending_deltas(dtype, T, H):
    """Two branch outputs still to be added: the result is that of adding them one after the
    other, bit for bit, with and without a row selection."""
    from clockwork_amd import ops

    resid = torch.randn(T, H, device=DEV)
    a = torch.randn(T, H, device=DEV).to(dtype)
    b = torch.randn(T, H, device=DEV).to(dtype)
    parts = torch.randn(3, T, H, device=DEV)
    w = (1 + 0.1 * torch.randn(H, device=DEV)).to(dtype)
    for second in (b, ops.PartialSums(parts)):
        r1 = resid.clone()
        ops.add_rmsnorm(r1, a, w, 1e-6, torch.empty(T, H, device=DEV, dtype=dtype))
        o1 = ops.add_rmsnorm(r1, second, w, 1e-6, torch.empty(T, H, device=DEV, dtype=dtype))
        r2 = resid.clone()
        o2 = ops.add_rmsnorm(r2, ops.PendingPair(a, second), w, 1e-6, torch.empty(T, H, device=DEV, dtype=dtype))
        assert torch.equal(r1, r2) and torch.equal(o1, o2)
        r3 = resid.clone()
        rows = torch.tensor([T - 1, 0], dtype=torch.int32, device=DEV)
        o3 = ops.add_rmsnorm(r3, ops.PendingPair(a, second), w, 1e-6, torch.empty(2, H, device=DEV, dtype=dtype), rows)
        assert torch.equal(r3, resid) and torch.equal(o3, o1[[T - 1, 0]])
    # a lazy norm computes its value without touching the residual
    r4 = resid.clone()
    lazy = ops.LazyAddNorm(r4, a, w, 1e-6, dtype)
    r5 = resid.clone()
    o5 = ops.add_rmsnorm(r5, a, w, 1e-6, torch.empty(T, H, device=DEV, dtype=dtype))
    assert torch.equal(lazy.value(), o5) and torch.equal(r4, resid)


@pytest.mark.parametrize("M", [1, 5, 16])
@pytest.mark.parametrize("norm_weight_dtype", [torch.bfloat16, torch.float32])
def test_swiglu_product_with_the_norm_inside(M, norm_weight_dtype):
    """gate/up product that makes its own input rmsnorm(resid + delta): against the two kernels
    it replaces and against float32 arithmetic; the residual is left alone."""
    from clockwork_amd import ops

    K, I = 1536, 4360 + 4
    resid = torch.randn(M, K, device=DEV)
    delta = torch.randn(M, K, device=DEV).to(torch.bfloat16)
    nw = (1 + 0.1 * torch.randn(K, device=DEV)).to(norm_weight_dtype)
    w = (torch.randn(2 * I, K, device=DEV) / K ** 0.5).to(torch.bfloat16)
    assert ops.swiglu_norm_fusable(M, 2 * I, K, torch.bfloat16, w, delta)
    before = resid.clone()
    got = ops.linear_swiglu(ops.LazyAddNorm(resid, delta, nw, 1e-6, torch.bfloat16), w)
    assert torch.equal(resid, before)
    x = ops.add_rmsnorm(resid.clone(), delta, nw, 1e-6, torch.empty(M, K, device=DEV, dtype=torch.bfloat16))
    two_kernels = ops.linear_swiglu(x, w)
    torch.testing.assert_close(got.float(), two_kernels.float(), rtol=2e-2, atol=2e-2)
    v = resid + delta.float()
    xn = (v * torch.rsqrt((v * v).mean(-1, keepdim=True) + 1e-6)).to(torch.bfloat16).float() * nw.float()
    y = xn.to(torch.bfloat16).float() @ w.float().t()
    torch.testing.assert_close(got.float(), torch.nn.functional.silu(y[:, :I]) * y[:, I:], rtol=2e-2, atol=2e-2)
    # a shape the fused kernel does not take falls back to the norm kernel and the plain product
    small = (torch.randn(2 * 96, K, device=DEV) / K ** 0.5).to(torch.bfloat16)
    assert not ops.swiglu_norm_fusable(M, 2 * 96, K, torch.bfloat16, small, delta)
    torch.testing.assert_close(ops.linear_swiglu(ops.LazyAddNorm(resid, delta, nw, 1e-6, torch.bfloat16), small).float(),
                               ops.linear_swiglu(x, small).float(), rtol=0, atol=0)


@pytest.mark.parametrize("M", [1, 8, 20, 64, 100])
@pytest.mark.parametrize("I,K", [(176, 64), (8960, 1536), (100, 80), (52, 200)])
def test_fused_swiglu_product(M, I, K):
    from clockwork_amd import ops

    x = torch.randn(M, K, device=DEV).to(torch.bfloat16)
    w = (torch.randn(2 * I, K, device=DEV) / K ** 0.5).to(torch.bfloat16)
    got = ops.linear_swiglu(x, w)
    y = x.float() @ w.float().t()
    want = torch.nn.functional.silu(y[:, :I]) * y[:, I:]
    torch.testing.assert_close(got.float(), want, rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("M,N,K", [(300, 1000, 200), (2048, 1536, 1536), (129, 130, 72), (64, 256, 8), (1000, 52, 2048)])
def test_tiled_product(M, N, K):
    """The LDS-tiled matrix-core product: plain with a bias of either type, and gated; sizes that
    are no multiples of the 128 x 128 x 64 tile; rows of x with a stride."""
    from clockwork_amd import ops

    wide = torch.randn(M, K + 16, device=DEV).to(torch.bfloat16)
    x = wide[:, :K]  # row stride K + 16
    w = (torch.randn(N, K, device=DEV) / K ** 0.5).to(torch.bfloat16)
    want = x.float() @ w.float().t()
    torch.testing.assert_close(ops.linear_tiled(x, w).float(), want, rtol=1e-2, atol=1e-2)
    for bias_dtype in (torch.bfloat16, torch.float32):
        b = torch.randn(N, device=DEV).to(bias_dtype)
        torch.testing.assert_close(ops.linear_tiled(x, w, b).float(), want + b.float(), rtol=1e-2, atol=2e-2)
    if N % 2 == 0:
        I = N // 2
        got = ops.linear_tiled(x, w, swiglu=True)
        assert tuple(got.shape) == (M, I)
        torch.testing.assert_close(got.float(), torch.nn.functional.silu(want[:, :I]) * want[:, I:], rtol=2e-2, atol=2e-2)
    # a row does not depend on the other rows of the batch
    alone = ops.linear_tiled(x[M - 1 :], w)
    assert torch.equal(alone[0], ops.linear_tiled(x, w)[M - 1])


@pytest.mark.parametrize("M,N,K", [(300, 1000, 256), (777, 2 * 489, 320), (1000, 2 * 488, 448), (257, 200, 1024),
                                   (2048, 2 * 1000, 1536), (513, 4000, 704)])
def test_wide_tile_product(M, N, K):
    """The product with 256 x 192 tiles, whose operands go from memory straight into LDS: plain
    with a bias of either type, and gated; sizes that are no multiples of the tile, outputs whose
    rows are no multiples of 16 bytes, rows of x with a stride, more tiles than one round of
    workgroups and fewer; a row does not depend on the other rows of the batch."""
    from clockwork_amd import ops

    padded = torch.randn(M, K + 24, device=DEV).to(torch.bfloat16)
    x = padded[:, :K]  # row stride K + 24
    w = (torch.randn(N, K, device=DEV) / K ** 0.5).to(torch.bfloat16)
    want = x.float() @ w.float().t()
    got = ops.linear_tiled(x, w, wide=True)
    torch.testing.assert_close(got.float(), want, rtol=1e-2, atol=1e-2)
    for bias_dtype in (torch.bfloat16, torch.float32):
        b = torch.randn(N, device=DEV).to(bias_dtype)
        torch.testing.assert_close(ops.linear_tiled(x, w, b, wide=True).float(), want + b.float(), rtol=1e-2, atol=2e-2)
    I = N // 2
    gated = ops.linear_tiled(x, w, swiglu=True, wide=True)
    assert tuple(gated.shape) == (M, I)
    torch.testing.assert_close(gated.float(), torch.nn.functional.silu(want[:, :I]) * want[:, I:], rtol=2e-2, atol=2e-2)
    alone = ops.linear_tiled(x[M - 1 :], w, wide=True)
    assert torch.equal(alone[0], got[M - 1])
    # the same bits as the kernel with the small tiles would not be promised; the same product is
    torch.testing.assert_close(got.float(), ops.linear_tiled(x, w, wide=False).float(), rtol=1e-2, atol=1e-2)


def test_wide_tile_product_finds_one_large_entry():
    """A product is a sum over all of K and over the right rows: one large element of x and of W
    shows in exactly one output, whatever stage, fragment and lane hold it."""
    from clockwork_amd import ops

    M, N, K = 520, 2 * 300, 1024
    g = torch.Generator(device="cpu").manual_seed(3)
    for _ in range(6):
        m, n, k = (int(torch.randint(0, hi, (1,), generator=g)) for hi in (M, N, K))
        x = torch.zeros(M, K, device=DEV, dtype=torch.bfloat16)
        w = torch.zeros(N, K, device=DEV, dtype=torch.bfloat16)
        x[m, k], w[n, k] = 3.0, 5.0
        y = ops.linear_tiled(x, w, wide=True).float()
        assert y[m, n].item() == 15.0 and torch.count_nonzero(y).item() == 1, (m, n, k)


def test_wide_tile_product_refuses_what_it_does_not_take():
    from clockwork_amd import ops
    from clockwork_amd.ops import KernelError

    x = torch.randn(300, 200, device=DEV).to(torch.bfloat16)   # K no multiple of 64
    w = torch.randn(128, 200, device=DEV).to(torch.bfloat16)
    with pytest.raises(KernelError):
        ops.linear_tiled(x, w, wide=True)
    assert not ops.wide_swiglu_pays(2048, 2 * 8960, 1500, 1500)
    # the gate/up product of the 1.5B and 7B shapes: long portions take the kernel, short ones do not
    assert ops.wide_swiglu_pays(2048, 2 * 8960, 1536, 1536) and ops.wide_swiglu_pays(512, 2 * 8960, 1536, 1536)
    assert not ops.wide_swiglu_pays(256, 2 * 8960, 1536, 1536)
    assert ops.wide_swiglu_pays(1024, 2 * 18944, 3584, 3584) and not ops.wide_swiglu_pays(512, 2 * 18944, 3584, 3584)


def test_gate_up_of_a_long_portion_goes_through_the_wide_tile_kernel():
    from clockwork_amd import ops

    x = torch.randn(1024, 1536, device=DEV).to(torch.bfloat16)
    w = (torch.randn(2 * 8960, 1536, device=DEV) / 40).to(torch.bfloat16)
    calls = []
    real = ops.linear_tiled
    ops.linear_tiled = lambda *a, **k: (calls.append(k), real(*a, **k))[1]
    try:
        got = ops.linear_swiglu(x, w)
        few = ops.linear_swiglu(x[:100], w)
    finally:
        ops.linear_tiled = real
    assert len(calls) == 1 and calls[0].get("wide") is True
    y = x.float() @ w.float().t()
    want = torch.nn.functional.silu(y[:, :8960]) * y[:, 8960:]
    torch.testing.assert_close(got.float(), want, rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(few.float(), want[:100], rtol=2e-2, atol=2e-2)


def test_a_tuning_start_up_measures_which_gate_up_product_is_faster():
    """While the library tunes, the first long portion of a weight shape times both ways and the
    choice is kept by the engine's own policy: later products of that shape follow it, and a
    call on behalf of another engine (another policy) knows nothing of it."""
    from clockwork_amd import ops

    x = torch.randn(1024, 1536, device=DEV).to(torch.bfloat16)
    w = (torch.randn(2 * 8960, 1536, device=DEV) / 40).to(torch.bfloat16)
    key = (2 * 8960, 1536)
    policy = ops.ProductPolicy()
    calls = []
    real = ops.linear_tiled
    ops.linear_tiled = lambda *a, **k: (calls.append(k), real(*a, **k))[1]
    try:
        policy.tuning = True   # what library_tuning(policy) sets, without touching the library's own tuner
        first = ops.linear_swiglu(x, w, policy=policy)
        policy.tuning = False
        assert key in policy.swiglu_choices and not ops.DEFAULT_POLICY.swiglu_choices
        for choice in (False, True):
            policy.swiglu_choices[key] = choice
            calls.clear()
            again = ops.linear_swiglu(x, w, policy=policy)
            assert bool(calls) == choice
            torch.testing.assert_close(again.float(), first.float(), rtol=2e-2, atol=2e-2)
        # fewer rows than the measurement speaks for: the rule, not the choice
        policy.swiglu_choices[key] = False
        calls.clear()
        ops.linear_swiglu(x[:512], w, policy=policy)
        assert calls
        # another engine's calls follow the rule too, whatever this one has measured
        calls.clear()
        ops.linear_swiglu(x, w, policy=ops.ProductPolicy())
        ops.linear_swiglu(x, w)
        assert len(calls) == 2
    finally:
        ops.linear_tiled = real


def test_a_tuning_start_up_times_plain_products_too():
    """A plain product of many rows is timed against the library's while the library tunes, if it
    has tiles enough; the choice then holds for the shape, and untimed shapes take the library."""
    from clockwork_amd import ops

    x = torch.randn(2048, 1024, device=DEV).to(torch.bfloat16)
    w = (torch.randn(3584, 1024, device=DEV) / 32).to(torch.bfloat16)     # 8 x 19 tiles
    small = (torch.randn(512, 1024, device=DEV) / 32).to(torch.bfloat16)  # 8 x 3 tiles
    b = torch.randn(3584, device=DEV).to(torch.bfloat16)
    policy = ops.ProductPolicy()
    calls = []
    real = ops.linear_tiled
    ops.linear_tiled = lambda *a, **k: (calls.append(k), real(*a, **k))[1]
    try:
        want = ops.linear(x, w, b, policy=policy)
        assert not calls and not policy.product_choices       # nothing is timed outside a tuning start-up
        policy.tuning = True
        ops.linear(x, w, b, policy=policy)
        ops.linear(x, small, policy=policy)
        policy.tuning = False
        assert (3584, 1024, True) in policy.product_choices and policy.product_choices[(512, 1024, False)] is False
        assert not ops.DEFAULT_POLICY.product_choices
        for choice in (True, False):
            policy.product_choices[(3584, 1024, True)] = choice
            calls.clear()
            got = ops.linear(x, w, b, policy=policy)
            assert bool(calls) == choice
            torch.testing.assert_close(got.float(), want.float(), rtol=2e-2, atol=2e-2)
        calls.clear()
        policy.product_choices[(3584, 1024, True)] = True
        ops.linear(x[:512], w, b, policy=policy)          # too few rows for the measurement to speak for
        ops.linear(x, w, policy=policy)                   # another shape (no bias): never timed
        ops.linear(x, w, b)                               # no engine behind the call: the library
        assert not calls
    finally:
        ops.linear_tiled = real


def test_hip_products_switch_routes_large_products_to_the_tiled_kernel():
    from clockwork_amd import ops

    x = torch.randn(200, 96, device=DEV).to(torch.bfloat16)
    w = (torch.randn(2 * 70, 96, device=DEV) / 10).to(torch.bfloat16)
    b = torch.randn(140, device=DEV).to(torch.bfloat16)
    lib_y, lib_g = ops.linear(x, w, b), ops.linear_swiglu(x, w)
    calls = []
    real = ops.linear_tiled
    ops.linear_tiled = lambda *a, **k: (calls.append(1), real(*a, **k))[1]
    own = ops.ProductPolicy(hip_products=True)
    try:
        own_y, own_g = ops.linear(x, w, b, policy=own), ops.linear_swiglu(x, w, policy=own)
        logits = ops.linear(x, w, out_dtype=torch.float32, policy=own)
        assert len(calls) == 3
        ops.linear(x, w, b)   # a call of another engine, or of none, stays with the library
        assert len(calls) == 3
    finally:
        ops.linear_tiled = real
    assert logits.dtype == torch.float32
    torch.testing.assert_close(own_y.float(), lib_y.float(), rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(own_g.float(), lib_g.float(), rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("dtype", DTYPES)
def test_linear_library_path_and_float32_logits(dtype):
    from clockwork_amd import ops

    x = torch.randn(70, 96, device=DEV).to(dtype)
    w = torch.randn(50, 96, device=DEV).to(dtype)
    got = ops.linear(x, w, out_dtype=torch.float32)
    assert got.dtype == torch.float32
    torch.testing.assert_close(got, x.float() @ w.float().t(), **(dict(rtol=1e-5, atol=1e-4) if dtype == torch.float32 else dict(rtol=2e-2, atol=1e-1)))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,I", [(3, 176), (1, 100), (17, 384)])
def test_silu_mul(dtype, T, I):
    from clockwork_amd import ops

    gu = (2 * torch.randn(T, 2 * I, device=DEV)).to(dtype)
    gu[0, 0] = 0.0
    out = torch.empty(T, I, device=DEV, dtype=dtype)
    ops.silu_mul(gu, out)
    want = torch.nn.functional.silu(gu[:, :I].float()) * gu[:, I:].float()
    torch.testing.assert_close(out.float(), want, **tol(dtype))
    assert float(out[0, 0]) == 0.0


def test_copy_pages():
    from clockwork_amd import ops

    pool = torch.randn(6, 10, 4, 2, 8, device=DEV)
    before = pool.clone()
    ops.copy_pages(pool.view(6, 10, -1), torch.tensor([[3, 7], [0, 9]], dtype=torch.int32, device=DEV))
    want = before.clone()
    want[:, 7] = before[:, 3]
    want[:, 9] = before[:, 0]
    assert torch.equal(pool, want)


# ---------------------------------------------------------------------------------- attention
def _paged_setup(dtype, nkv, hd, bs, num_blocks, tables, ctx_lens, poison=100.0):
    """Random keys/values per request laid into scrambled pages; unowned slots hold ``poison``."""
    kc = torch.full((num_blocks * bs, nkv, hd), poison, dtype=dtype, device=DEV)
    vc = torch.full((num_blocks * bs, nkv, hd), poison, dtype=dtype, device=DEV)
    ks, vs = [], []
    for table, ctx in zip(tables, ctx_lens):
        k = torch.randn(ctx, nkv, hd, device=DEV).to(dtype)
        v = torch.randn(ctx, nkv, hd, device=DEV).to(dtype)
        for p in range(ctx):
            slot = table[p // bs] * bs + p % bs
            kc[slot], vc[slot] = k[p], v[p]
        ks.append(k)
        vs.append(v)
    return kc, vc, ks, vs


def _run_attention(dtype, nh, nkv, hd, bs, tables, ctx_lens, q_lens, kc, vc, qs, window=0, splits=None, scale=None,
                   decode_kernel=False, prefill_kernel=False, fixed_ranges=False, key_parts=0):
    from clockwork_amd import ops
    from clockwork_amd.engine.batch import StepContext
    from clockwork_amd.parts.attention import attention_plan

    ctx = StepContext()
    ctx.device = torch.device(DEV)
    ctx.h_q_lens, ctx.h_ctx_lens = list(q_lens), list(ctx_lens)
    # prefill_kernel: True or 4 for workgroups of four row blocks, 2 for two (few work items here,
    # so the plan takes the small workgroups whenever it may)
    narrow = prefill_kernel == 2 and not isinstance(prefill_kernel, bool)
    plan = attention_plan(ctx, nh, nkv, narrow_ok=narrow)
    assert plan.mfma_row_blocks == (2 if narrow else 4)
    if splits is not None:
        plan.single_splits = splits
    R = len(q_lens)
    width = max(len(t) for t in tables)
    bt = torch.full((R, width), -1, dtype=torch.int32, device=DEV)
    for r, t in enumerate(tables):
        bt[r, : len(t)] = torch.tensor(t, dtype=torch.int32)
    cu = torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=torch.int32, device=DEV)
    cl = torch.tensor(ctx_lens, dtype=torch.int32, device=DEV)
    T = sum(q_lens)
    # queries sit inside a wider row, as they do in the fused qkv buffer
    pad = 24
    qbuf = torch.full((T, nh * hd + pad), 55.0, dtype=dtype, device=DEV)
    qbuf[:, : nh * hd] = torch.cat(qs).reshape(T, nh * hd)
    out = torch.full((T, nh * hd), -77.0, dtype=dtype, device=DEV)
    scale = scale if scale is not None else hd ** -0.5
    common = dict(q=qbuf, q_stride=qbuf.shape[1], out=out, k_cache=kc, v_cache=vc, block_tables=bt, ctx_lens=cl,
                  cu_q=cu, nh=nh, nkv=nkv, hd=hd, block_size=bs, window=window, scale=scale, n_tokens=T, n_requests=R)
    if plan.n_wide and prefill_kernel:
        assert ops.prefill_attention_supported(hd, dtype)
        items, n_items, ws = plan.mfma_items, plan.n_mfma, None
        if key_parts:  # every item's key range shared among this many workgroups (some parts may be empty)
            rec = items.cpu().numpy().reshape(-1, 4)[:n_items]
            rec = rec[(rec[:, 3] & 255) == 0]  # each item once, whatever the plan made of it
            rec = rec.repeat(key_parts, axis=0)
            rec[:, 3] = (torch.arange(len(rec)).numpy() % key_parts) | (key_parts << 8)
            items, n_items = torch.tensor(rec.reshape(-1), dtype=torch.int32, device=DEV), len(rec)
        if key_parts or plan.mfma_parts > 1:
            ws = torch.full((ops.prefill_attention_workspace_floats(hd, n_items, nh, nkv, plan.mfma_row_blocks),),
                            float("nan"), dtype=torch.float32, device=DEV)
        ops.attention_prefill(items=items, n_items=n_items, row_blocks=plan.mfma_row_blocks, workspace=ws, **common)
    elif plan.n_wide:
        n_splits, ws = key_parts or plan.wide_splits, None
        if n_splits > 1:
            chunks = -(-(nh // nkv) // plan.gh_wide)
            ws = torch.full((ops.attention_workspace_floats(hd, 64, plan.n_wide, nkv, chunks, n_splits),), float("nan"),
                            dtype=torch.float32, device=DEV)
        ops.attention(items=plan.wide_items, n_items=plan.n_wide, rows=64, gh=plan.gh_wide, n_splits=n_splits,
                      workspace=ws, **common)
    if plan.n_single and decode_kernel:
        assert ops.decode_attention_supported(hd, dtype)
        n_splits = splits if splits is not None else plan.decode_splits
        ws = None
        if n_splits > 1:
            ws = torch.full((ops.decode_attention_workspace_floats(hd, plan.n_single, nh, nkv, n_splits),), float("nan"),
                            dtype=torch.float32, device=DEV)
        extra = {}
        if fixed_ranges:  # every split at a fixed place; a batch of single tokens needs no items
            longest = max(c for c, q in zip(ctx_lens, q_lens) if q == 1)
            extra = dict(identity=plan.single_identity, split_keys=32 * -(-(-(-longest // n_splits)) // 32), max_ctx=longest)
        ops.attention_decode(items=plan.single_items, n_items=plan.n_single, n_splits=n_splits, workspace=ws, **common,
                             **extra)
    elif plan.n_single:
        ws = None
        if plan.single_splits > 1:
            ws = torch.empty(ops.attention_workspace_floats(hd, 16, plan.n_single, nkv, plan.chunks_single, plan.single_splits),
                             dtype=torch.float32, device=DEV)
        ops.attention(items=plan.single_items, n_items=plan.n_single, rows=16, gh=plan.gh_single,
                      n_splits=plan.single_splits, workspace=ws, **common)
    return out.view(T, nh, hd)


# the reference's decode cases (tests/test_triton_kernel.py:14-20) plus sizes of our own
DECODE_CASES = [
    (4, 4, 16, 4, [5, 12, 9]),
    (8, 2, 32, 4, [1, 7, 16, 3]),
    (6, 3, 64, 8, [23, 8, 31]),
    (12, 2, 128, 16, [17, 64, 49, 2]),
    (6, 1, 48, 16, [300, 33]),
    (40, 2, 16, 8, [70]),  # a group of 20 heads: more than one head chunk
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,hd,bs,ctx_lens", DECODE_CASES)
@pytest.mark.parametrize("splits", [1, 3])
def test_attention_single_tokens(dtype, nh, nkv, hd, bs, ctx_lens, splits):
    num_blocks = sum(-(-c // bs) for c in ctx_lens) + 5
    perm = torch.randperm(num_blocks).tolist()
    tables, at = [], 0
    for c in ctx_lens:
        n = -(-c // bs)
        tables.append(perm[at : at + n])
        at += n
    kc, vc, ks, vs = _paged_setup(dtype, nkv, hd, bs, num_blocks, tables, ctx_lens)
    qs = [torch.randn(1, nh, hd, device=DEV).to(dtype) for _ in ctx_lens]
    out = _run_attention(dtype, nh, nkv, hd, bs, tables, ctx_lens, [1] * len(ctx_lens), kc, vc, qs, splits=splits)
    assert not torch.isnan(out.float()).any()
    for r in range(len(ctx_lens)):
        want = plain.attention_dense(qs[r].float().cpu(), ks[r].float().cpu(), vs[r].float().cpu(), hd ** -0.5)
        torch.testing.assert_close(out[r : r + 1].float().cpu(), want, **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,hd,bs", [(4, 2, 16, 4), (6, 1, 32, 8), (3, 3, 48, 16), (12, 2, 128, 16), (2, 1, 256, 16)])
@pytest.mark.parametrize("key_parts", [0, 3])
def test_attention_portions_and_mixed_batches(dtype, nh, nkv, hd, bs, key_parts):
    """Portions (cached prefix + new tokens, end-aligned mask: clockwork/kernels/attention.py:45-65,
    tests/test_attention_kernels.py:49-62) next to single tokens, scrambled pages, poisoned free slots.
    key_parts: every portion item's keys cut three ways and merged (parts of short ranges are empty)."""
    ctx_lens = [21, 150, 2, 77, 1, 64]
    q_lens = [6, 150, 2, 1, 1, 33]
    num_blocks = sum(-(-c // bs) for c in ctx_lens) + 3
    perm = torch.randperm(num_blocks).tolist()
    tables, at = [], 0
    for c in ctx_lens:
        n = -(-c // bs)
        tables.append(perm[at : at + n])
        at += n
    kc, vc, ks, vs = _paged_setup(dtype, nkv, hd, bs, num_blocks, tables, ctx_lens)
    qs = [torch.randn(q, nh, hd, device=DEV).to(dtype) for q in q_lens]
    out = _run_attention(dtype, nh, nkv, hd, bs, tables, ctx_lens, q_lens, kc, vc, qs, key_parts=key_parts)
    at = 0
    for r, q_len in enumerate(q_lens):
        want = plain.attention_dense(qs[r].float().cpu(), ks[r].float().cpu(), vs[r].float().cpu(), hd ** -0.5)
        torch.testing.assert_close(out[at : at + q_len].float().cpu(), want, **tol(dtype))
        at += q_len


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [1, 5, 16, 40])
def test_attention_window(dtype, window):
    """A token reads itself and the window-1 tokens before it; pages behind the window may be gone
    (table entry -1) and are never dereferenced."""
    nh, nkv, hd, bs = 4, 2, 32, 8
    ctx_lens, q_lens = [90, 50, 70], [30, 1, 2]
    num_blocks = 40
    tables = [list(range(0, 12)), list(range(12, 19)), list(range(19, 28))]
    kc, vc, ks, vs = _paged_setup(dtype, nkv, hd, bs, num_blocks, tables, ctx_lens)
    tables_dev = [list(t) for t in tables]
    for r, (c, q) in enumerate(zip(ctx_lens, q_lens)):
        first_needed = max(0, (c - q) - window + 1) // bs
        for b in range(first_needed):
            tables_dev[r][b] = -1
    qs = [torch.randn(q, nh, hd, device=DEV).to(dtype) for q in q_lens]
    out = _run_attention(dtype, nh, nkv, hd, bs, tables_dev, ctx_lens, q_lens, kc, vc, qs, window=window)
    at = 0
    for r, q_len in enumerate(q_lens):
        want = plain.attention_dense(qs[r].float().cpu(), ks[r].float().cpu(), vs[r].float().cpu(), hd ** -0.5, window=window)
        torch.testing.assert_close(out[at : at + q_len].float().cpu(), want, **tol(dtype))
        at += q_len


# sizes of the bfloat16 decode kernel: head sizes 32..256, groups of 1 to 20 heads, pages of 4 to 32
DECODE_KERNEL_CASES = [
    (8, 2, 32, 4, [1, 7, 16, 3]),
    (6, 3, 64, 8, [23, 8, 31, 200]),
    (12, 2, 128, 16, [17, 64, 49, 2, 700]),
    (6, 1, 32, 16, [300, 33]),
    (40, 2, 64, 8, [70, 129]),
    (3, 3, 128, 32, [5, 1000]),
    (5, 1, 256, 16, [77, 300]),
    (14, 2, 128, 16, [2304]),
    (4, 2, 160, 16, [130, 9]),
    (3, 1, 224, 8, [400]),
]


@pytest.mark.parametrize("nh,nkv,hd,bs,ctx_lens", DECODE_KERNEL_CASES)
@pytest.mark.parametrize("splits", [1, 2, 7, 40, 256])
@pytest.mark.parametrize("fixed_ranges", [False, True])
def test_decode_attention_kernel(nh, nkv, hd, bs, ctx_lens, splits, fixed_ranges):
    dtype = torch.bfloat16
    from clockwork_amd import ops

    assert ops._load("attention", hd).cw_attention_decode_max_splits() == ops.DECODE_MAX_SPLITS == 256
    num_blocks = sum(-(-c // bs) for c in ctx_lens) + 5
    perm = torch.randperm(num_blocks).tolist()
    tables, at = [], 0
    for c in ctx_lens:
        n = -(-c // bs)
        tables.append(perm[at : at + n])
        at += n
    kc, vc, ks, vs = _paged_setup(dtype, nkv, hd, bs, num_blocks, tables, ctx_lens, poison=float("nan"))
    qs = [torch.randn(1, nh, hd, device=DEV).to(dtype) for _ in ctx_lens]
    out = _run_attention(dtype, nh, nkv, hd, bs, tables, ctx_lens, [1] * len(ctx_lens), kc, vc, qs, splits=splits,
                         decode_kernel=True, fixed_ranges=fixed_ranges)
    assert not torch.isnan(out.float()).any()
    for r in range(len(ctx_lens)):
        want = plain.attention_dense(qs[r].float().cpu(), ks[r].float().cpu(), vs[r].float().cpu(), hd ** -0.5)
        torch.testing.assert_close(out[r : r + 1].float().cpu(), want, **tol(dtype))


@pytest.mark.parametrize("nh,nkv,hd,bs", [(4, 2, 32, 4), (6, 1, 32, 8), (3, 3, 64, 16), (12, 2, 128, 16), (2, 1, 256, 16),
                                          (40, 1, 64, 8), (7, 7, 96, 16), (4, 2, 160, 16), (2, 2, 224, 8)])
@pytest.mark.parametrize("window", [0, 9, 40])
@pytest.mark.parametrize("row_blocks", [4, 2])
def test_prefill_attention_kernel(nh, nkv, hd, bs, window, row_blocks):
    """The matrix-core kernel for portions: cached prefix + new tokens, ragged sizes, groups that
    do not divide 32, a group larger than 32, single tokens in the same batch, poisoned pages."""
    dtype = torch.bfloat16
    if row_blocks == 2 and hd > 128:
        pytest.skip("head sizes beyond 128 have the kernel with four row blocks only")
    ctx_lens = [21, 150, 2, 77, 1, 64, 333]
    q_lens = [6, 150, 2, 1, 1, 33, 40]
    num_blocks = sum(-(-c // bs) for c in ctx_lens) + 3
    perm = torch.randperm(num_blocks).tolist()
    tables, at = [], 0
    for c in ctx_lens:
        n = -(-c // bs)
        tables.append(perm[at : at + n])
        at += n
    kc, vc, ks, vs = _paged_setup(dtype, nkv, hd, bs, num_blocks, tables, ctx_lens, poison=float("nan"))
    tables_dev = [list(t) for t in tables]
    if window:
        for r, (c, q) in enumerate(zip(ctx_lens, q_lens)):
            for b in range(max(0, (c - q) - window + 1) // bs):
                tables_dev[r][b] = -1
    qs = [torch.randn(q, nh, hd, device=DEV).to(dtype) for q in q_lens]
    out = _run_attention(dtype, nh, nkv, hd, bs, tables_dev, ctx_lens, q_lens, kc, vc, qs, window=window,
                         prefill_kernel=row_blocks, decode_kernel=ops_decode_ok(hd))
    assert not torch.isnan(out.float()).any()
    at = 0
    for r, q_len in enumerate(q_lens):
        want = plain.attention_dense(qs[r].float().cpu(), ks[r].float().cpu(), vs[r].float().cpu(), hd ** -0.5,
                                     window=window or None)
        torch.testing.assert_close(out[at : at + q_len].float().cpu(), want, **tol(dtype))
        at += q_len


@pytest.mark.parametrize("nh,nkv,hd,bs", [(4, 2, 32, 4), (12, 2, 128, 16), (2, 1, 256, 16), (40, 1, 64, 8), (7, 7, 96, 16)])
@pytest.mark.parametrize("window", [0, 40])
@pytest.mark.parametrize("row_blocks", [4, 2])
@pytest.mark.parametrize("key_parts", [2, 5])
def test_prefill_attention_kernel_with_shared_key_ranges(nh, nkv, hd, bs, window, row_blocks, key_parts):
    """Every item's keys in 2 or 5 parts, each a workgroup of its own, put together by the merge
    kernel: contexts of one stage (all parts but the first empty) up to many stages, a portion
    behind a cached prefix, single-token requests in between, NaN in unowned pages and in the
    workspace."""
    dtype = torch.bfloat16
    if row_blocks == 2 and hd > 128:
        pytest.skip("head sizes beyond 128 have the kernel with four row blocks only")
    ctx_lens = [21, 700, 2, 1, 333, 1100]
    q_lens = [6, 150, 2, 1, 333, 64]
    num_blocks = sum(-(-c // bs) for c in ctx_lens) + 3
    perm = torch.randperm(num_blocks).tolist()
    tables, at = [], 0
    for c in ctx_lens:
        n = -(-c // bs)
        tables.append(perm[at : at + n])
        at += n
    kc, vc, ks, vs = _paged_setup(dtype, nkv, hd, bs, num_blocks, tables, ctx_lens, poison=float("nan"))
    tables_dev = [list(t) for t in tables]
    if window:
        for r, (c, q) in enumerate(zip(ctx_lens, q_lens)):
            for b in range(max(0, (c - q) - window + 1) // bs):
                tables_dev[r][b] = -1
    qs = [torch.randn(q, nh, hd, device=DEV).to(dtype) for q in q_lens]
    out = _run_attention(dtype, nh, nkv, hd, bs, tables_dev, ctx_lens, q_lens, kc, vc, qs, window=window,
                         prefill_kernel=row_blocks, decode_kernel=ops_decode_ok(hd), key_parts=key_parts)
    assert not torch.isnan(out.float()).any()
    at = 0
    for r, q_len in enumerate(q_lens):
        want = plain.attention_dense(qs[r].float().cpu(), ks[r].float().cpu(), vs[r].float().cpu(), hd ** -0.5,
                                     window=window or None)
        torch.testing.assert_close(out[at : at + q_len].float().cpu(), want, **tol(dtype))
        at += q_len


def test_the_plan_shares_long_key_ranges_among_workgroups():
    """A short portion behind a long cached prefix makes few workgroups with long walks: its items
    are cut into as many parts as there are idle compute units for. A launch that fills the card
    (a whole prompt of 2048 tokens) and items with few keys are left alone."""
    import numpy as np

    from clockwork_amd.engine.batch import StepContext
    from clockwork_amd.parts.attention import MAX_PARTS, MIN_PART_KEYS, attention_plan

    def plan_of(q_lens, ctx_lens):
        ctx = StepContext()
        ctx.device = torch.device(DEV)
        ctx.h_q_lens, ctx.h_ctx_lens = list(q_lens), list(ctx_lens)
        assert ctx.num_compute_units == 256
        plan = attention_plan(ctx, 12, 2, narrow_ok=True)
        return plan, plan.mfma_items.cpu().numpy().reshape(-1, 4)[: plan.n_mfma]

    plan, items = plan_of([2048], [2048])
    assert plan.mfma_parts == 1 and (items[:, 3] == 0).all()
    plan, items = plan_of([200], [8392])  # 10 items of 20 tokens on 2 key/value heads: 20 workgroups, 12 parts each
    assert plan.mfma_row_blocks == 4 and plan.mfma_parts == 12 and plan.n_mfma == 120
    parts, part = (items[:, 3] >> 8) & 255, items[:, 3] & 255
    assert (parts == 12).all() and items[part == 0][:, 2].sum() == 200  # every token in one item before the items were repeated
    for i in np.flatnonzero(part == 0):  # the parts of an item follow one another
        assert (items[i : i + 12, :3] == items[i, :3]).all() and list(part[i : i + 12]) == list(range(12))
    plan, items = plan_of([16], [30016])  # 4 workgroups: as many parts as the kernel's list allows
    assert plan.mfma_parts == MAX_PARTS == 64 and 30000 // MAX_PARTS >= MIN_PART_KEYS
    plan, items = plan_of([100, 1, 1], [100, 500, 700])  # few workgroups, but of few keys
    assert plan.mfma_parts == 1 and (items[:, 3] == 0).all()


@pytest.mark.parametrize("window", [0, 700])
@pytest.mark.parametrize("row_blocks", [4, 2])
def test_prefill_attention_kernel_long_block_table(window, row_blocks):
    """More pages than the kernel holds of a block table at a time (pages of one key): the table
    window moves on while the keys are walked."""
    dtype = torch.bfloat16
    nh, nkv, hd, bs = 4, 2, 64, 1
    ctx, q_len = 2500, 200
    table = torch.randperm(ctx + 5).tolist()[:ctx]
    kc, vc, ks, vs = _paged_setup(dtype, nkv, hd, bs, ctx + 5, [table], [ctx], poison=float("nan"))
    q = torch.randn(q_len, nh, hd, device=DEV).to(dtype)
    # one far key that every query of head 0 looks at
    ks[0][37, 0] *= 0  # keep the reference tensors in step with the cache
    kc[table[37], 0] = 0
    kc[table[37], 0, :8] = 4.0
    ks[0][37, 0, :8] = 4.0
    q[:, 0, :8] = 4.0
    tables_dev = [list(table)]
    if window:
        for b in range(max(0, (ctx - q_len) - window + 1)):
            tables_dev[0][b] = -1
    out = _run_attention(dtype, nh, nkv, hd, bs, tables_dev, [ctx], [q_len], kc, vc, [q], window=window,
                         prefill_kernel=row_blocks)
    want = plain.attention_dense(q.float().cpu(), ks[0].float().cpu(), vs[0].float().cpu(), hd ** -0.5, window=window or None)
    torch.testing.assert_close(out.float().cpu(), want, **tol(dtype))


def ops_decode_ok(hd):
    from clockwork_amd import ops

    return ops.decode_attention_supported(hd, torch.bfloat16)


@pytest.mark.parametrize("row_blocks", [4, 2])
def test_prefill_attention_kernel_sharp_scores(row_blocks):
    """Scores of very different size, so that the running maximum moves from tile to tile and one
    far key dominates a row: rescaling and masking errors cannot hide behind near-uniform weights."""
    dtype = torch.bfloat16
    nh, nkv, hd, bs, T = 12, 2, 128, 16, 300
    tables = [torch.randperm(20).tolist()[:19]]
    kc, vc, ks, vs = _paged_setup(dtype, nkv, hd, bs, 20, tables, [T])
    q = (3.0 * torch.randn(T, nh, hd, device=DEV)).to(dtype)
    out = _run_attention(dtype, nh, nkv, hd, bs, tables, [T], [T], kc, vc, [q], prefill_kernel=row_blocks, scale=0.5)
    want = plain.attention_dense(q.float().cpu(), ks[0].float().cpu(), vs[0].float().cpu(), 0.5)
    torch.testing.assert_close(out.float().cpu(), want, rtol=3e-2, atol=3e-2)


@pytest.mark.parametrize("window", [1, 5, 16, 40])
@pytest.mark.parametrize("fixed_ranges", [False, True])
def test_decode_attention_kernel_window_and_mixed_batch(window, fixed_ranges):
    """Single tokens beside a portion in one batch; pages behind the window are gone (-1)."""
    dtype = torch.bfloat16
    nh, nkv, hd, bs = 4, 2, 32, 8
    ctx_lens, q_lens = [90, 50, 70, 9], [1, 1, 30, 1]
    tables = [list(range(0, 12)), list(range(12, 19)), list(range(19, 28)), [30, 31]]
    kc, vc, ks, vs = _paged_setup(dtype, nkv, hd, bs, 40, tables, ctx_lens, poison=float("nan"))
    tables_dev = [list(t) for t in tables]
    for r, (c, q) in enumerate(zip(ctx_lens, q_lens)):
        for b in range(max(0, (c - q) - window + 1) // bs):
            tables_dev[r][b] = -1
    qs = [torch.randn(q, nh, hd, device=DEV).to(dtype) for q in q_lens]
    out = _run_attention(dtype, nh, nkv, hd, bs, tables_dev, ctx_lens, q_lens, kc, vc, qs, window=window, decode_kernel=True,
                         splits=2 if fixed_ranges else None, fixed_ranges=fixed_ranges)
    at = 0
    for r, q_len in enumerate(q_lens):
        want = plain.attention_dense(qs[r].float().cpu(), ks[r].float().cpu(), vs[r].float().cpu(), hd ** -0.5, window=window)
        torch.testing.assert_close(out[at : at + q_len].float().cpu(), want, **tol(dtype))
        at += q_len


def test_decode_attention_many_requests_with_splits():
    """Fifty requests of lengths from 1 to 400 keys with 5 to 7 splits each (many of them empty),
    three launches in a row over the same pages."""
    dtype = torch.bfloat16
    nh, nkv, hd, bs = 12, 2, 128, 16
    gen = torch.Generator().manual_seed(5)
    ctx_lens = [int(c) for c in torch.randint(1, 400, (50,), generator=gen)]
    num_blocks = sum(-(-c // bs) for c in ctx_lens) + 5
    perm = torch.randperm(num_blocks, generator=gen).tolist()
    tables, at = [], 0
    for c in ctx_lens:
        n = -(-c // bs)
        tables.append(perm[at : at + n])
        at += n
    kc, vc, ks, vs = _paged_setup(dtype, nkv, hd, bs, num_blocks, tables, ctx_lens, poison=float("nan"))
    for launch in range(3):
        qs = [torch.randn(1, nh, hd, device=DEV).to(dtype) for _ in ctx_lens]
        out = _run_attention(dtype, nh, nkv, hd, bs, tables, ctx_lens, [1] * len(ctx_lens), kc, vc, qs, splits=5 + launch,
                             decode_kernel=True, fixed_ranges=launch == 1)
        for r in range(len(ctx_lens)):
            want = plain.attention_dense(qs[r].float().cpu(), ks[r].float().cpu(), vs[r].float().cpu(), hd ** -0.5)
            torch.testing.assert_close(out[r : r + 1].float().cpu(), want, **tol(dtype))


def test_decode_attention_far_key_stands_out():
    nh, nkv, hd, bs = 12, 2, 128, 16
    ctx = 700
    for where in (0, 15, 16, 511, 512, 698, 699):
        tables = [list(range(44))]
        kc, vc, ks, vs = _paged_setup(torch.bfloat16, nkv, hd, bs, 50, tables, [ctx])
        q = torch.randn(1, nh, hd, device=DEV).to(torch.bfloat16)
        slot = tables[0][where // bs] * bs + where % bs
        kc[slot, 1] = (60.0 * q[0, 7].float() / q[0, 7].float().norm()).to(torch.bfloat16)
        out = _run_attention(torch.bfloat16, nh, nkv, hd, bs, tables, [ctx], [1], kc, vc, [q], splits=3, decode_kernel=True,
                             fixed_ranges=where % 2 == 1)
        torch.testing.assert_close(out[0, 7].float(), vc[slot, 1].float(), rtol=2e-2, atol=2e-2)


def test_attention_far_key_stands_out():
    """One key among hundreds, scaled so that its score dominates: the output must be its value,
    wherever in the context (first page, page edge, last position) it sits."""
    nh, nkv, hd, bs = 2, 1, 64, 16
    ctx = 700
    for where in (0, 15, 16, 511, 512, 698, 699):
        tables = [list(range(44))]
        kc, vc, ks, vs = _paged_setup(torch.float32, nkv, hd, bs, 50, tables, [ctx])
        q = torch.randn(1, nh, hd, device=DEV)
        slot = tables[0][where // bs] * bs + where % bs
        kc[slot, 0] = 40.0 * q[0, 0] / q[0, 0].norm()
        out = _run_attention(torch.float32, nh, nkv, hd, bs, tables, [ctx], [1], kc, vc, [q], splits=4)
        torch.testing.assert_close(out[0, 0], vc[slot, 0], rtol=1e-3, atol=1e-3)


def test_attention_reduces_to_library_routine():
    """One head group, no rotation: equals F.scaled_dot_product_attention(is_causal=True)
    (tests/test_attention_kernels.py:137-145)."""
    nh, hd, bs, T = 4, 32, 8, 45
    tables = [list(range(6))]
    kc, vc, ks, vs = _paged_setup(torch.float32, nh, hd, bs, 8, tables, [T])
    q = torch.randn(T, nh, hd, device=DEV)
    out = _run_attention(torch.float32, nh, nh, hd, bs, tables, [T], [T], kc, vc, [q], scale=0.3)
    want = torch.nn.functional.scaled_dot_product_attention(
        q.transpose(0, 1)[None], ks[0].transpose(0, 1)[None], vs[0].transpose(0, 1)[None], is_causal=True, scale=0.3
    )[0].transpose(0, 1)
    torch.testing.assert_close(out, want, rtol=1e-5, atol=1e-5)


def test_attention_refuses_wrong_shapes():
    from clockwork_amd import ops
    from clockwork_amd.ops import KernelError

    with pytest.raises(ValueError):
        ops._load("attention", 24)
    kc = torch.zeros(64, 2, 32, device=DEV)
    with pytest.raises(KernelError):
        _run_attention(torch.float32, 4, 2, 32, 8, [[0]], [4], [1], kc[:, :1], kc, [torch.zeros(1, 4, 32, device=DEV)])


# ---------------------------------------------------------------------------------- sampling
@pytest.mark.parametrize("n,V", [(1, 1000), (5, 151936), (3, 17)])
def test_argmax_first_index_wins(n, V):
    from clockwork_amd import ops

    logits = torch.randn(n, V, device=DEV)
    logits[0, V // 2] = 50.0
    logits[0, V - 1] = 50.0
    got = ops.argmax(logits)
    assert got.tolist() == logits.argmax(-1).tolist()
    assert got[0] == V // 2


@pytest.mark.parametrize("V,scale", [(1000, 3.0), (4099, 1.0), (151936, 3.0), (151936, 0.3)])
def test_sampling_matches_plain_definition(V, scale):
    """Every combination of temperature, top-k and top-p against the plain definition with the same
    uniform number; a vocabulary of the model's size (a row is cut into chunks), one that no chunk
    size divides, peaked and nearly flat rows."""
    from clockwork_amd import ops

    n = 24
    logits = scale * torch.randn(n, V, device=DEV)
    logits[3, 7] = logits[3, V - 5] = logits[3].max() + 1.0  # equal maxima
    temps = torch.tensor([0.0, 0.8, 1.5, 1.0] * 6, device=DEV)
    top_k = torch.tensor(([-1] * 4 + [5] * 4 + [1] * 4 + [-1] * 4 + [50] * 4 + [V] * 4), dtype=torch.int32, device=DEV)
    top_p = torch.tensor(([1.0] * 12 + [0.9] * 4 + [0.5] * 4 + [0.05] * 4), device=DEV)
    seeds = torch.arange(n, dtype=torch.int64, device=DEV) * 7 + 1
    draws = torch.arange(n, dtype=torch.int64, device=DEV) % 5
    got = ops.sample(logits, temps, top_k, top_p, seeds, draws).tolist()
    for i in range(n):
        if temps[i] == 0:
            assert got[i] == int(logits[i].argmax())
            continue
        probs = plain.sampling_probs(logits[i].cpu(), float(temps[i]), int(top_k[i]), float(top_p[i]))
        u = plain.uniform01(int(seeds[i]), int(draws[i]))
        want, margin = plain.draw(probs, u)
        assert probs[got[i]] > 0, f"row {i}: a token outside the kept set was drawn"
        assert got[i] == want or margin < 1e-4, f"row {i}: got {got[i]}, plain draws {want} (margin {margin})"
        if int(top_k[i]) == 1:
            assert got[i] == int(logits[i].argmax())  # tests/test_server.py:323
    # the caller may say that no row has an option: the same tokens without those kernels
    plain_rows = [i for i in range(n) if int(top_k[i]) in (-1, V) and float(top_p[i]) == 1.0]
    sel = torch.tensor(plain_rows, device=DEV)
    again = ops.sample(logits[sel].contiguous(), temps[sel], top_k[sel], top_p[sel], seeds[sel], draws[sel],
                       any_top_k=False, any_top_p=False).tolist()
    assert again == [got[i] for i in plain_rows]


def test_sampling_of_rows_without_finite_logits_is_the_first_maximum():
    """Rows of -inf, a +inf among finite logits, NaNs among them: no weight can be formed for some
    of these rows; the kernels must neither fault nor leave the vocabulary."""
    from clockwork_amd import ops

    V = 5000
    rows = torch.randn(6, V, device=DEV)
    rows[0] = float("-inf")
    rows[1] = float("-inf"); rows[1, 123] = 0.5          # one finite logit
    rows[2, 777] = float("inf")                           # an infinite one wins
    rows[3, ::2] = float("nan")                           # NaN counts as -inf
    rows[4] = float("nan")
    n = rows.shape[0]
    for k, p in ((-1, 1.0), (20, 1.0), (-1, 0.7), (20, 0.7)):
        got = ops.sample(rows, torch.full((n,), 0.9, device=DEV), torch.full((n,), k, dtype=torch.int32, device=DEV),
                         torch.full((n,), p, device=DEV), torch.arange(n, dtype=torch.int64, device=DEV),
                         torch.zeros(n, dtype=torch.int64, device=DEV)).tolist()
        assert all(0 <= t < V for t in got)
        assert got[0] == 0 and got[1] == 123 and got[2] == 777 and got[4] == 0
        assert got[3] % 2 == 1
        probs = plain.sampling_probs(rows[5].cpu(), 0.9, k, p)
        assert probs[got[5]] > 0


def test_sampling_keeps_exactly_the_top_k_and_the_nucleus():
    """Many draws from one row: every token of the kept set comes up and no other does (a selection
    that is off by one place shows here, not in single draws)."""
    from clockwork_amd import ops

    torch.manual_seed(77)  # the same row every run: what must be seen below depends on it
    V, n = 3000, 6000
    row = torch.randn(V, device=DEV)
    row[torch.randperm(V, device=DEV)[:12]] += 6.0  # a dozen likely tokens
    logits = row.repeat(n, 1)
    seeds = torch.full((n,), 5, dtype=torch.int64, device=DEV)
    draws = torch.arange(n, dtype=torch.int64, device=DEV)
    ones = torch.ones(n, device=DEV)
    for k, p in ((8, 1.0), (-1, 0.6), (10, 0.8)):
        got = ops.sample(logits, ones, torch.full((n,), k, dtype=torch.int32, device=DEV), p * ones, seeds, draws)
        probs = plain.sampling_probs(row.cpu(), 1.0, k, p)
        kept = set(torch.nonzero(probs > 0).flatten().tolist())
        seen = set(got.tolist())
        assert seen <= kept
        likely = {i for i in kept if float(probs[i]) > 20.0 / n}  # missed with probability e^-20
        assert likely <= seen
        freq = torch.bincount(got.long(), minlength=V).float().cpu() / n
        assert float((freq - probs.float()).abs().max()) < 0.03


def test_sampling_is_reproducible_and_follows_the_distribution():
    from clockwork_amd import ops

    V, n = 8, 4000
    row = torch.tensor([2.0, 1.0, 0.0, -1.0, 0.5, -3.0, 1.5, 0.2], device=DEV)
    logits = row.repeat(n, 1)
    args = (torch.ones(n, device=DEV), torch.full((n,), -1, dtype=torch.int32, device=DEV), torch.ones(n, device=DEV))
    seeds = torch.full((n,), 42, dtype=torch.int64, device=DEV)
    draws = torch.arange(n, dtype=torch.int64, device=DEV)
    a = ops.sample(logits, *args, seeds, draws)
    b = ops.sample(logits, *args, seeds, draws)
    assert torch.equal(a, b)
    c = ops.sample(logits, *args, seeds + 1, draws)
    assert not torch.equal(a, c)
    freq = torch.bincount(a.long(), minlength=V).float() / n
    torch.testing.assert_close(freq.cpu(), torch.softmax(row, -1).cpu(), rtol=0, atol=0.03)


def test_fresh_state_rows_copies_the_template_into_the_slots_of_requests_that_begin():
    """pool [entries, slots, row]: the last slot is the template; a request whose step starts at
    position 0 gets it, every other row of the pool stays as it is."""
    from clockwork_amd import ops

    entries, slots, width = 3, 7, 10            # 5 request slots, the spare one, the template
    pool = torch.randn(entries, slots, width, device=DEV)
    before = pool.clone()
    rows = torch.tensor([4, 1, -1, 9, 5, 2, 6], dtype=torch.int32, device=DEV)     # -1 / 9: no request; 5: the spare slot
    starts = torch.tensor([0, 3, 0, 0, 0, 0, 0], dtype=torch.int32, device=DEV)    # slot 1 is in the middle of its request
    ops.fresh_state_rows(pool, rows, starts, 6)                                    # the seventh row is not part of the step
    torch.cuda.synchronize()
    want = before.clone()
    for slot in (4, 5, 2):
        want[:, slot] = before[:, 6]
    assert torch.equal(pool, want)   # slot 6 itself (the template) is never a target
    # half precision rows of an even width are whole words too
    half = torch.randn(2, 4, 6, device=DEV).to(torch.bfloat16)
    kept = half.clone()
    ops.fresh_state_rows(half, torch.tensor([0], dtype=torch.int32, device=DEV), torch.tensor([0], dtype=torch.int32, device=DEV), 1)
    torch.cuda.synchronize()
    kept[:, 0] = kept[:, 3]
    assert torch.equal(half, kept)
    with pytest.raises(ops.KernelError):
        ops.fresh_state_rows(pool[:, :1], rows, starts, 1)   # no room for a template


def test_the_parts_of_a_product_summed_over_k_are_as_many_as_the_engine_has_chosen():
    """A narrow output with a long K and few rows comes back as partial sums over K. How many
    parts is the kernel's rule, unless the engine's policy holds a count for the shape (what a
    tuning start-up measures): every count gives the same product, and the count is the same for
    every number of rows up to 16, so a row's sum does not depend on the rows beside it."""
    from clockwork_amd import ops

    N, K = 1536, 8960
    gen = torch.Generator(device=DEV).manual_seed(6)
    w = (torch.randn(N, K, device=DEV, generator=gen) / K ** 0.5).to(torch.bfloat16)
    x = torch.randn(16, K, device=DEV, generator=gen).to(torch.bfloat16)
    want = x.float() @ w.float().t()
    default = ops.linear(x[:8].contiguous(), w, partial_ok=True)
    assert isinstance(default, ops.PartialSums) and default.parts.shape[0] > 1
    one, all_rows = ops.linear(x[:1].contiguous(), w, partial_ok=True), ops.linear(x, w, partial_ok=True)
    assert one.parts.shape[0] == default.parts.shape[0] == all_rows.parts.shape[0]
    for splits in (2, 3, 6, 7, 12):
        policy = ops.ProductPolicy()
        policy.k_split_choices[(N, K)] = splits
        for rows in (1, 8, 16):
            got = ops.linear(x[:rows].contiguous(), w, partial_ok=True, policy=policy)
            assert got.parts.shape == (splits, rows, N)
            torch.testing.assert_close(got.sum(), want[:rows], rtol=2e-2, atol=2e-2)
        # one row alone and the same row in a batch: the same bits
        assert torch.equal(ops.linear(x[:1].contiguous(), w, partial_ok=True, policy=policy).parts[:, 0], got.parts[:, 0])
    # a tuning start-up measures the count once for the shape and keeps it
    policy = ops.ProductPolicy()
    policy.tuning = True
    first = ops.linear(x[:8].contiguous(), w, partial_ok=True, policy=policy)
    policy.tuning = False
    assert (N, K) in policy.k_split_choices and not ops.DEFAULT_POLICY.k_split_choices
    assert first.parts.shape[0] == policy.k_split_choices[(N, K)]
    assert ops.linear(x, w, partial_ok=True, policy=policy).parts.shape[0] == first.parts.shape[0]
    torch.testing.assert_close(first.sum(), want[:8], rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("M,N,K,splits", [(2048, 1536, 8960, 4), (1300, 1536, 8960, 5), (1030, 200, 2560, 2), (2048, 3584, 18944, 8),
                                          (257, 1536, 8960, 7)])
def test_wide_tile_product_in_partial_sums_over_k(M, N, K, splits):
    """The wide-tile kernel with K cut into runs, every run of every tile a work item that writes
    a float32 plane of partial sums: the planes add up to the product; rows and columns that end
    inside a tile, a width that is no multiple of 4 floats' alignment, several runs a workgroup."""
    from clockwork_amd import ops

    gen = torch.Generator(device=DEV).manual_seed(M + splits)
    x = torch.randn(M, K, device=DEV, generator=gen).to(torch.bfloat16)
    w = (torch.randn(N, K, device=DEV, generator=gen) / K ** 0.5).to(torch.bfloat16)
    got = ops.linear_wide_partial(x, w, splits)
    assert got.parts.shape == (splits, M, N) and got.parts.dtype == torch.float32
    run = K // splits
    for z in (0, splits - 1):
        want = x[:, z * run : (z + 1) * run].float() @ w[:, z * run : (z + 1) * run].float().t()
        torch.testing.assert_close(got.parts[z], want, rtol=1e-3, atol=1e-3)
    torch.testing.assert_close(got.sum(), x.float() @ w.float().t(), rtol=1e-3, atol=2e-3)
    # and through the norm that adds the planes up
    resid = torch.randn(M, N, device=DEV, generator=gen)
    before = resid.clone()
    weight = torch.ones(N, device=DEV)
    out = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    ops.add_rmsnorm(resid, got, weight, 1e-6, out)
    torch.testing.assert_close(resid, before + x.float() @ w.float().t(), rtol=1e-3, atol=3e-3)


def test_wide_tile_partial_sums_refuse_what_they_do_not_take():
    from clockwork_amd import ops

    x = torch.zeros(1024, 8960, device=DEV, dtype=torch.bfloat16)
    w = torch.zeros(1536, 8960, device=DEV, dtype=torch.bfloat16)
    for splits in (1, 3, 6, 17):   # 8960 is no multiple of 64 * 3 or 64 * 6
        with pytest.raises(ops.KernelError):
            ops.linear_wide_partial(x, w, splits)
    # the engine takes the kernel only where a tuning start-up has measured it to be the faster way
    policy = ops.ProductPolicy()
    assert isinstance(ops.linear(x, w, partial_ok=True, policy=policy), torch.Tensor)
    policy.wide_partial_choices[(1536, 8960)] = 4
    assert ops.linear(x, w, partial_ok=True, policy=policy).parts.shape == (4, 1024, 1536)
    assert isinstance(ops.linear(x[:512], w, partial_ok=True, policy=policy), torch.Tensor)   # too few rows
    assert isinstance(ops.linear(x, w, policy=policy), torch.Tensor)                           # a caller that wants a tensor


def test_attention_part_alone_as_the_benchmark_times_it(monkeypatch):
    """``bench.py --decode-attention-grid`` times ``PagedAttention.attend`` on a hand-made step of
    single tokens: the same call must give dense attention over each request's own pages, and the
    benchmark's record must hold a time for every point of its grid."""
    import argparse

    import bench
    from clockwork_amd.engine.batch import StepContext
    from clockwork_amd.parts.attention import PagedAttention
    from clockwork_amd.parts.specs import AttentionSpec

    nh, nkv, hd, bs = 12, 2, 128, 16
    part = PagedAttention(AttentionSpec(hidden_size=nh * hd, num_heads=nh, num_kv_heads=nkv, head_dim=hd,
                                        qkv_bias=False, out_bias=False, scale=hd ** -0.5))
    part.dtype = torch.bfloat16
    batch, context = 5, 700
    pages_each = -(-context // bs)
    gen = torch.Generator().manual_seed(11)
    k = torch.randn((batch * pages_each, bs, nkv, hd), generator=gen).to(DEV, torch.bfloat16)
    v = torch.randn((batch * pages_each, bs, nkv, hd), generator=gen).to(DEV, torch.bfloat16)
    q = torch.randn((batch, nh * hd), generator=gen).to(DEV, torch.bfloat16)
    tables = torch.randperm(batch * pages_each, generator=gen).view(batch, pages_each)
    ctx = StepContext()
    ctx.device, ctx.block_size = torch.device(DEV), bs
    ctx.num_tokens = ctx.num_requests = batch
    ctx.h_q_lens, ctx.h_ctx_lens = [1] * batch, [context] * batch
    ctx.block_tables = [tables.to(DEV, torch.int32)]
    ctx.ctx_lens = torch.full((batch,), context, dtype=torch.int32, device=DEV)
    ctx.cu_q = torch.arange(batch + 1, dtype=torch.int32, device=DEV)
    part.prepare(ctx)
    out = part.attend(q, ctx, argparse.Namespace(k=k, v=v, group=0, block_size=bs)).float().cpu().view(batch, 1, nh, hd)
    for r in range(batch):
        keys = k[tables[r]].reshape(-1, nkv, hd)[:context].float().cpu()
        values = v[tables[r]].reshape(-1, nkv, hd)[:context].float().cpu()
        want = plain.attention_dense(q[r].view(1, nh, hd).float().cpu(), keys, values, hd ** -0.5)
        torch.testing.assert_close(out[r], want, **tol(torch.bfloat16))

    monkeypatch.setattr(bench, "REFERENCE_DECODE_ATTENTION_MS", {(2, 128): 0.07, (4, 512): 0.27})
    record = bench.measure_decode_attention_grid()
    assert set(record["grid"]) == {"batch2_ctx128", "batch4_ctx512"}
    for point in record["grid"].values():
        assert 0 < point["ms"] < 1 and point["key_splits"] >= 1 and point["GB_per_s"] > 0


def test_candidates_are_timed_inside_graphs_over_copies_of_the_weights():
    """What a tuning start-up ranks its own kernels' variants by: each candidate runs inside a
    captured graph, round after round on another copy of the weights (together more than the
    caches hold). Twice the work must take clearly longer, the same work about the same, and the
    count of parts over K it chooses for a shape is one the kernel takes."""
    from clockwork_amd import ops

    N, K = 1536, 8960
    gen = torch.Generator(device=DEV).manual_seed(3)
    w = (torch.randn(N, K, device=DEV, generator=gen) / K ** 0.5).to(torch.bfloat16)
    x = torch.randn(8, K, device=DEV, generator=gen).to(torch.bfloat16)
    copies = ops._cold_copies(w)
    assert 2 <= len(copies) <= 16 and copies[0] is w
    assert sum(c.numel() * 2 for c in copies) > 256 << 20
    assert all(torch.equal(c, w) for c in copies[1:3])

    def once(i):
        ops.linear(x, copies[i % len(copies)])

    def twice(i):
        ops.linear(x, copies[(2 * i) % len(copies)])
        ops.linear(x, copies[(2 * i + 1) % len(copies)])

    times = ops._replayed_us({"once": once, "again": once, "twice": twice}, rounds=len(copies), flush=False)
    assert 2 < times["once"] < 60, times
    assert abs(times["again"] - times["once"]) < 0.2 * times["once"], times
    assert times["twice"] > 1.5 * times["once"], times
    # with the caches washed between the rounds instead (no memory for copies): the same ranking
    washed = ops._replayed_us({"once": lambda i: ops.linear(x, w), "twice": lambda i: (ops.linear(x, w), ops.linear(x, w))},
                              rounds=4, flush=True)
    assert washed["twice"] > 1.4 * washed["once"] > 0, washed
    chosen = ops._measure_k_splits(x, w, ops._load("gemm").cw_gemm_bf16_skinny_ksplits(8, N, K))
    policy = ops.ProductPolicy()
    policy.k_split_choices[(N, K)] = chosen
    got = ops.linear(x, w, partial_ok=True, policy=policy)
    assert got.parts.shape[0] == chosen
    torch.testing.assert_close(got.sum(), x.float() @ w.float().t(), rtol=2e-2, atol=2e-2)
