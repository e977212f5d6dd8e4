"""Pins for the plain implementation besides the reference's text: special cases that reduce
to a library routine, invariants, and vectors the reference's own tests hold. Each is chosen
so that a plausible mistake (a wrong sign or pairing, a norm in the wrong place) fails it."""

import math

import pytest
import torch
import torch.nn.functional as F

from tests.configs import TINY_A, TINY_B
from tests.plain import qwen2_plain as plain

torch.manual_seed(0)


# ------------------------------------------------------------------ norm, linear, feed-forward
def test_rmsnorm_is_the_library_routine_and_normalises():
    x = torch.randn(5, 48) * 3
    w = 1 + 0.1 * torch.randn(48)
    torch.testing.assert_close(plain.rmsnorm(x, w, 1e-6), F.rms_norm(x, (48,), w, 1e-6))
    ones = torch.ones(48)
    assert torch.allclose(plain.rmsnorm(x, ones, 1e-6).pow(2).mean(-1), torch.ones(5), atol=1e-4)
    torch.testing.assert_close(plain.rmsnorm(17 * x, ones, 1e-6), plain.rmsnorm(x, ones, 1e-6), rtol=1e-4, atol=1e-5)
    assert torch.all(plain.rmsnorm(torch.zeros(1, 48), w, 1e-6) == 0)
    # eps sits inside the root: a tiny row shows it
    tiny = torch.full((1, 48), 1e-4)
    assert abs(float(plain.rmsnorm(tiny, ones, 1e-6)[0, 0]) - 1e-4 / math.sqrt(1e-8 + 1e-6)) < 1e-6


def test_linear_is_x_w_transposed_plus_bias():
    x, w, b = torch.randn(3, 7), torch.randn(5, 7), torch.randn(5)
    torch.testing.assert_close(plain.linear(x, w, b), F.linear(x, w, b))


def test_swiglu_gates_with_the_first_matrix():
    x = torch.randn(4, 6)
    g, u, d = torch.randn(10, 6), torch.randn(10, 6), torch.randn(6, 10)
    want = F.linear(F.silu(F.linear(x, g)) * F.linear(x, u), d)
    torch.testing.assert_close(plain.swiglu(x, g, u, d), want)
    assert not torch.allclose(plain.swiglu(x, u, g, d), want, atol=1e-3)  # the halves are not interchangeable
    assert float(F.silu(torch.zeros(1))) == 0.0
    assert torch.all(plain.swiglu(torch.zeros(1, 6), g, u, d) == 0)


# ------------------------------------------------------------------ rotary
def test_rope_is_a_complex_rotation_of_half_split_pairs():
    hd, theta = 32, 1e4
    x = torch.randn(9, 3, hd, dtype=torch.float64)
    pos = torch.tensor([0, 1, 2, 5, 17, 100, 1000, 4000, 31])
    cos, sin = plain.rope_tables(pos, hd, theta, torch.float64)
    got = plain.apply_rope(x, cos, sin)
    # pair (i, i + hd/2) as a complex number times e^{i * pos * inv_freq_i}
    z = torch.complex(x[..., : hd // 2], x[..., hd // 2 :])
    angle = pos.double()[:, None] * plain.inv_frequencies(hd, theta).double()[None, :]
    rot = z * torch.polar(torch.ones_like(angle), angle)[:, None, :]
    want = torch.cat((rot.real, rot.imag), dim=-1)
    torch.testing.assert_close(got, want, rtol=1e-10, atol=1e-10)
    # the interleaved pairing (2i, 2i+1) is a different function: it must not pass
    zi = torch.view_as_complex(x.reshape(9, 3, hd // 2, 2).contiguous())
    roti = torch.view_as_real(zi * torch.polar(torch.ones_like(angle), angle)[:, None, :]).reshape(9, 3, hd)
    assert not torch.allclose(got, roti, atol=1e-3)


def test_rope_invariants():
    hd, theta = 16, 1e6
    q, k = torch.randn(1, 1, hd, dtype=torch.float64), torch.randn(1, 1, hd, dtype=torch.float64)

    def at(x, p):
        cos, sin = plain.rope_tables(torch.tensor([p]), hd, theta, torch.float64)
        return plain.apply_rope(x, cos, sin)

    torch.testing.assert_close(at(q, 0), q)  # position 0 is the identity
    assert abs(float(at(q, 37).norm()) - float(q.norm())) < 1e-12  # a rotation keeps the norm
    d1 = float((at(q, 9) * at(k, 4)).sum())
    d2 = float((at(q, 1009) * at(k, 1004)).sum())
    assert abs(d1 - d2) < 1e-9  # only the distance counts
    assert abs(d1 - float((at(q, 9) * at(k, 5)).sum())) > 1e-6
    # the sign: the first element of a pair turns towards minus the second
    e = torch.zeros(1, 1, hd, dtype=torch.float64)
    e[0, 0, hd // 2] = 1.0
    assert float(at(e, 1)[0, 0, 0]) < 0


def test_rope_tables_are_float32_exact_like_the_reference():
    # tests/test_hf_equivalence.py:156-171: inv_freq float32; cos/sin at 0, 1, 4000 close to exact
    inv = plain.inv_frequencies(32, 1e6)
    assert inv.dtype == torch.float32 and inv.shape == (16,) and float(inv[0]) == 1.0
    assert abs(float(inv[1]) - 1e6 ** (-2 / 32)) < 1e-7
    pos = torch.tensor([0, 1, 4000])
    cos, sin = plain.rope_tables(pos, 32, 1e6)
    cos64, sin64 = plain.rope_tables(pos, 32, 1e6, torch.float64)
    assert cos.shape == (3, 32) and torch.equal(cos[:, :16], cos[:, 16:])
    assert float((cos.double() - cos64).abs().max()) < 8e-3 and float((sin.double() - sin64).abs().max()) < 8e-3
    # the whole model's tables keep the reference's float32 angles in every precision: in float32
    # they are these tables, in float64 the exact cosines of the same float32 angles
    ref_cos, ref_sin = plain.reference_rope_tables(pos, 32, 1e6)
    assert torch.equal(ref_cos, cos) and torch.equal(ref_sin, sin)
    angles = pos.float()[:, None] * inv[None, :]
    cos_of_f32_angles, _ = plain.reference_rope_tables(pos, 32, 1e6, torch.float64)
    assert torch.equal(cos_of_f32_angles[:, :16], angles.double().cos())
    assert float((cos_of_f32_angles - cos.double()).abs().max()) < 2e-7     # float32's own cosine of the same angle
    assert float((cos_of_f32_angles - cos64).abs().max()) > 1e-5            # the angle's rounding at position 4000


# ------------------------------------------------------------------ attention
def test_attention_without_groups_is_the_library_routine():
    # tests/test_attention_kernels.py:137-145
    q, k, v = torch.randn(7, 4, 16), torch.randn(7, 4, 16), torch.randn(7, 4, 16)
    want = F.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1), is_causal=True, scale=0.31)
    torch.testing.assert_close(plain.attention_dense(q, k, v, 0.31), want.transpose(0, 1), rtol=1e-5, atol=1e-5)


def test_grouped_heads_read_kv_head_h_div_group():
    # tests/test_attention_kernels.py:148-190: a triple loop, kv heads set apart by large constants
    nh, nkv, hd, T = 6, 2, 8, 5
    q = torch.randn(T, nh, hd, dtype=torch.float64)
    k = torch.randn(T, nkv, hd, dtype=torch.float64)
    v = torch.randn(T, nkv, hd, dtype=torch.float64) + torch.tensor([0.0, 1000.0], dtype=torch.float64)[None, :, None]
    got = plain.attention_dense(q, k, v, hd ** -0.5)
    for h in range(nh):
        g = h // (nh // nkv)
        for i in range(T):
            s = torch.tensor([float(q[i, h] @ k[j, g]) * hd ** -0.5 for j in range(i + 1)], dtype=torch.float64)
            p = torch.softmax(s, 0)
            want = sum(p[j] * v[j, g] for j in range(i + 1))
            torch.testing.assert_close(got[i, h], want, rtol=1e-10, atol=1e-10)
    assert float(got[:, :3].abs().max()) < 100 and float(got[:, 3:].min()) > 900


def test_attention_invariants():
    nh, nkv, hd = 4, 2, 8
    q, k, v = torch.randn(9, nh, hd), torch.randn(9, nkv, hd), torch.randn(9, nkv, hd)
    out = plain.attention_dense(q, k, v, 0.3)
    torch.testing.assert_close(out[0], v[0].repeat_interleave(2, dim=0))  # the first token sees itself only
    # a suffix of the queries against all keys equals the slice of the full result (end-aligned mask)
    torch.testing.assert_close(plain.attention_dense(q[5:], k, v, 0.3), out[5:])
    # equal keys: the output is the running mean of the values
    same_k = k[:1].expand(9, -1, -1)
    mean = plain.attention_dense(q, same_k, v, 0.3)
    torch.testing.assert_close(mean[4, 0], v[:5, 0].mean(0), rtol=1e-5, atol=1e-6)
    # a window as long as the sequence changes nothing; a window of 1 returns the token's own value
    torch.testing.assert_close(plain.attention_dense(q, k, v, 0.3, window=9), out)
    torch.testing.assert_close(plain.attention_dense(q, k, v, 0.3, window=1), v.repeat_interleave(2, dim=1))
    # the scale multiplies the scores: it matters
    assert not torch.allclose(plain.attention_dense(q, k, v, 0.6), out, atol=1e-3)


# ------------------------------------------------------------------ the whole model
@pytest.fixture(scope="module")
def tiny(tmp_path_factory):
    from clockwork_amd.weights.random_init import write_random_model

    root = tmp_path_factory.mktemp("plain")
    return {"A": write_random_model(root / "A", TINY_A, 0), "B": write_random_model(root / "B", TINY_B, 1)}


def test_logits_are_causal_and_deterministic(tiny):
    model = plain.PlainQwen2(tiny["B"])
    toks = torch.randint(0, 1000, (20,), generator=torch.Generator().manual_seed(0)).tolist()
    full = model.logits(toks)
    assert full.shape == (20, 1000)
    torch.testing.assert_close(model.logits(toks[:11]), full[:11], rtol=1e-5, atol=1e-5)
    other = toks[:11] + [(t + 1) % 1000 for t in toks[11:]]
    torch.testing.assert_close(model.logits(other)[:11], full[:11], rtol=1e-5, atol=1e-5)
    assert not torch.allclose(model.logits(other)[12], full[12], atol=1e-4)


def test_the_models_score_scale_is_the_library_default_for_its_head_size(tmp_path, monkeypatch):
    """clockwork/engine/model.py:73: scale = head_dim ** -0.5, head_dim being the explicit key
    where a config has one (model.py:17-18), not hidden_size / heads. With the model's attention
    swapped for the library routine at its *default* scale (1 / sqrt of the queries' last
    dimension), configuration C (head_dim 48, hidden 80, 3 heads: 80 / 3 would give another
    scale) yields the same logits."""
    from clockwork_amd.weights.random_init import write_random_model
    from tests.configs import TINY_C

    model = plain.PlainQwen2(write_random_model(tmp_path / "C", TINY_C, 5), dtype=torch.float64)
    # sharper scores, so that the scale shows: with N(0, 0.02) weights every softmax is nearly flat
    for i in range(model.L):
        model.w[f"model.layers.{i}.self_attn.q_proj.weight"] *= 40.0
    toks = torch.randint(0, 777, (15,), generator=torch.Generator().manual_seed(2)).tolist()
    own = model.logits(toks)
    scales = []

    def library_attention(q, k, v, scale, window=None):
        scales.append(scale)
        assert q.shape[1] == k.shape[1] and window is None   # no groups in this configuration
        out = F.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1), is_causal=True)
        return out.transpose(0, 1)

    monkeypatch.setattr(plain, "attention_dense", library_attention)
    torch.testing.assert_close(model.logits(toks), own, rtol=1e-9, atol=1e-9)
    assert scales == [48 ** -0.5] * model.L
    # the bar bites: the scale that hidden_size / heads would give moves the logits
    model.scale = (80 / 3) ** -0.5
    monkeypatch.undo()
    assert not torch.allclose(model.logits(toks), own, rtol=1e-4, atol=1e-4)


def test_shifting_all_positions_changes_nothing(tiny):
    """Only distances count: running the layers with every position moved by a constant gives
    the same logits (a rotation applied to keys but not queries, or added positions, would not)."""
    model = plain.PlainQwen2(tiny["A"], dtype=torch.float64)
    toks = torch.randint(0, 512, (12,), generator=torch.Generator().manual_seed(1))

    def run(shift):
        h = plain.embedding(model.w["model.embed_tokens.weight"], toks)
        cos, sin = plain.rope_tables(torch.arange(12) + shift, model.hd, model.theta, torch.float64)
        for i in range(model.L):
            h = model.layer(i, h, cos, sin)
        return h

    torch.testing.assert_close(run(0), run(77), rtol=1e-9, atol=1e-9)


def _layer_setup(tiny, eps=None):
    """Layer 1 of model B in float64, a random stream h and its rotary tables."""
    model = plain.PlainQwen2(tiny["B"], dtype=torch.float64)
    if eps is not None:
        model.eps = eps
    T = 7
    h = torch.randn(T, 192, dtype=torch.float64, generator=torch.Generator().manual_seed(4)) * 0.3
    cos, sin = plain.rope_tables(torch.arange(T), model.hd, model.theta, torch.float64)
    return model, h, cos, sin


def _without(model, *names):
    """The same model with the named matrices of layer 1 zeroed."""
    import copy

    other = copy.copy(model)
    other.w = dict(model.w)
    for name in names:
        key = f"model.layers.1.{name}.weight"
        other.w[key] = torch.zeros_like(model.w[key])
    return other


def test_a_layer_with_both_output_matrices_zeroed_is_the_identity(tiny):
    """clockwork/engine/model.py:147-154: out = h + attn(...) + mlp(...). Both branches end in a
    matrix without bias, so zeroing o_proj and down_proj must leave the stream untouched; a norm
    applied to the stream itself (post-norm: h = norm(h + branch)) would not."""
    model, h, cos, sin = _layer_setup(tiny)
    still = _without(model, "self_attn.o_proj", "mlp.down_proj")
    assert torch.equal(still.layer(1, h, cos, sin), h)


def test_each_branch_reads_the_normed_stream_and_adds_to_the_raw_one(tiny):
    """Pre-norm wiring: a branch sees norm(stream), which does not change when the stream is
    scaled (eps aside: it is set to nothing here), and its output is added to the unscaled
    stream. With the other branch switched off, layer(c h) - c h == layer(h) - h for each of the
    two; a branch fed the raw stream, or a norm after the sum, breaks this."""
    model, h, cos, sin = _layer_setup(tiny, eps=1e-300)
    for off in ("mlp.down_proj", "self_attn.o_proj"):
        one = _without(model, off)
        branch = one.layer(1, h, cos, sin) - h
        assert float(branch.abs().max()) > 1e-3  # the branch that is left does something
        for c in (0.25, 9.0):
            torch.testing.assert_close(one.layer(1, c * h, cos, sin) - c * h, branch, rtol=1e-9, atol=1e-12)


def test_the_feed_forward_reads_the_stream_after_attention_was_added(tiny):
    """model.py:150-154: the second residual is h + attn, and the second norm reads it. Putting
    the layer together from its two branches, each measured alone, must give the layer; a
    feed-forward that read the layer's input, or the attention output alone, would not."""
    model, h, cos, sin = _layer_setup(tiny)
    a = _without(model, "mlp.down_proj").layer(1, h, cos, sin) - h          # attention branch
    only_ffn = _without(model, "self_attn.o_proj")
    m = only_ffn.layer(1, h + a, cos, sin) - (h + a)                        # feed-forward on h + a
    whole = model.layer(1, h, cos, sin)
    torch.testing.assert_close(whole, h + a + m, rtol=1e-12, atol=1e-12)
    m_wrong = only_ffn.layer(1, h, cos, sin) - h                            # feed-forward on h
    assert not torch.allclose(whole, h + a + m_wrong, atol=1e-5)


def test_each_norm_weight_feeds_its_own_branch(tiny):
    """input_layernorm scales what attention reads, post_attention_layernorm what the
    feed-forward reads (model.py:148, 152): with one branch off, the other norm's weight has no
    effect and the branch's own norm weight does; swapped weights change the layer."""
    model, h, cos, sin = _layer_setup(tiny)

    def with_norms(m, first, second):
        import copy

        other = copy.copy(m)
        other.w = dict(m.w)
        other.w["model.layers.1.input_layernorm.weight"] = first
        other.w["model.layers.1.post_attention_layernorm.weight"] = second
        return other

    w1 = model.w["model.layers.1.input_layernorm.weight"]
    w2 = model.w["model.layers.1.post_attention_layernorm.weight"]
    assert not torch.allclose(w1, w2)
    attn_only = _without(model, "mlp.down_proj")
    base = attn_only.layer(1, h, cos, sin)
    assert torch.equal(with_norms(attn_only, w1, 3 * w2).layer(1, h, cos, sin), base)
    assert not torch.allclose(with_norms(attn_only, 3 * w1, w2).layer(1, h, cos, sin), base, atol=1e-4)
    ffn_only = _without(model, "self_attn.o_proj")
    base = ffn_only.layer(1, h, cos, sin)
    assert torch.equal(with_norms(ffn_only, 3 * w1, w2).layer(1, h, cos, sin), base)
    assert not torch.allclose(with_norms(ffn_only, w1, 3 * w2).layer(1, h, cos, sin), base, atol=1e-4)
    assert not torch.allclose(with_norms(model, w2, w1).layer(1, h, cos, sin), model.layer(1, h, cos, sin), atol=1e-5)


def test_final_norm_comes_before_the_head_and_after_the_last_layer(tiny):
    """model.py:204, 228-233: logits = head(norm(h_L)). Scaling model.norm's weight scales every
    logit by the same factor (the head has no bias); a head applied to the raw stream would not
    notice, a norm per layer output would compound."""
    model = plain.PlainQwen2(tiny["B"], dtype=torch.float64)
    toks = [5, 900, 31, 7]
    before = model.logits(toks)
    model.w["model.norm.weight"] = 2.5 * model.w["model.norm.weight"]
    torch.testing.assert_close(model.logits(toks), 2.5 * before, rtol=1e-12, atol=1e-12)


def test_tied_head_is_the_embedding(tiny):
    model = plain.PlainQwen2(tiny["A"])
    assert model.w["lm_head.weight"] is model.w["model.embed_tokens.weight"]
    toks = [3, 9, 27]
    before = model.logits(toks)
    model.w["model.embed_tokens.weight"][400] += 0.5  # token 400 is not in the prompt
    after = model.logits(toks)
    changed = (after - before).abs().max(0).values
    assert float(changed[400]) > 1e-3 and float(changed[torch.arange(512) != 400].max()) < 1e-6


def test_greedy_is_the_argmax_of_the_last_row(tiny):
    model = plain.PlainQwen2(tiny["B"])
    out = model.greedy([5, 6, 7], 3)
    assert out[0] == int(model.logits([5, 6, 7])[-1].argmax())
    assert out[1] == int(model.logits([5, 6, 7, out[0]])[-1].argmax())


# ------------------------------------------------------------------ sampling
def test_philox_known_answers():
    # Random123's known-answer vectors for philox4x32-10 (first output word)
    assert plain.philox4x32_10(0, 0) == 0x6627E8D5
    assert 0.0 <= plain.uniform01(7, 3) < 1.0 and plain.uniform01(7, 3) != plain.uniform01(7, 4)


def test_sampling_probs_follow_the_reference_order():
    logits = torch.tensor([2.0, 1.0, 0.5, 0.0, -1.0])
    torch.testing.assert_close(plain.sampling_probs(logits, 0.5), torch.softmax(logits.double() / 0.5, -1))
    p = plain.sampling_probs(logits, 1.0, top_k=2)
    assert torch.count_nonzero(p) == 2 and abs(float(p.sum()) - 1) < 1e-12
    # top-p keeps the token that crosses the threshold (clockwork/engine/model_runner.py:153-163)
    base = torch.softmax(logits.double(), -1)
    p = plain.sampling_probs(logits, 1.0, top_p=float(base[0]) + 1e-3)
    assert torch.count_nonzero(p) == 2
    p = plain.sampling_probs(logits, 1.0, top_p=1e-9)
    assert torch.count_nonzero(p) == 1 and float(p[0]) == 1.0
    idx, margin = plain.draw(torch.tensor([0.25, 0.25, 0.5]), 0.6)
    assert idx == 2 and abs(margin - 0.1) < 1e-12
