"""A plain, slow Qwen2: whole sequences, no cache, one function per part.

Written from the reference's formulas (each function cites file:line in the reference's
source tree); it shares no code with ``clockwork_amd``: it parses config.json
and reads the safetensors file itself. Everything runs on the CPU in ``dtype``
(float32 by default, float64 for invariants).
"""

from __future__ import annotations

import json
import math
from pathlib import Path

import torch
from safetensors.torch import load_file


# ------------------------------------------------------------------------------- parts
def embedding(weight: torch.Tensor, ids: torch.Tensor) -> torch.Tensor:
    """clockwork/engine/model.py:200 - a row lookup, no scaling, no position added."""
    return weight[ids]


def inv_frequencies(head_dim: int, theta: float) -> torch.Tensor:
    """clockwork/engine/model.py:171-175 - 1 / theta^(2j/hd), j = 0..hd/2-1, in float32."""
    return 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim))


def rope_tables(positions: torch.Tensor, head_dim: int, theta: float, dtype=torch.float32):
    """clockwork/engine/model.py:186-191 - angles pos * inv_freq in float32, the half-table twice."""
    freqs = positions.to(torch.float32)[:, None] * inv_frequencies(head_dim, theta)[None, :]
    if dtype == torch.float64:
        freqs = positions.to(torch.float64)[:, None] * inv_frequencies(head_dim, theta).to(torch.float64)[None, :]
    emb = torch.cat((freqs, freqs), dim=-1)
    return emb.cos().to(dtype), emb.sin().to(dtype)


def reference_rope_tables(positions: torch.Tensor, head_dim: int, theta: float, dtype=torch.float32):
    """The tables as the reference's model has them whatever ``dtype`` the rest of the arithmetic
    runs in: the angle of a position is the float32 product pos * inv_freq (model.py:186-191;
    at position 2000 its rounding is 1e-4 of a radian, which a model with peaked attention
    shows in its logits), and only its cosine and sine are taken in ``dtype``. In float32 this
    is ``rope_tables``; in float64 it measures an engine against the reference's angles with
    everything else exact, where ``rope_tables`` would hold the engine's float32 angles against it."""
    freqs = positions.to(torch.float32)[:, None] * inv_frequencies(head_dim, theta)[None, :]
    emb = torch.cat((freqs, freqs), dim=-1).to(torch.float64 if dtype == torch.float64 else torch.float32)
    return emb.cos().to(dtype), emb.sin().to(dtype)


def rotate_half(x: torch.Tensor) -> torch.Tensor:
    """clockwork/engine/model.py:32-35 - (-second half, first half)."""
    half = x.shape[-1] // 2
    return torch.cat((-x[..., half:], x[..., :half]), dim=-1)


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """clockwork/engine/model.py:92-95 - x [T, heads, hd]; cos/sin [T, hd] broadcast over heads."""
    return x * cos[:, None, :] + rotate_half(x) * sin[:, None, :]


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """clockwork/engine/model.py:44-49 - mean of squares, rsqrt, then the weight."""
    variance = x.pow(2).mean(-1, keepdim=True)
    return weight * (x * torch.rsqrt(variance + eps))


def linear(x: torch.Tensor, weight: torch.Tensor, bias=None) -> torch.Tensor:
    """nn.Linear as the reference uses it (model.py:58-60, 74-77): y = x W^T + b, W [out, in]."""
    y = x @ weight.t()
    return y if bias is None else y + bias


def attention_dense(q, k, v, scale: float, window=None) -> torch.Tensor:
    """clockwork/kernels/attention.py:45-65 - q [Tq, nh, hd], k/v [Tk, nkv, hd].

    Query head h reads kv head h // (nh / nkv) (attention.py:35-42, repeat_interleave);
    scores are scaled after the dot product; query row i sits at position Tk - Tq + i and
    sees keys j <= that position (and j > position - window when a window is given: ours,
    the reference has no window)."""
    tq, nh, _ = q.shape
    tk, nkv, _ = k.shape
    rep = nh // nkv
    k = k.repeat_interleave(rep, dim=1)
    v = v.repeat_interleave(rep, dim=1)
    scores = torch.einsum("qhd,khd->hqk", q, k) * scale
    q_pos = torch.arange(tq)[:, None] + (tk - tq)
    k_pos = torch.arange(tk)[None, :]
    masked = k_pos > q_pos
    if window is not None:
        masked = masked | (k_pos <= q_pos - window)
    scores = scores.masked_fill(masked, float("-inf"))
    probs = torch.softmax(scores, dim=-1)
    return torch.einsum("hqk,khd->qhd", probs, v)


def swiglu(x, gate_w, up_w, down_w) -> torch.Tensor:
    """clockwork/engine/model.py:62-63 - down(silu(gate(x)) * up(x)), no biases."""
    return linear(torch.nn.functional.silu(linear(x, gate_w)) * linear(x, up_w), down_w)


# ------------------------------------------------------------------------------- the model
class PlainQwen2:
    def __init__(self, model_dir, dtype=torch.float32) -> None:
        model_dir = Path(model_dir)
        c = json.loads((model_dir / "config.json").read_text())
        assert c["model_type"] == "qwen2"  # clockwork/engine/loader.py:70-71
        self.cfg = c
        self.dtype = dtype
        self.L = c["num_hidden_layers"]
        self.nh = c["num_attention_heads"]
        self.nkv = c["num_key_value_heads"]
        # clockwork/engine/model.py:17-18
        self.hd = c.get("head_dim") or c["hidden_size"] // self.nh
        self.eps = c["rms_norm_eps"]
        self.theta = float(c["rope_theta"])
        self.tied = bool(c.get("tie_word_embeddings", False))
        self.scale = self.hd ** -0.5  # clockwork/engine/model.py:73
        self.w = {k: v.to(dtype) for k, v in load_file(str(model_dir / "model.safetensors")).items()}
        if self.tied and "lm_head.weight" not in self.w:
            # clockwork/engine/model.py:217-218
            self.w["lm_head.weight"] = self.w["model.embed_tokens.weight"]

    def layer(self, i: int, h: torch.Tensor, cos, sin) -> torch.Tensor:
        """clockwork/engine/model.py:147-154 (wiring) and 87-128 (attention)."""
        w, p = self.w, f"model.layers.{i}."
        T = h.shape[0]
        r = h
        x = rmsnorm(h, w[p + "input_layernorm.weight"], self.eps)
        q = linear(x, w[p + "self_attn.q_proj.weight"], w[p + "self_attn.q_proj.bias"]).view(T, self.nh, self.hd)
        k = linear(x, w[p + "self_attn.k_proj.weight"], w[p + "self_attn.k_proj.bias"]).view(T, self.nkv, self.hd)
        v = linear(x, w[p + "self_attn.v_proj.weight"], w[p + "self_attn.v_proj.bias"]).view(T, self.nkv, self.hd)
        q, k = apply_rope(q, cos, sin), apply_rope(k, cos, sin)
        a = attention_dense(q, k, v, self.scale)
        h = r + linear(a.reshape(T, self.nh * self.hd), w[p + "self_attn.o_proj.weight"])
        r = h
        x = rmsnorm(h, w[p + "post_attention_layernorm.weight"], self.eps)
        return r + swiglu(x, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])

    @torch.no_grad()
    def logits(self, token_ids) -> torch.Tensor:
        """All-position logits [T, vocab] of one whole sequence (model.py:200-204, 228-233)."""
        ids = torch.as_tensor(token_ids, dtype=torch.long)
        h = embedding(self.w["model.embed_tokens.weight"], ids)
        cos, sin = reference_rope_tables(torch.arange(len(ids)), self.hd, self.theta, self.dtype)
        for i in range(self.L):
            h = self.layer(i, h, cos, sin)
        h = rmsnorm(h, self.w["model.norm.weight"], self.eps)
        return linear(h, self.w["lm_head.weight"])

    def greedy(self, prompt, n: int) -> list[int]:
        """Greedy continuation by full recompute (tests/test_hf_equivalence.py:58-69)."""
        ids = list(prompt)
        out = []
        for _ in range(n):
            nxt = int(self.logits(ids)[-1].argmax())
            ids.append(nxt)
            out.append(nxt)
        return out


# ------------------------------------------------------------------------------- sampling
def philox4x32_10(seed: int, counter: int) -> int:
    """First output word of Philox4x32-10 (Salmon et al., "Parallel random numbers: as easy
    as 1, 2, 3"), key = seed's two halves, counter = (counter's two halves, 0, 0)."""
    M0, M1, W0, W1, mask = 0xD2511F53, 0xCD9E8D57, 0x9E3779B9, 0xBB67AE85, 0xFFFFFFFF
    c = [counter & mask, (counter >> 32) & mask, 0, 0]
    k = [seed & mask, (seed >> 32) & mask]
    for _ in range(10):
        p0, p1 = M0 * c[0], M1 * c[2]
        c = [((p1 >> 32) ^ c[1] ^ k[0]) & mask, p1 & mask, ((p0 >> 32) ^ c[3] ^ k[1]) & mask, p0 & mask]
        k = [(k[0] + W0) & mask, (k[1] + W1) & mask]
    return c[0]


def uniform01(seed: int, counter: int) -> float:
    return (philox4x32_10(seed, counter) >> 8) / 16777216.0


def sampling_probs(logits: torch.Tensor, temperature: float, top_k: int = -1, top_p: float = 1.0) -> torch.Tensor:
    """clockwork/engine/model_runner.py:147-164 - temperature, top-k, top-p, softmax; float64 here."""
    x = logits.to(torch.float64) / temperature
    if 0 < top_k < x.shape[-1]:
        kth = torch.topk(x, top_k).values[-1]
        x = x.masked_fill(x < kth, float("-inf"))
    if top_p < 1.0:
        sorted_x, order = torch.sort(x, descending=True)
        cum = torch.softmax(sorted_x, dim=-1).cumsum(-1)
        removed = cum > top_p
        removed[1:] = removed[:-1].clone()
        removed[0] = False
        mask = torch.zeros_like(removed)
        mask[order] = removed
        x = x.masked_fill(mask, float("-inf"))
    return torch.softmax(x, dim=-1)


def draw(probs: torch.Tensor, u: float) -> tuple[int, float]:
    """Inverse CDF in index order: the first index whose running sum exceeds u. Also returns the
    distance of u to the nearest boundary of that index's interval (for tests: a draw that
    close to a boundary may legitimately fall on either side in float32)."""
    cdf = probs.to(torch.float64).cumsum(-1)
    idx = int(torch.searchsorted(cdf, torch.tensor(u, dtype=torch.float64), right=True))
    idx = min(idx, probs.numel() - 1)
    lo = float(cdf[idx - 1]) if idx > 0 else 0.0
    return idx, min(abs(u - lo), abs(float(cdf[idx]) - u))
