"""Qwen2 / Qwen2.5 dense decoder: config.json keys -> typed config -> parts -> weight names.

The architecture as the reference runs it (clockwork/engine/model.py:17-233):
pre-norm blocks of grouped-query attention (q/k/v bias on, o bias off, NeoX
rotary, full causal) and a SwiGLU feed-forward, RMSNorm everywhere, optionally
tied output head.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

from clockwork_amd.config.spec import LayerSpec, ModelSpec, RunEntry, WeightTarget
from clockwork_amd.parts.specs import AttentionSpec, RMSNormSpec, RopeNeoxSpec, SwiGLUSpec
from clockwork_amd.registry import Architecture, register_architecture

_REQUIRED = (
    "vocab_size",
    "hidden_size",
    "num_hidden_layers",
    "num_attention_heads",
    "num_key_value_heads",
    "intermediate_size",
    "rms_norm_eps",
)


@dataclass(frozen=True)
class Qwen2Config:
    """The keys of a Qwen2 ``config.json`` that the model reads (clockwork/engine/model.py)."""

    vocab_size: int
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    rms_norm_eps: float
    rope_theta: float
    tie_word_embeddings: bool = False
    hidden_act: str = "silu"
    use_sliding_window: bool = False
    pad_token_id: Optional[int] = None
    eos_token_ids: tuple[int, ...] = ()
    max_position_embeddings: Optional[int] = None  # informative: the model does not read it

    @classmethod
    def from_dict(cls, d: dict) -> "Qwen2Config":
        if d.get("model_type") not in (None, "qwen2"):
            raise ValueError(f"expected a qwen2 model, got model_type={d.get('model_type')!r}")
        missing = [k for k in _REQUIRED if d.get(k) is None]
        if missing:
            raise ValueError(f"config.json lacks required keys: {missing}")
        hidden_act = d.get("hidden_act", "silu")
        if hidden_act != "silu":
            # clockwork/engine/model.py:55-57
            raise NotImplementedError(f"hidden_act {hidden_act!r} is not supported")
        if d.get("use_sliding_window", False):
            # clockwork/engine/model.py:211-212
            raise NotImplementedError("sliding-window attention is not supported")
        nh = int(d["num_attention_heads"])
        hidden = int(d["hidden_size"])
        # clockwork/engine/model.py:17-18: head_dim, else hidden_size // heads
        head_dim = d.get("head_dim") or hidden // nh
        eos = d.get("eos_token_id")
        if eos is None:
            eos_ids: tuple[int, ...] = ()
        elif isinstance(eos, int):
            eos_ids = (eos,)
        else:
            eos_ids = tuple(int(e) for e in eos)
        cfg = cls(
            vocab_size=int(d["vocab_size"]),
            hidden_size=hidden,
            num_hidden_layers=int(d["num_hidden_layers"]),
            num_attention_heads=nh,
            num_key_value_heads=int(d["num_key_value_heads"]),
            head_dim=int(head_dim),
            intermediate_size=int(d["intermediate_size"]),
            rms_norm_eps=float(d["rms_norm_eps"]),
            rope_theta=_rope_theta(d),
            tie_word_embeddings=bool(d.get("tie_word_embeddings", False)),
            hidden_act=hidden_act,
            use_sliding_window=False,
            pad_token_id=d.get("pad_token_id"),
            eos_token_ids=eos_ids,
            max_position_embeddings=d.get("max_position_embeddings"),
        )
        cfg.check()
        return cfg

    def check(self) -> None:
        for name in ("vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads",
                     "num_key_value_heads", "head_dim", "intermediate_size"):
            if getattr(self, name) <= 0:
                raise ValueError(f"{name} must be positive, got {getattr(self, name)}")
        if self.num_attention_heads % self.num_key_value_heads != 0:
            # clockwork/kernels/attention.py:39-40
            raise ValueError(
                f"num_heads {self.num_attention_heads} not a multiple of "
                f"num_kv_heads {self.num_key_value_heads}"
            )
        if self.head_dim % 2 != 0:
            raise ValueError(f"head_dim {self.head_dim} must be even for rotary pairs")
        if self.rms_norm_eps <= 0 or self.rope_theta <= 0:
            raise ValueError("rms_norm_eps and rope_theta must be positive")


def _rope_theta(d: dict) -> float:
    """clockwork/engine/model.py:21-29: rope_parameters{rope_type, rope_theta}, else rope_theta."""
    for key in ("rope_parameters", "rope_scaling"):
        params = d.get(key)
        if params:
            rope_type = params.get("rope_type", params.get("type", "default"))
            if rope_type != "default":
                raise NotImplementedError(f"rope_type {rope_type!r} is not supported")
            if "rope_theta" in params:
                return float(params["rope_theta"])
    if d.get("rope_theta") is None:
        raise ValueError("config.json lacks required keys: ['rope_theta']")
    return float(d["rope_theta"])


def build_spec(cfg: Qwen2Config) -> ModelSpec:
    attention = AttentionSpec(
        hidden_size=cfg.hidden_size,
        num_heads=cfg.num_attention_heads,
        num_kv_heads=cfg.num_key_value_heads,
        head_dim=cfg.head_dim,
        qkv_bias=True,   # clockwork/engine/model.py:74-76
        out_bias=False,  # clockwork/engine/model.py:77
        scale=cfg.head_dim ** -0.5,  # clockwork/engine/model.py:73
        window=None,
        position=RopeNeoxSpec(rotary_dim=cfg.head_dim, theta=cfg.rope_theta),
    )
    norm = RMSNormSpec(size=cfg.hidden_size, eps=cfg.rms_norm_eps)
    layer = LayerSpec(
        arrangement="prenorm",
        mixer=attention,
        feed_forward=SwiGLUSpec(cfg.hidden_size, cfg.intermediate_size),
        mixer_norm=norm,
        ffn_norm=norm,
    )
    n = cfg.num_hidden_layers
    spec = ModelSpec(
        architecture="Qwen2ForCausalLM",
        vocab_size=cfg.vocab_size,
        hidden_size=cfg.hidden_size,
        layers=[layer] * n,
        run=[RunEntry(layer=i) for i in range(n)],
        final_norm=norm,
        tie_embeddings=cfg.tie_word_embeddings,
        eos_token_ids=cfg.eos_token_ids,
        info={
            "layers": n,
            "hidden": cfg.hidden_size,
            "heads": cfg.num_attention_heads,
            "kv_heads": cfg.num_key_value_heads,
            "head_dim": cfg.head_dim,
            "intermediate": cfg.intermediate_size,
            "vocab": cfg.vocab_size,
            "rope_theta": cfg.rope_theta,
            "rms_norm_eps": cfg.rms_norm_eps,
            "tied": cfg.tie_word_embeddings,
        },
    )
    spec.validate()
    return spec


def weight_plan(cfg: Qwen2Config, spec: ModelSpec) -> list[WeightTarget]:
    """Checkpoint names (clockwork/engine/model.py module tree) -> the model's parameters.

    q/k/v and gate/up are stored apart and run as one product each, so they are
    concatenated along the output dimension here.
    """
    H, I = cfg.hidden_size, cfg.intermediate_size
    q = cfg.num_attention_heads * cfg.head_dim
    kv = cfg.num_key_value_heads * cfg.head_dim
    plan = [WeightTarget("embed.weight", ("model.embed_tokens.weight",), ((cfg.vocab_size, H),))]
    for i in range(cfg.num_hidden_layers):
        src = f"model.layers.{i}"
        dst = f"layers.{i}"
        attn = f"{src}.self_attn"
        plan += [
            WeightTarget(f"{dst}.mixer_norm.weight", (f"{src}.input_layernorm.weight",), ((H,),)),
            WeightTarget(
                f"{dst}.mixer.qkv_weight",
                (f"{attn}.q_proj.weight", f"{attn}.k_proj.weight", f"{attn}.v_proj.weight"),
                ((q, H), (kv, H), (kv, H)),
            ),
            WeightTarget(
                f"{dst}.mixer.qkv_bias",
                (f"{attn}.q_proj.bias", f"{attn}.k_proj.bias", f"{attn}.v_proj.bias"),
                ((q,), (kv,), (kv,)),
            ),
            WeightTarget(f"{dst}.mixer.out_weight", (f"{attn}.o_proj.weight",), ((H, q),)),
            WeightTarget(
                f"{dst}.ffn_norm.weight", (f"{src}.post_attention_layernorm.weight",), ((H,),)
            ),
            WeightTarget(
                f"{dst}.feed_forward.gate_up_weight",
                (f"{src}.mlp.gate_proj.weight", f"{src}.mlp.up_proj.weight"),
                ((I, H), (I, H)),
            ),
            WeightTarget(
                f"{dst}.feed_forward.down_weight", (f"{src}.mlp.down_proj.weight",), ((H, I),)
            ),
        ]
    plan.append(WeightTarget("final_norm.weight", ("model.norm.weight",), ((H,),)))
    # clockwork/engine/model.py:217-218 and loader.py:60-62: a tied head is the embedding,
    # and a tied checkpoint may leave lm_head.weight out.
    plan.append(
        WeightTarget(
            "lm_head.weight",
            ("lm_head.weight",),
            ((cfg.vocab_size, H),),
            optional=cfg.tie_word_embeddings,
        )
    )
    return plan


ARCHITECTURE = Architecture(
    name="Qwen2ForCausalLM",
    parse_config=Qwen2Config.from_dict,
    build_spec=build_spec,
    weight_plan=weight_plan,
)
register_architecture(["Qwen2ForCausalLM", "qwen2"], ARCHITECTURE)
