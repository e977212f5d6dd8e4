"""The decoder as data: an embedding, a list of blocks, a run list, a final norm, an output head.

Built from a :class:`ModelSpec` through the part registry; nothing here names an
architecture. Layer order is the spec's ``run`` list (clockwork/engine/model.py:200-204
is the special case "each layer once, in order").
"""

from __future__ import annotations

from typing import Optional

import torch

from clockwork_amd import ops
from clockwork_amd.config.spec import ModelSpec, ParamSpec
from clockwork_amd.registry import build_arrangement, build_part

_ROLES = ("mixer", "feed_forward", "mixer_norm", "ffn_norm")


def _build_layers(spec: ModelSpec) -> list:
    layers = []
    for layer_spec in spec.layers:
        # identical spec objects still get parts of their own: every layer has its own weights
        layers.append(
            build_arrangement(
                layer_spec.arrangement,
                mixer=build_part(layer_spec.mixer),
                feed_forward=build_part(layer_spec.feed_forward),
                mixer_norm=build_part(layer_spec.mixer_norm),
                ffn_norm=build_part(layer_spec.ffn_norm),
            )
        )
    return layers


def _param_specs(spec: ModelSpec, layers, final_norm) -> dict[str, ParamSpec]:
    out = {"embed.weight": ParamSpec((spec.vocab_size, spec.hidden_size))}
    for i, layer in enumerate(layers):
        for role, part in layer.parts().items():
            for name, p in part.param_specs().items():
                out[f"layers.{i}.{role}.{name}"] = p
    for name, p in final_norm.param_specs().items():
        out[f"final_norm.{name}"] = p
    out["lm_head.weight"] = ParamSpec((spec.vocab_size, spec.hidden_size))
    return out


def model_param_specs(spec: ModelSpec) -> dict[str, ParamSpec]:
    """Every tensor the model owns, by its internal name. Needs no GPU."""
    return _param_specs(spec, _build_layers(spec), build_part(spec.final_norm))


class DecoderModel:
    def __init__(self, spec: ModelSpec) -> None:
        spec.validate()
        self.spec = spec
        self.layers = _build_layers(spec)
        self.final_norm = build_part(spec.final_norm)

    def param_specs(self) -> dict[str, ParamSpec]:
        return _param_specs(self.spec, self.layers, self.final_norm)

    def mixers(self) -> list:
        return [layer.mixer for layer in self.layers]

    def head_dims(self) -> list[int]:
        """Head sizes whose attention kernels this model runs."""
        dims = []
        for layer in self.layers:
            hd = getattr(getattr(layer.mixer, "spec", None), "head_dim", None)
            if hd is not None and hasattr(layer.mixer, "position"):
                dims.append(int(hd))
        return dims

    def attention_geometries(self) -> list[tuple[int, int]]:
        """(heads, kv heads) of every attention mixer: what attention work plans are made for."""
        found = []
        for layer in self.layers:
            spec = getattr(layer.mixer, "spec", None)
            if hasattr(layer.mixer, "position") and spec is not None:
                geo = (spec.num_heads, spec.num_kv_heads)
                if geo not in found:
                    found.append(geo)
        return found

    def graph_safe(self) -> bool:
        """True when every part says its step is a fixed sequence of GPU launches (no host reads,
        no data-dependent shapes), so that a decode step can be captured into a HIP graph."""
        parts = [self.final_norm]
        for layer in self.layers:
            parts += list(layer.parts().values())
        return all(getattr(part, "graph_safe", False) for part in parts)

    def bind(self, params: dict, device, dtype) -> None:
        self.device, self.dtype = device, dtype
        self.embed = params["embed.weight"]
        if "lm_head.weight" in params:
            self.lm_head = params["lm_head.weight"]
        elif self.spec.tie_embeddings:
            # one buffer, two uses (clockwork/engine/model.py:217-218)
            self.lm_head = self.embed
        else:
            raise RuntimeError("lm_head.weight is missing and the embeddings are not tied")
        for i, layer in enumerate(self.layers):
            for role, part in layer.parts().items():
                prefix = f"layers.{i}.{role}."
                part.bind({k[len(prefix):]: v for k, v in params.items() if k.startswith(prefix)}, device, dtype)
        self.final_norm.bind({k[len("final_norm."):]: v for k, v in params.items() if k.startswith("final_norm.")}, device, dtype)
        self.params = params

    def weight_bytes_per_step(self) -> int:
        """Bytes of weights a decode step reads: every matrix once; of the embedding table only
        the rows of the step's tokens (not counted), the output head whole."""
        total = 0
        seen = set()
        for name, t in self.params.items():
            if name == "embed.weight" or t.data_ptr() in seen:
                continue
            seen.add(t.data_ptr())
            total += t.numel() * t.element_size()
        if self.lm_head.data_ptr() not in seen:
            total += self.lm_head.numel() * self.lm_head.element_size()
        return total

    def forward(self, ctx, caches) -> Optional[torch.Tensor]:
        """Run the step's tokens; returns float32 logits [len(ctx.logit_rows), vocab] or None
        when no logits are wanted. ``caches[i]`` is the EntryCache of run entry i."""
        T = ctx.num_tokens
        resid = torch.empty((T, self.spec.hidden_size), dtype=torch.float32, device=self.device)
        ops.embedding(self.embed, ctx.token_ids, resid)
        delta = None
        run = self.spec.run
        for i, entry in enumerate(run):
            # may this block hand on two pending outputs? Only if the norm that comes next takes them
            nxt = self.layers[run[i + 1].layer].parts().get("mixer_norm") if i + 1 < len(run) else self.final_norm
            ctx.next_norm_accepts_pending = bool(getattr(nxt, "accepts_pending", False))
            delta = self.layers[entry.layer].forward(resid, delta, ctx, caches[i])
        if ctx.num_logit_rows == 0:
            return None
        rows = self.final_norm.forward(resid, delta, rows=ctx.logit_rows)
        return ops.linear(rows, self.lm_head, out_dtype=torch.float32)
