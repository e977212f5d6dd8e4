"""The decoder as data: an embedding, a list of blocks, a run list, a final norm, an output head.

Built from a :class:`ModelSpec` through the part registry; nothing here names an
architecture or holds a formula: every tensor operation belongs to a part. Layer order
is the spec's ``run`` list (clockwork/engine/model.py:200-204 is the special case "each
layer once, in order").
"""

from __future__ import annotations

from typing import Optional

import torch

from clockwork_amd.config.spec import ModelSpec, ParamSpec
from clockwork_amd.parts.specs import LinearHeadSpec, TokenEmbeddingSpec
from clockwork_amd.registry import build_arrangement, build_part


def _embedding_spec(spec: ModelSpec):
    return spec.embedding if spec.embedding is not None else TokenEmbeddingSpec(spec.vocab_size, spec.hidden_size)


def _head_spec(spec: ModelSpec):
    return spec.head if spec.head is not None else LinearHeadSpec(spec.vocab_size, spec.hidden_size, spec.tie_embeddings)


def _build_layers(spec: ModelSpec) -> list:
    # identical spec objects still get parts of their own: every layer has its own weights
    return [
        build_arrangement(layer.arrangement, **{name: build_part(part) for name, part in layer.named_parts().items()})
        for layer in spec.layers
    ]


def _named_parts(embedding, layers, final_norm, head) -> list:
    """(prefix of its parameters' names, part) for every part of the model."""
    named = [("embed.", embedding)]
    for i, layer in enumerate(layers):
        named += [(f"layers.{i}.{role}.", part) for role, part in layer.parts().items()]
    named += [("final_norm.", final_norm), ("lm_head.", head)]
    return named


def model_param_specs(spec: ModelSpec) -> dict[str, ParamSpec]:
    """Every tensor the model owns, by its internal name. Needs no GPU."""
    named = _named_parts(build_part(_embedding_spec(spec)), _build_layers(spec), build_part(spec.final_norm),
                         build_part(_head_spec(spec)))
    return {prefix + name: p for prefix, part in named for name, p in part.param_specs().items()}


class DecoderModel:
    def __init__(self, spec: ModelSpec) -> None:
        spec.validate()
        self.spec = spec
        self.embedding = build_part(_embedding_spec(spec))
        self.layers = _build_layers(spec)
        self.final_norm = build_part(spec.final_norm)
        self.head = build_part(_head_spec(spec))

    def named_parts(self) -> list:
        return _named_parts(self.embedding, self.layers, self.final_norm, self.head)

    def param_specs(self) -> dict[str, ParamSpec]:
        return {prefix + name: p for prefix, part in self.named_parts() for name, p in part.param_specs().items()}

    def mixers(self) -> list:
        """Per layer the part that owns its cache (the one named ``mixer``), or None."""
        return [layer.parts().get("mixer") for layer in self.layers]

    def kernel_libraries(self) -> list:
        """(library, head size or None) pairs that the parts say they run: compiled and loaded
        before the first step."""
        jobs = []
        for _, part in self.named_parts():
            for job in getattr(part, "kernel_libraries", lambda: [])():
                if job not in jobs:
                    jobs.append(job)
        return jobs

    def graph_safe(self) -> bool:
        """True when every part says its step is a fixed sequence of GPU launches (no host reads,
        no data-dependent shapes), so that a step can be captured into a HIP graph."""
        return all(getattr(part, "graph_safe", False) for _, part in self.named_parts())

    def prepare(self, ctx) -> None:
        """Let every part make what it needs of this step's shape ahead of its ``forward`` (work
        items of its kernels, uploaded): a step that is captured as a graph must not plan, and so
        upload, inside the capture. Parts keep such things in ``ctx.plans``."""
        for _, part in self.named_parts():
            prepare = getattr(part, "prepare", None)
            if prepare is not None:
                prepare(ctx)

    def shape_class(self, q_lens, ctx_lens) -> tuple:
        """What of a step's shape, beyond its token counts, decides which kernels the parts
        launch: a captured graph serves the steps of its own class only."""
        out = []
        for _, part in self.named_parts():
            classify = getattr(part, "shape_class", None)
            if classify is not None:
                label = classify(q_lens, ctx_lens)
                if label not in out:
                    out.append(label)
        return tuple(out)

    def bind(self, params: dict, device, dtype) -> None:
        self.device, self.dtype = device, dtype
        params = dict(params)
        if getattr(getattr(self.head, "spec", None), "tied", False) and hasattr(self.head, "use_embedding"):
            self.head.use_embedding(self.embedding)
        for prefix, part in self.named_parts():
            part.bind({k[len(prefix):]: v for k, v in params.items() if k.startswith(prefix)}, device, dtype)
        if getattr(self.head, "shares_embedding", False):
            # a head's tensor that the checkpoint brought beside the table it is tied to is not kept
            for name in [k for k in params if k.startswith("lm_head.")]:
                del params[name]
        self.params = params

    def weight_bytes_per_step(self) -> int:
        """Bytes of weights a decode step reads: every matrix once; of the embedding's tensors
        only the rows of the step's tokens (not counted), the output head's whole."""
        total = 0
        seen = set()

        def count(t):
            nonlocal total
            if t.data_ptr() not in seen:
                seen.add(t.data_ptr())
                total += t.numel() * t.element_size()

        for name, t in self.params.items():
            if not name.startswith("embed."):
                count(t)
        for t in getattr(self.head, "matrices", lambda: [])():
            count(t)
        return total

    def forward(self, ctx, caches) -> Optional[torch.Tensor]:
        """Run the step's tokens; returns float32 logits [len(ctx.logit_rows), vocab] or None
        when no logits are wanted. ``caches[i]`` is the EntryCache of run entry i."""
        # what ``ctx.positions`` holds is the embedding part's to say: without its word every token
        # carries its index in its request (``ctx.sequence_positions``, which stays what it is)
        positions_of = getattr(self.embedding, "positions", None)
        if positions_of is not None:
            ctx.positions = positions_of(ctx)
        resid = self.embedding.forward(ctx)
        delta = None
        run = self.spec.run
        for i, entry in enumerate(run):
            # may this block hand on two pending outputs? Only if the norm that takes them next (the
            # next block's first norm, as that block's arrangement names it, or the final norm) can
            if i + 1 < len(run):
                first_norm = getattr(self.layers[run[i + 1].layer], "first_norm", None)
                nxt = first_norm() if first_norm is not None else None
            else:
                nxt = self.final_norm
            ctx.next_norm_accepts_pending = bool(getattr(nxt, "accepts_pending", False))
            delta = self.layers[entry.layer].forward(resid, delta, ctx, caches[i])
        if ctx.num_logit_rows == 0:
            return None
        rows = self.final_norm.forward(resid, delta, rows=ctx.logit_rows)
        return self.head.forward(rows, ctx)
