"""The two ends of the decoder: token ids to the residual stream, final rows to logits.

Both are parts like any other (clockwork/engine/model.py:200 and 216-233 are the plain table
lookup and the plain product that these two implement); another architecture registers its own
(a scaled embedding, positions added at the input, a capped or biased output) under its own spec.

Interfaces: an embedding has ``forward(ctx) -> resid`` (float32 [T, hidden], the residual
stream of the step's tokens) and may offer ``table()``, the [vocab, hidden] matrix a tied head
uses. A head has ``forward(rows, ctx) -> logits`` (float32 [n, vocab]) for the normed rows the
step wants logits of; a head whose spec has ``tied`` set is handed the embedding part through
``use_embedding(part)`` before it is bound.
"""

from __future__ import annotations

import torch

from clockwork_amd import ops
from clockwork_amd.config.spec import ParamSpec
from clockwork_amd.parts.base import Part
from clockwork_amd.parts.specs import LinearHeadSpec, TokenEmbeddingSpec


class TokenEmbedding(Part):
    graph_safe = True

    def __init__(self, spec: TokenEmbeddingSpec) -> None:
        self.spec = spec

    def param_specs(self):
        return {"weight": ParamSpec((self.spec.vocab_size, self.spec.hidden_size))}

    def bind(self, params, device, dtype) -> None:
        self.weight = params["weight"]
        self.device = device

    def table(self) -> torch.Tensor:
        return self.weight

    def forward(self, ctx) -> torch.Tensor:
        resid = torch.empty((ctx.num_tokens, self.spec.hidden_size), dtype=torch.float32, device=self.device)
        return ops.embedding(self.weight, ctx.token_ids, resid)


class LinearHead(Part):
    graph_safe = True

    def __init__(self, spec: LinearHeadSpec) -> None:
        self.spec = spec
        self._embedding = None
        self.shares_embedding = False

    def param_specs(self):
        return {"weight": ParamSpec((self.spec.vocab_size, self.spec.hidden_size))}

    def use_embedding(self, embedding) -> None:
        self._embedding = embedding

    def bind(self, params, device, dtype) -> None:
        own = params.get("weight")
        if not self.spec.tied:
            if own is None:
                raise RuntimeError("the output head's matrix is missing and the embeddings are not tied")
            self.weight = own
            return
        # one buffer, two uses (clockwork/engine/model.py:217-218). A tied checkpoint may still
        # carry the head's tensor; the reference loads it into the shared parameter, so it has to
        # be the table itself: it is checked and let go, not kept as a second matrix.
        table = getattr(self._embedding, "table", lambda: None)() if self._embedding is not None else None
        if table is None:
            raise RuntimeError("a tied output head needs an embedding part that offers its table()")
        if own is not None and not (own.shape == table.shape and torch.equal(own, table)):
            raise ValueError(
                "the checkpoint ties the output head to the embedding (tie_word_embeddings) but "
                "carries an lm_head tensor that differs from the embedding table"
            )
        self.weight = table
        self.shares_embedding = True

    def matrices(self) -> list:
        """The matrices a step streams through this part (for the step's byte count)."""
        return [self.weight]

    def forward(self, rows: torch.Tensor, ctx) -> torch.Tensor:
        return ops.linear(rows, self.weight, out_dtype=torch.float32, policy=getattr(ctx, "products", None))
