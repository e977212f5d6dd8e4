"""Block arrangements: how norms, mixer and feed-forward sit around the residual stream."""

from __future__ import annotations

from clockwork_amd import ops


class PreNormBlock:
    """x = x + mixer(norm(x)); x = x + ffn(norm(x)) (clockwork/engine/model.py:139-154).

    The residual stream is float32 and is only ever touched by the norms' fused add, so
    each branch output is added exactly once, in float32. ``forward`` takes the previous
    block's pending output ``delta`` and returns its own.
    """

    def __init__(self, mixer, feed_forward, mixer_norm, ffn_norm) -> None:
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.mixer_norm = mixer_norm
        self.ffn_norm = ffn_norm

    def parts(self) -> dict:
        return {
            "mixer": self.mixer,
            "feed_forward": self.feed_forward,
            "mixer_norm": self.mixer_norm,
            "ffn_norm": self.ffn_norm,
        }

    def first_norm(self):
        """The norm that takes what the block before hands on (may it be two pending outputs?)."""
        return self.mixer_norm

    def forward(self, resid, delta, ctx, cache):
        x = self.mixer_norm.forward(resid, delta)
        a = self.mixer.forward(x, ctx, cache)
        # Few rows: the second norm can run inside the feed-forward's first product, which saves a
        # launch. That kernel writes no residual, so the mixer's output stays pending and is
        # handed on together with the feed-forward's (the next norm must be able to take both).
        fuses = getattr(self.feed_forward, "fuses_input_norm", None)
        lazy = getattr(self.ffn_norm, "lazy", None)
        if (fuses is not None and lazy is not None and getattr(ctx, "next_norm_accepts_pending", False)
                and fuses(resid.shape[0], x.dtype, a)):
            return ops.PendingPair(a, self.feed_forward.forward(lazy(resid, a), ctx))
        x = self.ffn_norm.forward(resid, a)
        return self.feed_forward.forward(x, ctx)
