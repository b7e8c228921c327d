"""Pre-norm residual block: ``h += mixer(norm_in(h)); h += ffn(norm_post(h))``.

Order of the parts as in /root/reference/utils/model.py:15-35.  The block keeps the reference's
fused dataflow (/root/reference/utils/model.py:87-100): the residual stream and the update that
is still to be added travel as a pair, so every "add, then normalise" is one kernel.
"""
from __future__ import annotations

from .base import Block, FeedForward, Mixer, Norm


class PreNormBlock(Block):
    def __init__(self, mixer_norm: Norm, mixer: Mixer, ffn_norm: Norm, ffn: FeedForward,
                 names=("input_layernorm", "self_attn", "post_attention_layernorm", "mlp")):
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn = mixer_norm, mixer, ffn_norm, ffn
        self.names = tuple(names)

    def _parts(self):
        return dict(zip(self.names, (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn)))

    def param_specs(self):
        return {f"{prefix}.{name}": spec for prefix, part in self._parts().items() for name, spec in part.param_specs().items()}

    def assign(self, name, tensor):
        prefix, rest = name.split(".", 1)
        self._parts()[prefix].assign(rest, tensor)

    def finalize(self):
        for part in self._parts().values():
            part.finalize()

    @staticmethod
    def _feed(norm, consumer, resid, delta, ctx, *args):
        """Run ``consumer`` on ``norm(resid + delta)``; returns ``(resid + delta, consumer's output)``.

        A consumer that starts with a projection gets the normalisation still pending, so that the
        projection's kernel may do the sum and the norm itself (few rows); otherwise the norm runs
        first, in its own kernel."""
        if consumer.accepts_pending_norm and hasattr(norm, "defer"):
            pending = norm.defer(resid, delta, ctx)
            out = consumer.forward(pending, ctx, *args)
            if pending.delta is not None:          # nobody used it: the update must still be added
                pending.tensor()
            return pending.resid, out
        return resid, consumer.forward(norm.add_norm(resid, delta, ctx), ctx, *args)

    def forward(self, resid, delta, ctx, cache):
        resid, mixed = self._feed(self.mixer_norm, self.mixer, resid, delta, ctx, cache)
        return self._feed(self.ffn_norm, self.ffn, resid, mixed, ctx)
