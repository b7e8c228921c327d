"""Pre-norm residual block: ``h += mixer(norm_in(h)); h += ffn(norm_post(h))``.

Order of the parts as in utils/model.py:15-35.  The block keeps the reference's
fused dataflow (utils/model.py:87-100): the residual stream and the update that
is still to be added travel as a pair, so every "add, then normalise" is one kernel.
"""
from __future__ import annotations

from .base import Block, FeedForward, Mixer, Norm, ResidualSink, StreamUpdate


class PreNormBlock(Block):
    takes_following = True

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
    def _feed(norm, consumer, resid, delta, ctx, *args, following=None):
        """Run ``consumer`` on ``norm(resid + delta)``; returns ``(resid + delta, consumer's output)``.

        A consumer that starts with a projection gets the normalisation still pending, so that the
        projection may apply a norm that the previous projection prepared (``delta`` is then a
        :class:`StreamUpdate`); otherwise the norm runs first, in its own kernel.  A consumer that
        ends with a projection is told the norm that follows its output (``following``), so that
        this projection may in turn add its result to the stream and prepare that norm."""
        if consumer.accepts_pending_norm:
            pending = norm.defer(resid, delta, ctx)
            kwargs = {}
            if following is not None and consumer.takes_sink:
                kwargs["sink"] = ResidualSink(pending, following)
            out = consumer.forward(pending, ctx, *args, **kwargs)
            if pending.delta is not None:          # nobody used it: the update must still be added
                pending.tensor()
            return pending.resid, out
        if isinstance(delta, StreamUpdate):
            resid, delta = delta.resid, None
        return resid, consumer.forward(norm.add_norm(resid, delta, ctx), ctx, *args)

    def entry_norm(self):
        return self.mixer_norm

    def forward(self, resid, delta, ctx, cache, following=None):
        """``following``: the norm that will be applied to this block's output, if the caller knows it."""
        resid, mixed = self._feed(self.mixer_norm, self.mixer, resid, delta, ctx, cache, following=self.ffn_norm)
        return self._feed(self.ffn_norm, self.ffn, resid, mixed, ctx, following=following)
