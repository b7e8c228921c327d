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

    def forward(self, resid, delta, ctx, cache):
        normed = self.mixer_norm.add_norm(resid, delta, ctx)
        mixed = self.mixer.forward(normed, ctx, cache)
        normed = self.ffn_norm.add_norm(resid, mixed, ctx)
        return self.ffn.forward(normed, ctx)
