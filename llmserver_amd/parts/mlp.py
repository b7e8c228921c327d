"""Gated feed-forward ``down(act(gate(x)) * up(x))``; ``act`` is SiLU in every model built so far.

Gate and up are one stacked product, gate first (utils/layers.py:194-218;
utils/fused_ops.py:59-61, 80-88).  Sigmoid and the product run in 32-bit inside
the activation kernel.
"""
from __future__ import annotations

import dataclasses
from typing import Tuple

from .base import FeedForward, PendingNorm
from .linear import Linear


@dataclasses.dataclass(frozen=True)
class GatedMLPNames:
    """Checkpoint names of the layer's tensors.  ``gate_up``: the gate and the up projection, or one tensor that holds
    the gate's rows followed by the up projection's."""
    gate_up: Tuple[str, ...] = ("gate_proj", "up_proj")
    down: str = "down_proj"


class GatedMLP(FeedForward):
    accepts_pending_norm = True
    takes_sink = True

    # config.json's names of an activation -> the name the kernels know it by (utils/layers.py:182 in the
    # reference lists more; a further one is an entry here and a branch in the activation kernel and the gated epilogues)
    ACTIVATIONS = {"silu": "silu", "swish": "silu"}

    def __init__(self, width: int, intermediate: int, activation: str = "silu", bias: bool = False,
                 names: GatedMLPNames = GatedMLPNames()):
        if activation not in self.ACTIVATIONS:
            raise ValueError(f"Unsupported activation {activation!r}; supported: {sorted(self.ACTIVATIONS)}")
        self.activation = self.ACTIVATIONS[activation]
        self.width = width
        self.intermediate = intermediate
        if len(names.gate_up) not in (1, 2):
            raise ValueError(f"gate and up projection come in one or two checkpoint tensors, not {len(names.gate_up)}")
        self.names = names
        self.gate_up = Linear(width, names.gate_up, (intermediate, intermediate) if len(names.gate_up) == 2 else (2 * intermediate,), bias)
        self.down = Linear(intermediate, (names.down,), (width,), bias)

    def param_specs(self):
        return {**self.gate_up.param_specs(), **self.down.param_specs()}

    def assign(self, name, tensor):
        owner = name.rsplit(".", 1)[0]
        if owner == self.names.down:
            self.down.assign(name, tensor)
        elif owner in self.names.gate_up:
            self.gate_up.assign(name, tensor)
        else:
            raise KeyError(name)

    def finalize(self):
        self.gate_up.finalize()
        self.down.finalize()

    def forward(self, x, ctx, sink=None):
        ops = ctx.ops
        if self.gate_up.bias is None:
            # Few rows: one launch for both products with the activation in its epilogue.
            row_scale = None
            tensor = x
            if isinstance(x, PendingNorm):
                scaled = x.row_scale() if ops.fuse_stream_updates else None
                if scaled is not None and ops.row_scale_fits(scaled[0], self.gate_up.weight, scaled[1]):
                    tensor, row_scale = scaled
                else:
                    tensor = x.tensor()
            hidden = ops.linear_gated(tensor, self.gate_up.weight, row_scale=row_scale, activation=self.activation)
            if hidden is not None:
                return self.down.forward(hidden, ctx, sink=sink)
            if row_scale is not None:
                tensor = x.tensor()
            x = tensor
        gate_up = self.gate_up.forward(x, ctx)
        hidden = ctx.empty((gate_up.shape[0], self.intermediate))
        ops.swiglu(gate_up, hidden, activation=self.activation)
        return self.down.forward(hidden, ctx, sink=sink)
