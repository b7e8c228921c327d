"""Linear projection ``y = x W^T (+ b)`` with ``W [out, in]`` as checkpoints store it.

The matrix product itself is a library call, as in the reference's engine, which runs every
projection through the vendor GEMM behind ``nn.Linear`` (utils/attention.py:33-37,
utils/layers.py:188-191).  Several checkpoint matrices can be stacked along the
output dimension into one product (utils/attention.py:54-66,
utils/layers.py:194-203).
"""
from __future__ import annotations

from typing import Dict, Sequence

import torch

from .base import MATRIX, VECTOR, ParamSpec, Part, PendingNorm, StreamUpdate


class Linear(Part):
    """One GEMM over one or several stacked checkpoint matrices.

    ``names``/``out_features`` list the stacked pieces in output order, e.g. ``("q_proj",
    "k_proj", "v_proj")``.  Tensor names are ``<piece>.weight`` and ``<piece>.bias``.
    """

    def __init__(self, in_features: int, pieces: Sequence[str], out_features: Sequence[int], bias: bool = False,
                 out_float32: bool = False):
        self.in_features = in_features
        self.pieces = tuple(pieces)
        self.piece_out = tuple(out_features)
        self.out_features = sum(out_features)
        self.has_bias = bias
        self.out_float32 = out_float32
        self._w: Dict[str, torch.Tensor] = {}
        self._b: Dict[str, torch.Tensor] = {}
        self.weight = None   # [out, in] compute dtype
        self.bias = None     # [out] float32
        self.bias_rounded = None   # the bias in the weight's type, if that type holds it exactly (a library's product takes it so)

    def param_specs(self):
        specs = {}
        for piece, n in zip(self.pieces, self.piece_out):
            specs[f"{piece}.weight"] = ParamSpec((n, self.in_features), MATRIX, "normal")
            if self.has_bias:
                specs[f"{piece}.bias"] = ParamSpec((n,), VECTOR, "bias")
        return specs

    def assign(self, name, tensor):
        piece, kind = name.rsplit(".", 1)
        (self._w if kind == "weight" else self._b)[piece] = tensor

    def share_weight(self, tensor: torch.Tensor) -> None:
        """Use an existing matrix (a tied output head aliases the embedding table, no copy)."""
        self.weight = tensor

    def finalize(self):
        if self.weight is None:
            ws = [self._w[p] for p in self.pieces]
            self.weight = ws[0] if len(ws) == 1 else torch.cat(ws, dim=0)
        if self.has_bias and self.bias is None:
            bs = [self._b[p] for p in self.pieces]
            self.bias = bs[0] if len(bs) == 1 else torch.cat(bs, dim=0)
        if self.bias is not None and self.weight.dtype != torch.float32:
            rounded = self.bias.to(self.weight.dtype)
            self.bias_rounded = rounded if torch.equal(rounded.to(self.bias.dtype), self.bias) else None
        self._w.clear()
        self._b.clear()

    def forward(self, x, ctx, out=None, sink=None):
        """``x`` is a tensor or a :class:`PendingNorm`.  With ``sink`` (a :class:`ResidualSink`) the result may
        come back as a :class:`StreamUpdate`: already added to the residual stream, the following norm prepared
        or carried out."""
        ops = ctx.ops
        fused = ops.fuse_stream_updates
        row_scale = None
        if isinstance(x, PendingNorm):
            scaled = x.row_scale() if fused else None
            if scaled is not None and ops.row_scale_fits(scaled[0], self.weight, scaled[1]) \
                    and not ops.library_is_faster("plain", scaled[0], self.weight, True, self.out_float32):
                x, row_scale = scaled            # the norm becomes a scale of the product's rows
            else:
                x = x.tensor()
        following = sink.norm.row_scale_form() if sink is not None and fused and self.bias is None and not self.out_float32 else None
        if following is not None:
            # The product may leave its result as partial sums, which the kernel of the sum and the norm adds up on
            # its way: that is the way of 17 rows and more, and of fewer where it has been measured to be faster.
            split_few_rows = row_scale is None and ops.partial_sums_are_faster(x, self.weight)
            if not split_few_rows:
                done = ops.linear_into_stream(x, self.weight, sink.stream(), following[0], row_scale=row_scale)
                if done is not None:
                    return StreamUpdate(sink.norm, *done)
            sums = None
            if row_scale is None:
                sums = ops.linear_partial_sums(x, self.weight, few_rows_too=split_few_rows)
            if sums is not None:
                stream = sink.stream()
                return StreamUpdate(sink.norm, stream, normed=sink.norm.add_norm(stream, sums, ctx))
        if self.bias is not None and ops.fuses_bias:
            # The bias joins the product's float32 sums, which are then rounded once.
            if row_scale is not None:
                return ops.linear_few_rows(x, self.weight, out=out, out_float32=self.out_float32, row_scale=row_scale, bias=self.bias)
            return ops.linear(x, self.weight, out=out, out_float32=self.out_float32, bias=self.bias, bias_rounded=self.bias_rounded)
        if row_scale is not None:
            y = ops.linear_few_rows(x, self.weight, out=out, out_float32=self.out_float32, row_scale=row_scale)
        else:
            y = ops.linear(x, self.weight, out=out, out_float32=self.out_float32)
        if self.bias is not None:
            ops.add_bias_(y, self.bias)
        return y
