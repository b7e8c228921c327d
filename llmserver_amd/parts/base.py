"""Interfaces of the parts a layer is put together from.

A model is a list of blocks and a list that says in which order they run.  A block arranges
a mixer (attention here), a feed-forward, norms and a position encoding.  Every part takes its
sizes and constants as constructor parameters, declares its tensors with :class:`ParamSpec`,
says what cache it needs with a :class:`CacheSpec`, and runs on a flat batch of tokens described
by a step context.  No part knows which model it is in.

Shapes used below: ``T`` tokens in the step, ``R`` request rows in the step, ``H`` model width.
"""
from __future__ import annotations

import dataclasses
from typing import Dict, Optional, Tuple

import torch

MATRIX = "matrix"      # follows the compute dtype (bfloat16 for serving, float32 on the 32-bit path)
VECTOR = "vector"      # small per-channel vectors: always held in float32
INT_TABLE = "int"      # integer tables: held as int32


@dataclasses.dataclass(frozen=True)
class ParamSpec:
    """One checkpoint tensor of a part: its shape, how it is stored and how random weights draw it."""
    shape: Tuple[int, ...]
    role: str = MATRIX
    init: str = "normal"          # "normal" | "norm" | "bias" | "zeros"
    optional: bool = False         # may be absent from the checkpoint
    # The share of the tensor that one token's pass uses: 1 for a dense layer's matrix, k/n for one of n experts of
    # which a token chooses k, 0 for a table of which a token reads a row.  (What a step costs is summed from this.)
    share_per_token: float = 1.0


@dataclasses.dataclass(frozen=True)
class PagedKVSpec:
    """Keys and values of every token, in pages.  ``window`` None keeps all keys; a number keeps
    only the last ``window`` keys a query can see, so earlier pages can be given back."""
    n_kv_heads: int
    head_dim: int
    window: Optional[int] = None


@dataclasses.dataclass(frozen=True)
class StateSpec:
    """Per-request state of fixed size (one slot per live request)."""
    shape: Tuple[int, ...]
    dtype: str = "float32"


class Part:
    """Common base: named tensors in, nothing model-specific."""

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {}

    def assign(self, name: str, tensor: torch.Tensor) -> None:
        raise KeyError(name)

    def finalize(self) -> None:
        """Called once after all tensors were assigned (fuse, re-lay-out, free the originals)."""


class Norm(Part):
    """Normalisation fused with the residual sum.

    ``add_norm(resid, delta, ctx, rows=None)`` computes ``s = resid + delta`` in 32-bit (``delta``
    may be None), stores ``s`` back into ``resid`` and returns ``norm(s)``; with ``rows`` (int32
    device tensor) only those token rows are normalised and returned, ``resid`` is left alone.

    ``row_scale_form()`` is how a norm tells the projections around it that it can be folded into them: a norm of
    the form ``s * rsqrt(mean(s^2) + eps) * weight`` returns ``(weight, eps)`` and must then also accept ``delta`` as
    float32 partial sums ``[parts, T, H]`` (a projection that was told this norm follows it may leave its result so);
    any other norm returns None and always runs in a kernel of its own.
    """

    def add_norm(self, resid, delta, ctx, rows=None):
        raise NotImplementedError

    def row_scale_form(self):
        return None

    def defer(self, resid, delta, ctx) -> "PendingNorm":
        """The same normalisation, left to whoever consumes it (a projection may fold it in)."""
        return PendingNorm(self, resid, delta, ctx)


class StreamUpdate:
    """What a part may return instead of a plain update of the residual stream, when its last
    projection has already added the update and prepared the norm that follows.

    ``resid [T, H]`` is the stream with the update added, ``norm`` the norm that was prepared, in one of two ways.
    Either ``weighted [T, H] = resid * norm.weight`` and ``square_sums [T, P]``, float32 partial sums of
    ``resid^2`` over P parts of each row: a projection that reads ``weighted`` and divides its result rows by
    ``sqrt(sum(square_sums) / H + eps)`` has multiplied the normalised stream.  Or ``normed [T, H]``, the norm's
    result itself (the update came as partial sums, and the kernel that added them up went on to normalise)."""

    def __init__(self, norm: "Norm", resid, weighted=None, square_sums=None, normed=None):
        self.norm, self.resid, self.weighted, self.square_sums, self.normed = norm, resid, weighted, square_sums, normed


class PendingNorm:
    """A normalisation that has not run yet: ``norm(resid + delta)``.

    A part that starts with a projection can hand this to its :class:`~llmserver_amd.parts.linear.Linear`.
    If ``delta`` came as a :class:`StreamUpdate` prepared for this very norm, the sum is done already
    and ``prepared`` holds what lets the projection apply the norm in its epilogue.  ``tensor()``
    carries the normalisation out the plain way.  Afterwards ``resid`` is the residual stream with
    ``delta`` added."""

    def __init__(self, norm: "Norm", resid, delta, ctx):
        self.prepared = None
        if isinstance(delta, StreamUpdate):
            if delta.norm is norm:
                self.prepared = delta
            resid, delta = delta.resid, None
        self.norm, self.resid, self.delta, self.ctx = norm, resid, delta, ctx
        self._done = self.prepared.normed if self.prepared is not None else None

    def tensor(self):
        if self._done is None:
            self._done = self.norm.add_norm(self.resid, self.delta, self.ctx)
            self.delta = None
        return self._done

    def row_scale(self):
        """``(weighted stream, (square_sums, eps))`` if a projection may apply the norm as a row scale, else None."""
        form = self.norm.row_scale_form()
        if self.prepared is None or self.prepared.weighted is None or self._done is not None or form is None:
            return None
        return self.prepared.weighted, (self.prepared.square_sums, form[1])


class ResidualSink:
    """Told to a part with ``takes_sink``: its output will be added to the residual stream and
    ``norm`` will follow.  The part's last projection may then do both (returning a
    :class:`StreamUpdate`); ``stream()`` is the residual stream it has to add to."""

    def __init__(self, pending: PendingNorm, norm: "Norm"):
        self.pending, self.norm = pending, norm

    def stream(self):
        if self.pending.delta is not None:          # nobody has added the previous update yet
            self.pending.tensor()
        return self.pending.resid


class PositionEncoding(Part):
    """How token positions enter a mixer.  ``rotary_table()`` returns the float32 inverse
    frequencies ``[rotary_dim/2]`` of a rotate-half rotation, or None if nothing is rotated.  ``rotary_dim`` says how
    many dimensions of a head the encoding rotates (None: none); a mixer checks it against what its kernels rotate."""

    rotary_dim: Optional[int] = None

    def rotary_table(self, device) -> Optional[torch.Tensor]:
        return None

    def cos_sin(self, ctx) -> Optional[torch.Tensor]:
        """float32 ``[T, rotary_dim]`` (cos of every pair, then sin) for the step's tokens, or None."""
        return None


class Mixer(Part):
    """Token mixer: reads and writes its own cache through the view the step gives it."""

    # True if ``forward`` only launches work whose shapes and addresses follow from the step's
    # staged arrays (no host-side loops over rows, no host reads): such a step can be captured
    # into a graph once and replayed.
    graph_safe = False
    # True if ``forward`` passes its input straight to a Linear and so can take a PendingNorm.
    accepts_pending_norm = False
    # True if ``forward`` takes ``sink=`` (a ResidualSink or None) and may return a StreamUpdate.
    takes_sink = False

    def cache_spec(self):
        """:class:`PagedKVSpec`, :class:`StateSpec` or None."""
        return None

    def prepare(self, ctx) -> None:
        """Stage per-step metadata (host arrays) before the single upload of the step."""

    def graph_shape(self, rows: int, longest_context: int):
        """What a captured step of ``rows`` single tokens, the longest of whose contexts is ``longest_context``, depends
        on in this mixer beyond the number of rows and the width of the block tables: anything hashable, None for
        nothing.  Steps to which every mixer of the model gives equal answers share a graph, so the answer has to be
        a pure function of the two numbers; the mixer asks itself the same question when it prepares such a step."""
        return None

    def graph_shape_edges(self):
        """Contexts at which :meth:`graph_shape` changes its answer (a warm-up captures a graph on either side)."""
        return ()

    def mixing_flops(self, new_tokens: int, context: int) -> float:
        """Floating-point operations between the mixer's projections for a row of ``new_tokens`` tokens that ends at a
        context of ``context`` tokens (attention: scores and weighted values); the projections are counted from
        ``param_specs``.  Only measurement reads this."""
        return 0.0

    def forward(self, x, ctx, cache):
        """``x [T, H]`` normalised input -> ``[T, H]`` update to add to the residual stream."""
        raise NotImplementedError


class FeedForward(Part):
    accepts_pending_norm = False
    takes_sink = False

    def forward(self, x, ctx):
        raise NotImplementedError


class Block(Part):
    """An arrangement of parts.  ``forward(resid, delta, ctx, cache) -> (resid', delta')``:
    ``resid`` is the residual stream, ``delta`` the pending update not yet added to it (a tensor,
    None, or a :class:`StreamUpdate`, which carries the stream it was added to)."""

    mixer: Mixer
    # True if ``forward`` takes ``following=``: the norm that will be applied to the block's
    # output (the next block's ``entry_norm()``), or None.  Such a block may return a StreamUpdate.
    takes_following = False

    def entry_norm(self):
        """The norm this block applies first to what it is given, or None."""
        return None

    def forward(self, resid, delta, ctx, cache):
        raise NotImplementedError
