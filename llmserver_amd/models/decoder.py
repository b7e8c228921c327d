"""A decoder assembled from parts: embedding, blocks, the order they run in, final norm, head.

The order is data: ``order`` is a list of :class:`LayerCall`, each naming a block and the cache
it uses.  A block may be named twice (its weights are shared) and a call may read the cache that
another call writes.  The plain stacked model is ``[LayerCall(i, i) for i in range(L)]``
(utils/model.py:124-132).  Rows whose logits are wanted are selected before the
final norm and the head (utils/model.py:147-158).
"""
from __future__ import annotations

import dataclasses
from typing import Dict, Optional, Sequence

import torch

from ..parts.base import Block, Norm, ParamSpec, StreamUpdate
from ..parts.embedding import TokenEmbedding
from ..parts.linear import Linear


@dataclasses.dataclass(frozen=True)
class LayerCall:
    block: int                  # index into ``blocks``
    cache: int                  # index of the cache this call uses
    writes_cache: bool = True   # False: read the cache another call has written


class DecoderModel:
    def __init__(self, config, embedding: TokenEmbedding, blocks: Sequence[Block], final_norm: Norm, head: Linear,
                 tie_head: bool, order: Optional[Sequence[LayerCall]] = None,
                 names=("model.embed_tokens", "model.layers", "model.norm")):
        self.config = config
        self.embedding = embedding
        self.blocks = list(blocks)
        self.final_norm = final_norm
        self.head = head
        self.tie_head = tie_head
        self.order = list(order) if order is not None else [LayerCall(i, i) for i in range(len(self.blocks))]
        self.embed_name, self.layers_name, self.norm_name = names
        self.device = None
        self.dtype = None
        self._check_order()

    # -- structure ---------------------------------------------------------------------
    def _check_order(self):
        writers = {}
        for call in self.order:
            if not 0 <= call.block < len(self.blocks):
                raise ValueError(f"order names block {call.block}, the model has {len(self.blocks)}")
            if call.writes_cache:
                if call.cache in writers:
                    raise ValueError(f"cache {call.cache} is written by two calls of the order")
                writers[call.cache] = call.block
        for call in self.order:
            spec = self.blocks[call.block].mixer.cache_spec()
            if spec is None:
                continue
            if call.cache not in writers:
                raise ValueError(f"cache {call.cache} is read but never written")
            if self.blocks[writers[call.cache]].mixer.cache_spec() != spec:
                raise ValueError(f"cache {call.cache} is shared by mixers with different cache needs")

    def cache_specs(self) -> Dict[int, object]:
        """cache index -> what its writer stores."""
        specs = {}
        for call in self.order:
            spec = self.blocks[call.block].mixer.cache_spec()
            if spec is not None and call.writes_cache:
                specs[call.cache] = spec
        return specs

    # -- parameters --------------------------------------------------------------------
    def param_specs(self) -> Dict[str, ParamSpec]:
        specs = {f"{self.embed_name}.{k}": v for k, v in self.embedding.param_specs().items()}
        for i, block in enumerate(self.blocks):
            specs.update({f"{self.layers_name}.{i}.{k}": v for k, v in block.param_specs().items()})
        specs.update({f"{self.norm_name}.{k}": v for k, v in self.final_norm.param_specs().items()})
        for k, v in self.head.param_specs().items():
            # Tied when the configuration says so or the checkpoint holds no head
            # (utils/model_loader.py:56-59).
            specs[k] = dataclasses.replace(v, optional=True)
        return specs

    def ignored_names(self):
        """Checkpoint tensors that may be present but are not read."""
        return set(self.head.param_specs()) if self.tie_head else set()

    def assign(self, name: str, tensor: torch.Tensor) -> None:
        if name.startswith(self.embed_name + "."):
            self.embedding.assign(name[len(self.embed_name) + 1:], tensor)
        elif name.startswith(self.layers_name + "."):
            index, rest = name[len(self.layers_name) + 1:].split(".", 1)
            self.blocks[int(index)].assign(rest, tensor)
        elif name.startswith(self.norm_name + "."):
            self.final_norm.assign(name[len(self.norm_name) + 1:], tensor)
        else:
            self.head.assign(name, tensor)

    def finalize(self, assigned: Sequence[str], device, dtype) -> None:
        head_names = set(self.head.param_specs())
        if self.tie_head or not (head_names & set(assigned)):
            self.head.share_weight(self.embedding.weight)   # alias, not a copy
            self.tie_head = True
        for part in (self.embedding, *self.blocks, self.final_norm, self.head):
            part.finalize()
        self.device, self.dtype = torch.device(device), dtype

    # -- the forward pass over one flat batch ----------------------------------------------
    def prepare(self, ctx) -> None:
        for call in self.order:
            self.blocks[call.block].mixer.prepare(ctx)

    def forward(self, ctx, caches) -> torch.Tensor:
        """Run the step's tokens through every call of the order; float32 logits ``[n_out, vocab]``."""
        resid = self.embedding.forward(ctx.token_ids, ctx)
        delta = None
        for index, call in enumerate(self.order):
            block = self.blocks[call.block]
            if block.takes_following and index + 1 < len(self.order):
                # The block may add its last update itself and prepare the next block's first norm.
                following = self.blocks[self.order[index + 1].block].entry_norm()
                resid, delta = block.forward(resid, delta, ctx, caches.view(call), following=following)
            else:
                resid, delta = block.forward(resid, delta, ctx, caches.view(call))
        if isinstance(delta, StreamUpdate):
            resid, delta = delta.resid, None
        if ctx.n_out == 0:
            return torch.empty((0, self.head.out_features), device=resid.device, dtype=torch.float32)
        selected = self.final_norm.add_norm(resid, delta, ctx, rows=ctx.logit_idx)
        return self.head.forward(selected, ctx)
