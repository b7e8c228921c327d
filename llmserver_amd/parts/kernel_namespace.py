"""What the parts, the step function and the engine ask of the object that carries the kernels (``ctx.ops``).

The package ships one such object, ``llmserver_amd.kernels.HipOps`` (hand-written HIP for gfx950); the tests pass
plain torch twins in its place.  Both derive from :class:`KernelNamespace`, which names every call: the ones every
namespace must answer raise ``NotImplementedError`` here, and the ones that only a namespace with fused or tuned
kernels answers have neutral answers here ("not offered"), so that no caller has to ask whether a method exists.
"""
from __future__ import annotations

import contextlib
from typing import Optional


class KernelNamespace:
    name = ""                       # "hip": the step function may record single-token steps into graphs
    fuse_stream_updates = False     # the few-row products fold the residual sum and the norm around them in
    fuses_bias = False              # linear() and linear_few_rows() take a bias themselves (one rounding)
    attention_tuning = None         # an AttentionTuning for this GPU, or None: the attention part's neutral defaults

    # -- what every namespace must do (shapes and meanings: see HipOps, whose docstrings are the contract) -----------
    def preload(self, head_dims, dtype) -> None:
        """Load (compile, if need be) what models of these head sizes and this type will call."""

    def linear(self, x, weight, out=None, out_float32=False, bias=None, bias_rounded=None):
        raise NotImplementedError

    def embedding(self, table, token_ids, out):
        raise NotImplementedError

    def add_rmsnorm(self, resid, delta, weight, eps, out, rows=None):
        raise NotImplementedError

    def swiglu(self, gate_up, out, activation="silu"):
        """``out = act(gate) * up`` with ``gate_up [T, 2I]``, gate first; a namespace refuses an ``activation`` it has not built."""
        raise NotImplementedError

    def add_bias_(self, y, bias):
        raise NotImplementedError

    def rotary_table(self, positions, inv_freq):
        raise NotImplementedError

    def qk_norm_rope_kv_write(self, qkv, keys, values, table, token_row, positions, q_weight, k_weight, eps, cos_sin,
                              page_size, n_q, n_kv, head_dim, write_cache=True):
        raise NotImplementedError

    def paged_attention(self, qkv, out, keys, values, table, row_start, row_len, row_ctx, plan, scale, window, page_size,
                        n_q, n_kv, head_dim, ctx, decode_fusion=None):
        raise NotImplementedError

    def sample(self, logits, temperature, uniform, out):
        raise NotImplementedError

    # -- what a namespace may offer; the answers here mean "not offered" --------------------------------------------
    def check_cache_geometry(self, cache_specs, page_size: int, num_pages=None) -> None:
        """Raise ``ValueError`` for a cache that the kernels cannot read (asked before anything is allocated):
        ``page_size`` keys a page, ``num_pages`` pages (one number, or one per group of caches; None: not said)."""

    def row_scale_fits(self, x, weight, row_scale) -> bool:
        """Whether the few-row product of these sizes can apply a norm as a scale of its rows."""
        return False

    def linear_few_rows(self, x, weight, out=None, out_float32=False, rows_per_workgroup=0, row_scale=None, bias=None):
        """The weight-streaming product (taking a pending norm as ``row_scale``), or None: no case for it."""
        return None

    def linear_into_stream(self, x, weight, resid, norm_weight, rows_per_workgroup=0, row_scale=None):
        """The product as an update of the residual stream with the following norm prepared, or None."""
        return None

    def linear_partial_sums(self, x, weight, few_rows_too=False):
        """The product as float32 partial sums ``[parts, T, out]`` for :meth:`add_rmsnorm` to add up, or None."""
        return None

    def partial_sums_are_faster(self, x, weight) -> bool:
        return False

    def library_is_faster(self, kind, x, weight, scaled=False, out_float32=False) -> bool:
        return False

    def linear_gated(self, x, gate_up_weight, pairs_per_workgroup=0, row_scale=None, activation="silu"):
        """Gate and up products with the activation in one launch, or None (also for an ``activation`` it has not built)."""
        return None

    def attention_tuning_for(self, dtype, head_dim=None):
        """``attention_tuning`` as it holds for tensors of ``dtype`` and heads of ``head_dim`` (kernels of different types
        may step through their keys differently, and costs grow with the head); here: the same for all."""
        return self.attention_tuning

    def attention_workgroup_tiles(self, dtype, head_dim, page_size=None) -> int:
        """Most tiles a workgroup of a prompt-portion attention kernel takes together; 0: there is no such kernel."""
        return 0

    def attention_tile_halves(self, dtype, head_dim) -> int:
        return 1

    def attention_tile_key_ranges(self, dtype, head_dim) -> int:
        """Most ranges the keys of a workgroup's tiles may be cut into for workgroups of their own (1: not offered)."""
        return 1

    def attention_tile_min_workgroups(self, dtype) -> int:
        return 0

    def decode_fusion_fits(self, dtype, head_dim) -> bool:
        """Whether ``paged_attention`` takes q/k norm, rotation and the cache write on itself in single-token steps."""
        return False

    def measuring(self):
        """A context in which unknown shapes may be timed and entered into a table of choices; here: nothing happens."""
        return contextlib.nullcontext(None)


def tuning_of(ops: KernelNamespace, default, dtype=None, head_dim=None):
    """The namespace's attention tuning for steps of this type and head size, or ``default`` where it has none."""
    tuning: Optional[object] = ops.attention_tuning_for(dtype, head_dim) if dtype is not None else ops.attention_tuning
    return tuning if tuning is not None else default
