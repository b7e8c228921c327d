"""The kernels as Python calls on torch tensors.

Every call checks on the host that shapes, dtypes and strides are what the kernel and its grid
assume, then launches on torch's current stream.  There is no CPU path and no library fallback
for the hand-written kernels: if the compiled extension is missing and cannot be built, loading
raises.  Matrix products are library calls (hipBLASLt/rocBLAS behind ``torch``), in bfloat16 with
32-bit accumulation for serving and in plain float32, with every reduced-precision matrix mode
switched off, on the 32-bit path.
"""
from __future__ import annotations

import torch

from ..parts.attention import group_tiling
from . import build, library

_DTYPE_CODE = {torch.float32: 0, torch.bfloat16: 1}
SKINNY_GEMM_ROWS = 8        # up to this many rows the hand-written weight-streaming product beats the library (measured)


def _code(tensor: torch.Tensor) -> int:
    try:
        return _DTYPE_CODE[tensor.dtype]
    except KeyError:
        raise TypeError(f"kernels take float32 or bfloat16 tensors, got {tensor.dtype}") from None


def _check(tensor, name, dtype=None, shape=None):
    if not tensor.is_cuda:
        raise ValueError(f"{name} must live on the GPU, it is on {tensor.device}")
    if not tensor.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    if dtype is not None and tensor.dtype != dtype:
        raise TypeError(f"{name} must be {dtype}, got {tensor.dtype}")
    if shape is not None and tuple(tensor.shape) != tuple(shape):
        raise ValueError(f"{name} must have shape {tuple(shape)}, got {tuple(tensor.shape)}")


def _ptr(tensor):
    return None if tensor is None else tensor.data_ptr()


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _launched(code: int, what: str):
    if code != 0:
        raise RuntimeError(f"launch of {what} failed with HIP error {code}")


class HipOps:
    """Kernel namespace handed to the parts through the step context."""

    name = "hip"

    def __init__(self):
        if not torch.cuda.is_available():
            raise library.KernelLibraryMissing("no GPU is visible; the engine has no CPU path")
        # True 32-bit matrix products on the float32 path: no reduced-precision mode.
        torch.backends.cuda.matmul.allow_tf32 = False
        torch.backends.cudnn.allow_tf32 = False
        torch.set_float32_matmul_precision("highest")
        self._elementwise = library.load("elementwise")
        self._rope_kv = library.load("rope_kv")
        self._sampling = library.load("sampling")
        self._gemm = library.load("gemm")
        self._attention = {}
        self.skinny_rows = SKINNY_GEMM_ROWS
        # The few-row product can take the residual sum + RMSNorm, or SwiGLU, as a prologue.  Every
        # workgroup then redoes that work for its 16 output columns, and measured on Qwen3-8B shapes
        # the fused launches are slower than the separate kernels (gate/up 60 vs 42 us, down 57 vs
        # 25 us at 1 row), so the parts do not use them unless this is switched on.
        self.fuse_prologues = False

    @staticmethod
    def required_modules(head_dims, dtype):
        names = list(build.BASE_MODULES)
        for dim in sorted(set(head_dims)):
            names.append(build.attention_module(dtype == torch.bfloat16, dim))
        return names

    def preload(self, head_dims, dtype):
        library.preload(self.required_modules(head_dims, dtype))

    # -- library matrix product ------------------------------------------------------------
    def linear(self, x, weight, out=None, out_float32=False, tiling=0):
        """``x [T, in] @ weight[out, in]^T``; float32 result if asked (the output head).  ``tiling`` picks the
        few-row kernel's workgroup shape (1 or 2 tiles of the weight; 0 lets the size decide)."""
        if x.shape[1] != weight.shape[1]:
            raise ValueError(f"linear: x {tuple(x.shape)} does not fit weight {tuple(weight.shape)}")
        rows, width = x.shape
        if x.dtype == torch.bfloat16 and 0 < rows <= self.skinny_rows and width % 8 == 0:
            # Few rows: the product is a stream over the weights; the hand-written kernel reads them once at HBM rate.
            _check(x, "x", torch.bfloat16)
            _check(weight, "weight", torch.bfloat16)
            if out is None or out_float32:
                out = torch.empty((rows, weight.shape[0]), device=x.device, dtype=torch.float32 if out_float32 else torch.bfloat16)
            _check(out, "out", None, (rows, weight.shape[0]))
            _launched(self._gemm.lsa_gemm_skinny(1 if out_float32 else 0, _ptr(x), _ptr(weight), _ptr(out), rows,
                                                 weight.shape[0], width, int(tiling), _stream()), "gemm_skinny")
            return out
        if out_float32 and x.dtype != torch.float32:
            return torch.mm(x, weight.t(), out_dtype=torch.float32)
        return torch.mm(x, weight.t(), out=out) if out is not None else torch.mm(x, weight.t())

    def linear_gated(self, x, gate_up_weight, tiling=0):
        """``silu(x @ gate^T) * (x @ up^T)`` with ``gate_up_weight [2I, K]`` in one launch for few rows (the
        activation sits in the product's epilogue), or None if this is not such a case."""
        rows, width = x.shape
        inter = gate_up_weight.shape[0] // 2
        if x.dtype != torch.bfloat16 or not 0 < rows <= self.skinny_rows or width % 8 or inter % 8 or gate_up_weight.shape[1] != width:
            return None
        _check(x, "x", torch.bfloat16)
        _check(gate_up_weight, "gate_up_weight", torch.bfloat16)
        out = torch.empty((rows, inter), device=x.device, dtype=torch.bfloat16)
        _launched(self._gemm.lsa_gemm_skinny_gated(_ptr(x), _ptr(gate_up_weight), _ptr(out), rows, inter, width, int(tiling), _stream()),
                  "gemm_skinny_gated")
        return out

    def swiglu_linear(self, gate_up, weight, force=False):
        """``(silu(gate) * up) @ weight^T`` in one launch for few rows, or None if this is not such a case."""
        rows, inter = gate_up.shape[0], gate_up.shape[1] // 2
        if not (self.fuse_prologues or force):
            return None
        if gate_up.dtype != torch.bfloat16 or not 0 < rows <= self.skinny_rows or inter % 8 or weight.shape[1] != inter:
            return None
        _check(gate_up, "gate_up", torch.bfloat16)
        _check(weight, "weight", torch.bfloat16)
        out = torch.empty((rows, weight.shape[0]), device=gate_up.device, dtype=torch.bfloat16)
        _launched(self._gemm.lsa_gemm_skinny_swiglu(_ptr(gate_up), _ptr(weight), _ptr(out), rows, weight.shape[0], inter, _stream()),
                  "gemm_skinny_swiglu")
        return out

    def norm_linear(self, resid, delta, norm_weight, eps, weight, out_float32=False, force=False):
        """``rmsnorm(resid + delta) * norm_weight @ weight^T`` in one launch for few rows.

        Returns ``(y, resid_after)`` where ``resid_after`` holds ``resid + delta`` (a new tensor; ``resid`` itself
        when ``delta`` is None), or None if this is not a case for the fused kernel."""
        rows, width = resid.shape
        if not (self.fuse_prologues or force):
            return None
        if resid.dtype != torch.bfloat16 or not 0 < rows <= self.skinny_rows or width % 8 or width > 16384 or weight.shape[1] != width:
            return None
        _check(resid, "resid", torch.bfloat16)
        _check(weight, "weight", torch.bfloat16)
        _check(norm_weight, "norm_weight", torch.float32, (width,))
        resid_after = resid
        if delta is not None:
            _check(delta, "delta", torch.bfloat16, (rows, width))
            resid_after = torch.empty_like(resid)
        out = torch.empty((rows, weight.shape[0]), device=resid.device, dtype=torch.float32 if out_float32 else torch.bfloat16)
        _launched(self._gemm.lsa_gemm_skinny_norm(1 if out_float32 else 0, _ptr(resid), _ptr(delta), _ptr(norm_weight), float(eps),
                                                  _ptr(resid_after), _ptr(weight), _ptr(out), rows, weight.shape[0], width,
                                                  _stream()), "gemm_skinny_norm")
        return out, resid_after

    # -- hand-written kernels ----------------------------------------------------------------
    def embedding(self, table, token_ids, out):
        n, width = out.shape
        _check(table, "table", out.dtype)
        _check(token_ids, "token_ids", torch.int32, (n,))
        _check(out, "out")
        if table.shape[1] != width:
            raise ValueError(f"embedding: table width {table.shape[1]} != out width {width}")
        _launched(self._elementwise.lsa_embedding(_code(out), _ptr(table), _ptr(token_ids), _ptr(out), n, width,
                                                  table.shape[0], _stream()), "embedding")

    def add_rmsnorm(self, resid, delta, weight, eps, out, rows=None):
        n_tokens, width = resid.shape
        _check(resid, "resid")
        _check(weight, "weight", torch.float32, (width,))
        if delta is not None:
            _check(delta, "delta", resid.dtype, (n_tokens, width))
        n_out = n_tokens if rows is None else rows.shape[0]
        _check(out, "out", resid.dtype, (n_out, width))
        if rows is not None:
            _check(rows, "rows", torch.int32, (n_out,))
        _launched(self._elementwise.lsa_add_rmsnorm(_code(resid), _ptr(resid), _ptr(delta), _ptr(weight), float(eps),
                                                    _ptr(out), _ptr(rows), n_out, width, _stream()), "add_rmsnorm")

    def swiglu(self, gate_up, out):
        n, inter = out.shape
        _check(gate_up, "gate_up", out.dtype, (n, 2 * inter))
        _check(out, "out")
        _launched(self._elementwise.lsa_swiglu(_code(out), _ptr(gate_up), _ptr(out), n, inter, _stream()), "swiglu")

    def add_bias_(self, y, bias):
        n, width = y.shape
        _check(y, "y")
        _check(bias, "bias", torch.float32, (width,))
        _launched(self._elementwise.lsa_add_bias(_code(y), _ptr(y), _ptr(bias), n, width, _stream()), "add_bias")

    def rotary_table(self, positions, inv_freq):
        """cos and sin of ``position * inv_freq`` for every token: float32 ``[T, 2 * len(inv_freq)]``, cos first."""
        n, half = positions.shape[0], inv_freq.shape[0]
        _check(positions, "positions", torch.int32)
        _check(inv_freq, "inv_freq", torch.float32)
        out = torch.empty((n, 2 * half), device=positions.device, dtype=torch.float32)
        _launched(self._rope_kv.lsa_rotary_table(_ptr(positions), _ptr(inv_freq), _ptr(out), half, n, _stream()), "rotary_table")
        return out

    def qk_norm_rope_kv_write(self, qkv, keys, values, table, token_row, positions, q_weight, k_weight, eps, cos_sin,
                              page_size, n_q, n_kv, head_dim, write_cache=True):
        n = qkv.shape[0]
        _check(qkv, "qkv", None, (n, (n_q + 2 * n_kv) * head_dim))
        _check(keys, "keys", qkv.dtype)
        _check(values, "values", qkv.dtype)
        pages = keys.shape[0]
        if tuple(keys.shape) != (pages, n_kv, page_size, head_dim) or tuple(values.shape) != (pages, n_kv, head_dim, page_size):
            raise ValueError(f"cache pages have shapes {tuple(keys.shape)} / {tuple(values.shape)}, expected "
                             f"{(pages, n_kv, page_size, head_dim)} / {(pages, n_kv, head_dim, page_size)}")
        _check(table, "table", torch.int32)
        _check(token_row, "token_row", torch.int32, (n,))
        _check(positions, "positions", torch.int32, (n,))
        if head_dim % 16:
            raise ValueError(f"the q/k kernel takes head sizes in steps of 16, got {head_dim}")
        for name, w in (("q_weight", q_weight), ("k_weight", k_weight)):
            if w is not None:
                _check(w, name, torch.float32, (head_dim,))
        if (q_weight is None) != (k_weight is None):
            raise ValueError("q and k norm weights must come together")
        if cos_sin is not None:
            _check(cos_sin, "cos_sin", torch.float32, (n, head_dim))
        _launched(self._rope_kv.lsa_qk_norm_rope_kv_write(
            _code(qkv), _ptr(qkv), _ptr(keys), _ptr(values), _ptr(table), table.shape[1], _ptr(token_row), _ptr(positions),
            _ptr(q_weight), _ptr(k_weight), float(eps), _ptr(cos_sin), page_size, n_q, n_kv, head_dim,
            1 if write_cache else 0, n, _stream()), "qk_norm_rope_kv_write")

    def _attention_library(self, dtype, head_dim):
        key = (dtype, head_dim)
        if key not in self._attention:
            self._attention[key] = library.load(build.attention_module(dtype == torch.bfloat16, head_dim))
        return self._attention[key]

    def paged_attention(self, qkv, out, keys, values, table, row_start, row_len, row_ctx, plan, scale, window, page_size,
                        n_q, n_kv, head_dim, ctx):
        """Attention of the step's tokens over their requests' pages.

        ``qkv [T, (n_q + 2 n_kv) * d]`` holds the normalised, rotated queries in its first
        ``n_q * d`` columns; ``out [T, n_q * d]``; ``plan`` is the staged work list.
        """
        n = qkv.shape[0]
        _check(qkv, "qkv", None, (n, (n_q + 2 * n_kv) * head_dim))
        _check(out, "out", qkv.dtype, (n, n_q * head_dim))
        _check(keys, "keys", qkv.dtype)
        _check(values, "values", qkv.dtype)
        pages = keys.shape[0]
        if tuple(keys.shape) != (pages, n_kv, page_size, head_dim) or tuple(values.shape) != (pages, n_kv, head_dim, page_size):
            raise ValueError("cache pages do not have the layout the attention kernel reads")
        if page_size % 4:
            raise ValueError(f"the attention kernel reads values four keys at a time: page_size must be a multiple of 4, got {page_size}")
        if n_q % n_kv:
            raise ValueError(f"query heads {n_q} must be a multiple of KV heads {n_kv}")
        _check(table, "table", torch.int32)
        rows = table.shape[0]
        for name, tensor in (("row_start", row_start), ("row_len", row_len), ("row_ctx", row_ctx)):
            _check(tensor, name, torch.int32, (rows,))
        n_items, n_merges, n_slots = plan["n_items"], plan["n_merges"], plan["n_slots"]
        _check(plan["items"], "plan items", torch.int32, (n_items, 4))
        _check(plan["item_slot"], "plan item_slot", torch.int32, (n_items,))
        _check(plan["merges"], "plan merges", torch.int32, (n_merges, 4))
        n_tiles = plan.get("n_tiles", 0)
        tiles = plan.get("tiles") if n_tiles else None
        if n_tiles:
            _check(tiles, "plan tiles", torch.int32, (n_tiles, 4))
            if qkv.dtype != torch.bfloat16:
                raise TypeError("the workgroup-tile attention kernel exists for bfloat16 only")
        gheads, tokens_per_tile, gtiles = group_tiling(n_q // n_kv)
        part_acc = part_ml = None
        if n_slots:
            part_acc = ctx.empty((n_slots, n_kv * gtiles, 16, head_dim), dtype=torch.float32)
            part_ml = ctx.empty((n_slots, n_kv * gtiles, 16, 2), dtype=torch.float32)
        lib = self._attention_library(qkv.dtype, head_dim)
        _launched(lib.lsa_paged_attention(
            _ptr(qkv), qkv.shape[1], _ptr(out), _ptr(keys), _ptr(values), _ptr(table), table.shape[1], _ptr(row_start),
            _ptr(row_len), _ptr(row_ctx), _ptr(plan["items"]), _ptr(plan["item_slot"]), n_items, _ptr(plan["merges"]),
            n_merges, _ptr(part_acc), _ptr(part_ml), _ptr(tiles), n_tiles, float(scale), int(window) if window else 0,
            page_size, n_q, n_kv, gheads, tokens_per_tile, gtiles, _stream()), "paged_attention")

    def sample(self, logits, temperature, uniform, out):
        n, vocab = logits.shape
        _check(logits, "logits", torch.float32)
        _check(temperature, "temperature", torch.float32, (n,))
        _check(uniform, "uniform", torch.float32, (n,))
        _check(out, "out", torch.int32, (n,))
        chunks = self._sampling.lsa_sample_chunks(vocab)
        workspace = torch.empty((n, chunks, 4), device=logits.device, dtype=torch.float32)
        _launched(self._sampling.lsa_sample(_ptr(logits), _ptr(temperature), _ptr(uniform), _ptr(out), _ptr(workspace), n, vocab,
                                            _stream()), "sample")


_default = None


def default_ops() -> HipOps:
    global _default
    if _default is None:
        _default = HipOps()
    return _default
