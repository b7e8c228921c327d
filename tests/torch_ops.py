"""Plain torch twins of the HIP kernels, with the same call signatures and the same page layout.

Two uses: each is the reference its kernel is tested against on the GPU, and together they let
the tests drive the engine's step function, cache and scheduler on a CPU (the product has no CPU
path of its own; the tests pass this object in place of the kernel namespace).  Arithmetic is
float32 inside, like the kernels.
"""
from __future__ import annotations

import torch

from llmserver_amd.parts.attention import group_tiling  # noqa: F401  (kept for symmetry of imports)
from llmserver_amd.parts.kernel_namespace import KernelNamespace


class TorchOps(KernelNamespace):
    """``fused=True`` also offers the twins of the fused kernels (sum and norm folded into the few-row products, q/k
    norm, rotation and cache write inside the attention of single-token steps), for any type and size, so that the
    parts' fused dataflow runs on the CPU as it does on the GPU."""
    name = "torch"
    FUSED_ROWS = 16

    def __init__(self, fused: bool = False):
        self.fuse_stream_updates = fused
        self.fused = fused
        self.fused_calls = {"row_scale": 0, "into_stream": 0, "gated": 0, "decode_attention": 0, "partial_sums": 0}

    def preload(self, head_dims, dtype):
        pass

    # -- twins of the fused few-row products ------------------------------------------------------
    def row_scale_fits(self, x, weight, row_scale) -> bool:
        return self.fused and x.shape[1] == weight.shape[1] and 0 < x.shape[0] <= self.FUSED_ROWS

    @staticmethod
    def _scaled(y, row_scale, width):
        if row_scale is None:
            return y
        square_sums, eps = row_scale
        return y * torch.rsqrt(square_sums.float().sum(dim=1, keepdim=True) / width + eps)

    def linear_few_rows(self, x, weight, out=None, out_float32=False, rows_per_workgroup=0, row_scale=None):
        if not self.row_scale_fits(x, weight, row_scale):
            return None
        self.fused_calls["row_scale"] += row_scale is not None
        y = self._scaled(x.float() @ weight.float().t(), row_scale, x.shape[1])
        return y if (out_float32 or x.dtype == torch.float32) else y.to(x.dtype)

    def linear_into_stream(self, x, weight, resid, norm_weight, rows_per_workgroup=0, row_scale=None):
        if not self.row_scale_fits(x, weight, row_scale):
            return None
        self.fused_calls["into_stream"] += 1
        y = self._scaled(x.float() @ weight.float().t(), row_scale, x.shape[1]).to(x.dtype)
        stream = (resid.float() + y.float()).to(resid.dtype)
        weighted = (stream.float() * norm_weight).to(resid.dtype)
        squares = stream.float() ** 2
        parts = torch.stack([squares[:, i::3].sum(dim=1) for i in range(3)], dim=1)      # any split of the row will do
        return stream, weighted, parts

    def linear_gated(self, x, gate_up_weight, pairs_per_workgroup=0, row_scale=None, activation="silu"):
        beyond = self.fused and row_scale is None and 16 < x.shape[0] <= 32            # the kernel for more rows has no row scale
        if not beyond and not self.row_scale_fits(x, gate_up_weight, row_scale):
            return None
        self.fused_calls["gated"] += 1
        gate_up = self._scaled(x.float() @ gate_up_weight.float().t(), row_scale, x.shape[1])
        inter = gate_up.shape[1] // 2
        gate, up = gate_up[:, :inter], gate_up[:, inter:]
        return (gate * torch.sigmoid(gate) * up).to(x.dtype)

    def linear_partial_sums(self, x, weight, few_rows_too=False):
        if not self.fused or not (0 if few_rows_too else 16) < x.shape[0] <= 128:
            return None
        self.fused_calls["partial_sums"] += 1
        bounds = [0, x.shape[1] // 3, x.shape[1] // 2, x.shape[1]]                      # any split of the inner dimension
        return torch.stack([x[:, a:b].float() @ weight[:, a:b].float().t() for a, b in zip(bounds, bounds[1:])])

    def decode_fusion_fits(self, dtype, head_dim) -> bool:
        return self.fused

    def linear(self, x, weight, out=None, out_float32=False):
        y = (x.float() @ weight.float().t())
        y = y if (out_float32 or x.dtype == torch.float32) else y.to(x.dtype)
        if out is not None:
            out.copy_(y)
            return out
        return y

    def embedding(self, table, token_ids, out):
        out.copy_(table[token_ids.long()])

    def add_rmsnorm(self, resid, delta, weight, eps, out, rows=None):
        if delta is not None and delta.dim() == 3:                                       # partial sums of the update
            delta = delta.sum(dim=0).to(resid.dtype)
        if rows is None:
            total = resid.float()
            if delta is not None:
                total = (total + delta.float()).to(resid.dtype)
                resid.copy_(total)
                total = total.float()
        else:
            index = rows.long()
            total = resid[index].float()
            if delta is not None:
                total = (total + delta[index].float()).to(resid.dtype).float()
        normed = total * torch.rsqrt(total.pow(2).mean(dim=-1, keepdim=True) + eps) * weight
        out.copy_(normed.to(out.dtype))

    def swiglu(self, gate_up, out, activation="silu"):
        inter = out.shape[1]
        gate, up = gate_up[:, :inter].float(), gate_up[:, inter:].float()
        out.copy_((gate * torch.sigmoid(gate) * up).to(out.dtype))

    def add_bias_(self, y, bias):
        y.copy_((y.float() + bias).to(y.dtype))

    def rotary_table(self, positions, inv_freq):
        angles = positions.float()[:, None] * inv_freq[None, :]
        return torch.cat([torch.cos(angles), torch.sin(angles)], dim=1)

    def qk_norm_rope_kv_write(self, qkv, keys, values, table, token_row, positions, q_weight, k_weight, eps, cos_sin,
                              page_size, n_q, n_kv, head_dim, write_cache=True):
        n = qkv.shape[0]
        heads = qkv.view(n, n_q + 2 * n_kv, head_dim)
        qk = heads[:, :n_q + n_kv].float()
        if q_weight is not None:
            weight = torch.cat([q_weight.expand(n_q, -1), k_weight.expand(n_kv, -1)], dim=0)
            qk = qk * torch.rsqrt(qk.pow(2).mean(dim=-1, keepdim=True) + eps) * weight
        if cos_sin is not None:
            half = head_dim // 2
            cos, sin = cos_sin[:, None, :half], cos_sin[:, None, half:]
            x1, x2 = qk[..., :half], qk[..., half:]
            qk = torch.cat([x1 * cos - x2 * sin, x2 * cos + x1 * sin], dim=-1)
        heads[:, :n_q] = qk[:, :n_q].to(qkv.dtype)
        if not write_cache:
            return
        pos = positions.long()
        pages = table.long()[token_row.long(), pos // page_size]
        slots = pos % page_size
        keys[pages, :, slots, :] = qk[:, n_q:].to(keys.dtype)
        values[pages, :, :, slots] = heads[:, n_q + n_kv:].to(values.dtype)

    def paged_attention(self, qkv, out, keys, values, table, row_start, row_len, row_ctx, plan, scale, window, page_size,
                        n_q, n_kv, head_dim, ctx, decode_fusion=None):
        """Per request row: gather its keys/values through the block table, one softmax over all
        keys a query may see (no tiles, no splits).  ``decode_fusion``: the step's rows bring one token each and
        ``qkv`` is the raw projection, which is left as it is."""
        if decode_fusion is not None:
            self.fused_calls["decode_attention"] += 1
            q_weight, k_weight, eps, cos_sin, write_cache = decode_fusion
            rows = table.shape[0]
            assert qkv.shape[0] == rows and all(int(n) == 1 for n in row_len)
            qkv = qkv.clone()
            token_row = torch.arange(rows, dtype=torch.int32, device=qkv.device)
            positions = (row_ctx - 1).to(torch.int32)
            self.qk_norm_rope_kv_write(qkv, keys, values, table, token_row, positions, q_weight, k_weight, eps, cos_sin, page_size,
                                       n_q, n_kv, head_dim, write_cache)
        n = qkv.shape[0]
        q_all = qkv.view(n, n_q + 2 * n_kv, head_dim)[:, :n_q].float()
        group = n_q // n_kv
        for row in range(table.shape[0]):
            start, length, ctx_len = int(row_start[row]), int(row_len[row]), int(row_ctx[row])
            first = 0 if not window else max(0, ctx_len - length - window + 1)
            place = torch.arange(first, ctx_len, device=qkv.device)
            pages = table[row].long()[place // page_size]
            k = keys[pages, :, place % page_size, :].float()            # [keys, n_kv, d]
            v = values[pages, :, :, place % page_size].float()          # [keys, n_kv, d]
            q = q_all[start:start + length]                               # [len, n_q, d]
            k = k.repeat_interleave(group, dim=1)
            v = v.repeat_interleave(group, dim=1)
            scores = torch.einsum("qhd,khd->hqk", q, k) * scale
            q_pos = torch.arange(ctx_len - length, ctx_len, device=qkv.device)
            hidden = place[None, :] > q_pos[:, None]
            if window:
                hidden = hidden | (place[None, :] <= q_pos[:, None] - window)
            scores = scores.masked_fill(hidden[None], float("-inf"))
            result = torch.einsum("hqk,khd->qhd", torch.softmax(scores, dim=-1), v)
            out[start:start + length] = result.reshape(length, n_q * head_dim).to(out.dtype)

    def sample(self, logits, temperature, uniform, out):
        for row in range(logits.shape[0]):
            temp = float(temperature[row])
            if not temp > 0.0:
                out[row] = int(torch.argmax(logits[row]))
                continue
            weights = torch.exp((logits[row] - logits[row].max()) / temp)
            running = torch.cumsum(weights.double(), dim=0)
            target = float(uniform[row]) * float(running[-1])
            index = int(torch.searchsorted(running, torch.tensor(target, dtype=torch.float64), right=True))
            out[row] = min(index, logits.shape[1] - 1)
