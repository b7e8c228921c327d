"""The step function: a batch of (request, its next tokens) in, logits at the wanted places out.

It runs only the tokens it is given, as one flat batch, against the cache earlier steps left:
portions of prompts beside single decoded tokens, cut anywhere.  The reference runs two kinds of
forward per engine step, padded prefill batches and a decode batch
(utils/engine.py:437-443, utils/model.py:76-158); here there is
one pass, and one code path serves generation, the benchmark and trace replay.

A step that brings one token per request is launch-bound, so it is captured once into a HIP
graph per (rows, block-table width, wanted rows) and replayed afterwards: the kernels read
everything that changes from the staged arrays, whose addresses and shapes stay the same.  Decoding
steps are filled up with rows of nobody's to one of a few sizes, so that few graphs serve every batch.  The
reference replays its decode pass from a CUDA graph in the same way
(utils/cuda_graph.py:51-99).

Such a step can be laid out on the host while the GPU still runs the step before it (``prepare_ahead``: everything but
the token ids is known then), and started before the host has seen those tokens (``launch_ahead``: the ids are copied
on the device from the sampler's output); ``step`` then finds its work done, or drops it if the step that comes is
another one.

Small steps that bring portions of prompts are captured too, where launching their kernels one by one would take the
host longer than running them takes the GPU (``_portion_key``).
"""
from __future__ import annotations

import warnings
from collections import OrderedDict
from typing import Dict, Optional, Sequence

import numpy as np
import torch

from ..cache.manager import CacheManager
from .batch import Staging, StepContext, StepEntry

TABLE_WIDTH_STEP = 64      # captured steps serve block tables up to the next multiple of this many pages
MAX_GRAPHS = 96
# Steps that bring portions of prompts are captured too while they are small (there the host's work per launch, not the
# GPU's, bounds the step): up to this many rows, their tokens filled up to one of these numbers.
PORTION_ROWS = 16
PORTION_TOKENS = (8, 16, 24, 32, 48, 64, 96, 128, 192, 256, 384, 512)
PORTION_MEETINGS = 2        # a shape of such a step is captured when it is met for this many times (shapes are many, captures cost a step or two)
# ... and only where the host is what bounds it.  Launched one by one, a step takes the longer of the host's and the GPU's
# time; replayed, the GPU's (and somewhat more of that: a captured step's attention cannot choose its kernel by the rows'
# lengths).  The host's time is about 140 us a layer call (nine or ten launches from Python, a library product 20 us each);
# the GPU's is estimated from what the step reads and multiplies at the rates that small steps reach.
HOST_SECONDS_PER_LAYER_CALL = 140e-6
SMALL_STEP_BYTES_PER_SECOND = 4e12
SMALL_STEP_FLOPS_PER_SECOND = 1e15


def padded_rows(rows: int) -> int:
    """The number of rows a captured step of ``rows`` single tokens runs with: the next of 1, 2, 3, 4, 6, 8, ..., 16,
    20, 24, ..., 32, 40, 48, ..., 64, 80, 96, ...  (at most a quarter more, never 16 more), so that requests that
    come and go do not ask for a graph of every size."""
    if rows <= 4:
        return rows
    step = 2 if rows <= 16 else 4 if rows <= 32 else 8 if rows <= 64 else 16
    return -(-rows // step) * step


def padded_tokens(tokens: int) -> Optional[int]:
    """The number of tokens a captured step with portions of ``tokens`` tokens runs with; None: too many to capture."""
    for size in PORTION_TOKENS:
        if tokens <= size:
            return size
    return None


class _CapturedStep:
    def __init__(self, graph, logits, layout, staging):
        self.graph, self.logits, self.layout, self.staging = graph, logits, layout, staging


class ModelRunner:
    def __init__(self, model, cache: CacheManager, ops=None, use_graphs: Optional[bool] = None):
        if ops is None:
            from ..kernels import default_ops
            ops = default_ops()
        self.model, self.cache, self.ops = model, cache, ops
        # (whoever made the cache may have asked already, before allocating it; a runner never reads a cache unasked)
        ops.check_cache_geometry(model.cache_specs(), cache.page_size, [group.pool.num_pages for group in cache.groups] or None)
        self.device, self.dtype = model.device, model.dtype
        self._staging = [Staging(self.device), Staging(self.device)]
        self._flip = 0
        self.vocab = model.head.out_features
        self._mixers = list({id(block.mixer): block.mixer for block in model.blocks}.values())
        graph_safe = all(mixer.graph_safe for mixer in self._mixers) and not cache.state_specs
        if use_graphs is None:
            use_graphs = self.device.type == "cuda" and ops.name == "hip"
        self.use_graphs = bool(use_graphs and graph_safe)
        self.capture_portions = True      # small steps that bring prompt portions are replayed from graphs as well
        self._graphs: "OrderedDict[tuple, _CapturedStep]" = OrderedDict()
        self._met: Dict[tuple, int] = {}  # how often a shape of a step with portions has been met (see PORTION_MEETINGS)
        self._host_bound: Dict[tuple, bool] = {}
        self.graph_replays = 0
        self._ahead = None          # (graph key, request ids, staged context) of a decoding step prepared ahead
        self._launched = None       # (request ids, their contexts after it, logits) of a step started ahead of its tokens
        self.steps_prepared_ahead = 0
        self.steps_launched_ahead = 0

    def build_context(self, entries: Sequence[StepEntry], staging: Optional[Staging] = None,
                      table_width: Optional[int] = None, filler_rows: int = 0, filler_tokens: Optional[int] = None,
                      want_last: Optional[bool] = None) -> StepContext:
        """Check the entries against the cache, allocate their pages, lay out the flat batch.  ``filler_rows`` more rows
        follow the entries', each a first token of nobody's on a scratch page of its own, its logits wanted: they
        bring a step of single tokens to the shape of a captured one.  ``filler_tokens`` (a number, possibly 0): one
        more row of nobody's with that many tokens, the start of a prompt on scratch pages, which brings the step's
        tokens to a captured number.  ``want_last``: instead of the entries' own wanted places, the last token of
        every row (True) or nothing (False), so that the wanted places have a captured shape as well."""
        if not entries:
            raise ValueError("a step needs at least one entry")
        seen = set()
        token_ids, positions, token_row = [], [], []         # one array per row
        row_start, row_len, row_ctx, logit_idx, request_ids = [], [], [], [], []
        n_tokens = 0
        for row, entry in enumerate(entries):
            if entry.request_id in seen:
                raise ValueError(f"request {entry.request_id!r} appears twice in one step")
            seen.add(entry.request_id)
            tokens = np.asarray(entry.tokens, dtype=np.int64).reshape(-1)
            count = tokens.size
            if not count:
                raise ValueError(f"request {entry.request_id!r} brings no tokens")
            if int(tokens.min()) < 0 or int(tokens.max()) >= self.vocab:
                token = int(tokens[(tokens < 0) | (tokens >= self.vocab)][0])
                raise ValueError(f"token id {token} of request {entry.request_id!r} is outside the vocabulary of {self.vocab}")
            record = self.cache.record(entry.request_id)
            start = record.num_computed
            for place in entry.want:
                if not 0 <= place < count:
                    raise ValueError(f"wanted place {place} is outside the {count} tokens of request {entry.request_id!r}")
                if want_last is None:
                    logit_idx.append(n_tokens + place)
            if want_last:
                logit_idx.append(n_tokens + count - 1)
            row_start.append(n_tokens)
            row_len.append(count)
            row_ctx.append(start + count)
            request_ids.append(entry.request_id)
            token_ids.append(tokens)
            positions.append(np.arange(start, start + count, dtype=np.int64))
            token_row.append(np.full(count, row, dtype=np.int64))
            n_tokens += count
        for entry, ctx_len in zip(entries, row_ctx):
            self.cache.ensure(entry.request_id, ctx_len)
        if filler_rows:
            fillers = np.arange(filler_rows, dtype=np.int64)
            if want_last is not False:
                logit_idx.extend((n_tokens + fillers).tolist())
            row_start.extend((n_tokens + fillers).tolist())
            row_len.extend([1] * filler_rows)
            row_ctx.extend([1] * filler_rows)
            token_row.append(len(entries) + fillers)
            token_ids.append(np.zeros(filler_rows, dtype=np.int64))
            positions.append(np.zeros(filler_rows, dtype=np.int64))
        extra_rows = filler_rows
        if filler_tokens is not None:
            first = n_tokens + filler_rows
            if want_last:
                logit_idx.append(first + max(filler_tokens, 1) - 1 if filler_tokens else 0)     # (an empty row has no last token: any place will do)
            row_start.append(first)
            row_len.append(filler_tokens)
            row_ctx.append(filler_tokens)
            token_row.append(np.full(filler_tokens, len(entries) + filler_rows, dtype=np.int64))
            token_ids.append(np.zeros(filler_tokens, dtype=np.int64))
            positions.append(np.arange(filler_tokens, dtype=np.int64))
            extra_rows += 1
        token_ids, positions, token_row = np.concatenate(token_ids), np.concatenate(positions), np.concatenate(token_row)
        tables = []
        records = [self.cache.record(rid) for rid in request_ids]
        for group in self.cache.groups:
            rows_pages = [record.table_array(group.index) for record in records]
            width = table_width if table_width is not None else max(1, max(len(pages) for pages in rows_pages))
            table = np.full((len(entries) + extra_rows, width), -1, dtype=np.int32)
            for row, pages in enumerate(rows_pages):
                table[row, :len(pages)] = pages
            for filler in range(filler_rows):           # (from the end of the scratch pages: the row of several tokens has their start)
                table[len(entries) + filler, 0] = group.scratch_page(group.scratch_pages - 1 - filler)
            if filler_tokens:
                for block in range(-(-filler_tokens // group.page_size)):
                    table[len(entries) + filler_rows, block] = group.scratch_page(block)
            tables.append(table)
        request_ids = request_ids + [None] * extra_rows
        slots = None
        if self.cache.state_specs:
            slots = np.asarray([self.cache.record(rid).state_slot for rid in request_ids], dtype=np.int32)
        if staging is None:
            self._flip ^= 1
            staging = self._staging[self._flip]
        ctx = StepContext(self.ops, self.device, self.dtype, staging)
        ctx.page_size = self.cache.page_size
        ctx.fill(token_ids, positions, token_row, row_start, row_len, row_ctx, logit_idx, tables, slots, request_ids)
        return ctx

    # -- captured single-token steps ---------------------------------------------------------
    def _graph_key(self, entries: Sequence[StepEntry]):
        if not self.use_graphs:
            return None
        if any(len(entry.tokens) != 1 for entry in entries):
            return self._portion_key(entries)
        longest = 1
        for entry in entries:
            record = self.cache.requests.get(entry.request_id)
            if record is None:
                return None
            longest = max(longest, record.num_computed + 1)
        blocks = -(-longest // self.cache.page_size)
        width = -(-blocks // TABLE_WIDTH_STEP) * TABLE_WIDTH_STEP
        rows, wanted = len(entries), sum(len(entry.want) for entry in entries)
        if all(len(entry.want) == 1 for entry in entries):
            rows = wanted = padded_rows(rows)          # decoding: filled up to one of a few sizes
        # what the mixers' captured work depends on beyond that (each asks itself the same when it prepares the step)
        shapes = tuple(dict.fromkeys(mixer.graph_shape(rows, longest) for mixer in self._mixers))
        return (rows, width, wanted, shapes)

    def _host_bounds_a_step(self, tokens: int, keys: int) -> bool:
        """Whether a step of ``tokens`` tokens behind up to ``keys`` keys takes the GPU less time than launching its
        kernels takes the host (an estimate from the model's own sizes: the same answer in every run)."""
        known = self._host_bound.get((tokens, keys))
        if known is None:
            from .cost import StepRow, step_bytes, step_flops
            row = [StepRow(tokens, keys, 1)]
            gpu = step_bytes(self.model, row, self.dtype) / SMALL_STEP_BYTES_PER_SECOND + step_flops(self.model, row) / SMALL_STEP_FLOPS_PER_SECOND
            known = self._host_bound[(tokens, keys)] = gpu < len(self.model.order) * HOST_SECONDS_PER_LAYER_CALL
        return known

    def _portion_key(self, entries: Sequence[StepEntry]):
        """The captured shape of a small step that brings portions of prompts (beside single tokens, possibly), or None
        if it runs eagerly: too many rows or tokens, logits wanted elsewhere than at a row's last token (the engine
        never asks for others; a trace may), a step that the GPU, not the host, bounds anyway, or a shape that has not
        been met often enough yet.

        Such a step is filled up with rows of nobody's: rows of one token as in decoding steps, and one more row (empty
        if the numbers fit) with the tokens that are missing to the captured number, the start of a prompt on scratch
        pages.  Its wanted places are every row's last token, or none."""
        if not self.capture_portions or len(entries) > PORTION_ROWS:
            return None
        tokens, longest = 0, 1
        for entry in entries:
            record = self.cache.requests.get(entry.request_id)
            want = list(entry.want)
            if record is None or (want and want != [len(entry.tokens) - 1]):
                return None
            tokens += len(entry.tokens)
            longest = max(longest, record.num_computed + len(entry.tokens))
        rows = padded_rows(len(entries)) + 1
        size = padded_tokens(tokens + rows - 1 - len(entries))          # the rows of one token that fill the rows up bring a token each
        if size is None:
            return None
        longest = max(longest, size - tokens - (rows - 1 - len(entries)))
        blocks = -(-longest // self.cache.page_size)
        width = -(-blocks // TABLE_WIDTH_STEP) * TABLE_WIDTH_STEP
        if not self._host_bounds_a_step(size, width * self.cache.page_size):
            return None
        wanted = rows if any(entry.want for entry in entries) else 0
        shapes = tuple(dict.fromkeys(mixer.graph_shape(rows, longest) for mixer in self._mixers))
        key = ("portions", rows, size, width, wanted, shapes)
        if key not in self._graphs:
            met = self._met[key] = self._met.get(key, 0) + 1
            if len(self._met) > 4 * MAX_GRAPHS:
                self._met.clear()
            if met < PORTION_MEETINGS:
                return None
        return key

    @torch.inference_mode()
    def prepare_ahead(self, request_ids: Sequence[object]) -> bool:
        """Do the host's share of the next step now, while the GPU still works on the last one.

        The caller expects the next step to bring one token, as yet unknown, for each of ``request_ids`` in this order,
        and to want its logits: a decoding step.  Pages are allocated, the batch and the mixers' plans are laid out in
        the staging buffer of the captured step of that shape; :meth:`step` then only fills in the token ids, copies
        and replays.  If the next step turns out to be another one, what was prepared is dropped (pages that were
        allocated for a request stay in its table until they are needed or the request ends).  Returns whether a
        step was prepared; shapes that have not been captured yet are not prepared."""
        self._ahead = None
        request_ids = list(request_ids)
        if not self.use_graphs or not request_ids or len(set(request_ids)) != len(request_ids) \
                or any(rid not in self.cache.requests for rid in request_ids):
            return False
        entries = [StepEntry(rid, (0,), (0,)) for rid in request_ids]
        key = self._graph_key(entries)
        captured = self._graphs.get(key) if key is not None else None
        if captured is None:
            return False
        try:
            ctx = self.build_context(entries, staging=captured.staging, table_width=key[1], filler_rows=key[0] - len(entries))
        except BufferError:          # no page for one of them: the step itself will say so, or the caller makes room
            return False
        ctx.static_max_keys = key[1] * self.cache.page_size
        self.model.prepare(ctx)
        ctx.stage()
        if ctx.layout != captured.layout:
            return False
        self._ahead = (key, request_ids, ctx)
        return True

    @torch.inference_mode()
    def launch_ahead(self, device_tokens: torch.Tensor) -> bool:
        """Start the step that :meth:`prepare_ahead` laid out, with token ids that are still on the device: row ``i``
        gets ``device_tokens[i]`` (int32, one per request of the prepared step; the sampler's output for the step
        before).  The host has not seen the tokens yet, so the GPU goes from one step to the next without waiting
        for it.  The next :meth:`step` must bring these requests, in this order, with one token each and its logits
        wanted: it then takes the result.  Any other step drops it: what it wrote into the pages lies at places that
        are written again, with the same values, by the step that takes their tokens, or that nobody reads."""
        ahead, self._ahead = self._ahead, None
        if ahead is None or self._launched is not None:
            return False
        key, request_ids, ctx = ahead
        captured = self._graphs.get(key)
        if captured is None or device_tokens.dtype != torch.int32 or tuple(device_tokens.shape) != (len(request_ids),) \
                or device_tokens.device != ctx.token_ids.device:
            return False
        self._graphs.move_to_end(key)
        ctx.staging.upload()
        ctx.token_ids[:len(request_ids)].copy_(device_tokens)       # on the device, in stream order behind the upload
        captured.graph.replay()
        self.graph_replays += 1
        self.steps_launched_ahead += 1
        self._launched = (request_ids, [int(c) for c in ctx.h_row_ctx[:len(request_ids)]], captured.logits[:len(request_ids)])
        return True

    def _take_launched(self, entries) -> Optional[torch.Tensor]:
        """The logits of the step started ahead if ``entries`` are that step; it is dropped otherwise."""
        launched, self._launched = self._launched, None
        if launched is None or len(launched[0]) != len(entries):
            return None
        for entry, rid, ctx_len in zip(entries, launched[0], launched[1]):
            record = self.cache.requests.get(rid)
            if entry.request_id != rid or len(entry.tokens) != 1 or list(entry.want) != [0] or record is None \
                    or record.num_computed + 1 != ctx_len:
                return None
        return launched[2]

    def _take_ahead(self, entries, key) -> Optional[StepContext]:
        """The context prepared ahead if it is this step's: same shape, same requests in the same order at the same
        places of their sequences, one token each with its logits wanted."""
        ahead, self._ahead = self._ahead, None
        if ahead is None or ahead[0] != key or len(ahead[1]) != len(entries):
            return None
        ctx = ahead[2]
        for row, (entry, rid) in enumerate(zip(entries, ahead[1])):
            if entry.request_id != rid or len(entry.tokens) != 1 or list(entry.want) != [0] \
                    or self.cache.requests[rid].num_computed + 1 != int(ctx.h_row_ctx[row]):
                return None
        tokens = np.fromiter((entry.tokens[0] for entry in entries), dtype=np.int64, count=len(entries))
        if int(tokens.min()) < 0 or int(tokens.max()) >= self.vocab:
            return None              # the usual way names the token and the request
        ids = ctx.h_token_ids.copy()
        ids[:len(entries)] = tokens
        ctx.set_token_ids(ids)
        return ctx

    def _step_captured(self, entries, key) -> torch.Tensor:
        captured = self._graphs.get(key)
        portions = key[0] == "portions"
        ctx = self._take_ahead(entries, key) if captured is not None and not portions else None
        if ctx is not None:
            self._graphs.move_to_end(key)
            ctx.staging.upload()
            captured.graph.replay()
            self.graph_replays += 1
            self.steps_prepared_ahead += 1
            return captured.logits[:len(entries)]
        staging = captured.staging if captured is not None else Staging(self.device, capacity=4096)
        if portions:
            _, rows, size, width, wanted_rows, _ = key
            tokens = sum(len(entry.tokens) for entry in entries)
            filler_rows = rows - 1 - len(entries)
            ctx = self.build_context(entries, staging=staging, table_width=width, filler_rows=filler_rows,
                                     filler_tokens=size - tokens - filler_rows, want_last=bool(wanted_rows))
            # every row's last token was computed: the rows that asked are handed out (the fillers' come last)
            asked = [row for row, entry in enumerate(entries) if entry.want]

            def select(logits):
                if len(asked) == len(entries) or not len(asked):
                    return logits[:len(asked)]
                return logits[torch.tensor(asked, device=logits.device)]
        else:
            width = key[1]
            ctx = self.build_context(entries, staging=staging, table_width=width, filler_rows=key[0] - len(entries))
            wanted = sum(len(entry.want) for entry in entries)           # the fillers' logits come last and are dropped

            def select(logits):
                return logits[:wanted]
        ctx.static_max_keys = width * self.cache.page_size
        self.model.prepare(ctx)
        if captured is None:
            ctx.static_max_keys = None           # the first upload may size the staging buffer
            ctx.upload()
            ctx.static_max_keys = width * self.cache.page_size
            logits = self.model.forward(ctx, self.cache)              # this step's result, run eagerly
            torch.cuda.synchronize(self.device)
            ctx.forget_computed()                # what the eager run computed on the device must be recorded too
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                static_logits = self.model.forward(ctx, self.cache)   # recorded, not run
            self._graphs[key] = _CapturedStep(graph, static_logits, ctx.layout, staging)
            while len(self._graphs) > MAX_GRAPHS:
                self._graphs.popitem(last=False)
            return select(logits)
        self._graphs.move_to_end(key)
        ctx.upload()
        if ctx.layout != captured.layout:
            warnings.warn("a captured step met arrays of another shape; running it eagerly")
            return select(self.model.forward(ctx, self.cache))
        captured.graph.replay()
        self.graph_replays += 1
        return select(captured.logits)

    def graph_count(self) -> int:
        return len(self._graphs)

    def drop_graphs(self) -> None:
        self._graphs.clear()

    @torch.inference_mode()
    def step(self, entries: Sequence[StepEntry]) -> torch.Tensor:
        """Run one step; returns float32 logits ``[wanted, vocab]`` in the order of the entries and their ``want``.

        The tensor a captured step returns is overwritten by the next step of the same shape."""
        logits = self._take_launched(entries) if self._launched is not None else None
        key = self._graph_key(entries) if logits is None else None
        if logits is not None or key is not None:
            if logits is None:
                logits = self._step_captured(entries, key)
            ctx_rows = [(entry.request_id, self.cache.record(entry.request_id).num_computed + len(entry.tokens)) for entry in entries]
        else:
            self._ahead = None
            ctx = self.build_context(entries)
            self.model.prepare(ctx)
            ctx.upload()
            logits = self.model.forward(ctx, self.cache)
            ctx_rows = list(zip(ctx.request_ids, (int(c) for c in ctx.h_row_ctx)))
        for rid, ctx_len in ctx_rows:
            self.cache.advance(rid, ctx_len)
        return logits
