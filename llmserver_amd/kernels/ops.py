"""The kernels as Python calls on torch tensors.

Every call checks on the host that shapes, dtypes and strides are what the kernel and its grid
assume, then launches on torch's current stream.  There is no CPU path and no library fallback
for the hand-written kernels: if the compiled extension is missing and cannot be built, loading
raises.  Matrix products are library calls (hipBLASLt/rocBLAS behind ``torch``), in bfloat16 with
32-bit accumulation for serving and in plain float32, with every reduced-precision matrix mode
switched off, on the 32-bit path.
"""
from __future__ import annotations

import dataclasses

import torch

from ..parts.attention import AttentionTuning, TileLaunchCost, group_tiling
from ..parts.kernel_namespace import KernelNamespace
from . import build, library
from .choices import ChoiceTable, choice_key

_DTYPE_CODE = {torch.float32: 0, torch.bfloat16: 1}
SKINNY_GEMM_ROWS = 16       # up to this many rows the hand-written weight-streaming products, with the sums, norms and the
                            # activation between them folded in, beat the library's products plus those kernels (measured)


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


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream():
    """Handle of torch's current stream on the current device (asked for at every launch, a few hundred times a step:
    the short way if torch has it; whoever launches a kernel holds a tensor on the GPU, so torch's runtime is up)."""
    if _raw_stream is not None and _raw_device is not None:
        return _raw_stream(_raw_device())
    return torch.cuda.current_stream().cuda_stream


def _launched(code: int, what: str):
    if code != 0:
        raise RuntimeError(f"launch of {what} failed with HIP error {code}")


class HipOps(KernelNamespace):
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
        # Whether projections may fold the residual sum and the norm between two few-row products into their
        # epilogues (see linear_into_stream); off, every such sum and norm is a kernel of its own.
        self.fuse_stream_updates = True
        # Whether projections whose result is added to the residual stream may leave it as partial sums at 17 to 128 rows.
        self.split_products = True
        self._split_parts = {}      # (rows, out, in) -> partial sums the split product writes for that size
        # The few-row products win on most shapes but not on all (on Qwen3-32B's gate/up the library is a third faster).
        # Which way a shape goes is looked up in a table per GPU model (see choices.py); a shape the table does not
        # know goes the hand-written way.  Nothing is timed unless somebody asks for it (``measuring()``).
        self.consult_choices = True
        properties = torch.cuda.get_device_properties(torch.cuda.current_device())
        # (the marketing name is the same for several chips; the architecture and the number of compute units tell them apart)
        self.device_kind = f"{str(getattr(properties, 'gcnArchName', properties.name)).split(':')[0]}-{properties.multi_processor_count}cu"
        self.choices = ChoiceTable.load(self.device_kind)
        self._measuring = False
        self._flush = None
        self._replay_overhead = None
        self._tunings = {}

    # What the prompt-portion kernel's launches cost, per kind of GPU: measured at head size 128 (a launch of one prompt of
    # 512 to 4,096 tokens, of several, and of portions behind long prefixes; eight tiles to a workgroup do more with each
    # key they load but start later, two halves shorten the longest workgroup's walk but make every step dearer).  A GPU
    # that is not listed plans with the attention part's neutral costs; other head sizes scale the trips and steps by
    # head size / 128 (loads and products of a step grow with the head; untuned beyond that).
    TILE_COSTS = {"gfx950-256cu": (((False, 1), TileLaunchCost(3.2, 0.89, 1.55)), ((True, 1), TileLaunchCost(8.7, 0.94, 2.45)),
                                   ((False, 2), TileLaunchCost(3.3, 1.11, 2.08)), ((True, 2), TileLaunchCost(8.8, 1.44, 2.84)))}
    TILE_COSTS_HEAD_DIM = 128

    @property
    def attention_tuning(self) -> AttentionTuning:
        """What the attention plan should know of this GPU: four wavefronts in flight per compute unit (more and shorter
        key ranges cost more in the merge than they gain), and what the prompt-portion kernel costs in each of its four
        forms on this kind of GPU, if that has been measured."""
        return self.attention_tuning_for(torch.bfloat16, self.TILE_COSTS_HEAD_DIM)

    def attention_tuning_for(self, dtype, head_dim=None) -> AttentionTuning:
        """The float32 kernels step through 16 keys at a time (16x16x4 products), the bfloat16 ones through 32."""
        head_dim = int(head_dim or self.TILE_COSTS_HEAD_DIM)
        key = (dtype == torch.float32, head_dim)
        if key not in self._tunings:
            units = torch.cuda.get_device_properties(torch.cuda.current_device()).multi_processor_count
            tuning = AttentionTuning(target_waves=4 * units, key_step=16 if dtype == torch.float32 else 32)
            costs = self.TILE_COSTS.get(self.device_kind)
            if costs is not None:
                scale = head_dim / self.TILE_COSTS_HEAD_DIM
                costs = tuple((form, TileLaunchCost(cost.start_us, cost.trip_us * scale, cost.step_ns * scale)) for form, cost in costs)
                tuning = dataclasses.replace(tuning, tile_costs=costs)
            self._tunings[key] = tuning
        return self._tunings[key]

    @staticmethod
    def check_cache_geometry(cache_specs, page_size: int, num_pages=None) -> None:
        """Refuse, before anything is allocated, a cache that the attention kernels cannot read.  ``num_pages`` (one
        number, or one per group of caches) bounds how long a request's context can get."""
        if page_size % 4:
            raise ValueError(f"the attention kernel reads values four keys at a time: page_size must be a multiple of 4, got {page_size}")
        if num_pages is not None:
            # A key's page is found as the high half of key * ceil(2^32 / page_size), which is key // page_size only for
            # keys below 2^32 / page_size; no request can hold more keys than the pool has room for.
            most = max(num_pages) if isinstance(num_pages, (list, tuple)) else int(num_pages)
            if most * page_size >= (1 << 32) // page_size:
                raise ValueError(f"a pool of {most} pages of {page_size} keys lets a context reach {most * page_size} keys; the attention "
                                 f"kernels find a key's page exactly only below 2^32 / page_size = {(1 << 32) // page_size} keys")
        for spec in cache_specs.values():
            head_dim = getattr(spec, "head_dim", None)
            if head_dim is not None:
                build.attention_module(True, head_dim)      # raises with the sizes the kernels take

    @staticmethod
    def required_modules(head_dims, dtype):
        names = list(build.BASE_MODULES)
        for dim in sorted(set(head_dims)):
            names.append(build.attention_module(dtype == torch.bfloat16, dim))
        return names

    def preload(self, head_dims, dtype):
        library.preload(self.required_modules(head_dims, dtype))

    # -- matrix products -------------------------------------------------------------------
    FUSED_ROWS = 16         # most rows the few-row product's fused epilogues take
    SCALE_PARTS = 512       # most partial sums per row its row scale takes (half as many from 9 rows on)

    def _few_rows(self, x, weight):
        rows, width = x.shape
        return x.dtype == torch.bfloat16 and 0 < rows <= self.skinny_rows and width % 8 == 0 and width >= 8 \
            and weight.dtype == torch.bfloat16

    LIBRARY_MARGIN = 0.93       # the library replaces a few-row kernel only if it takes less than this share of its time

    def _median_time(self, run, repeats=5):
        """Milliseconds of ``run()``, replayed from a graph of its own (several launches then follow one another as
        they do in a captured step, with no host between them), weights cold (a buffer larger than the caches is
        read before every replay)."""
        if self._flush is None:
            self._flush = torch.zeros(96 << 20, device="cuda", dtype=torch.int32)
        run()                                             # loads what the first call of a kernel loads
        current = torch.cuda.current_stream()
        side = torch.cuda.Stream()
        side.wait_stream(current)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            graph.capture_begin()
            try:
                run()
            finally:
                graph.capture_end()                       # whatever happened, the stream must not stay in capture
        current.wait_stream(side)
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        times = []
        for _ in range(repeats):
            self._flush.sum()
            start.record()
            graph.replay()
            end.record()
            end.synchronize()
            times.append(start.elapsed_time(end))
        return sorted(times)[repeats // 2]

    def _second_is_faster(self, first, second) -> bool:
        """Times both; a measurement that fails (something that cannot be recorded into a graph) keeps the first."""
        try:
            overhead = self._replay_cost()
            return self._median_time(second) - overhead < self.LIBRARY_MARGIN * (self._median_time(first) - overhead)
        except RuntimeError as error:
            import warnings
            warnings.warn(f"timing two ways of a product failed ({error!r}); keeping the few-row kernel")
            return False

    def _replay_cost(self):
        """What a replay takes between its events beside its kernels (milliseconds): a replay of next to nothing."""
        if self._replay_overhead is None:
            cell = torch.zeros(1, device="cuda")
            self._replay_overhead = self._median_time(lambda: cell.zero_(), repeats=7)
        return self._replay_overhead

    def library_is_faster(self, kind, x, weight, scaled=False, out_float32=False) -> bool:
        """Whether, for these sizes, the library's product (with a norm kernel before it if ``scaled``, and the
        activation kernel after it if ``kind`` is "gated") beats the kernel of this repository that does it all;
        ``kind`` "partial": the product in partial sums and the norm kernel that adds them up, against the library's
        product and the plain norm kernel.  Looked up in the table of choices; measured only inside ``measuring()``."""
        if not self.consult_choices:
            return False
        rows, width = x.shape
        # Beyond the few-row kernels one entry stands for eight neighbouring numbers of rows (portions of prompts
        # come in every length).
        key = choice_key(kind, rows if rows <= 16 else -(-rows // 8) * 8, weight.shape[0], width, scaled, out_float32)
        known = self.choices.get(key)
        if known is not None:
            return known
        if not self._measuring or torch.cuda.is_current_stream_capturing():
            return False                                  # unknown shape: this repository's kernel
        sums = torch.ones((rows, 16), device=x.device, dtype=torch.float32) if scaled else None
        row_scale = (sums, 1e-6) if scaled else None
        stream = torch.zeros_like(x) if scaled else None
        norm_weight = torch.ones(width, device=x.device, dtype=torch.float32) if scaled else None
        normed = torch.empty_like(x) if scaled else None
        saved, self.consult_choices = self.consult_choices, False
        try:
            if kind == "partial":
                stream = torch.zeros((rows, weight.shape[0]), device=x.device, dtype=x.dtype)
                norm_weight = torch.ones(weight.shape[0], device=x.device, dtype=torch.float32)
                normed = torch.empty_like(stream)

                def few():
                    sums = self.linear_partial_sums(x, weight, few_rows_too=True)
                    if sums is not None:
                        self.add_rmsnorm(stream, sums, norm_weight, 1e-6, normed)
                    return sums

                def library():
                    self.add_rmsnorm(stream, torch.mm(x, weight.t()), norm_weight, 1e-6, normed)
            elif kind == "gated":
                hidden = torch.empty((rows, weight.shape[0] // 2), device=x.device, dtype=x.dtype)

                def few():
                    return self.linear_gated(x, weight, row_scale=row_scale)

                def library():
                    if scaled:
                        self.add_rmsnorm(stream, None, norm_weight, 1e-6, normed)
                    self.swiglu(torch.mm(x, weight.t()), hidden)
            else:
                def few():
                    return self.linear_few_rows(x, weight, out_float32=out_float32, row_scale=row_scale)

                def library():
                    if scaled:
                        self.add_rmsnorm(stream, None, norm_weight, 1e-6, normed)
                    return torch.mm(x, weight.t(), out_dtype=torch.float32) if out_float32 else torch.mm(x, weight.t())
            if few() is None:
                return False                              # no case for this repository's kernel: nothing to choose
            faster = self._second_is_faster(few, library)
        finally:
            self.consult_choices = saved
        self.choices.record(key, faster)
        return faster

    def measuring(self):
        """A context in which shapes that the table of choices does not know are timed the first time they are met
        (a few milliseconds each) and entered into ``self.choices``; afterwards the buffer that the timing uses to
        empty the caches is given back.  Never entered by a step that serves a request."""
        import contextlib

        @contextlib.contextmanager
        def context():
            saved, self._measuring = self._measuring, True
            try:
                yield self.choices
            finally:
                self._measuring = saved
                self._flush = None
        return context()

    def partial_sums_are_faster(self, x, weight) -> bool:
        """For a projection of few rows into the residual stream: whether the product in partial sums plus the kernel
        that adds them up and normalises beats the few-row kernel that does it all (long inner dimensions at 9 to 16
        rows, where every workgroup of the few-row kernel moves as many activations as weights); measured once."""
        rows, width = x.shape
        if not self.consult_choices or not self.split_products or not self.fuse_stream_updates \
                or not 8 < rows <= self.skinny_rows or not self._few_rows(x, weight):
            return False
        key = choice_key("stream", rows, weight.shape[0], width, False, False)
        known = self.choices.get(key)
        if known is not None:
            return known
        if not self._measuring or torch.cuda.is_current_stream_capturing():
            return False
        resid = torch.zeros((rows, weight.shape[0]), device=x.device, dtype=x.dtype)
        norm_weight = torch.ones(weight.shape[0], device=x.device, dtype=torch.float32)
        normed = torch.empty_like(resid)
        saved, self.consult_choices = self.consult_choices, False
        try:
            def few():
                return self.linear_into_stream(x, weight, resid, norm_weight)

            def split():
                self.add_rmsnorm(resid, self.linear_partial_sums(x, weight, few_rows_too=True), norm_weight, 1e-6, normed)
            if few() is None or self.linear_partial_sums(x, weight, few_rows_too=True) is None:
                faster = False
            else:
                faster = self._second_is_faster(few, split)
        finally:
            self.consult_choices = saved
        self.choices.record(key, faster)
        return faster

    def _row_scale_args(self, row_scale, rows):
        """``row_scale = (square_sums [rows, P] float32, eps)`` or None -> kernel arguments."""
        if row_scale is None:
            return None, 0, 0.0
        square_sums, eps = row_scale
        _check(square_sums, "square_sums", torch.float32)
        if square_sums.dim() != 2 or square_sums.shape[0] != rows:
            raise ValueError(f"square_sums: expected [{rows}, parts], got {tuple(square_sums.shape)}")
        return _ptr(square_sums), square_sums.shape[1], float(eps)

    def _row_scale_fits(self, row_scale, rows):
        most = self.SCALE_PARTS if rows <= 8 else self.SCALE_PARTS // 2
        return row_scale is None or (rows <= self.FUSED_ROWS and 0 < row_scale[0].shape[1] <= most)

    def row_scale_fits(self, x, weight, row_scale) -> bool:
        """Whether the few-row products take ``x`` with this ``row_scale`` (then they do not return None for it)."""
        return x.shape[1] == weight.shape[1] and self._few_rows(x, weight) and self._row_scale_fits(row_scale, x.shape[0])

    fuses_bias = True       # linear() and linear_few_rows() take the bias themselves

    def linear(self, x, weight, out=None, out_float32=False, rows_per_workgroup=0, bias=None, bias_rounded=None):
        """``x [T, in] @ weight[out, in]^T``; float32 result if asked (the output head).  ``rows_per_workgroup``
        fixes the few-row kernel's share of the weight per workgroup (1 to 32; 0 lets the size decide).

        ``bias [out]`` (float32) is added to the product.  In bfloat16 the sum is rounded once, as a library's
        product with a bias rounds it: by the few-row kernel, or by the library if ``bias_rounded`` gives the same
        numbers in ``x``'s type; a bias that has no such form is added to the rounded product."""
        if x.shape[1] != weight.shape[1]:
            raise ValueError(f"linear: x {tuple(x.shape)} does not fit weight {tuple(weight.shape)}")
        if bias is not None:
            _check(bias, "bias", torch.float32, (weight.shape[0],))
        if self._few_rows(x, weight) and (rows_per_workgroup or not self.library_is_faster("plain", x, weight, False, out_float32)):
            # Few rows: the product is a stream over the weights; the hand-written kernel reads them once at HBM rate.
            return self.linear_few_rows(x, weight, out=out, out_float32=out_float32, rows_per_workgroup=rows_per_workgroup, bias=bias)
        if out_float32 and x.dtype != torch.float32:
            y = torch.mm(x, weight.t(), out_dtype=torch.float32)
        elif bias is not None and bias_rounded is not None and bias_rounded.dtype == x.dtype and x.dtype != torch.float32:
            _check(bias_rounded, "bias_rounded", x.dtype, (weight.shape[0],))
            return torch.addmm(bias_rounded, x, weight.t(), out=out) if out is not None else torch.addmm(bias_rounded, x, weight.t())
        else:
            y = torch.mm(x, weight.t(), out=out) if out is not None else torch.mm(x, weight.t())
        if bias is not None:
            self.add_bias_(y, bias)
        return y

    def linear_few_rows(self, x, weight, out=None, out_float32=False, rows_per_workgroup=0, row_scale=None, bias=None):
        """The weight-streaming product, or None if this is no case for it.

        ``row_scale = (square_sums [T, P], eps)``: ``x`` is a residual stream already multiplied by a norm's
        weights, ``square_sums`` are partial sums of the stream's squares, and the result rows are divided by the
        stream's root mean square, so that the result is the product of the normalised stream (up to 16 rows).
        ``bias [out]`` (float32) is added before the result is rounded."""
        rows, width = x.shape
        if x.shape[1] != weight.shape[1] or not self._few_rows(x, weight) or not self._row_scale_fits(row_scale, rows) \
                or (rows_per_workgroup > 16 and rows > 16):
            return None
        _check(x, "x", torch.bfloat16)
        _check(weight, "weight", torch.bfloat16)
        if out is None or out_float32:
            out = torch.empty((rows, weight.shape[0]), device=x.device, dtype=torch.float32 if out_float32 else torch.bfloat16)
        _check(out, "out", None, (rows, weight.shape[0]))
        sums, parts, eps = self._row_scale_args(row_scale, rows)
        if bias is not None:
            _check(bias, "bias", torch.float32, (weight.shape[0],))
        _launched(self._gemm.lsa_gemm_skinny(1 if out_float32 else 0, _ptr(x), _ptr(weight), _ptr(out), rows, weight.shape[0], width,
                                             int(rows_per_workgroup), sums, parts, eps, _ptr(bias) if bias is not None else None,
                                             _stream()), "gemm_skinny")
        return out

    SPLIT_ROWS = 128        # most rows the product that leaves partial sums takes (it starts above the few-row kernels')
    PARTS_ROWS = 1024       # most rows for which the library's product is tried in ranges of the inner dimension

    @staticmethod
    def _parts_bucket(rows: int) -> int:
        """One table entry stands for 64 neighbouring numbers of rows up to 256, for 128 beyond."""
        step = 64 if rows <= 256 else 128
        return -(-rows // step) * step

    @staticmethod
    def _in_parts(x, weight, parts: int):
        """``x @ weight^T`` as ``parts`` products over ranges of the inner dimension, one batched call of the library
        with float32 results ``[parts, T, out]`` (views only: nothing is copied)."""
        rows, width = x.shape
        return torch.bmm(x.view(rows, parts, width // parts).transpose(0, 1),
                         weight.view(weight.shape[0], parts, width // parts).permute(1, 2, 0), out_dtype=torch.float32)

    def library_parts(self, x, weight) -> int:
        """In how many ranges of the inner dimension the library's product of these sizes goes, when its result joins
        the residual stream anyway (the kernel of the sum and the norm adds float32 partial sums up as it goes): 0
        (whole), 2 or 4.  With a few hundred rows and an inner dimension of many thousands the library's whole product
        leaves compute units idle (a tile to each, walking all of the inner dimension); as a batched product of
        ranges it has several times the tiles.  Looked up in the table of choices; measured only inside
        ``measuring()``."""
        rows, width = x.shape
        if not self.consult_choices or not self.split_products or not self.fuse_stream_updates or x.dtype != torch.bfloat16 \
                or weight.dtype != torch.bfloat16 or not self.SPLIT_ROWS < rows <= self.PARTS_ROWS or not x.is_contiguous() \
                or not weight.is_contiguous():
            return 0
        ways = [parts for parts in (2, 4) if width % (8 * parts) == 0]
        if not ways:
            return 0
        bucket = self._parts_bucket(rows)
        keys = {parts: choice_key(f"parts{parts}", bucket, weight.shape[0], width, False, False) for parts in ways}
        known = {parts: self.choices.get(key) for parts, key in keys.items()}
        if all(value is not None for value in known.values()):
            return max((parts for parts, best in known.items() if best), default=0)
        if not self._measuring or torch.cuda.is_current_stream_capturing():
            return 0
        stream = torch.zeros((rows, weight.shape[0]), device=x.device, dtype=x.dtype)
        norm_weight = torch.ones(weight.shape[0], device=x.device, dtype=torch.float32)
        normed = torch.empty_like(stream)
        saved, self.consult_choices = self.consult_choices, False
        try:
            overhead = self._replay_cost()
            times = {0: self._median_time(lambda: self.add_rmsnorm(stream, torch.mm(x, weight.t()), norm_weight, 1e-6, normed)) - overhead}
            for parts in ways:
                times[parts] = self._median_time(
                    lambda: self.add_rmsnorm(stream, self._in_parts(x, weight, parts), norm_weight, 1e-6, normed)) - overhead
            best = min(ways, key=lambda parts: times[parts])
            if times[best] >= self.LIBRARY_MARGIN * times[0]:
                best = 0
        except RuntimeError as error:
            import warnings
            warnings.warn(f"timing the library's product in parts failed ({error!r}); keeping it whole")
            best = 0
        finally:
            self.consult_choices = saved
        for parts, key in keys.items():
            self.choices.record(key, parts == best)
        return best

    def linear_partial_sums(self, x, weight, few_rows_too=False):
        """``x @ weight^T`` for 17 to 128 rows (fewer if ``few_rows_too``) as float32 partial sums ``[parts, T, out]``
        over ranges of the inner dimension (their sum is the product), or None if this is no case for it.  Whoever
        adds the result to the residual stream adds the parts up (:meth:`add_rmsnorm` takes them).  Beyond 128 rows
        the library multiplies, in ranges where the table of choices says that this is faster (see
        :meth:`library_parts`)."""
        rows, width = x.shape
        if rows > self.SPLIT_ROWS and x.shape[1] == weight.shape[1]:
            parts = self.library_parts(x, weight)      # beyond this repository's product: the library's, whole or in ranges
            return self._in_parts(x, weight, parts) if parts else None
        if not ((0 if few_rows_too else self.skinny_rows) < rows <= self.SPLIT_ROWS) or x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16 \
                or x.shape[1] != weight.shape[1] or not self.split_products:
            return None
        if not few_rows_too and self.library_is_faster("partial", x, weight):
            return None
        size = (rows, weight.shape[0], width)
        parts = self._split_parts.get(size)
        if parts is None:
            parts = self._split_parts[size] = self._gemm.lsa_gemm_split_parts(*size)
        if parts < 2:           # refused, or so many rows of the weight that nothing is split: the library is as fast
            return None
        _check(x, "x", torch.bfloat16)
        _check(weight, "weight", torch.bfloat16)
        out = torch.empty((parts, rows, weight.shape[0]), device=x.device, dtype=torch.float32)
        _launched(self._gemm.lsa_gemm_split(_ptr(x), _ptr(weight), _ptr(out), rows, weight.shape[0], width, _stream()), "gemm_split")
        return out

    def linear_into_stream(self, x, weight, resid, norm_weight, rows_per_workgroup=0, row_scale=None):
        """The few-row product as an update of the residual stream ``resid [T, out]`` that a norm with weights
        ``norm_weight`` follows, in one launch: returns ``(stream, weighted, square_sums)`` with
        ``stream = resid + x @ weight^T`` (a new tensor), ``weighted = stream * norm_weight`` and
        ``square_sums [T, P]`` partial sums of ``stream^2`` (one per tile of the kernel's workgroups), which is what
        ``row_scale`` of the next product takes.  None if this is no case for it (more than 16 rows, other types)."""
        rows, width = x.shape
        n = weight.shape[0]
        if x.shape[1] != weight.shape[1] or not self._few_rows(x, weight) or rows > self.FUSED_ROWS \
                or not self._row_scale_fits(row_scale, rows) or resid.dtype != torch.bfloat16:
            return None
        _check(x, "x", torch.bfloat16)
        _check(weight, "weight", torch.bfloat16)
        _check(resid, "resid", torch.bfloat16, (rows, n))
        _check(norm_weight, "norm_weight", torch.float32, (n,))
        stream = torch.empty_like(resid)
        weighted = torch.empty_like(resid)
        n_sums = self._gemm.lsa_gemm_skinny_parts(rows, n, int(rows_per_workgroup))
        if n_sums <= 0:
            raise ValueError(f"linear_into_stream: no layout for {rows} x {n} with {rows_per_workgroup} rows per workgroup")
        square_sums = torch.empty((rows, n_sums), device=x.device, dtype=torch.float32)
        sums, parts, eps = self._row_scale_args(row_scale, rows)
        _launched(self._gemm.lsa_gemm_skinny_stream(_ptr(x), _ptr(weight), rows, n, width, int(rows_per_workgroup), sums, parts, eps, _ptr(resid),
                                                    _ptr(norm_weight), _ptr(stream), _ptr(weighted), _ptr(square_sums), _stream()),
                  "gemm_skinny_stream")
        return stream, weighted, square_sums

    ACTIVATIONS = ("silu",)       # what the activation kernel and the gated products' epilogues compute

    def linear_gated(self, x, gate_up_weight, pairs_per_workgroup=0, row_scale=None, activation="silu"):
        """``silu(x @ gate^T) * (x @ up^T)`` with ``gate_up_weight [2I, K]`` in one launch for few rows (the
        activation sits in the product's epilogue), or None if this is not such a case (another activation is none).  ``pairs_per_workgroup``:
        1 to 16 pairs of a gate and an up row in two tiles, -1 for 8 pairs in one tile, 0 lets the size decide.
        ``row_scale`` as in :meth:`linear_few_rows`."""
        rows, width = x.shape
        inter = gate_up_weight.shape[0] // 2
        if activation not in self.ACTIVATIONS:
            return None
        if rows > self.skinny_rows:
            return self._linear_gated_beyond_few_rows(x, gate_up_weight) if row_scale is None and pairs_per_workgroup == 0 else None
        if not self._few_rows(x, gate_up_weight) or inter % 8 or gate_up_weight.shape[1] != width or rows > 16 \
                or not self._row_scale_fits(row_scale, rows):
            return None
        if pairs_per_workgroup == 0 and self.library_is_faster("gated", x, gate_up_weight, row_scale is not None):
            return None
        _check(x, "x", torch.bfloat16)
        _check(gate_up_weight, "gate_up_weight", torch.bfloat16)
        out = torch.empty((rows, inter), device=x.device, dtype=torch.bfloat16)
        sums, parts, eps = self._row_scale_args(row_scale, rows)
        _launched(self._gemm.lsa_gemm_skinny_gated(_ptr(x), _ptr(gate_up_weight), _ptr(out), rows, inter, width, int(pairs_per_workgroup), sums, parts,
                                                   eps, _stream()), "gemm_skinny_gated")
        return out

    def _linear_gated_beyond_few_rows(self, x, gate_up_weight):
        """The same for 17 to 32 rows where the weight has so many rows that one workgroup can take the whole inner
        dimension (the kernel of :meth:`linear_partial_sums` with the activation in its epilogue), else None."""
        rows, width = x.shape
        inter = gate_up_weight.shape[0] // 2
        if x.dtype != torch.bfloat16 or gate_up_weight.dtype != torch.bfloat16 or gate_up_weight.shape[1] != width \
                or gate_up_weight.shape[0] % 2 or not self.split_products:
            return None
        size = ("gated", rows, inter, width)
        fits = self._split_parts.get(size)
        if fits is None:
            fits = self._split_parts[size] = self._gemm.lsa_gemm_split_gated_fits(rows, inter, width)
        if not fits or self.library_is_faster("gated", x, gate_up_weight):
            return None
        _check(x, "x", torch.bfloat16)
        _check(gate_up_weight, "gate_up_weight", torch.bfloat16)
        out = torch.empty((rows, inter), device=x.device, dtype=torch.bfloat16)
        _launched(self._gemm.lsa_gemm_split_gated(_ptr(x), _ptr(gate_up_weight), _ptr(out), rows, inter, width, _stream()), "gemm_split_gated")
        return out

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
        """``resid += delta`` (unless ``rows`` selects), ``out = rmsnorm(resid) * weight``.  ``delta``: None, a tensor
        like ``resid``, or float32 partial sums ``[parts, T, width]`` of one (see :meth:`linear_partial_sums`)."""
        n_tokens, width = resid.shape
        _check(resid, "resid")
        _check(weight, "weight", torch.float32, (width,))
        n_out = n_tokens if rows is None else rows.shape[0]
        _check(out, "out", resid.dtype, (n_out, width))
        if rows is not None:
            _check(rows, "rows", torch.int32, (n_out,))
        if delta is not None and delta.dim() == 3:
            _check(delta, "delta", torch.float32, (delta.shape[0], n_tokens, width))
            _launched(self._elementwise.lsa_add_rmsnorm_partial_sums(
                _code(resid), _ptr(resid), _ptr(delta), delta.shape[0], n_tokens * width, _ptr(weight), float(eps), _ptr(out),
                _ptr(rows), n_out, width, _stream()), "add_rmsnorm")
            return
        if delta is not None:
            _check(delta, "delta", resid.dtype, (n_tokens, width))
        _launched(self._elementwise.lsa_add_rmsnorm(_code(resid), _ptr(resid), _ptr(delta), _ptr(weight), float(eps),
                                                    _ptr(out), _ptr(rows), n_out, width, _stream()), "add_rmsnorm")

    def swiglu(self, gate_up, out, activation="silu"):
        if activation not in self.ACTIVATIONS:
            raise ValueError(f"the activation kernel computes {', '.join(self.ACTIVATIONS)}; {activation!r} is not built")
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

    def attention_workgroup_tiles(self, dtype, head_dim, page_size=None) -> int:
        """Most tiles of 16 (token, head) pairs that a workgroup of the prompt-portion attention kernel takes together
        (an entry of a plan's ``tiles`` spans four, or this many); 0 if that kernel does not take pages of
        ``page_size`` keys (its loads bring 8 keys of a value row at a time in bfloat16)."""
        lib = self._attention_library(dtype, head_dim)
        if page_size is not None and int(page_size) % int(lib.lsa_attention_tile_page_multiple()):
            return 0
        return int(lib.lsa_attention_workgroup_tiles())

    def attention_tile_min_workgroups(self, dtype) -> int:
        """Workgroups below which a launch of the prompt-portion kernel does not pay.  The float32 kernel's steps are
        slow (true 32-bit products, 16 keys a step), so with few workgroups its longest one decides: measured at head
        size 128, 1,024 workgroups finish 1.4 times sooner than wavefronts of their own, 256 (one for every compute
        unit) take a third longer.  Wanted: a quarter more workgroups than compute units."""
        if dtype == torch.bfloat16:
            return 0
        return 5 * torch.cuda.get_device_properties(torch.cuda.current_device()).multi_processor_count // 4

    def attention_tile_halves(self, dtype, head_dim) -> int:
        """Halves that a workgroup of the prompt-portion kernel can split its tiles' keys between (1: it cannot)."""
        return int(self._attention_library(dtype, head_dim).lsa_attention_tile_halves())

    def attention_tile_key_ranges(self, dtype, head_dim) -> int:
        """Most ranges that the keys of a workgroup's tiles may be cut into, each range another workgroup's (their
        partial results are merged afterwards); 1: the kernel does not offer that."""
        return int(self._attention_library(dtype, head_dim).lsa_attention_tile_key_ranges())

    @staticmethod
    def decode_fusion_fits(dtype, head_dim) -> bool:
        """Whether the attention kernel can take the q/k norm, the rotation and the new token's way into the cache
        on itself in a step in which every row brings one token."""
        return dtype == torch.bfloat16 and head_dim % 64 == 0

    def paged_attention(self, qkv, out, keys, values, table, row_start, row_len, row_ctx, plan, scale, window, page_size,
                        n_q, n_kv, head_dim, ctx, decode_fusion=None):
        """Attention of the step's tokens over their requests' pages.

        ``qkv [T, (n_q + 2 n_kv) * d]`` holds the normalised, rotated queries in its first
        ``n_q * d`` columns; ``out [T, n_q * d]``; ``plan`` is the staged work list.

        ``decode_fusion = (q_weight, k_weight, eps, cos_sin, write_cache)`` instead of a call of
        :meth:`qk_norm_rope_kv_write` before this one: ``qkv`` is then the raw projection, every row of the step
        must bring exactly one token, and the kernel normalises and rotates q and the new key itself and (with
        ``write_cache``) takes the new key and value from ``qkv`` and puts them into the pages.
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
            most = self.attention_workgroup_tiles(qkv.dtype, head_dim, page_size)
            if not most:
                raise ValueError(f"the kernel for prompt portions in workgroups does not take pages of {page_size} keys: "
                                 "plan this step with attention_workgroup_tiles(dtype, head_dim, page_size), which says so")
            if int(plan.get("tiles_per_workgroup", 0)) not in (4, most):
                raise ValueError(f"the plan gives a workgroup {plan.get('tiles_per_workgroup')} tiles, this kernel takes 4 or {most}")
        tile_slots = plan.get("tile_slots") if n_tiles else None
        if tile_slots is not None:
            _check(tile_slots, "plan tile_slots", torch.int32, (n_tiles, 2))
            if self.attention_tile_key_ranges(qkv.dtype, head_dim) <= 1 or not n_slots or not n_merges:
                raise ValueError("the plan shares the keys of a workgroup's tiles between workgroups: that takes a kernel that "
                                 "offers it (attention_tile_key_ranges), slots for the partial results and their merges")
        gheads, tokens_per_tile, gtiles = group_tiling(n_q // n_kv)
        part_acc = part_ml = None
        if n_slots:
            part_acc = ctx.empty((n_slots, n_kv * gtiles, 16, head_dim), dtype=torch.float32)
            part_ml = ctx.empty((n_slots, n_kv * gtiles, 16, 2), dtype=torch.float32)
        fusion_mode, q_weight, k_weight, norm_eps, cos_sin = 0, None, None, 0.0, None
        if decode_fusion is not None:
            q_weight, k_weight, norm_eps, cos_sin, write_cache = decode_fusion
            if not self.decode_fusion_fits(qkv.dtype, head_dim) or n_tiles or n != rows:
                raise ValueError("decode fusion takes bfloat16, head sizes in steps of 64 and steps of one token per row")
            for name, w in (("q_weight", q_weight), ("k_weight", k_weight)):
                if w is not None:
                    _check(w, name, torch.float32, (head_dim,))
            if (q_weight is None) != (k_weight is None):
                raise ValueError("q and k norm weights must come together")
            if cos_sin is not None:
                _check(cos_sin, "cos_sin", torch.float32, (n, head_dim))
            fusion_mode = 3 if write_cache else 1
        merge_in_workgroup = int(plan.get("merge_in_workgroup", 0))
        if merge_in_workgroup and (n_items % 4 or n_merges or n_slots or n_tiles or (merge_in_workgroup == 2 and n != rows)
                                   or (decode_fusion is not None and (q_weight is None or cos_sin is None))):
            raise ValueError("merging in the workgroup takes a plan that gives every tile four key ranges (or, in steps of one token "
                             "per row, two, with tiles in pairs) and no slots, and, with decode fusion, both norm weights and a rotation")
        lib = self._attention_library(qkv.dtype, head_dim)
        if n_tiles and int(plan.get("tile_halves", 1)) not in (1, lib.lsa_attention_tile_halves()):
            raise ValueError(f"the plan splits a workgroup's keys into {plan['tile_halves']} halves, this kernel takes 1 or {lib.lsa_attention_tile_halves()}")
        if plan.get("most_splits", 0) > lib.lsa_attention_most_splits():
            raise ValueError(f"the plan splits a tile's keys into {plan['most_splits']} ranges, the merge kernel takes {lib.lsa_attention_most_splits()}")
        _launched(lib.lsa_paged_attention(
            _ptr(qkv), qkv.shape[1], _ptr(out), _ptr(keys), _ptr(values), _ptr(table), table.shape[1], _ptr(row_start),
            _ptr(row_len), _ptr(row_ctx), _ptr(plan["items"]), _ptr(plan["item_slot"]), n_items, _ptr(plan["merges"]),
            n_merges, n_slots, _ptr(part_acc), _ptr(part_ml), _ptr(tiles), _ptr(tile_slots), n_tiles, float(scale), int(window) if window else 0,
            page_size, n_q, n_kv, gheads, tokens_per_tile, gtiles, fusion_mode, _ptr(q_weight), _ptr(k_weight), float(norm_eps),
            _ptr(cos_sin), int(plan.get("tiles_per_workgroup", 0)), merge_in_workgroup, int(plan.get("tile_halves", 1)), _stream()),
            "paged_attention")

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

    def sample_no_alloc(self, logits, temperature, uniform, out):
        """:meth:`sample` for callers that must not allocate (a graph under capture, for one): the per-chunk statistics
        lie in a fixed array inside the library instead of a workspace tensor.  At most
        ``lsa_sample_static_max_rows()`` rows; calls that overlap on one GPU race on that array."""
        n, vocab = logits.shape
        _check(logits, "logits", torch.float32)
        _check(temperature, "temperature", torch.float32, (n,))
        _check(uniform, "uniform", torch.float32, (n,))
        _check(out, "out", torch.int32, (n,))
        most = self._sampling.lsa_sample_static_max_rows()
        if n > most:
            raise ValueError(f"sampling without a workspace takes at most {most} rows, got {n}")
        code = self._sampling.lsa_sample_static(_ptr(logits), _ptr(temperature), _ptr(uniform), _ptr(out), n, vocab, _stream())
        if code:
            raise RuntimeError(f"sample_static failed ({code}): {self._sampling.lsa_sample_static_error(code).decode()}")


_default = None


def default_ops() -> HipOps:
    global _default
    if _default is None:
        _default = HipOps()
    return _default
