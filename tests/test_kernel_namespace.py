"""The calls that the parts, the step function and the engine make on ``ctx.ops`` are the methods of
``parts.KernelNamespace``: the shipped HIP namespace and the tests' torch twins both answer the required ones, and a
namespace that offers nothing beyond them (the base class's neutral answers) still runs a model."""
import inspect
import os
import re

import pytest
import torch

from llmserver_amd.parts import KernelNamespace
from torch_ops import TorchOps

REQUIRED = ("linear", "embedding", "add_rmsnorm", "swiglu", "add_bias_", "rotary_table", "qk_norm_rope_kv_write", "paged_attention", "sample")
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_both_namespaces_answer_what_must_be_answered():
    from llmserver_amd.kernels.ops import HipOps
    for cls in (HipOps, TorchOps):
        assert issubclass(cls, KernelNamespace)
        for name in REQUIRED:
            assert getattr(cls, name) is not getattr(KernelNamespace, name), (cls.__name__, name)
    for name in REQUIRED:                       # the base class refuses them
        method = getattr(KernelNamespace(), name)
        arguments = [None] * len([p for p in inspect.signature(method).parameters.values() if p.default is p.empty])
        try:
            method(*arguments)
        except NotImplementedError:
            continue
        raise AssertionError(f"KernelNamespace.{name} should be abstract")


def test_every_call_on_ops_in_the_package_is_named_by_the_interface():
    """No caller outside the kernels' own folder uses a method that the interface does not name, and none asks
    whether a method exists."""
    used = set()
    for folder in ("parts", "models", "engine", "sampling", "cache"):
        for base, _, files in os.walk(os.path.join(ROOT, "llmserver_amd", folder)):
            for file in files:
                if file.endswith(".py"):
                    text = open(os.path.join(base, file)).read()
                    assert not re.search(r"(getattr|hasattr)\([^)]*\bops\b", text), (file, "asks whether the namespace has something")
                    used.update(re.findall(r"\bops\.([A-Za-z_]\w*)", text))
    used -= {"py"}                                # (a file name in a comment)
    missing = sorted(name for name in used if not hasattr(KernelNamespace, name))
    assert not missing, missing


def test_a_namespace_that_offers_nothing_runs_a_model():
    """The torch twins with every offer withdrawn (the base class's answers) give the same logits as with them."""
    import numpy as np
    from helpers import model_folder
    from llmserver_amd.engine.replay import make_runner
    from llmserver_amd.engine.step import StepEntry

    class Bare(TorchOps):
        row_scale_fits = KernelNamespace.row_scale_fits
        linear_few_rows = KernelNamespace.linear_few_rows
        linear_into_stream = KernelNamespace.linear_into_stream
        linear_partial_sums = KernelNamespace.linear_partial_sums
        linear_gated = KernelNamespace.linear_gated
        decode_fusion_fits = KernelNamespace.decode_fusion_fits

    outs = []
    for ops in (TorchOps(fused=True), Bare(fused=False)):
        runner = make_runner(model_folder("A"), "float32", 128, 16, device="cpu", ops=ops)
        runner.cache.open("r")
        runner.cache.ensure("r", 9)
        first = runner.step([StepEntry("r", [3, 1, 4, 1, 5, 9, 2, 6], [7])])
        runner.cache.advance("r", 8)
        second = runner.step([StepEntry("r", [5], [0])])
        outs.append(np.concatenate([first.float().cpu().numpy(), second.float().cpu().numpy()]))
    np.testing.assert_allclose(outs[0], outs[1], atol=2e-5, rtol=1e-5)


def test_pools_that_let_a_context_outgrow_the_kernels_page_lookup_are_refused():
    """The attention kernels find a key's page as the high half of key * ceil(2^32 / page_size), exact only for keys
    below 2^32 / page_size: a pool whose pages could hold a longer context is refused when the engine or a runner
    is made, with the numbers; page sizes the kernels cannot read, and head sizes, are refused there too."""
    from llmserver_amd.kernels.ops import HipOps
    from llmserver_amd.parts.base import PagedKVSpec
    specs = {0: PagedKVSpec(2, 64, None)}
    HipOps.check_cache_geometry(specs, 16, (1 << 24) - 1)                  # 2^28 - 16 keys: the last context that is exact
    HipOps.check_cache_geometry(specs, 500, [17_179, 10])                  # 8,589,500 < 2^32 / 500 = 8,589,934
    for page_size, pages in ((16, 1 << 24), (500, 17_180), (16, [8, 1 << 24]), (4, 1 << 28)):
        with pytest.raises(ValueError, match="2\\^32 / page_size"):
            HipOps.check_cache_geometry(specs, page_size, pages)
    # the arithmetic the refusal protects: exact below the limit, wrong at some key beyond it
    for page_size in (500, 12, 16):
        magic = -(-(1 << 32) // page_size)
        limit = (1 << 32) // page_size
        keys = [0, 1, page_size - 1, page_size, limit - 1, limit - page_size, (limit - 1) // page_size * page_size]
        assert all((key * magic) >> 32 == key // page_size for key in keys)
    with pytest.raises(ValueError, match="multiple of 4"):
        HipOps.check_cache_geometry(specs, 6, 10)
    with pytest.raises(ValueError):
        HipOps.check_cache_geometry({0: PagedKVSpec(2, 40, None)}, 16, 10)


def test_parts_refuse_what_their_kernels_do_not_compute_when_they_are_made():
    """A position encoding that rotates a part of the head, or an activation that the kernels do not compute, is refused
    with the reason by the part's constructor, not by a shape check at the first step."""
    from llmserver_amd.parts import GatedMLP, GQAttention, NoPosition, RotaryPosition
    with pytest.raises(ValueError, match="rotates 16 of a head's 32 dimensions"):
        GQAttention(64, 4, 2, 32, RotaryPosition(16, 1e4))
    assert GQAttention(64, 4, 2, 32, RotaryPosition(32, 1e4)).position.rotary_dim == 32
    assert GQAttention(64, 4, 2, 32, NoPosition()).position.rotary_dim is None
    with pytest.raises(ValueError, match="Unsupported activation 'gelu'"):
        GatedMLP(64, 128, "gelu")
    assert GatedMLP(64, 128, "swish").activation == "silu"
    # a namespace's fused product declines an activation it has not built (the caller then takes the separate kernels,
    # whose activation kernel refuses it by name)
    from llmserver_amd.kernels.ops import HipOps
    assert HipOps.linear_gated(HipOps.__new__(HipOps), torch.zeros(2, 8), torch.zeros(16, 8), activation="gelu") is None
    with pytest.raises(ValueError, match="'gelu' is not built"):
        HipOps.swiglu(HipOps.__new__(HipOps), torch.zeros(2, 8), torch.zeros(2, 4), activation="gelu")


def test_a_mixer_tells_the_step_what_its_captured_work_depends_on():
    """The step function knows nothing of attention's short contexts: a mixer answers ``graph_shape`` (and names the
    contexts at which its answer changes), steps with equal answers share a graph."""
    from llmserver_amd.parts import GQAttention, Mixer, NoPosition
    from llmserver_amd.parts.attention import SHORT_CONTEXT
    attention = GQAttention(64, 4, 2, 32, NoPosition())
    assert attention.graph_shape(8, SHORT_CONTEXT) == attention.graph_shape(1, 1) != attention.graph_shape(8, SHORT_CONTEXT + 1)
    assert attention.graph_shape(8, 10 ** 6) is None and attention.graph_shape_edges() == (SHORT_CONTEXT,)
    assert Mixer().graph_shape(3, 5) is None and Mixer().graph_shape_edges() == ()
    import llmserver_amd.engine.step as step
    import llmserver_amd.engine.batch as batch
    assert "SHORT_CONTEXT" not in vars(step) and "short_contexts" not in inspect.getsource(batch)
