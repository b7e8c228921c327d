"""Python entry points in the reference's manner: ``model_loader(...)`` then ``Engine(...)``
(utils/model_loader.py:18, utils/engine.py:47)."""
from __future__ import annotations

from typing import List, Sequence

from .engine.engine import Engine
from .engine.loading import load_model


def model_loader(model_name: str, device="cuda", dtype="bfloat16"):
    """Load a model folder; the name and the first arguments follow the reference's loader."""
    return load_model(model_name, device, dtype)


def generate(model, prompts: Sequence[Sequence[int]], max_new_tokens: int = 16, dtype="bfloat16", device="cuda",
             temperature: float = 0.0, seed: int = 0, block_size: int = 16, num_blocks: int = None,
             max_batch_size: int = None, max_num_batched_tokens: int = 2048, ignore_eos: bool = True,
             prefill_chunk_size: int = None, ops=None) -> List[List[int]]:
    """Generate from token-id prompts with a model folder (or a loaded model); returns token ids."""
    if isinstance(model, str):
        model = load_model(model, device, dtype)
    if num_blocks is None:
        num_blocks = sum(-(-(len(p) + max_new_tokens) // block_size) for p in prompts) + 8
    engine = Engine(model, None, max_new_tokens=max_new_tokens, max_batch_size=max_batch_size or max(1, len(prompts)),
                    max_num_batched_tokens=max(max_num_batched_tokens, max_batch_size or len(prompts)),
                    prefill_chunk_size=prefill_chunk_size, kv_cache_num_blocks=num_blocks, kv_cache_block_size=block_size,
                    stream_text=False, ignore_eos=ignore_eos, temperature=temperature, seed=seed, ops=ops)
    return engine.generate(prompts)
