"""Fills the table of kernel choices for given model sizes on the GPU at hand.

    python -m llmserver_amd.kernels.calibrate --model DIR [--model DIR ...] [--out FILE] [--max-batch-size 64]
    python -m llmserver_amd.kernels.calibrate --config config.json [...]      (random weights of those sizes, two layers)
    python -m llmserver_amd.kernels.calibrate --random-config qwen3-8b [...]  (a size known by name, see llmserver_amd/config/named_sizes.py)

Every product shape of the models is timed both ways (a hand-written kernel with what it folds in; the library's
product and the kernels it would have absorbed; the library's product whole or in ranges of its inner dimension) at 1
to ``--max-batch-size`` decoding rows and at prompt portions of 17 to 1,024 tokens, and the faster way is written to ``--out`` (default: the table that ships with the package) under
the GPU's name.  Serving never measures; it reads this table.
"""
from __future__ import annotations

import argparse
import json
import sys

from .choices import SHIPPED


def main(argv=None) -> int:
    parser = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    parser.add_argument("--model", action="append", default=[], help="a model folder (config.json + safetensors)")
    parser.add_argument("--config", action="append", default=[], help="a config.json whose sizes are measured with random weights")
    parser.add_argument("--random-config", action="append", default=[], help="a named size (llmserver_amd/config/named_sizes.py)")
    parser.add_argument("--layers", type=int, default=2, help="layers of a --config model (shapes do not depend on the number)")
    parser.add_argument("--out", default=SHIPPED)
    parser.add_argument("--max-batch-size", type=int, default=64)
    parser.add_argument("--dtype", default="bfloat16")
    args = parser.parse_args(argv)
    if not args.model and not args.config and not args.random_config:
        parser.error("name at least one --model, --config or --random-config")
    import torch

    from .. import models  # noqa: F401
    from ..config import config_from_dict, named_size
    from ..engine import Engine, load_model, parse_dtype
    from ..weights import random_model_on_device
    total = 0
    sources = [("model", m) for m in args.model] + [("config", c) for c in args.config] + [("named", n) for n in args.random_config]
    for kind, source in sources:
        if kind == "model":
            model = load_model(source, "cuda", args.dtype)
        else:
            if kind == "named":
                raw = named_size(source)
            else:
                with open(source) as handle:
                    raw = json.load(handle)
            raw["num_hidden_layers"] = min(int(raw.get("num_hidden_layers", args.layers)), args.layers)
            model = random_model_on_device(config_from_dict(raw), "cuda", parse_dtype(args.dtype))
        engine = Engine(model, None, max_new_tokens=1, max_batch_size=args.max_batch_size, max_num_batched_tokens=max(1024, args.max_batch_size),
                        kv_cache_num_blocks=args.max_batch_size * 8 + 64, kv_cache_block_size=16, enable_prefix_caching=False)
        measured = engine.calibrate(save_to=args.out)
        total += measured
        print(f"{source}: {measured} shapes measured on {engine.runner.ops.device_kind}", flush=True)
        del engine, model
        torch.cuda.empty_cache()
    print(f"{total} shapes in all; table: {args.out}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
