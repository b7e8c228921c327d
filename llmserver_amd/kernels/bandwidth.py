"""What this GPU's memory delivers to a kernel that only reads: the scale the step's kernels are read against.

    python -m llmserver_amd.kernels.bandwidth [--megabytes 134,1240] [--workgroups 32,64,128,256,512,1024] [--threads 256,1024]
    python -m llmserver_amd.kernels.bandwidth --chain 50,134,34,201,100 --layers 36

Every launch reads cold memory (a different stretch of a buffer larger than the caches each time) from the given
number of workgroups and is timed with events; the best of five is printed with its rate, and the rate per workgroup
(up to one workgroup per compute unit that is what a single compute unit pulls).

``--chain``: launches that each read so many megabytes, one after the other as the kernels of a decoding step follow one
another (a layer's products and its attention, ``--layers`` times, every launch its own stretch of memory), replayed from
a graph: what a step of that many launches of those sizes takes if its kernels did nothing but read.
"""
from __future__ import annotations

import argparse
import sys


def measure(megabytes, workgroups, threads, repeats=5):
    import torch

    from . import library
    from .ops import _ptr, _stream
    lib = library.load("elementwise")
    total = int(megabytes) << 20
    buffer = torch.zeros(8 * total // 4, dtype=torch.float32, device="cuda")            # eight stretches: none is met again soon
    sink = torch.zeros(1, dtype=torch.float32, device="cuda")
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    best = float("inf")
    for repeat in range(repeats + 1):
        stretch = buffer[(repeat % 8) * (total // 4):]
        start.record()
        code = lib.lsa_plain_read(_ptr(stretch), _ptr(sink), total, workgroups, threads, _stream())
        end.record()
        end.synchronize()
        if code:
            raise RuntimeError(f"launch of plain_read failed with HIP error {code}")
        if repeat:
            best = min(best, start.elapsed_time(end) * 1e-3)
    return best


def measure_chain(megabytes, layers, workgroups=256, threads=512, repeats=5):
    """Seconds of one replay of ``layers`` times the launches of ``megabytes`` (best of ``repeats``), and the bytes read."""
    import torch

    from . import library
    from .ops import _ptr, _stream
    lib = library.load("elementwise")
    sizes = [int(m) * 1_000_000 // (16 * workgroups) * (16 * workgroups) for m in megabytes]
    buffer = torch.zeros(layers * sum(sizes) // 4, dtype=torch.float32, device="cuda")
    sink = torch.zeros(1, dtype=torch.float32, device="cuda")

    def launches():
        at = 0
        for _ in range(layers):
            for size in sizes:
                code = lib.lsa_plain_read(_ptr(buffer[at // 4:]), _ptr(sink), size, workgroups, threads, _stream())
                if code:
                    raise RuntimeError(f"launch of plain_read failed with HIP error {code}")
                at += size
    launches()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        launches()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    best = float("inf")
    for repeat in range(repeats + 1):
        start.record()
        graph.replay()
        end.record()
        end.synchronize()
        if repeat:
            best = min(best, start.elapsed_time(end) * 1e-3)
    return best, layers * sum(sizes)


def main(argv=None) -> int:
    parser = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    parser.add_argument("--megabytes", default="134,1240")
    parser.add_argument("--workgroups", default="32,64,128,256,512,1024")
    parser.add_argument("--threads", default="256,1024")
    parser.add_argument("--chain", default=None, help="megabytes of the launches of one layer, read one after the other from a graph")
    parser.add_argument("--layers", type=int, default=36)
    args = parser.parse_args(argv)
    numbers = lambda text: [int(item) for item in text.split(",") if item.strip()]
    if args.chain:
        sizes = numbers(args.chain)
        seconds, total = measure_chain(sizes, args.layers)
        count = args.layers * len(sizes)
        print(f"{count} launches of {', '.join(map(str, sizes))} MB x {args.layers}: {seconds * 1e3:7.3f} ms for {total / 1e9:.2f} GB, "
              f"{total / seconds / 1e12:.2f} TB/s, {seconds * 1e6 / count:.2f} us a launch", flush=True)
        return 0
    for megabytes in numbers(args.megabytes):
        for threads in numbers(args.threads):
            for workgroups in numbers(args.workgroups):
                seconds = measure(megabytes, workgroups, threads)
                rate = (megabytes << 20) / seconds
                print(f"{megabytes:6d} MB  {threads:4d} threads x {workgroups:4d} workgroups: {seconds * 1e6:8.1f} us  {rate / 1e12:5.2f} TB/s"
                      f"  {rate / 1e9 / workgroups:6.1f} GB/s a workgroup", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
