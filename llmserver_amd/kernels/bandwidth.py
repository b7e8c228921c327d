"""What this GPU's memory delivers to a kernel that only reads: the scale the step's kernels are read against.

    python -m llmserver_amd.kernels.bandwidth [--megabytes 134,1240] [--workgroups 32,64,128,256,512,1024] [--threads 256,1024]

Every launch reads cold memory (a different stretch of a buffer larger than the caches each time) from the given
number of workgroups and is timed with events; the best of five is printed with its rate, and the rate per workgroup
(up to one workgroup per compute unit that is what a single compute unit pulls).
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


def main(argv=None) -> int:
    parser = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    parser.add_argument("--megabytes", default="134,1240")
    parser.add_argument("--workgroups", default="32,64,128,256,512,1024")
    parser.add_argument("--threads", default="256,1024")
    args = parser.parse_args(argv)
    numbers = lambda text: [int(item) for item in text.split(",") if item.strip()]
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
