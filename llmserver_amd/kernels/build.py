"""Compiles the HIP sources under ``csrc/`` for gfx950 into shared libraries and finds them again.

Every library is one ``hipcc`` call.  Its file name carries a hash of the sources and flags it
was built from, so a stale library is never loaded.  Libraries live in ``kernels/_lib`` inside
the package (they travel with the tree); if that folder cannot be written they go to a per-user
folder under the system's temporary directory.  What a model needs and is not there yet is
compiled at first use, several libraries at a time, with a progress line every few seconds.
"""
from __future__ import annotations

import concurrent.futures
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from typing import Dict, Iterable, List, Tuple

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")
LIB_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "_lib")
ARCH = "gfx950"
FLAGS = ["-O3", f"--offload-arch={ARCH}", "-shared", "-fPIC", "-std=c++17",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
HEAD_DIMS = tuple(range(16, 257, 16))
BASE_MODULES = ("elementwise", "rope_kv", "sampling", "gemm")


class KernelBuildError(RuntimeError):
    pass


def attention_module(bf16: bool, head_dim: int) -> str:
    if head_dim % 16 or not 16 <= head_dim <= 256:
        raise ValueError(f"the attention kernels take head sizes 16, 32, ..., 256; got {head_dim}")
    return f"attention_{'bf16' if bf16 else 'f32'}_d{head_dim}"


def module_recipe(name: str) -> Tuple[str, List[str]]:
    """(source file, extra flags) of a library."""
    if name.startswith("attention_"):
        _, kind, dim = name.split("_")
        return "attention.hip", [f"-DLSA_BF16={1 if kind == 'bf16' else 0}", f"-DLSA_ND={int(dim[1:]) // 16}"]
    if name in BASE_MODULES:
        return f"{name}.hip", []
    raise KeyError(f"unknown kernel library {name!r}")


def all_modules(head_dims: Iterable[int] = (64, 128)) -> List[str]:
    names = list(BASE_MODULES)
    for dim in head_dims:
        names += [attention_module(True, dim), attention_module(False, dim)]
    return names


def _hash(name: str) -> str:
    source, extra = module_recipe(name)
    digest = hashlib.sha256()
    own_header = os.path.join(CSRC, os.path.splitext(source)[0] + ".h")          # its entry points' declarations, if it has any
    paths = [os.path.join(CSRC, source), os.path.join(CSRC, "common.hpp")] + ([own_header] if os.path.isfile(own_header) else [])
    for path in paths:
        with open(path, "rb") as handle:
            digest.update(handle.read())
    digest.update(" ".join(FLAGS + extra).encode())
    return digest.hexdigest()[:12]


def _file_name(name: str) -> str:
    return f"{name}-{_hash(name)}.so"


def _fallback_dir() -> str:
    return os.path.join(tempfile.gettempdir(), f"llmserver_amd-{os.getuid()}", "lib")


def find_library(name: str):
    file_name = _file_name(name)
    for folder in (os.environ.get("LLMSERVER_AMD_LIB_DIR"), LIB_DIR, _fallback_dir()):
        if folder and os.path.isfile(os.path.join(folder, file_name)):
            return os.path.join(folder, file_name)
    return None


def _output_dir() -> str:
    for folder in (os.environ.get("LLMSERVER_AMD_LIB_DIR"), LIB_DIR, _fallback_dir()):
        if not folder:
            continue
        try:
            os.makedirs(folder, exist_ok=True)
            probe = os.path.join(folder, f".probe-{os.getpid()}")
            with open(probe, "w"):
                pass
            os.remove(probe)
            return folder
        except OSError:
            continue
    raise KernelBuildError("no writable folder for compiled kernels")


def _hipcc() -> str:
    for candidate in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if candidate and os.path.exists(candidate):
            return candidate
    raise KernelBuildError("hipcc was not found; the HIP kernels cannot be compiled")


def compile_library(name: str, folder: str = None) -> str:
    source, extra = module_recipe(name)
    folder = folder or _output_dir()
    target = os.path.join(folder, _file_name(name))
    scratch = f"{target}.{os.getpid()}.tmp"
    command = [_hipcc(), *FLAGS, *extra, os.path.join(CSRC, source), "-o", scratch]
    env = dict(os.environ)
    env.setdefault("HOME", tempfile.gettempdir())     # hipcc wants a home for its caches
    result = subprocess.run(command, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env, cwd=folder)
    if result.returncode != 0 or not os.path.exists(scratch):
        raise KernelBuildError(f"compiling {name} failed:\n{' '.join(command)}\n{result.stdout}")
    os.replace(scratch, target)
    for other in os.listdir(folder):                   # drop libraries built from older sources
        if other.startswith(name + "-") and other.endswith(".so") and other != os.path.basename(target):
            try:
                os.remove(os.path.join(folder, other))
            except OSError:
                pass
    return target


def build(names: Iterable[str], force: bool = False, quiet: bool = False) -> Dict[str, str]:
    """Make sure the named libraries exist; returns name -> path.  Compiles up to 8 at a time."""
    names = list(dict.fromkeys(names))
    found = {} if force else {name: find_library(name) for name in names}
    todo = [name for name in names if not found.get(name)]
    if not todo:
        return found
    folder = _output_dir()
    started = time.time()
    if not quiet:
        print(f"[llmserver_amd] compiling {len(todo)} HIP kernel librar{'y' if len(todo) == 1 else 'ies'} for {ARCH}: "
              + ", ".join(todo), file=sys.stderr, flush=True)
    done = threading.Event()

    def ticker():
        while not done.wait(10.0):
            print(f"[llmserver_amd] still compiling ... {time.time() - started:.0f} s", file=sys.stderr, flush=True)

    thread = threading.Thread(target=ticker, daemon=True)
    if not quiet:
        thread.start()
    try:
        with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(todo))) as pool:
            for name, path in zip(todo, pool.map(lambda n: compile_library(n, folder), todo)):
                found[name] = path
    finally:
        done.set()
    if not quiet:
        print(f"[llmserver_amd] compiled in {time.time() - started:.1f} s", file=sys.stderr, flush=True)
    return found
