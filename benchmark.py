#!/usr/bin/env python3
"""Command line of the engine's benchmark; see llmserver_amd/cli/benchmark.py for the options."""
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

from llmserver_amd.cli.benchmark import main  # noqa: E402

if __name__ == "__main__":
    sys.exit(main())
