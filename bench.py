#!/usr/bin/env python3
"""python bench.py --gpus 1 --steps K --warmup W: one JSON line with decode and prefill throughput."""
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
from leone_amd.benchmark import main  # noqa: E402

if __name__ == "__main__":
    sys.exit(main())
