#!/usr/bin/env python3
"""The reference's example.py as a command: generate from a few prompts and print them.

    python example.py --model DIR --prompt-ids 1,2,3 --prompt "introduce yourself"

Defaults follow the reference (example.py:7-13 there): temperature 0.6, 256 new tokens."""
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

from nano_vllm_amd.cli import main  # noqa: E402

if __name__ == "__main__":
    sys.exit(main(["generate"] + sys.argv[1:]))
