#!/usr/bin/env python3
"""python cli.py --checkpoints_dir DIR [--temperature 0.6 --top_p 0.9 --max_gen_len 1024 ...]"""
import sys

from pytriton_llama_amd.cli import main

if __name__ == "__main__":
    sys.exit(main())
