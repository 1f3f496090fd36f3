"""Command line in the reference's manner (cli.py:11-66): the same option names
with the same meanings (temperature, top_p, max_seq_len, max_gpu_num_blocks,
max_gen_len, load_model, compiled_model, triton_weight; compiled_model is on
unless switched off, because the replayed step is the fast path here), the checkpoint folder
as an option instead of a line to edit in the source, and a prompt loop that
ends at "exit". With a tokenizer.json in the folder prompts are text; without
one they are token ids separated by blanks or commas.
"""
from __future__ import annotations

import argparse
import json
import sys
import tempfile
from typing import List, Optional


def _bool(s: str) -> bool:
    return str(s).lower() in ("1", "true", "yes", "on")


def build_parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(prog="cli.py", description="Generate with a Llama model folder on one MI355X")
    ap.add_argument("--checkpoints_dir", "--model", dest="checkpoints_dir", default=None,
                    help="folder with config.json and model.safetensors")
    ap.add_argument("--temperature", type=float, default=0.6)
    ap.add_argument("--top_p", type=float, default=0.9)
    ap.add_argument("--max_seq_len", type=int, default=2048)
    ap.add_argument("--max_gpu_num_blocks", type=int, default=None, help="cache pages (None: from free memory)")
    ap.add_argument("--max_gen_len", type=int, default=1024)
    ap.add_argument("--load_model", type=_bool, default=True, help="false: random weights from --seed")
    ap.add_argument("--compiled_model", type=_bool, default=True,
                    help="replay decode steps and single prompt portions as HIP graphs (false: launch "
                         "every kernel from the host)")
    ap.add_argument("--triton_weight", type=_bool, default=True, help="accepted, without effect")
    ap.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--page_size", type=int, default=16)
    ap.add_argument("--max_batch_size", type=int, default=64)
    ap.add_argument("--max_num_batched_tokens", type=int, default=2048)
    ap.add_argument("--prefill_chunk", type=int, default=None)
    ap.add_argument("--random_config", default=None,
                    help="a config.json to build a random-weights model folder from (with --seed)")
    ap.add_argument("--prompt", action="append", default=None, help="text prompt (repeatable)")
    ap.add_argument("--prompt_ids", action="append", default=None,
                    help="prompt as token ids, e.g. '1,5,17' (repeatable)")
    ap.add_argument("--stream", type=_bool, default=True)
    return ap


def parse_ids(s: str) -> List[int]:
    return [int(x) for x in s.replace(",", " ").split()]


def main(argv: Optional[List[str]] = None) -> int:
    args = build_parser().parse_args(argv)
    from .generate import GenerateStreamText

    folder = args.checkpoints_dir
    if args.random_config:
        from .weights import write_random_model
        with open(args.random_config) as f:
            cfg = json.load(f)
        folder = folder or tempfile.mkdtemp(prefix="random_model_")
        write_random_model(cfg, folder, seed=args.seed)
        print(f"random model written to {folder}", file=sys.stderr)
    if not folder:
        print("give --checkpoints_dir (or --random_config)", file=sys.stderr)
        return 2
    gen = GenerateStreamText(
        checkpoints_dir=folder, tokenizer_path=folder, max_seq_len=args.max_seq_len,
        max_gpu_num_blocks=args.max_gpu_num_blocks, load_model=args.load_model,
        triton_weight=args.triton_weight, compiled_model=args.compiled_model, dtype=args.dtype,
        seed=args.seed, page_size=args.page_size, max_batch_size=args.max_batch_size,
        max_num_batched_tokens=args.max_num_batched_tokens, prefill_chunk=args.prefill_chunk)

    def run(prompts_text, prompts_ids):
        if prompts_ids is not None:
            stream = gen.generate_stream(prompts_ids, args.max_gen_len, args.temperature, args.top_p)
            done = [[] for _ in prompts_ids]
            for batch in stream:
                for i, new in enumerate(batch):
                    done[i].extend(new)
                if args.stream and len(prompts_ids) == 1 and batch[0]:
                    print(" ".join(map(str, batch[0])), end=" ", flush=True)
            if not (args.stream and len(prompts_ids) == 1):
                for ids in done:
                    print(" ".join(map(str, ids)))
            else:
                print()
        else:
            shown = ""
            last = None
            for comps in gen.text_completion_stream(prompts_text, args.temperature, args.top_p,
                                                    args.max_gen_len):
                last = comps
                if args.stream and len(prompts_text) == 1:
                    text = comps[0]["generation"]
                    print(text[len(shown):], end="", flush=True)
                    shown = text
            if args.stream and len(prompts_text) == 1:
                print()
            elif last:
                for c in last:
                    print(c["generation"])

    if args.prompt_ids:
        run(None, [parse_ids(s) for s in args.prompt_ids])
        return 0
    if args.prompt:
        run(args.prompt, None)
        return 0
    text_mode = gen.tokenizer is not None
    while True:
        try:
            line = input("prompt ('exit' to quit)" + ("" if text_mode else " as token ids") + ":\n")
        except EOFError:
            break
        if line.strip().lower() == "exit":
            break
        if not line.strip():
            continue
        if text_mode:
            run([line], None)
        else:
            run(None, [parse_ids(line)])
        print("\n==================================\n")
    return 0


if __name__ == "__main__":
    sys.exit(main())
