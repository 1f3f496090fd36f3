#!/usr/bin/env python3
"""Decode and prefill throughput of the engine at Llama-3.2-1B shape on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one decode step of the whole engine (schedule, model step over the
paged cache, sampling, bookkeeping) for a batch of requests whose prompts are
already in the cache. The default run: random weights N(0, 0.02) of the 1B
shape, batch 8, 2,048-token prompts of seeded uniform-random token ids, greedy
sampling, EOS ignored, 256 timed steps: the contexts grow from 2,048 to 2,304
tokens while the clock runs (the warm-up steps are taken by a batch of the same
shape that is thrown away before the timed one goes in; the timed requests end
with the token of the last timed step, so the engine, which otherwise launches
every decode step ahead of the tokens of the step before, starts no step inside
the clock whose tokens nobody takes). One JSON line is
printed: decoded tokens a second at batch 8, the prefill of one 2,048-token
prompt, the decode step's HBM roofline, the decode rates at batch 1 and 64, and
(points.generate_call_b8) the tokens a second of one whole generate() call for 8
short prompts with temperature 0.6 and top_p 0.9, which is how the reference's
own benchmark measures.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# MI355X published peaks
PEAK_HBM_GBS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}

LLAMA_1B = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "num_hidden_layers": 16, "hidden_size": 2048, "num_attention_heads": 32,
    "num_key_value_heads": 8, "head_dim": 64, "intermediate_size": 8192, "vocab_size": 128256,
    "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 32.0, "low_freq_factor": 1.0,
                     "high_freq_factor": 4.0, "original_max_position_embeddings": 8192},
    "max_position_embeddings": 131072, "rms_norm_eps": 1e-5, "tie_word_embeddings": True,
    "torch_dtype": "bfloat16", "hidden_act": "silu", "initializer_range": 0.02,
}


SHAPES = {
    "1b": {},
    # Llama-3.2-3B shape
    "3b": {"num_hidden_layers": 28, "hidden_size": 3072, "num_attention_heads": 24,
           "num_key_value_heads": 8, "head_dim": 128, "intermediate_size": 8192},
    # Llama-3.1-8B shape
    "8b": {"num_hidden_layers": 32, "hidden_size": 4096, "num_attention_heads": 32,
           "num_key_value_heads": 8, "head_dim": 128, "intermediate_size": 14336,
           "tie_word_embeddings": False,
           "rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0,
                            "high_freq_factor": 4.0, "original_max_position_embeddings": 8192}},
}


SHAPE_NAMES = {"1b": "Llama-3.2-1B", "3b": "Llama-3.2-3B", "8b": "Llama-3.1-8B"}


def log(msg):
    print(f"[bench] {msg}", file=sys.stderr, flush=True)


def model_numbers(cfg, dtype_bytes):
    L, H, I, V = cfg["num_hidden_layers"], cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    Hq, Hkv, D = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    layer_params = (Hq + 2 * Hkv) * D * H + H * Hq * D + 3 * I * H
    return {
        "layer_params": layer_params,
        "weight_bytes": (L * (layer_params + 2 * H) + V * H + H) * dtype_bytes,   # every weight a step uses
        "kv_bytes_per_token": 2 * L * Hkv * D * dtype_bytes,
        "linear_flops_per_token": 2 * L * layer_params,
        "attn_flops": lambda S: L * 4 * D * Hq * S * (S + 1) // 2,              # causal, one prompt
        "head_flops_per_row": 2 * V * H,
    }


def mixed_workload(args, cfg, short):
    """The secondary workload: a continuous batch of N requests with prompts of
    128..4096 tokens, computed in 512-token portions beside the decodes of the
    others, 256 greedy tokens each. Reports generated tokens per second of the
    whole run and the prompt tokens per second that went in beside them. The
    workload runs twice and the second run is timed: the first records the HIP
    graphs of the step shapes it meets (a server does that once, at its start)."""
    import torch
    from pytriton_llama_amd.config import EngineConfig
    from pytriton_llama_amd.engine import Engine, SamplingParams
    N, new = args.mixed, 256
    g = torch.Generator().manual_seed(99)
    lens = torch.randint(128, 4097, (N,), generator=g).tolist()
    page = 16
    pages = sum(-(-(n + new + 8) // page) for n in lens) + 8
    ec = EngineConfig(dtype=args.dtype, page_size=page, num_pages=pages, max_num_seqs=N,
                      max_num_batched_tokens=512 + N, prefill_chunk=512, max_model_len=4096 + new + 8, seed=0)
    t0 = time.time()
    log(f"building the {cfg['num_hidden_layers']}-layer {args.shape} model with random weights ({args.dtype})")
    engine = Engine(cfg, ec, random_seed=0)
    log(f"model ready in {time.time() - t0:.1f}s")
    sp = SamplingParams(temperature=0.0, max_new_tokens=new, ignore_eos=True)
    warm = engine.generate([torch.randint(0, cfg["vocab_size"], (600,), generator=g).tolist()],
                           SamplingParams(temperature=0.0, max_new_tokens=8, ignore_eos=True))
    prompts = [torch.randint(0, cfg["vocab_size"], (n,), generator=g).tolist() for n in lens]
    nums = model_numbers(cfg, 2 if short == "bf16" else 4)
    t0 = time.time()
    engine.generate(prompts, sp)
    log(f"untimed pass of the workload: {time.time() - t0:.2f}s")
    torch.cuda.synchronize()
    t = time.perf_counter()
    steps = 0
    ids = [engine.add_request(p, sp) for p in prompts]
    reqs = [engine.requests[i] for i in ids]
    # what the steps have to do, counted from what every step computed: the flops of the
    # products and of the attention, and the bytes a step must read (every weight once, the keys
    # and values of every sequence it touches once)
    flops = bytes_read = 0
    before = [0] * N
    attn_unit = nums["attn_flops"](1)                      # per (query, key) pair of all layers
    while engine.has_work:
        engine.step()
        steps += 1
        touched = 0
        for k, r in enumerate(reqs):
            now = r.num_computed
            n = now - before[k]
            if n > 0:
                touched += 1
                flops += nums["linear_flops_per_token"] * n + attn_unit * (n * before[k] + n * (n + 1) // 2)
                bytes_read += now * nums["kv_bytes_per_token"]
                before[k] = now
        if touched:
            bytes_read += nums["weight_bytes"]
    flops += nums["head_flops_per_row"] * N * new
    torch.cuda.synchronize()
    dt = time.perf_counter() - t
    out = {"metric": f"mixed continuous batch, {SHAPE_NAMES[args.shape]} shape: {N} requests, prompts 128..4096, "
                     f"512-token portions beside decodes, {new} new tokens each",
           "value": round(N * new / dt, 1), "unit": "generated tokens/s", "seconds": round(dt, 3),
           "engine_steps": steps, "prompt_tokens": sum(lens),
           "prompt_tokens_per_s": round(sum(lens) / dt, 1), "preemptions": engine.scheduler.num_preemptions,
           "tflops": round(flops / dt / 1e12, 1), "flops_frac": round(flops / dt / PEAK_FLOPS[short], 4),
           "roofline": {"bound": "hbm", "achieved": round(bytes_read / dt / 1e9, 1), "peak": PEAK_HBM_GBS,
                        "unit": "GB/s", "frac": round(bytes_read / dt / 1e9 / PEAK_HBM_GBS, 4)},
           "config": {"model": f"{SHAPE_NAMES[args.shape]} shape, random weights N(0,0.02)",
                      "layers": cfg["num_hidden_layers"], "hidden_size": cfg["hidden_size"],
                      "heads": cfg["num_attention_heads"], "kv_heads": cfg["num_key_value_heads"],
                      "head_dim": cfg["head_dim"], "intermediate_size": cfg["intermediate_size"],
                      "vocab_size": cfg["vocab_size"], "requests": N, "prefill_chunk": 512, "page_size": page,
                      "untimed_passes_before": 1},
           "dtype": short, "data": "synthetic", "n_gpus": 1}
    print(json.dumps(out), flush=True)
    return 0


def like_reference(args, cfg, short):
    """The measurement the reference publishes (examples/benchmark.py:42-74,175-190;
    docs/benchmark_models.md:364-604): one ``generate`` call of the Python entry point for a
    batch of short prompts with temperature 0.6 and top_p 0.9, one warm-up call before it,
    tokens/s = generated tokens / wall time of the whole call (prompt, decoding, bookkeeping).
    The reference runs English prompts of roughly 10 to 60 tokens through a tokenizer and real
    weights in fp16; here the prompts are 10 to 60 random token ids and the weights random."""
    import tempfile
    import torch
    from pytriton_llama_amd.generate import GenerateText
    B, new = args.like_reference, 256
    folder = tempfile.mkdtemp(prefix="bench_like_reference_")
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    t0 = time.time()
    gen = GenerateText(folder, max_seq_len=2048, load_model=False, compiled_model=True,
                       dtype=args.dtype, max_batch_size=B)
    log(f"model ready in {time.time() - t0:.1f}s")
    g = torch.Generator().manual_seed(7)
    lens = torch.randint(10, 61, (B,), generator=g).tolist()
    prompts = [torch.randint(0, cfg["vocab_size"], (n,), generator=g).tolist() for n in lens]
    gen.generate(prompts, new, temperature=0.6, top_p=0.9)                 # the warm-up call
    best = None
    for _ in range(3):
        torch.cuda.synchronize()
        t = time.perf_counter()
        outs, _ = gen.generate(prompts, new, temperature=0.6, top_p=0.9)
        dt = time.perf_counter() - t
        made = sum(len(o) for o in outs)
        if best is None or made / dt > best[0] / best[1]:
            best = (made, dt)
    made, dt = best
    published = {2: 481.50, 4: 400.99, 8: 620.0, 16: 963.15}               # the best run of each batch size
    out = {"metric": f"one generate() call as the reference measures it: {SHAPE_NAMES[args.shape]} shape, "
                     f"batch {B}, prompts of 10..60 tokens, {new} new tokens, temperature 0.6, top_p 0.9",
           "value": round(made / dt, 1), "unit": "generated tokens/s", "seconds": round(dt, 4),
           "generated_tokens": made, "ms_per_token": round(dt / made * 1e3, 4),
           "reference_published": published.get(B) if args.shape == "1b" else None,
           "reference_published_note": "lite_llama's own best run at this batch size, other hardware, real "
                                       "weights and prompts (docs/benchmark_models.md)",
           "vs_reference_published": (round(made / dt / published[B], 2)
                                      if args.shape == "1b" and B in published else None),
           "dtype": short, "data": "synthetic", "n_gpus": 1}
    print(json.dumps(out), flush=True)
    return 0


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--prompt-len", type=int, default=2048)
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the 1B shape has")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--points", default="1,16,32,64", help="other batch sizes to report, '' for none")
    ap.add_argument("--long-context", type=int, default=8192, metavar="S",
                    help="with the default run: one more point, batch 8 decoding behind prompts of S tokens "
                         "(0: none)")
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--no-probes", action="store_true",
                    help="skip the two probes of the box (streaming read, MFMA loop)")
    ap.add_argument("--prefill-only", action="store_true", help="measure the prefill and stop (for profiles)")
    ap.add_argument("--prefill-chunk", type=int, default=0, metavar="N",
                    help="compute a prompt in portions of N tokens, one step each (default: the whole prompt "
                         "in one step, as the 2,048-token measurement does)")
    ap.add_argument("--shape", default="1b", choices=sorted(SHAPES),
                    help="layer sizes: the default 1b is the benchmark; 3b and 8b are the secondary shapes")
    ap.add_argument("--mixed", type=int, default=0, metavar="N",
                    help="instead of the decode measurement: N requests with prompts of 128..4096 tokens "
                         "through the scheduler in 512-token portions beside decodes, 256 new tokens each")
    ap.add_argument("--like-reference", type=int, default=0, metavar="B",
                    help="instead of the decode measurement: one generate() call of the Python entry point "
                         "for B short prompts, 256 new tokens, temperature 0.6, top_p 0.9, as the "
                         "reference's examples/benchmark.py measures")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU: this engine has no multi-GPU path, --gpus {args.gpus} is not run")
        return 2

    import torch
    from pytriton_llama_amd.config import EngineConfig
    from pytriton_llama_amd.engine import Engine, SamplingParams

    cfg = dict(LLAMA_1B)
    cfg.update(SHAPES[args.shape])
    full_layers = cfg["num_hidden_layers"]
    if args.layers:
        cfg["num_hidden_layers"] = args.layers
    short = "bf16" if args.dtype == "bfloat16" else "fp32"
    dbytes = 2 if short == "bf16" else 4
    nums = model_numbers(cfg, dbytes)
    point_batches = [int(x) for x in args.points.split(",") if x]
    max_batch = max([args.batch] + point_batches)
    K, W, S = args.steps, args.warmup, args.prompt_len
    page = 16
    # requests whose prompt is in first go on decoding while the others' prompts are computed
    slack = max_batch * -(-S // (args.prefill_chunk or max(S, 2048))) + 8
    per_req_pages = -(-(S + max(W, K) + slack) // page)
    if args.mixed:
        return mixed_workload(args, cfg, short)
    if args.like_reference:
        return like_reference(args, cfg, short)
    ec = EngineConfig(dtype=args.dtype, page_size=page, num_pages=per_req_pages * max_batch + 8,
                      max_num_seqs=max_batch,
                      max_num_batched_tokens=args.prefill_chunk or max(S, 2048),
                      prefill_chunk=args.prefill_chunk or None,
                      max_model_len=S + max(W, K) + slack, seed=0)
    t0 = time.time()
    log(f"building the {cfg['num_hidden_layers']}-layer {args.shape.upper()}-shape model with random weights "
        f"({args.dtype})")
    engine = Engine(cfg, ec, random_seed=0)
    log(f"model ready in {time.time() - t0:.1f}s")
    g = torch.Generator().manual_seed(1234)

    def prompts(n, length=None):
        return [torch.randint(0, cfg["vocab_size"], (length or S,), generator=g).tolist() for _ in range(n)]

    def sync():
        torch.cuda.synchronize()

    # ---- prefill of one 2,048-token prompt --------------------------------------
    prefill = None
    if not args.no_prefill:
        times = []
        for i in range(8):
            rid = engine.add_request(prompts(1)[0], SamplingParams(temperature=0.0, max_new_tokens=1,
                                                                    ignore_eos=True))
            sync()
            t = time.perf_counter()
            while engine.has_work:              # the whole prompt in one step (or portion by portion),
                engine.step()                   # first token sampled
            sync()
            times.append(time.perf_counter() - t)
            engine.requests.pop(rid, None)
            assert not engine.has_work
        best = min(times[1:])
        flops = nums["linear_flops_per_token"] * S + nums["attn_flops"](S) + nums["head_flops_per_row"]
        prefill = {"value": round(S / best, 1), "tokens": S, "ms": round(best * 1e3, 3),
                   "frac": round(flops / best / PEAK_FLOPS[short], 4)}
        if args.prefill_chunk:
            prefill["portions_of"] = args.prefill_chunk
        log(f"prefill {S} tokens: {best * 1e3:.2f} ms ({S / best:.0f} tok/s)")

    if args.prefill_only:
        print(json.dumps({"prefill": prefill}), flush=True)
        return 0

    # ---- decode ---------------------------------------------------------------------
    def prefilled(batch, new_tokens, ends_there=False, engine=engine, S=S, slack=slack):
        """``batch`` requests with their prompts in the cache and their first tokens sampled.
        ``ends_there``: every request ends with the token of decode step number ``new_tokens``
        from here, as the workload says (N new tokens each); the engine then launches no step
        ahead of the last one, so the timed steps are all that the GPU does inside the clock."""
        ids = [engine.add_request(p, SamplingParams(temperature=0.0, max_new_tokens=new_tokens + slack - 4,
                                                    ignore_eos=True)) for p in prompts(batch, S)]
        while any(engine.requests[i].num_computed < S for i in ids):
            engine.step()                       # prompts go in, portion by portion
        if ends_there:
            for i in ids:                       # (those whose prompt went in first have decoded a few tokens)
                engine.requests[i].params.max_new_tokens = len(engine.requests[i].output) + new_tokens
        return ids

    def drop(ids, engine=engine):
        for i in ids:
            engine.abort(i)                     # (nothing left to stop for a request that has ended)
        assert not engine.has_work

    def decode_rate(batch, steps, warmup, engine=engine, S=S, slack=slack):
        """(tokens/s, seconds a step, mean context while timed, GB/s of what a step must read)"""
        def prefilled_(b, n, ends_there=False):
            return prefilled(b, n, ends_there, engine, S, slack)
        if warmup:
            ids = prefilled_(batch, warmup)     # a batch of the same shape takes the warm-up steps
            for _ in range(warmup):
                engine.step()
            drop(ids, engine)
        ids = prefilled_(batch, steps, ends_there=True)
        reqs = [engine.requests[i] for i in ids]
        first_ctx = [r.num_computed for r in reqs]
        sync()
        t = time.perf_counter()
        produced = 0
        for _ in range(steps):
            produced += len(engine.step())
        sync()
        dt = time.perf_counter() - t
        assert produced == batch * steps, (produced, batch, steps)
        assert all(r.finish_reason == "length" for r in reqs) and not engine.has_work
        ctx = [r.num_computed for r in reqs]
        drop(ids, engine)
        mean_ctx = (sum(first_ctx) + sum(ctx)) / (2.0 * len(ctx))
        bytes_step = nums["weight_bytes"] + batch * mean_ctx * nums["kv_bytes_per_token"]
        return batch * steps / dt, dt / steps, mean_ctx, bytes_step * steps / dt / 1e9

    rate, step_s, mean_ctx, achieved = decode_rate(args.batch, K, W)
    log(f"decode batch {args.batch}: {rate:.0f} tok/s, {step_s * 1e3:.3f} ms/step")
    points = {}
    for b in point_batches:
        r, st, _, gbs = decode_rate(b, max(16, K // 2), max(4, W // 2))
        points[f"decode_b{b}"] = round(r, 1)
        points[f"decode_b{b}_ms_per_step"] = round(st * 1e3, 4)
        points[f"decode_b{b}_hbm_frac"] = round(gbs / PEAK_HBM_GBS, 4)
        log(f"decode batch {b}: {r:.0f} tok/s, {st * 1e3:.3f} ms/step, {gbs:.0f} GB/s")

    # One whole generate() call as the reference's own benchmark times it (examples/benchmark.py:
    # short prompts, temperature 0.6, top_p 0.9, 256 new tokens, tokens/s over the whole call),
    # on the engine that is there; --like-reference B is the same through GenerateText.
    if args.points and args.batch >= 8 and not args.no_prefill:
        try:
            lens = torch.randint(10, 61, (8,), generator=g).tolist()
            short_prompts = [torch.randint(0, cfg["vocab_size"], (n,), generator=g).tolist() for n in lens]
            sp = SamplingParams(temperature=0.6, top_p=0.9, max_new_tokens=256)
            engine.generate(short_prompts, sp)                             # the warm-up call
            sync()
            t = time.perf_counter()
            made = sum(len(o) for o in engine.generate(short_prompts, sp))
            dt = time.perf_counter() - t
            points["generate_call_b8"] = round(made / dt, 1)
            log(f"generate() call, 8 prompts of 10..60 tokens, 256 new tokens, temperature 0.6, top_p 0.9: "
                f"{made / dt:.0f} tok/s ({dt * 1e3:.0f} ms; the reference publishes 558 to 620 tok/s at batch 8)")
        except Exception as e:                                              # (never at the cost of the line)
            log(f"generate() call not measured: {e!r}")

    # One point at a longer context: batch 8 decoding behind prompts of --long-context tokens, on a
    # second engine that shares the weights (its recorded steps are planned for its own longest
    # request, so the engine above keeps the plans of the workload it measures).
    if args.points and args.long_context and args.long_context > S and not args.layers:
        try:
            model, S2, B2, K2, W2 = engine.model, args.long_context, 8, 32, 4
            slack2 = B2 * -(-S2 // 2048) + 8
            ec2 = EngineConfig(dtype=args.dtype, page_size=page,
                               num_pages=-(-(S2 + K2 + slack2) // page) * B2 + 8, max_num_seqs=B2,
                               max_num_batched_tokens=2048, prefill_chunk=2048,
                               max_model_len=S2 + K2 + slack2, seed=0)
            long_engine = Engine(model, ec2)
            r, st, ctx2, gbs = decode_rate(B2, K2, W2, long_engine, S2, slack2)
            points[f"decode_b{B2}_ctx{S2}"] = round(r, 1)
            points[f"decode_b{B2}_ctx{S2}_ms_per_step"] = round(st * 1e3, 4)
            points[f"decode_b{B2}_ctx{S2}_hbm_frac"] = round(gbs / PEAK_HBM_GBS, 4)
            log(f"decode batch {B2} behind {S2}-token prompts: {r:.0f} tok/s, {st * 1e3:.3f} ms/step, {gbs:.0f} GB/s")
            del long_engine
        except Exception as e:                                              # (never at the cost of the line)
            log(f"long-context point not measured: {e!r}")

    out = {
        "metric": f"decode tokens/s, {SHAPE_NAMES[args.shape]} shape, batch {args.batch}, {S}-token prompts",
        "value": round(rate, 1), "unit": "tokens/s", "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": round(step_s * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": short, "data": "synthetic",
        "config": {
            "model": f"{SHAPE_NAMES[args.shape]} shape, random weights N(0,0.02)", "layers": cfg["num_hidden_layers"],
            "layers_of_full_model": full_layers, "hidden_size": cfg["hidden_size"],
            "heads": cfg["num_attention_heads"], "kv_heads": cfg["num_key_value_heads"],
            "head_dim": cfg["head_dim"], "intermediate_size": cfg["intermediate_size"],
            "vocab_size": cfg["vocab_size"], "tied_embeddings": cfg["tie_word_embeddings"],
            "rope": f"llama3 factor {cfg['rope_scaling']['factor']:g}",
            "global_batch": args.batch, "seq_len": S, "new_tokens": K, "context_at_timing": round(mean_ctx),
            "page_size": page, "kv_dtype": short, "sampling": "greedy", "parallelism": "single GPU",
        },
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS,
                     "unit": "GB/s", "frac": round(achieved / PEAK_HBM_GBS, 4)},
        "points": points,
    }
    if prefill is not None:
        out["prefill"] = prefill
    if not args.no_probes and args.dtype == "bfloat16":
        # what this box gives beside the published peaks the fractions above are taken of
        peaks = measured_peaks()
        out["measured_peaks"] = peaks
        out["roofline"]["frac_of_measured"] = round(achieved / peaks["hbm_read_gbs"], 4)
        log(f"probes: streaming read {peaks['hbm_read_gbs']:.0f} GB/s, bf16 MFMA loop "
            f"{peaks['mfma_bf16_tflops']:.0f} TFLOP/s")
    print(json.dumps(out), flush=True)
    return 0


def measured_peaks():
    """Streaming-read bandwidth (1 GiB that no cache holds, read by a kernel that does nothing
    else, one workgroup a CU) and the rate of a loop of independent bfloat16 MFMAs (eight
    workgroups of four waves a CU)."""
    import torch
    from pytriton_llama_amd import ops
    buf = torch.empty(1 << 30, dtype=torch.uint8, device="cuda").zero_()

    def timed(f, reps):
        f()
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(reps):
            f()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) * 1e-3 / reps

    t = timed(lambda: ops.probe_stream_read(buf, 256), 5)      # one workgroup a CU reads fastest
    iters, blocks = 4096, 2048
    t2 = timed(lambda: ops.probe_mfma(iters, blocks), 3)
    return {"hbm_read_gbs": round(buf.numel() / t / 1e9, 1),
            "mfma_bf16_tflops": round(blocks * iters * ops.PROBE_MFMA_FLOPS_PER_ITER / t2 / 1e12, 1)}


if __name__ == "__main__":
    sys.exit(main())
