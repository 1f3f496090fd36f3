"""Generation through the entry points: greedy against the plain implementation,
seeded temperature sampling, preemption, the command line."""
import os
import subprocess
import sys

import pytest
import torch

import plain_llama
from engine_helpers import make_folder
from tiny_configs import tiny

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def folder_a(tmp_path_factory, gpu_device):
    return make_folder(tmp_path_factory, "A", seed=21)


@pytest.fixture(scope="module")
def folder_b(tmp_path_factory, gpu_device):
    return make_folder(tmp_path_factory, "B", seed=22)


def prompts_a():
    g = torch.Generator().manual_seed(1)
    return [torch.randint(0, 256, (n,), generator=g).tolist() for n in (5, 9, 13, 17)]


def test_greedy_generation_matches_the_plain_implementation(folder_a):
    """The first tiny workload: 4 requests, prompts 5/9/13/17, 8 greedy tokens, pages of 4."""
    from pytriton_llama_amd.generate import GenerateText
    folder, page = folder_a
    cfg, w = plain_llama.read_model_folder(folder)
    prompts = prompts_a()
    want = [plain_llama.greedy_generate(cfg, w, p, 8) for p in prompts]
    gen = GenerateText(folder, max_seq_len=64, max_gpu_num_blocks=64, dtype="float32", page_size=page,
                       max_batch_size=4)
    got, _ = gen.generate(prompts, max_gen_len=8, temperature=0.0)
    assert got == want
    echoed, _ = gen.generate(prompts[:1], max_gen_len=3, temperature=0.0, echo=True)
    assert echoed[0] == prompts[0] + want[0][:3]


def test_stream_yields_the_same_tokens(folder_a):
    from pytriton_llama_amd.generate import GenerateStreamText
    folder, page = folder_a
    prompts = prompts_a()
    gen = GenerateStreamText(folder, max_seq_len=64, max_gpu_num_blocks=64, dtype="float32",
                             page_size=page, max_batch_size=4)
    whole, _ = gen.generate(prompts, 8, temperature=0.0)
    streamed = [[] for _ in prompts]
    for batch in gen.generate_stream(prompts, 8, temperature=0.0):
        for i, new in enumerate(batch):
            streamed[i].extend(new)
    assert streamed == whole


def test_preemption_does_not_change_greedy_output(folder_a):
    from pytriton_llama_amd.config import EngineConfig
    from pytriton_llama_amd.engine import Engine, SamplingParams
    folder, page = folder_a
    prompts = prompts_a()
    sp = SamplingParams(temperature=0.0, max_new_tokens=12)
    roomy = Engine(folder, EngineConfig(dtype="float32", page_size=page, num_pages=64, max_num_seqs=4,
                                        max_model_len=64))
    want = roomy.generate(prompts, sp)
    tight = Engine(folder, EngineConfig(dtype="float32", page_size=page, num_pages=14, max_num_seqs=4,
                                        max_model_len=64, max_num_batched_tokens=16, prefill_chunk=6))
    got = tight.generate(prompts, sp)
    assert tight.scheduler.num_preemptions > 0
    assert got == want
    m = tight.runner.manager
    m.check()
    assert m.paged[0].pool.num_free == 14 and m.num_free_slots == 4


def test_seeded_temperature_sampling(folder_b):
    """The second tiny workload: 3 requests, prompts 31/70/100, 12 tokens at
    temperature 0.8, pages of 16, 32-token portions. The same seed gives the same
    tokens whatever the batching; another seed gives others."""
    from pytriton_llama_amd.config import EngineConfig
    from pytriton_llama_amd.engine import Engine, SamplingParams
    folder, page = folder_b
    g = torch.Generator().manual_seed(2)
    prompts = [torch.randint(0, 384, (n,), generator=g).tolist() for n in (31, 70, 100)]
    params = [SamplingParams(temperature=0.8, top_p=0.9, max_new_tokens=12, seed=100 + i) for i in range(3)]

    def run(seed, **kw):
        eng = Engine(folder, EngineConfig(dtype="float32", page_size=page, num_pages=32, max_num_seqs=4,
                                          max_model_len=128, seed=seed, **kw))
        return eng.generate(prompts, params)

    a = run(7, prefill_chunk=32, max_num_batched_tokens=64)
    b = run(7, prefill_chunk=None, max_num_batched_tokens=512)
    c = run(8, prefill_chunk=32, max_num_batched_tokens=64)
    assert a == b
    assert a != c
    assert all(len(x) == 12 for x in a)
    # one request alone draws what it drew in the batch
    eng = Engine(folder, EngineConfig(dtype="float32", page_size=page, num_pages=32, max_num_seqs=4,
                                      max_model_len=128, seed=7))
    assert eng.generate(prompts[1:2], params[1:2])[0] == a[1]


@pytest.mark.parametrize("compiled", ["true", "false"])
def test_command_line(folder_a, compiled):
    folder, page = folder_a
    cfg, w = plain_llama.read_model_folder(folder)
    prompt = [7, 1, 30, 200, 11]
    want = plain_llama.greedy_generate(cfg, w, prompt, 5)
    out = subprocess.run(
        [sys.executable, os.path.join(ROOT, "cli.py"), "--checkpoints_dir", folder, "--dtype", "float32",
         "--temperature", "0", "--max_gen_len", "5", "--max_seq_len", "64", "--max_gpu_num_blocks", "32",
         "--page_size", str(page), "--compiled_model", compiled,
         "--prompt_ids", ",".join(map(str, prompt))],
        capture_output=True, text=True, timeout=110)
    assert out.returncode == 0, out.stderr[-2000:]
    assert [int(x) for x in out.stdout.split()] == want


def test_entry_points_replay_graphs_unless_told_otherwise(folder_a):
    from pytriton_llama_amd.cli import build_parser
    from pytriton_llama_amd.generate import GenerateText
    folder, page = folder_a
    assert build_parser().parse_args([]).compiled_model is True
    assert build_parser().parse_args(["--compiled_model", "false"]).compiled_model is False
    kw = dict(max_seq_len=64, max_gpu_num_blocks=32, dtype="float32", page_size=page, max_batch_size=2)
    assert GenerateText(folder, **kw).engine.runner.graphs is not None
    assert GenerateText(folder, compiled_model=False, **kw).engine.runner.graphs is None


def word_tokenizer(folder, vocab_size):
    """tokenizer.json with one word "w<i>" per token id, built offline."""
    from tokenizers import Tokenizer, models, pre_tokenizers
    tok = Tokenizer(models.WordLevel({f"w{i}": i for i in range(vocab_size)}, unk_token="w0"))
    tok.pre_tokenizer = pre_tokenizers.WhitespaceSplit()
    tok.save(os.path.join(folder, "tokenizer.json"))


@pytest.fixture(scope="module")
def folder_with_words(tmp_path_factory, gpu_device):
    """Tiny A with a word-level tokenizer and, as end-of-sequence token, the fourth token that
    greedy decoding of the test prompt gives: text generation must stop there."""
    import json
    folder, page = make_folder(tmp_path_factory, "A", seed=21)
    cfg, w = plain_llama.read_model_folder(folder)
    prompt = [7, 1, 30, 200, 11]
    free = plain_llama.greedy_generate(cfg, w, prompt, 8)
    stop_at = next(i for i in range(3, 8) if free[i] not in free[:i])
    cfg["eos_token_id"] = free[stop_at]
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    word_tokenizer(folder, cfg["vocab_size"])
    return folder, page, prompt, free, stop_at


def test_text_completion_matches_the_token_path(folder_with_words):
    """lite_llama/generate.py:156-177: prompts are encoded, generated from, and decoded without
    the end-of-sequence token."""
    from pytriton_llama_amd.generate import GenerateText
    folder, page, prompt, free, stop_at = folder_with_words
    gen = GenerateText(folder, max_seq_len=64, max_gpu_num_blocks=64, dtype="float32", page_size=page,
                       max_batch_size=4)
    assert gen.tokenizer is not None
    text = " ".join(f"w{t}" for t in prompt)
    other = [3, 9, 250]
    ids, _ = gen.generate([prompt, other], max_gen_len=8, temperature=0.0)
    assert ids[0] == free[:stop_at + 1]                       # stops with the end-of-sequence token
    outs = gen.text_completion([text, "w3 w9 w250"], temperature=0.0, max_gen_len=8)
    words = lambda ts: " ".join(f"w{t}" for t in ts if t != free[stop_at])
    assert [o["generation"] for o in outs] == [words(ids[0]), words(ids[1])]
    echoed = gen.text_completion([text], temperature=0.0, max_gen_len=8, echo=True)
    assert echoed[0]["generation"] == text + " " + words(ids[0])
    # a limit on new tokens ends the text earlier
    short = gen.text_completion([text], temperature=0.0, max_gen_len=2)
    assert short[0]["generation"] == words(free[:2])


def test_text_completion_stream_grows_to_the_same_text(folder_with_words):
    """lite_llama/generate_stream.py:190-216: every yield holds the text so far."""
    from pytriton_llama_amd.generate import GenerateStreamText
    folder, page, prompt, free, stop_at = folder_with_words
    gen = GenerateStreamText(folder, max_seq_len=64, max_gpu_num_blocks=64, dtype="float32",
                             page_size=page, max_batch_size=4)
    texts = [" ".join(f"w{t}" for t in prompt), "w3 w9 w250"]
    whole = gen.text_completion(texts, temperature=0.0, max_gen_len=8)
    seen = ["", ""]
    yields = 0
    for batch in gen.text_completion_stream(texts, temperature=0.0, max_gen_len=8):
        yields += 1
        for i, c in enumerate(batch):
            assert c["generation"].startswith(seen[i])
            seen[i] = c["generation"]
    assert yields >= 2 and seen == [w["generation"] for w in whole]


@pytest.mark.parametrize("stream", ["true", "false"])
def test_command_line_with_text_prompts(folder_with_words, stream):
    """cli.py --prompt (the reference's prompt loop, cli.py:40-66, fed from the command line)."""
    folder, page, prompt, free, stop_at = folder_with_words
    text = " ".join(f"w{t}" for t in prompt)
    out = subprocess.run(
        [sys.executable, os.path.join(ROOT, "cli.py"), "--checkpoints_dir", folder, "--dtype", "float32",
         "--temperature", "0", "--max_gen_len", "8", "--max_seq_len", "64", "--max_gpu_num_blocks", "32",
         "--page_size", str(page), "--stream", stream, "--prompt", text],
        capture_output=True, text=True, timeout=110)
    assert out.returncode == 0, out.stderr[-2000:]
    assert out.stdout.split() == [f"w{t}" for t in free[:stop_at]]
    # the prompt loop on standard input
    out = subprocess.run(
        [sys.executable, os.path.join(ROOT, "cli.py"), "--checkpoints_dir", folder, "--dtype", "float32",
         "--temperature", "0", "--max_gen_len", "8", "--max_seq_len", "64", "--max_gpu_num_blocks", "32",
         "--page_size", str(page)],
        input=text + "\nexit\n", capture_output=True, text=True, timeout=110)
    assert out.returncode == 0, out.stderr[-2000:]
    assert " ".join(f"w{t}" for t in free[:stop_at]) in out.stdout


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_decode_graphs_match_eager_steps(folder_b, dtype):
    """Decode-only steps replayed as HIP graphs give the logits of the same
    steps launched kernel by kernel: every replay is checked, with eager work
    (prompt portions of a newcomer, a request ending, another batch size) and
    synchronisations between the replays."""
    from pytriton_llama_amd.config import build_model, read_config_json
    from pytriton_llama_amd.engine.batch import StepEntry
    from pytriton_llama_amd.engine.runner import ModelRunner
    from pytriton_llama_amd.weights import load_weights
    folder, page = folder_b
    model = build_model(read_config_json(folder))
    load_weights(model, folder, dtype, "cuda:0")
    eager = ModelRunner(model, page, 40, 6)
    graphed = ModelRunner(model, page, 40, 6, max_model_len=200, use_graphs=True)
    assert graphed.graphs is not None and eager.graphs is None
    g = torch.Generator().manual_seed(12)
    toks = {r: torch.randint(0, 384, (160,), generator=g).tolist() for r in "abcd"}
    fed = {r: 0 for r in toks}

    def both(spec):
        entries = []
        for r, n in spec:
            entries.append(StepEntry(r, toks[r][fed[r]:fed[r] + n], [n - 1]))
            fed[r] += n
        le = eager.step(entries).float().cpu()
        lg = graphed.step(entries).float().cpu()
        scale = float(le.abs().max())
        assert float((le - lg).abs().max()) / scale < (1e-5 if dtype == torch.float32 else 2e-2)

    both([("a", 37), ("b", 5), ("c", 70)])                # prompts: eager in both runners
    replays = 0
    for i in range(40):
        both([("a", 1), ("b", 1), ("c", 1)])              # bucket of 4, three live rows
        replays += 1
        if i == 10:
            both([("d", 33), ("a", 1)])                   # mixed step between replays: eager
        if i > 10 and i % 2:
            both([("d", 1)])                              # another bucket
        if i == 25:
            for r in (eager, graphed):
                r.end("b")
            toks["b"] = toks["b"][::-1]
            fed["b"] = 0
            both([("b", 9)])                              # a new request in the freed pages
    assert graphed.graphs.buckets[4].graph is not None and graphed.graphs.buckets[1].graph is not None
    assert replays == 40


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("which", ["A", "B"])
def test_portion_graphs_match_eager_steps(folder_a, folder_b, which, dtype):
    """Steps that bring one portion of one prompt, alone or beside decoding requests, replayed
    as HIP graphs (padded to 32, 64, ... tokens and 1, 2, 4, ... decoding rows), give the
    logits of the same steps launched kernel by kernel: every replay is checked, with a prefix
    already in the cache, the wanted place last, in the middle or absent, steps of other kinds
    and a request's end between the replays, and pages that are used again."""
    from pytriton_llama_amd.config import build_model, read_config_json
    from pytriton_llama_amd.engine.batch import StepEntry
    from pytriton_llama_amd.engine.runner import ModelRunner
    from pytriton_llama_amd.weights import load_weights
    folder, page = folder_a if which == "A" else folder_b
    cfg = read_config_json(folder)
    model = build_model(cfg)
    load_weights(model, folder, dtype, "cuda:0")
    pages = -(-600 // page)                                # not many more than are held at once
    eager = ModelRunner(model, page, pages, 4)
    graphed = ModelRunner(model, page, pages, 4, max_model_len=260, use_graphs=True)
    assert graphed.portion_graphs is not None and eager.portion_graphs is None
    g = torch.Generator().manual_seed(13)
    toks = {r: torch.randint(0, model.vocab_size, (260,), generator=g).tolist() for r in "abc"}
    fed = {r: 0 for r in toks}
    # float32: the same arithmetic on both sides. bfloat16: a padded portion takes the library
    # products where the eager step of up to 16 rows takes the fused kernels, so the two differ
    # as two bfloat16 runs do (the tolerance of the engine against the plain implementation).
    tol = 1e-5 if dtype == torch.float32 else 4e-2

    def both(spec):
        entries = []
        for r, n, want in spec:
            entries.append(StepEntry(r, toks[r][fed[r]:fed[r] + n], want))
            fed[r] += n
        le = eager.step(entries).float().cpu()
        lg = graphed.step(entries).float().cpu()
        assert le.shape == lg.shape
        if le.numel():
            assert float((le - lg).abs().max()) / float(le.abs().max()) < tol

    both([("a", 2, [1])])                                   # bucket of 32
    both([("a", 31, [30])])
    both([("a", 33, [7])])                                  # bucket of 64, a place in the middle
    both([("b", 70, [])])                                   # bucket of 128, nothing wanted
    both([("b", 5, [4]), ("a", 1, [0])])                    # a decoding row beside the portion
    both([("a", 64, [63])])
    for i in range(12):                                     # the same buckets again and again
        both([("a" if i % 2 else "b", 3 + i, [2 + i])])
        if i == 5:
            both([("b", 1, [0])])                           # a decode step (its own graph)
            torch.cuda.synchronize()
    for r in (eager, graphed):
        r.end("a")
    toks["a"] = toks["a"][::-1]
    fed["a"] = 0
    both([("a", 100, [99])])                                # a new request in the freed pages
    both([("c", 40, [39])])
    both([("c", 129, [128])])                               # bucket of 256
    # decoding rows beside a portion, in any order of the entries, wanted or not
    both([("a", 1, [0]), ("c", 9, []), ("b", 1, [])])
    both([("c", 35, [0]), ("b", 1, [0]), ("a", 1, [0])])
    for i in range(4):
        both([("b", 1, [0]), ("c", 2 + i, [1 + i]), ("a", 1, [0])])
        both([("a", 1, [0]), ("b", 1, [0])])                # decode-only steps between them
    both([("a", 7, [6]), ("b", 3, [2])])                    # two portions: launched kernel by kernel
    used = graphed.portion_graphs.buckets
    assert {(0, 32), (0, 64), (0, 128), (0, 256), (1, 32), (2, 32), (2, 64)} <= set(used)
    assert all(b.graph is not None for b in used.values())


def test_warm_up_captures_the_graphs_and_changes_nothing(folder_b):
    """Engine.warm_up makes the graphs of every bucket the limits allow and gives everything
    back; generation afterwards is what it is without it."""
    from pytriton_llama_amd.config import EngineConfig
    from pytriton_llama_amd.engine import Engine, SamplingParams
    folder, page = folder_b
    g = torch.Generator().manual_seed(3)
    prompts = [torch.randint(0, 384, (n,), generator=g).tolist() for n in (20, 45, 3)]
    params = SamplingParams(temperature=0.0, max_new_tokens=6, ignore_eos=True)

    def engine():
        return Engine(folder, EngineConfig(dtype="float32", page_size=page, num_pages=24, max_num_seqs=4,
                                           max_model_len=128, max_num_batched_tokens=100))
    plain = engine().generate(prompts, params)
    eng = engine()
    free = [g.pool.num_free for g in eng.runner.manager.paged]
    eng.warm_up()
    assert [g.pool.num_free for g in eng.runner.manager.paged] == free and not eng.has_work
    assert sorted(eng.runner.portion_graphs.buckets) == [(0, 32), (0, 64)]      # 128 > the budget of 100
    assert sorted(eng.runner.graphs.buckets) == [1, 2, 4]
    assert eng.generate(prompts, params) == plain
    eng.add_request(prompts[0], params)
    with pytest.raises(RuntimeError):
        eng.warm_up()


def test_logprobs_of_generated_tokens(folder_a):
    """log_softmax of the plain logits at the tokens the engine chose."""
    from pytriton_llama_amd.generate import GenerateText
    folder, page = folder_a
    cfg, w = plain_llama.read_model_folder(folder)
    prompts = prompts_a()[:2]
    gen = GenerateText(folder, max_seq_len=64, max_gpu_num_blocks=64, dtype="float32", page_size=page,
                       max_batch_size=4)
    toks, lps = gen.generate(prompts, max_gen_len=5, temperature=0.0, logprobs=True)
    assert gen.generate(prompts, max_gen_len=5, temperature=0.0)[1] is None
    for p, t, lp in zip(prompts, toks, lps):
        assert len(lp) == len(t) == 5
        for i in range(5):
            logits = plain_llama.forward(cfg, w, list(p) + t[:i])[-1]
            want = float(torch.log_softmax(logits.double(), -1)[t[i]])
            assert abs(lp[i] - want) < 1e-4


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_steps_launched_ahead_give_the_same_tokens(folder_b, dtype):
    """With async_decode every decode step is launched before the tokens of the step before it
    have reached the host. The tokens, the log-probabilities and the finish reasons are those of
    the engine that waits for every step: greedy and seeded sampling side by side, a request that
    stops at an end-of-sequence token while the others go on, one that joins later."""
    from pytriton_llama_amd.config import EngineConfig
    from pytriton_llama_amd.engine import Engine, SamplingParams
    folder, page = folder_b
    g = torch.Generator().manual_seed(5)
    prompts = [torch.randint(0, 384, (n,), generator=g).tolist() for n in (31, 7, 50, 18)]

    def run(async_decode, eos=None):
        eng = Engine(folder, EngineConfig(dtype=dtype, page_size=page, num_pages=40, max_num_seqs=4,
                                          max_model_len=128, seed=3, async_decode=async_decode))
        if eos is not None:
            eng.scheduler.eos_token_ids = (eos,)
        params = [SamplingParams(temperature=0.0, max_new_tokens=20, logprobs=True),
                  SamplingParams(temperature=0.9, top_p=0.8, max_new_tokens=14, seed=11),
                  SamplingParams(temperature=0.0, max_new_tokens=9),
                  SamplingParams(temperature=0.7, top_p=1.0, max_new_tokens=12, seed=12, logprobs=True)]
        ids = [eng.add_request(p, sp) for p, sp in zip(prompts[:3], params[:3])]
        steps, ahead = 0, 0
        while eng.has_work:
            eng.step()
            ahead += eng._inflight is not None
            steps += 1
            if steps == 5:
                ids.append(eng.add_request(prompts[3], params[3]))
        reqs = [eng.requests[i] for i in ids]
        eng.runner.manager.check()
        assert eng.runner.manager.paged[0].pool.num_free == 40
        return [(r.output, r.finish_reason) for r in reqs], [r.output_logprobs for r in reqs], ahead

    plain_out, plain_lp, n0 = run(False)
    ahead_out, ahead_lp, n1 = run(True)
    assert n0 == 0 and n1 > 10                   # it did run ahead
    assert ahead_out == plain_out
    # (the late request joins one step later when steps run ahead, so in bfloat16 some rows
    # pass through other kernels, batched otherwise, and differ in their roundings)
    tol = 1e-5 if dtype == "float32" else 5e-2
    for a, b in zip(ahead_lp, plain_lp):
        assert len(a) == len(b)
        torch.testing.assert_close(torch.tensor(a), torch.tensor(b), atol=tol, rtol=tol)
    # an end-of-sequence token in the middle of request 0's greedy output
    eos = plain_out[0][0][6]
    cut = plain_out[0][0].index(eos) + 1
    stop_plain, _, _ = run(False, eos)
    stop_ahead, _, n2 = run(True, eos)
    assert stop_plain[0] == (plain_out[0][0][:cut], "eos")
    assert stop_ahead == stop_plain and n2 > 5


def test_random_traffic_with_and_without_steps_ahead(folder_a):
    """Forty requests of random lengths arriving at random steps, greedy and sampled, some ending
    at an end-of-sequence token, with so few pages that requests are preempted: every request
    gets the same tokens and the same finish reason whether steps are launched ahead or not and
    whether they replay graphs or not, and no page or slot is lost."""
    from pytriton_llama_amd.config import EngineConfig
    from pytriton_llama_amd.engine import Engine, SamplingParams
    import random
    folder, page = folder_a

    def run(async_decode, use_graphs=True):
        rng = random.Random(11)
        g = torch.Generator().manual_seed(12)
        eng = Engine(folder, EngineConfig(dtype="float32", page_size=page, num_pages=36, max_num_seqs=6,
                                          max_num_batched_tokens=48, prefill_chunk=16, max_model_len=72,
                                          seed=5, async_decode=async_decode, use_graphs=use_graphs))
        eng.scheduler.eos_token_ids = (7, 91, 200)
        todo, done, ahead = [], {}, 0
        for i in range(40):
            n = rng.randint(2, 30)
            sp = SamplingParams(temperature=rng.choice([0.0, 0.0, 0.8]), top_p=rng.choice([1.0, 0.9]),
                                max_new_tokens=rng.randint(1, 24), seed=1000 + i)
            todo.append((rng.randint(0, 60), torch.randint(0, 256, (n,), generator=g).tolist(), sp, i))
        todo.sort(key=lambda t: t[0])
        step = 0
        while todo or eng.has_work:
            while todo and todo[0][0] <= step:
                _, prompt, sp, i = todo.pop(0)
                eng.add_request(prompt, sp, request_id=i)
            if eng.has_work:
                eng.step()
                ahead += eng._inflight is not None
            step += 1
            assert step < 5000
        eng.runner.manager.check()
        assert eng.runner.manager.paged[0].pool.num_free == 36 and eng.runner.manager.num_free_slots == 6
        return {i: (r.output, r.finish_reason) for i, r in eng.requests.items()}, ahead, \
            eng.scheduler.num_preemptions

    plain, n0, p0 = run(False)
    fast, n1, p1 = run(True)
    assert len(plain) == 40 and n0 == 0 and n1 > 0
    assert p0 > 0 and p1 > 0                   # requests were preempted and recomputed
    assert fast == plain
    assert {r for _, r in plain.values()} >= {"length", "eos"}
    # and whether steps replay graphs (padded to buckets) or are launched kernel by kernel
    eager, _, _ = run(False, use_graphs=False)
    assert eager == plain


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_decode_graph_of_a_request_name_that_comes_again(folder_a, dtype):
    """A request ends and another one comes under the same name, as long or longer (what a
    preempted request does when it is recomputed): its pages are other ones, in another order,
    and the decode graph's copy of the block table has to follow."""
    from pytriton_llama_amd.config import build_model, read_config_json
    from pytriton_llama_amd.engine.batch import StepEntry
    from pytriton_llama_amd.engine.runner import ModelRunner
    from pytriton_llama_amd.weights import load_weights
    folder, page = folder_a
    model = build_model(read_config_json(folder))
    load_weights(model, folder, dtype, "cuda:0")
    eager = ModelRunner(model, page, 40, 4)
    graphed = ModelRunner(model, page, 40, 4, max_model_len=64, use_graphs=True)
    g = torch.Generator().manual_seed(3)
    for turn in range(5):
        n = 20 + 4 * turn
        toks = torch.randint(0, model.vocab_size, (n + 3,), generator=g).tolist()
        outs = []
        for runner in (eager, graphed):
            if turn == 2:                       # another request holds some pages meanwhile
                runner.step([StepEntry("other", toks[:9], [])])
            runner.step([StepEntry("r", toks[:n], [])])
            outs.append(torch.cat([runner.step([StepEntry("r", [t], [0])]).float().cpu()
                                   for t in toks[n:]]))
            runner.end("r")
            if turn == 3:
                runner.end("other")
            runner.manager.check()
        err = float((outs[0] - outs[1]).abs().max()) / float(outs[0].abs().max())
        assert err < (1e-5 if dtype == torch.float32 else 4e-2), f"turn {turn}: {err}"
