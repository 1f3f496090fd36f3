"""The engine against the plain implementation under every way of cutting the
work, in float32 and in bfloat16, for three tiny configurations and for some drawn at random."""
import pytest
import torch

import cuttings
from engine_helpers import (TOL, first_mismatch, load_runner, make_folder, plain_logits,
                            random_sequences, replay)
from tiny_configs import tiny

pytestmark = pytest.mark.gpu

LENGTHS = {"A": [5, 9, 13, 17, 70, 41], "B": [31, 70, 100, 45, 64, 129], "C": [33, 80, 16, 97, 50]}
DTYPES = [torch.float32, torch.bfloat16]


@pytest.fixture(scope="module")
def cases(tmp_path_factory, gpu_device):
    out = {}
    for name in ("A", "B", "C"):
        folder, page = make_folder(tmp_path_factory, name, seed=11)
        cfg = tiny(name)[0]
        seqs = random_sequences(cfg["vocab_size"], LENGTHS[name], seed=5)
        want = {torch.float32: plain_logits(folder, seqs),
                torch.bfloat16: plain_logits(folder, seqs, torch.bfloat16)}
        out[name] = (folder, page, seqs, want)
    return out


def run_cutting(cases, name, dtype, steps, num_pages=None):
    folder, page, seqs, want = cases[name]
    if num_pages is None:
        num_pages = -(-cuttings.max_live_tokens(steps) // page)
    runner = load_runner(folder, dtype, page, num_pages)
    got = replay(runner, steps, seqs)
    bad = first_mismatch(got, want[dtype], TOL[dtype])
    assert bad is None, f"config {name} {dtype}: first wrong place (request, position, error) = {bad}"
    assert all(g.pool.num_free == g.pool.num_pages for g in runner.manager.paged)


@pytest.mark.parametrize("dtype", DTYPES, ids=["fp32", "bf16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_whole(cases, name, dtype):
    run_cutting(cases, name, dtype, cuttings.whole(cases[name][2]))


@pytest.mark.parametrize("dtype", DTYPES, ids=["fp32", "bf16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_last_tokens_one_by_one(cases, name, dtype):
    run_cutting(cases, name, dtype, cuttings.tail_decode(cases[name][2], 32))


@pytest.mark.parametrize("dtype", DTYPES, ids=["fp32", "bf16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_portions_of_changing_size(cases, name, dtype):
    run_cutting(cases, name, dtype, cuttings.portions(cases[name][2]))


@pytest.mark.parametrize("dtype", DTYPES, ids=["fp32", "bf16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_mixed_with_page_reuse(cases, name, dtype):
    seqs = cases[name][2]
    steps = cuttings.mixed(seqs, seed=3, max_live=4)
    page = cases[name][1]
    need = cuttings.max_live_tokens(steps, round_to=page) // page
    total = sum(-(-len(t) // page) for t in seqs.values())
    assert need < total, "the pool must be too small to hold all requests at once"
    run_cutting(cases, name, dtype, steps, need)


@pytest.mark.parametrize("dtype", DTYPES, ids=["fp32", "bf16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_cuttings_replayed_as_graphs(cases, name, dtype):
    """The same cuttings with decode steps and single portions replayed as HIP graphs (their
    padded layouts of a step against the plain model, not against the eager layout): the last
    tokens one by one, portions of changing size, and the mixed trace. A replayed portion has
    one wanted place, so only the last row of every entry is asked for."""
    from engine_helpers import first_wrong_row, load_graph_runner, plain_rows, replay_wanted
    folder, page, seqs, _ = cases[name]
    for steps in (cuttings.tail_decode(seqs, 32), cuttings.portions(seqs), cuttings.mixed(seqs, seed=3)):
        for st in steps:
            for e in st["entries"]:
                e["want"] = e["want"][-1:]
        places = cuttings.wanted_places(steps)
        want = plain_rows(folder, seqs, places, dtype)
        runner = load_graph_runner(folder, dtype, page, -(-cuttings.max_live_tokens(steps) // page),
                                   max_model_len=160, max_num_seqs=4)
        got = replay_wanted(runner, steps)
        bad = first_wrong_row(got, want, places, TOL[dtype])
        assert bad is None, f"config {name} {dtype}: first wrong place (request, position, error) = {bad}"
        assert runner.graphs.buckets and runner.portion_graphs.buckets


@pytest.mark.parametrize("dtype", DTYPES, ids=["fp32", "bf16"])
def test_a_replayed_portion_gives_the_logits_of_any_one_of_its_rows(cases, dtype):
    """A replayed step with a portion computes the logits of one row of the portion: the row the
    entry names, not only its last (first, a middle and the last row of portions of changing
    size, alone and beside decoded tokens of another request), against the plain model."""
    from engine_helpers import first_wrong_row, load_graph_runner, plain_rows, replay_wanted
    folder, page, seqs, _ = cases["B"]
    again = {r + "_again": t for r, t in seqs.items()}        # the same requests under other names
    steps = cuttings.mixed(seqs, seed=11, max_live=3) + cuttings.portions(again, sizes=(9, 40, 2, 17))
    for i, st in enumerate(steps):
        st["step"] = i
        for j, e in enumerate(st["entries"]):
            n = len(e["tokens"])
            e["want"] = [(0, n // 2, n - 1)[(i + j) % 3]] if n > 1 else [0]
    assert any(e["want"] == [0] and len(e["tokens"]) > 2 for st in steps for e in st["entries"])
    both = dict(seqs, **again)
    places = cuttings.wanted_places(steps)
    want = plain_rows(folder, both, places, dtype)
    runner = load_graph_runner(folder, dtype, page, -(-cuttings.max_live_tokens(steps) // page),
                               max_model_len=160, max_num_seqs=4)
    got = replay_wanted(runner, steps)
    bad = first_wrong_row(got, want, places, TOL[dtype])
    assert bad is None, f"{dtype}: first wrong place (request, position, error) = {bad}"
    assert runner.portion_graphs.buckets


@pytest.mark.parametrize("dtype", DTYPES, ids=["fp32", "bf16"])
def test_first_tokens_of_a_sequence(cases, dtype):
    """Positions 0, 1, 2: one token whole, then one by one from an empty cache."""
    folder, page, seqs, want = cases["B"]
    toks = seqs["r0"][:3]
    runner = load_runner(folder, dtype, page, 4)
    from pytriton_llama_amd.engine.batch import StepEntry
    got = []
    for i, t in enumerate(toks):
        got.append(runner.step([StepEntry("x", [t], [0])]).float().cpu()[0])
    runner.end("x")
    ref = want[dtype]["r0"][:3]
    scale = float(ref.abs().max())
    err = (torch.stack(got) - ref).abs().max() / scale
    assert err < TOL[dtype], err
    # the very first token attends only itself
    one = runner.step([StepEntry("y", toks[:1], [0])]).float().cpu()[0]
    assert (one - ref[0]).abs().max() / scale < TOL[dtype]


@pytest.mark.parametrize("dtype", DTYPES, ids=["fp32", "bf16"])
def test_long_decoding(cases, dtype):
    """A short prompt and then 300 tokens one by one across many pages."""
    folder, page, _, _ = cases["A"]
    cfg = tiny("A")[0]
    seqs = random_sequences(cfg["vocab_size"], [308], seed=9)
    want = plain_logits(folder, seqs, dtype)
    steps = cuttings.tail_decode(seqs, tail=300)
    runner = load_runner(folder, dtype, page, -(-320 // page))
    got = replay(runner, steps, seqs)
    bad = first_mismatch(got, want, TOL[dtype])
    assert bad is None, bad


def _drawn_configuration(rng):
    """A Llama configuration with every size drawn: head sizes in steps of 16 up to 256, any
    number of kv heads and of query heads a kv head, widths, feed-forward sizes and
    vocabularies that are no power of two (some no multiple of 8, which the bfloat16 matrix
    kernels refuse and the general ones take), both spellings of the scaling's type key."""
    kv_heads = rng.choice([1, 2, 3, 5])
    scaling = None
    if rng.random() < 0.6:
        scaling = {rng.choice(["rope_type", "type"]): "llama3", "factor": rng.choice([2.0, 8.0, 32.0]),
                   "low_freq_factor": 1.0, "high_freq_factor": rng.choice([2.0, 4.0]),
                   "original_max_position_embeddings": rng.choice([32, 64, 256])}
    return {"architectures": ["LlamaForCausalLM"], "model_type": "llama",
            "num_hidden_layers": rng.randint(1, 3),
            "hidden_size": rng.choice([8 * rng.randint(4, 40), 2 * rng.randint(17, 99)]),
            "num_attention_heads": kv_heads * rng.choice([1, 2, 3, 4, 6, 7, 8, 16]),
            "num_key_value_heads": kv_heads,
            "head_dim": rng.choice([16, 32, 48, 64, 80, 96, 112, 128, 160, 192, 256]),
            "intermediate_size": rng.choice([8 * rng.randint(5, 60), 2 * rng.randint(21, 150)]),
            "vocab_size": rng.choice([rng.randint(100, 2000), rng.randint(2000, 40000) | 1]),
            "rope_theta": rng.choice([1e3, 1e4, 5e5]), "rope_scaling": scaling,
            "rms_norm_eps": rng.choice([1e-3, 1e-5, 1e-6]), "tie_word_embeddings": rng.random() < 0.5,
            "torch_dtype": "float32", "hidden_act": "silu", "max_position_embeddings": 4096}


@pytest.mark.parametrize("seed", [1, 3, 10, 17, 33, 40, 48, 58])
def test_drawn_configurations_mixed_with_page_reuse(tmp_path, gpu_device, seed):
    """Configurations drawn at random (sizes, options, page size), five requests of 2 to 420
    tokens in a mixed batch with so few pages that they are used again, in both dtypes."""
    import random
    from pytriton_llama_amd.weights import write_random_model
    rng = random.Random(seed)
    cfg = _drawn_configuration(rng)
    page = rng.choice([4, 8, 16, 32, 64])
    lengths = [rng.randint(2, 40), rng.randint(40, 140), rng.randint(140, 420), rng.randint(3, 90),
               rng.randint(60, 300)]
    folder = str(tmp_path)
    write_random_model(cfg, folder, seed=seed, dtype=torch.float32, norm_std=0.1,
                       std=0.8 / cfg["hidden_size"] ** 0.5)
    seqs = random_sequences(cfg["vocab_size"], lengths, seed=seed)
    steps = cuttings.mixed(seqs, seed=seed, max_live=rng.choice([2, 3, 4]))
    pages = cuttings.max_live_tokens(steps, round_to=max(64, page)) // page
    for dtype in DTYPES:
        want = plain_logits(folder, seqs, dtype)
        got = replay(load_runner(folder, dtype, page, pages, max_num_seqs=4), steps, seqs)
        bad = first_mismatch(got, want, TOL[dtype])
        assert bad is None, f"{cfg}, page size {page}, {dtype}: first wrong place {bad}"
