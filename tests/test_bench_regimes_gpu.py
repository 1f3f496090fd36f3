"""Logits against the plain implementation where the measurements run: steps with 9 to 64
decoding rows (the products change from the skinny kernel to the library's at 9 rows, the fused
decode kernels end at 16, the decode attention stops splitting once the batch fills the chip),
contexts of 2,304 and 4,640 keys (128-row query blocks, work lists shared by workgroups, eight
and more splits of a decoding row's keys), and the head sizes and head counts of the 1B, 3B
and 8B shapes at their real widths, two layers each. The head of the plain model is applied
to the wanted rows only."""
import random

import pytest
import torch

import cuttings
from engine_helpers import (TOL, first_wrong_row, load_graph_runner, load_runner, make_folder,
                            plain_rows, random_sequences, replay_wanted)
from tiny_configs import tiny

pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.bfloat16]


def many_decoders(vocab, n_short, seed, long_len=90, want_prompt_rows="all", lengths=(8, 40),
                  portion=24):
    """``n_short`` short requests whose last 5 to 9 tokens are decoded one by one (so the rows of
    a step fall by about a fifth in each of the last steps) and one long prompt that arrives in
    three or four portions beside them."""
    rng = random.Random(seed)
    lens = [rng.randint(*lengths) for _ in range(n_short)]
    seqs = random_sequences(vocab, lens + [long_len], seed=seed)
    ids = list(seqs)
    long_id = ids[-1]
    shorts = {r: seqs[r] for r in ids[:-1]}
    tails = {r: min(len(shorts[r]) - 1, 5 + i % 5) for i, r in enumerate(shorts)}
    steps = cuttings.decoders_beside_a_portion(shorts, long_id, seqs[long_id], tails, portion=portion,
                                               want_prompt_rows=want_prompt_rows)
    return seqs, steps


@pytest.fixture(scope="module")
def tiny_folders(tmp_path_factory, gpu_device):
    return {name: make_folder(tmp_path_factory, name, seed=13) for name in ("B", "C")}


@pytest.mark.parametrize("graphs", [False, True], ids=["eager", "graphs"])
@pytest.mark.parametrize("dtype", DTYPES, ids=["fp32", "bf16"])
@pytest.mark.parametrize("n_short", [12, 24, 64])
@pytest.mark.parametrize("name", ["B", "C"])
def test_many_decoding_rows_beside_a_portion(tiny_folders, name, n_short, dtype, graphs):
    """12, 24 and 64 requests decoding in one step beside a portion of another prompt, then on
    their own as they end one after the other; launched kernel by kernel and replayed as HIP
    graphs (whose padded layouts of the step are then compared with the plain model directly)."""
    folder, page = tiny_folders[name]
    vocab = tiny(name)[0]["vocab_size"]
    seqs, steps = many_decoders(vocab, n_short, seed=n_short,
                                want_prompt_rows="last" if graphs else "all")
    rows_in_a_step = max(sum(len(e["tokens"]) == 1 for e in st["entries"]) for st in steps)
    assert rows_in_a_step == n_short
    pages = cuttings.max_live_tokens(steps, round_to=page) // page
    if graphs:
        runner = load_graph_runner(folder, dtype, page, pages, max_model_len=128,
                                   max_num_seqs=n_short + 1)
    else:
        runner = load_runner(folder, dtype, page, pages, max_num_seqs=n_short + 1)
    places = cuttings.wanted_places(steps)
    want = plain_rows(folder, seqs, places, dtype)
    got = replay_wanted(runner, steps)
    bad = first_wrong_row(got, want, places, TOL[dtype])
    assert bad is None, f"config {name}, {n_short} decoding rows, {dtype}: first wrong place {bad}"
    assert all(g.pool.num_free == g.pool.num_pages for g in runner.manager.paged)
    if graphs:
        assert runner.graphs.buckets and runner.portion_graphs.buckets, "no step was replayed"


def shape_config(hidden, heads, kv_heads, head_dim, inter, vocab, factor, tied):
    return {
        "architectures": ["LlamaForCausalLM"], "model_type": "llama", "num_hidden_layers": 2,
        "hidden_size": hidden, "num_attention_heads": heads, "num_key_value_heads": kv_heads,
        "head_dim": head_dim, "intermediate_size": inter, "vocab_size": vocab,
        "rope_theta": 500000.0,
        "rope_scaling": {"rope_type": "llama3", "factor": factor, "low_freq_factor": 1.0,
                         "high_freq_factor": 4.0, "original_max_position_embeddings": 8192},
        "max_position_embeddings": 131072, "rms_norm_eps": 1e-5, "tie_word_embeddings": tied,
        "torch_dtype": "bfloat16", "hidden_act": "silu"}


# two layers of the Llama-3.2-1B, Llama-3.2-3B and Llama-3.1-8B shapes (the last two with a
# shorter vocabulary than theirs: the head at 128,256 columns is run by the 1B shape)
SHAPES = {
    "1b": shape_config(2048, 32, 8, 64, 8192, 128256, 32.0, True),
    "3b": shape_config(3072, 24, 8, 128, 8192, 20008, 32.0, True),
    "8b": shape_config(4096, 32, 8, 128, 14336, 12347, 8.0, False),
}


@pytest.fixture(scope="module")
def shape_folders(tmp_path_factory, gpu_device):
    made = {}

    def get(name):
        if name not in made:
            from pytriton_llama_amd.weights import write_random_model
            folder = str(tmp_path_factory.mktemp("shape_" + name))
            # bfloat16 values in the file: one plain result serves both engine dtypes. std 0.03:
            # scores spread over about two, so that a key in the wrong place moves the logits
            write_random_model(dict(SHAPES[name]), folder, seed=4, dtype=torch.bfloat16, std=0.03)
            made[name] = folder
        return made[name]
    return get


def long_requests_steps(seqs):
    """Request "whole": all but the last 32 tokens in one step, then one by one. Request
    "portions": 512-token portions (logits wanted at both sides of two page edges, in the
    middle and at the end of every portion), then the last 32 tokens one by one."""
    steps = []
    toks = seqs["whole"]
    head = len(toks) - 32
    steps.append({"step": 0, "entries": [{"id": "whole", "tokens": toks[:head],
                                          "want": [0, 1, 15, 16, head // 2, head - 2, head - 1]}],
                  "end": []})
    for i in range(head, len(toks)):
        steps.append({"step": len(steps), "entries": [{"id": "whole", "tokens": toks[i:i + 1], "want": [0]}],
                      "end": ["whole"] if i == len(toks) - 1 else []})
    toks = seqs["portions"]
    head = len(toks) - 32
    for lo in range(0, head, 512):
        hi = min(head, lo + 512)
        n = hi - lo
        steps.append({"step": len(steps), "entries": [{"id": "portions", "tokens": toks[lo:hi],
                                                       "want": [0, 15, 16, n // 2, n - 1]}], "end": []})
    for i in range(head, len(toks)):
        steps.append({"step": len(steps), "entries": [{"id": "portions", "tokens": toks[i:i + 1], "want": [0]}],
                      "end": ["portions"] if i == len(toks) - 1 else []})
    return steps


@pytest.fixture(scope="module")
def long_cases(shape_folders):
    cache = {}

    def get(name):
        if name not in cache:
            folder = shape_folders(name)
            seqs = random_sequences(SHAPES[name]["vocab_size"], [2304, 4640], seed=31)
            seqs = {"whole": seqs["r0"], "portions": seqs["r1"]}
            steps = long_requests_steps(seqs)
            places = cuttings.wanted_places(steps)
            cache[name] = (folder, seqs, steps, places, plain_rows(folder, seqs, places))
        return cache[name]
    return get


@pytest.mark.parametrize("graphs", [False, True], ids=["eager", "graphs"])
@pytest.mark.parametrize("dtype", DTYPES, ids=["fp32", "bf16"])
@pytest.mark.parametrize("name", ["1b", "3b", "8b"])
def test_long_contexts_at_real_widths(long_cases, name, dtype, graphs):
    """2,304 tokens (2,272 at once, 32 decoded) and 4,640 tokens (nine portions of 512, 32
    decoded) through two layers of each shape, launched kernel by kernel and with the portions
    and the decoded tokens replayed as HIP graphs (planned for the longest request)."""
    folder, seqs, steps, places, want = long_cases(name)
    pages = (2304 + 4640) // 16 + 2
    if graphs:
        runner = load_graph_runner(folder, dtype, 16, pages, max_model_len=4640, max_num_seqs=2)
    else:
        runner = load_runner(folder, dtype, 16, pages, max_num_seqs=2)
    got = replay_wanted(runner, steps)
    bad = first_wrong_row(got, want, places, TOL[dtype])
    assert bad is None, f"shape {name}, {dtype}: first wrong place (request, position, error) = {bad}"


@pytest.mark.parametrize("graphs", [False, True], ids=["eager", "graphs"])
@pytest.mark.parametrize("dtype", DTYPES, ids=["fp32", "bf16"])
@pytest.mark.parametrize("name", ["1b", "3b", "8b"])
def test_many_decoding_rows_at_real_widths(shape_folders, name, dtype, graphs):
    """64 requests of 20 to 120 tokens decoding together at the real widths (with eight kv heads
    the decode attention runs without splits from 32 rows on), beside a prompt of 300 tokens in
    portions of 100; the rows fall to 9 and below as the requests end. At the 8B widths the
    fused decode products run over 4,096 and 14,336 columns."""
    folder = shape_folders(name)
    seqs, steps = many_decoders(SHAPES[name]["vocab_size"], 64, seed=7, long_len=300,
                                want_prompt_rows="last", lengths=(20, 120), portion=100)
    counts = {sum(len(e["tokens"]) == 1 for e in st["entries"]) for st in steps}
    assert 64 in counts and any(17 <= c < 64 for c in counts) and any(9 <= c <= 16 for c in counts)
    pages = cuttings.max_live_tokens(steps, round_to=16) // 16
    if graphs:
        runner = load_graph_runner(folder, dtype, 16, pages, max_model_len=320, max_num_seqs=65)
    else:
        runner = load_runner(folder, dtype, 16, pages, max_num_seqs=65)
    places = cuttings.wanted_places(steps)
    want = plain_rows(folder, seqs, places)
    got = replay_wanted(runner, steps)
    bad = first_wrong_row(got, want, places, TOL[dtype])
    assert bad is None, f"shape {name}, {dtype}: first wrong place (request, position, error) = {bad}"


def test_recorded_steps_without_timed_products_give_the_same_bits_twice(shape_folders):
    """Two runners made one after the other with ``timed_library_products`` off replay the same
    steps (64 decoding rows beside portions, where the products are the library's) to logits
    that are equal bit for bit: every product runs the library's first proposal, whatever a
    runner before them has timed. With the timing on the same steps stay within the tolerance
    of the plain model (the tests above) but need not give the same bits in another process."""
    folder = shape_folders("1b")
    seqs, steps = many_decoders(SHAPES["1b"]["vocab_size"], 64, seed=9, long_len=200,
                                want_prompt_rows="last", lengths=(20, 60), portion=100)
    pages = cuttings.max_live_tokens(steps, round_to=16) // 16
    # a runner that times the shapes of its recorded steps comes first
    replay_wanted(load_graph_runner(folder, torch.bfloat16, 16, pages, max_model_len=320, max_num_seqs=65),
                  steps)
    got = []
    for _ in range(2):
        runner = load_graph_runner(folder, torch.bfloat16, 16, pages, max_model_len=320, max_num_seqs=65,
                                   timed_library_products=False)
        got.append(replay_wanted(runner, steps))
        assert runner.graphs.buckets and runner.portion_graphs.buckets, "no step was replayed"
        del runner
    for rid in got[0]:
        assert torch.equal(got[0][rid], got[1][rid]), f"request {rid}: the two runs differ"


@pytest.fixture(scope="module")
def full_depth(tmp_path_factory, gpu_device):
    """All sixteen layers of the 1B shape, as the measurements run it."""
    from pytriton_llama_amd.weights import write_random_model
    cfg = dict(SHAPES["1b"], num_hidden_layers=16)
    folder = str(tmp_path_factory.mktemp("full_depth"))
    write_random_model(cfg, folder, seed=6, dtype=torch.bfloat16, std=0.02)
    seqs = random_sequences(cfg["vocab_size"], [260, 45, 150], seed=12)
    steps = cuttings.mixed(seqs, seed=2, max_live=3)
    for st in steps:                       # the last row of every entry is enough here
        for e in st["entries"]:
            e["want"] = e["want"][-1:]
    places = cuttings.wanted_places(steps)
    return folder, seqs, steps, places, plain_rows(folder, seqs, places)


@pytest.mark.parametrize("dtype", DTYPES, ids=["fp32", "bf16"])
def test_sixteen_layers_mixed(full_depth, dtype):
    """The whole depth of the 1B shape (weights N(0, 0.02) as in the measurements): portions of
    three prompts beside decoded tokens, against the plain model."""
    folder, seqs, steps, places, want = full_depth
    runner = load_runner(folder, dtype, 16, cuttings.max_live_tokens(steps) // 16, max_num_seqs=4)
    got = replay_wanted(runner, steps)
    bad = first_wrong_row(got, want, places, TOL[dtype])
    assert bad is None, f"16 layers, {dtype}: first wrong place (request, position, error) = {bad}"
