"""Two layers at the widths of the Llama-3.2-1B shape (hidden 2048, 32/8 heads of
64, feed-forward 8192, vocabulary 128256, llama3 scaling factor 32): the sizes at
which the matrix-core kernels, the split-KV decode and the skinny products really
run. Whole, last tokens one by one, portions, and a mixed batch, against the
plain implementation, in float32 and bfloat16."""
import pytest
import torch

import cuttings
from engine_helpers import TOL, first_mismatch, load_runner, plain_logits, random_sequences, replay

pytestmark = pytest.mark.gpu

WIDE = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "num_hidden_layers": 2, "hidden_size": 2048, "num_attention_heads": 32,
    "num_key_value_heads": 8, "head_dim": 64, "intermediate_size": 8192, "vocab_size": 128256,
    "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 32.0, "low_freq_factor": 1.0,
                     "high_freq_factor": 4.0, "original_max_position_embeddings": 8192},
    "max_position_embeddings": 131072, "rms_norm_eps": 1e-5, "tie_word_embeddings": True,
    "torch_dtype": "bfloat16", "hidden_act": "silu",
}


@pytest.fixture(scope="module")
def wide(tmp_path_factory, gpu_device):
    from pytriton_llama_amd.weights import write_random_model
    folder = str(tmp_path_factory.mktemp("wide"))
    # std 0.03 instead of 0.02: scores then have a spread of about two, so that a key in the
    # wrong place moves the logits
    write_random_model(dict(WIDE), folder, seed=2, dtype=torch.bfloat16, std=0.03)
    seqs = random_sequences(WIDE["vocab_size"], [300, 77, 150], seed=8)
    want = plain_logits(folder, seqs)      # the file holds bfloat16 values: one plain result for both
    return folder, seqs, want


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_wide_model_all_cuttings(wide, dtype):
    folder, seqs, want = wide
    for make in (cuttings.whole, lambda s: cuttings.tail_decode(s, 32),
                 lambda s: cuttings.portions(s, (64, 2, 130, 2, 33, 7)),
                 lambda s: cuttings.mixed(s, seed=5, max_live=3)):
        steps = make(seqs)
        runner = load_runner(folder, dtype, 16, cuttings.max_live_tokens(steps) // 16)
        got = replay(runner, steps, seqs)
        bad = first_mismatch(got, want, TOL[dtype])
        assert bad is None, f"{dtype}: first wrong place (request, position, error) = {bad}"


def test_wide_model_graph_replays_of_long_portions(wide):
    """Portions of 2,048 and 1,500 tokens at the real widths, where the library picks other
    kernels than for short ones (its stream-K product among them): a step replayed as a HIP
    graph gives the logits of the same step launched kernel by kernel, on every replay, with
    eager steps and synchronisations between the replays."""
    from pytriton_llama_amd.config import build_model, read_config_json
    from pytriton_llama_amd.engine.batch import StepEntry
    from pytriton_llama_amd.engine.runner import ModelRunner
    from pytriton_llama_amd.weights import load_weights
    folder, _, _ = wide
    model = build_model(read_config_json(folder))
    load_weights(model, folder, torch.bfloat16, "cuda:0")
    pages = 2 * 2112 // 16
    eager = ModelRunner(model, 16, pages, 4)
    graphed = ModelRunner(model, 16, pages, 4, max_model_len=2112, use_graphs=True)
    g = torch.Generator().manual_seed(21)
    for i, n in enumerate([2048, 2048, 1500, 2048, 1500]):
        toks = torch.randint(0, WIDE["vocab_size"], (n + 1,), generator=g).tolist()
        got, want = [], []
        for runner, out in ((eager, want), (graphed, got)):
            assert (runner.portion_graphs is not None) == (runner is graphed)
            out.append(runner.step([StepEntry("r", toks[:n], [n - 1])]).float().cpu())
            out.append(runner.step([StepEntry("r", toks[n:], [0])]).float().cpu())   # one decoded token
            runner.end("r")
        torch.cuda.synchronize()
        for a, b in zip(got, want):
            err = float((a - b).abs().max()) / float(b.abs().max())
            assert err < 2e-2, f"replay {i} ({n} tokens): {err}"
