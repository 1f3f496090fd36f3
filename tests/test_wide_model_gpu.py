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
