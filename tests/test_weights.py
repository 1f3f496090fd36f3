"""The safetensors loader's errors and the random-weights mode (CPU)."""
import copy
import json
import os

import pytest
import torch
from safetensors.torch import load_file, save_file

import pytriton_llama_amd  # noqa: F401
from pytriton_llama_amd.config import build_model
from pytriton_llama_amd.weights import WeightError, load_weights, write_random_model
from tiny_configs import TINY_A, TINY_B


@pytest.fixture()
def folder(tmp_path):
    return write_random_model(copy.deepcopy(TINY_B), str(tmp_path / "m"), seed=4,
                              dtype=torch.float32, norm_std=0.1)


def rewrite(folder, fn):
    path = os.path.join(folder, "model.safetensors")
    t = load_file(path)
    fn(t)
    save_file(t, path)


def test_written_folder_reads_back(folder):
    m = build_model(TINY_B)
    load_weights(m, folder, torch.float32, "cpu")
    t = load_file(os.path.join(folder, "model.safetensors"))
    att = m.blocks[1].mixer
    want = torch.cat([t[f"model.layers.1.self_attn.{n}_proj.weight"] for n in "qkv"])
    assert torch.equal(att.qkv, want) and att.qkv.dtype == torch.float32
    assert torch.equal(m.blocks[0].feed_forward.gate_up[:320], t["model.layers.0.mlp.gate_proj.weight"])
    assert torch.equal(m.head.weight, t["lm_head.weight"])
    assert not torch.equal(m.blocks[0].input_norm.weight, torch.ones(128))    # 1 + N(0, 0.1)


def test_dtypes_as_held(folder):
    m = build_model(TINY_B)
    load_weights(m, folder, torch.bfloat16, "cpu")
    assert m.embedding.weight.dtype == torch.bfloat16 and m.blocks[0].mixer.o.dtype == torch.bfloat16
    # a vector stays in 32 bit
    assert m.final_norm.weight.dtype == torch.float32
    t = load_file(os.path.join(folder, "model.safetensors"))
    assert torch.equal(m.final_norm.weight, t["model.norm.weight"])
    assert torch.equal(m.embedding.weight, t["model.embed_tokens.weight"].to(torch.bfloat16))


def test_one_error_lists_everything(folder):
    def damage(t):
        del t["model.layers.0.mlp.up_proj.weight"]
        del t["model.norm.weight"]
        t["model.layers.7.extra.weight"] = torch.zeros(2)
        t["model.layers.2.self_attn.k_proj.weight"] = torch.zeros(32, 127)
        t["lm_head.weight"] = t["lm_head.weight"].t().contiguous()
    rewrite(folder, damage)
    with pytest.raises(WeightError) as ei:
        load_weights(build_model(TINY_B), folder, torch.float32, "cpu")
    e = ei.value
    assert e.missing == ["model.layers.0.mlp.up_proj.weight", "model.norm.weight"]
    assert e.unexpected == ["model.layers.7.extra.weight"]
    assert sorted(n for n, _, _ in e.wrong_shape) == ["lm_head.weight",
                                                       "model.layers.2.self_attn.k_proj.weight"]
    msg = str(e)
    for word in ("up_proj", "model.norm.weight", "extra", "[32, 127]", "[32, 128]"):
        assert word in msg


def test_tied_checkpoint(tmp_path):
    f = write_random_model(copy.deepcopy(TINY_A), str(tmp_path / "a"), seed=1)
    assert "lm_head.weight" not in load_file(os.path.join(f, "model.safetensors"))
    m = build_model(TINY_A)
    load_weights(m, f, torch.float32, "cpu")
    assert m.head.weight is m.embedding.weight
    # a tied checkpoint that still carries the copy, and rotary buffers, load too
    rewrite(f, lambda t: t.update({"lm_head.weight": t["model.embed_tokens.weight"].clone(),
                                   "model.layers.0.self_attn.rotary_emb.inv_freq": torch.zeros(4)}))
    load_weights(build_model(TINY_A), f, torch.float32, "cpu")
    # untied without a head is an error
    d = copy.deepcopy(TINY_A)
    d["tie_word_embeddings"] = False
    rewrite(f, lambda t: t.pop("lm_head.weight"))
    with pytest.raises(WeightError, match="lm_head.weight"):
        load_weights(build_model(d), f, torch.float32, "cpu")


def test_no_tensor_file(tmp_path):
    (tmp_path / "config.json").write_text(json.dumps(TINY_A))
    with pytest.raises(WeightError, match="model.safetensors"):
        load_weights(build_model(TINY_A), str(tmp_path), torch.float32, "cpu")


def test_sharded_folder(folder):
    path = os.path.join(folder, "model.safetensors")
    t = load_file(path)
    names = sorted(t)
    a, b = names[: len(names) // 2], names[len(names) // 2:]
    save_file({n: t[n] for n in a}, os.path.join(folder, "model-00001-of-00002.safetensors"))
    save_file({n: t[n] for n in b}, os.path.join(folder, "model-00002-of-00002.safetensors"))
    os.remove(path)
    wm = {n: "model-00001-of-00002.safetensors" for n in a}
    wm.update({n: "model-00002-of-00002.safetensors" for n in b})
    with open(os.path.join(folder, "model.safetensors.index.json"), "w") as f:
        json.dump({"weight_map": wm}, f)
    m = build_model(TINY_B)
    load_weights(m, folder, torch.float32, "cpu")
    assert torch.equal(m.head.weight, t["lm_head.weight"])
    os.remove(os.path.join(folder, "model-00002-of-00002.safetensors"))
    with pytest.raises(WeightError, match="absent"):
        load_weights(build_model(TINY_B), folder, torch.float32, "cpu")


def test_random_weights_depend_on_seed_and_name_only(tmp_path):
    f1 = write_random_model(copy.deepcopy(TINY_A), str(tmp_path / "1"), seed=7, dtype=torch.float32)
    f2 = write_random_model(copy.deepcopy(TINY_A), str(tmp_path / "2"), seed=7, dtype=torch.bfloat16)
    f3 = write_random_model(copy.deepcopy(TINY_A), str(tmp_path / "3"), seed=8, dtype=torch.float32)
    t1, t2, t3 = (load_file(os.path.join(f, "model.safetensors")) for f in (f1, f2, f3))
    for n in t1:
        assert torch.equal(t1[n].to(torch.bfloat16), t2[n])
    w = t1["model.layers.0.mlp.gate_proj.weight"]
    assert not torch.equal(w, t3["model.layers.0.mlp.gate_proj.weight"])
    assert abs(float(w.std()) - 0.02) < 0.002 and torch.all(t1["model.norm.weight"] == 1)
    # a model with more layers has the same first layers
    d = copy.deepcopy(TINY_A)
    d["num_hidden_layers"] = 3
    t4 = load_file(os.path.join(write_random_model(d, str(tmp_path / "4"), seed=7, dtype=torch.float32),
                                "model.safetensors"))
    assert torch.equal(t4["model.layers.1.self_attn.q_proj.weight"],
                       t1["model.layers.1.self_attn.q_proj.weight"])
    assert json.load(open(os.path.join(f1, "config.json")))["hidden_size"] == 64


def test_init_hints_of_a_part_go_before_the_rule_of_the_kind():
    """A part may say how its tensors are drawn in the random-weights mode (biases, decay rates,
    gates are no norm weights); a hint nobody knows is an error."""
    from pytriton_llama_amd.weights.random_init import random_tensor
    d = random_tensor(3, "x.decay", (4000,), "vector", 0.02, 0.1, init=("uniform", 0.5, 0.9))
    assert d.dtype == torch.float32 and 0.5 <= float(d.min()) and float(d.max()) <= 0.9
    assert abs(float(d.mean()) - 0.7) < 0.01
    b = random_tensor(3, "x.bias", (4000,), "vector", 0.02, 0.1, init=("normal", 0.0, 0.3))
    assert abs(float(b.mean())) < 0.03 and abs(float(b.std()) - 0.3) < 0.02
    c = random_tensor(3, "x.gate", (5, 7), "matrix", 0.02, 0.1, init=("constant", -2.5))
    assert c.shape == (5, 7) and bool((c == -2.5).all())
    assert torch.equal(d, random_tensor(3, "x.decay", (4000,), "vector", 0.5, 0.0, init=("uniform", 0.5, 0.9)))
    n = random_tensor(3, "x.norm", (4000,), "vector", 0.02, 0.1)            # no hint: a norm weight
    assert abs(float(n.mean()) - 1.0) < 0.01
    with pytest.raises(ValueError, match="unknown init hint"):
        random_tensor(3, "x", (4,), "vector", 0.02, 0.1, init=("xavier",))
    # through a model: the toy mixer's decay rates and bias in a written folder
    import toy_parts  # noqa: F401
    from pytriton_llama_amd.config import build_model
    from pytriton_llama_amd.weights.random_init import random_tensors
    model = build_model({"architectures": ["ToyStateLM"], "vocab_size": 30, "hidden_size": 16, "inner": 24,
                         "layers": ["state_on_device"], "toy_norm": False, "toy_ffn": True})
    drawn = {name: t for name, _, _, t in random_tensors(model, 1, norm_std=0.1)}
    assert 0.5 <= float(drawn["l0.mixer.decay"].min()) and float(drawn["l0.mixer.decay"].max()) <= 0.9
    assert abs(float(drawn["l0.mixer.bias"].mean())) < 0.1
    assert abs(float(drawn["l0.input_norm.weight"].mean()) - 1.0) < 0.1


def test_without_the_key_the_file_decides_whether_the_head_is_tied(tmp_path):
    """config.json without tie_word_embeddings means tied (the reference's default) unless the
    file brings lm_head.weight: then that is the head, never the embedding table in its place."""
    import json
    from tiny_configs import tiny
    from pytriton_llama_amd.config import build_model, read_config_json
    from pytriton_llama_amd.weights import WeightError, load_weights, write_random_model
    cfg = tiny("A")[0]
    cfg["tie_word_embeddings"] = False
    write_random_model(cfg, str(tmp_path), seed=1, dtype=torch.float32)
    del cfg["tie_word_embeddings"]
    with open(tmp_path / "config.json", "w") as f:
        json.dump(cfg, f)
    from safetensors.torch import load_file, save_file
    tensors = load_file(str(tmp_path / "model.safetensors"))
    model = build_model(read_config_json(str(tmp_path)))
    load_weights(model, str(tmp_path), torch.float32, "cpu")
    assert model.head.tied_to is None and torch.equal(model.head.weight, tensors["lm_head.weight"])
    assert not torch.equal(model.head.weight, model.embedding.weight)
    # the same folder without the head: tied
    head = tensors.pop("lm_head.weight")
    save_file(tensors, str(tmp_path / "model.safetensors"))
    model = build_model(read_config_json(str(tmp_path)))
    load_weights(model, str(tmp_path), torch.float32, "cpu")
    assert model.head.weight is model.embedding.weight
    # config.json says untied and the head is absent: an error that names it
    cfg["tie_word_embeddings"] = False
    with open(tmp_path / "config.json", "w") as f:
        json.dump(cfg, f)
    with pytest.raises(WeightError) as e:
        load_weights(build_model(read_config_json(str(tmp_path))), str(tmp_path), torch.float32, "cpu")
    assert e.value.missing == ["lm_head.weight"]
    tensors["lm_head.weight"] = head
    save_file(tensors, str(tmp_path / "model.safetensors"))
    # said in so many words, a tied checkpoint may carry the copy
    cfg["tie_word_embeddings"] = True
    with open(tmp_path / "config.json", "w") as f:
        json.dump(cfg, f)
    load_weights(build_model(read_config_json(str(tmp_path))), str(tmp_path), torch.float32, "cpu")
