"""``LlamaForCausalLM``: the dense Llama decoder as a list of layer specs.

Reference: lite_llama/models/llama.py:165-226 (model), :122-162 (layer),
:10-105 (attention), :107-120 (MLP). Tensor names are the HF checkpoint's
(lite_llama/executor/weight_convert.py:193-212 lists them while renaming;
here they are read as they are).
"""
from __future__ import annotations

from typing import Any, Dict, List

from ..config.model_config import LlamaConfig
from ..config.registry import register_model
from ..parts.base import build_part
from .causal_lm import CausalLM, LayerCall

# role of a part inside a block -> its checkpoint prefix below "model.layers.{i}."
LLAMA_BLOCK_PREFIXES = {
    "input_norm": "input_layernorm.",
    "mixer": "self_attn.",
    "post_norm": "post_attention_layernorm.",
    "feed_forward": "mlp.",
}


def llama_layer_specs(cfg: LlamaConfig) -> List[Dict[str, Any]]:
    """One spec per layer: which part, by registry name, with which numbers.
    All layers of Llama are alike, but the list is what the builder reads, so
    a model whose layers differ only needs another list."""
    rs = cfg.rope_scaling
    position = ("rotary", dict(
        head_dim=cfg.head_dim, theta=cfg.rope_theta, rope_type=rs.rope_type, factor=rs.factor,
        low_freq_factor=rs.low_freq_factor, high_freq_factor=rs.high_freq_factor,
        original_max_position_embeddings=rs.original_max_position_embeddings))
    spec = {
        "block": "prenorm",
        "norm": ("rmsnorm", dict(size=cfg.hidden_size, eps=cfg.rms_norm_eps)),
        "mixer": ("paged_attention", dict(
            hidden_size=cfg.hidden_size, num_heads=cfg.num_attention_heads,
            num_kv_heads=cfg.num_key_value_heads, head_dim=cfg.head_dim)),
        "position": position,
        "feed_forward": ("swiglu", dict(hidden_size=cfg.hidden_size,
                                        intermediate_size=cfg.intermediate_size)),
    }
    return [spec for _ in range(cfg.num_hidden_layers)]


def build_block(spec: Dict[str, Any]):
    norm_name, norm_kw = spec["norm"]
    mixer_name, mixer_kw = spec["mixer"]
    ffn_name, ffn_kw = spec["feed_forward"]
    mixer_kw = dict(mixer_kw)
    if spec.get("position") is not None:
        pos_name, pos_kw = spec["position"]
        mixer_kw["position"] = build_part("position", pos_name, **pos_kw)
    return build_part(
        "block", spec["block"],
        input_norm=build_part("norm", norm_name, **norm_kw),
        mixer=build_part("mixer", mixer_name, **mixer_kw),
        post_norm=build_part("norm", norm_name, **norm_kw),
        feed_forward=build_part("feed_forward", ffn_name, **ffn_kw))


def build_llama(cfg: LlamaConfig) -> CausalLM:
    embedding = build_part("embedding", "token_embedding", vocab_size=cfg.vocab_size,
                           hidden_size=cfg.hidden_size)
    blocks = [build_block(s) for s in llama_layer_specs(cfg)]
    final_norm = build_part("norm", "rmsnorm", size=cfg.hidden_size, eps=cfg.rms_norm_eps)
    head = build_part("head", "linear_head", vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size,
                      tied_to=embedding if cfg.tie_word_embeddings else None)
    prefixes = [("model.embed_tokens.", embedding)]
    for i, b in enumerate(blocks):
        for role, part in b.children().items():
            prefixes.append((f"model.layers.{i}.{LLAMA_BLOCK_PREFIXES[role]}", part))
    prefixes += [("model.norm.", final_norm), ("lm_head.", head)]
    ignorable = ["*.rotary_emb.inv_freq"]
    if cfg.tie_word_embeddings and cfg.tie_word_embeddings_given:
        # a checkpoint that says it is tied may still carry the copy
        ignorable.append("lm_head.weight")
    cache_layers = [b.cache_spec() for b in blocks]
    schedule = [LayerCall(i, i) for i in range(len(blocks))]
    model = CausalLM(cfg, embedding, blocks, final_norm, head, cache_layers, schedule, prefixes,
                     ignorable)
    if not cfg.tie_word_embeddings_given:
        # config.json does not say: tied is the reference's default
        # (lite_llama/models/model_config.py:30), but a file that brings a head of its own is an
        # untied model, and running it with the embedding table would give wrong logits quietly
        def the_file_decides(names):
            head.tied_to = None if "lm_head.weight" in names else embedding
        model.before_load = the_file_decides
    return model


register_model("LlamaForCausalLM", LlamaConfig, build_llama, model_type="llama")
