from .causal_lm import CausalLM, LayerCall
from .llama import build_block, build_llama, llama_layer_specs
