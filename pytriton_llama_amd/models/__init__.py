from .causal_lm import CausalLM, LayerCall
from .llama import build_block, build_llama, llama_layer_specs
from .rubasun import build_rubasun
from .virusun import build_virusun
from .matusun import build_matusun
from .senavik import build_senavik
