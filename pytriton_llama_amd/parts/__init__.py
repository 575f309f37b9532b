from .base import (PART_KINDS, PART_REGISTRY, PagedSpec, PagedTensor, ParamSource, Part, StateSpec, WorkList,
                   build_part, paged_kv_spec,
                   place, register_part)
from .linear import linear
from .norm import DynamicTanh, RMSNorm
from .rotary import RotaryEncoding, banded_inv_freq, default_inv_freq, llama3_inv_freq, ramp_inv_freq
from .attention import PagedAttention
from .feedforward import GatedMLP, PlainMLP, RoutedExperts, SwiGLU
from .latent_attention import LatentAttention
from .token_input import GatedTokenInput, TokenTable
from .embedding import LinearHead, TokenEmbedding
from .normed_attention import NormedAttention
from .recurrent import GatedDeltaRule, MatrixMemory, ParallelMixers, SelectiveScan
from .block import HyperConnectionBlock, OutputNormBlock, PreNormBlock, SandwichBlock
