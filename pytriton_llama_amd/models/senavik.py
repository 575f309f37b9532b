"""``Senavik``: pre-norm layers given as a list, each with one of two mixers (grouped-query
attention inside a sliding window that also keeps a sequence's first tokens, rotated with
frequencies rescaled by wavelength band; attention over a latent that all heads share, with the
queries through a latent of their own and a rotated part whose frequencies follow a ramp), a
learned term a head in every softmax denominator, a dense (squared-ReLU) or routed (sigmoid
scores, a correction for the choice, groups of experts) feed-forward or none, norms whose
weights are stored around zero, a norm behind the embedding and a head matrix of its own. The
residual stream is float32. The model is a list of layer specs over the engine's parts; tensor
names are the checkpoint's own ("embed", "embed.norm", "l<i>.mix.q", "l<i>.mix.sink",
"l<i>.mlp.e0.gate", "l<i>.norm1", "final.norm", "head").
"""
from __future__ import annotations

from ..config.registry import register_model
from ..config.senavik_config import SenavikConfig
from ..parts.base import build_part
from .causal_lm import CausalLM, LayerCall

# role of a part inside a block -> what follows "l<i>." in its tensors' names
SENAVIK_BLOCK_PREFIXES = {"norm1": "norm1", "norm2": "norm2", "mixer": "mix.", "feed_forward": "mlp."}


def _norm(cfg: SenavikConfig):
    """x / rms(x) * (1 + w): the checkpoint holds w."""
    return build_part("norm", "rmsnorm", size=cfg.hidden_size, eps=cfg.norm_eps, weight_name="", offset=1.0)


def _mixer(cfg: SenavikConfig, layer):
    W, m = cfg.hidden_size, layer.mixer
    if layer.kind == "attention":
        return build_part("mixer", "normed_attention", hidden_size=W, num_heads=m.heads, num_kv_heads=m.kv_heads,
                          dim=m.dim, vdim=m.vdim, scale=m.scale, eps=cfg.norm_eps, qk_norm=None, maps=1,
                          bias=False, gated=False, rot_dims=m.rot_dims, rot_base=m.rot_base,
                          rot_scaling=m.rot_scaling, window=m.window, keep_first=m.keep_first if m.window else 0,
                          sink_name="sink")
    return build_part("mixer", "latent_attention", hidden_size=W, num_heads=m.heads, dim=m.dim, rot_dim=m.rot_dim,
                      vdim=m.vdim, kv_rank=m.kv_rank, scale=m.scale, rot_base=m.rot_base, rot_dims=m.rot_dims,
                      eps=cfg.norm_eps, gated=False, q_rank=m.q_rank, rot_layout="half",
                      rot_scaling=m.rot_scaling, sink_name="sink")


def _feed_forward(cfg: SenavikConfig, mlp):
    if mlp is None:
        return None
    W = cfg.hidden_size
    if mlp.kind == "dense":
        return build_part("feed_forward", "mlp", hidden_size=W, intermediate_size=mlp.ff, activation="relu2")
    return build_part("feed_forward", "routed_experts", hidden_size=W, intermediate_size=mlp.ff,
                      num_experts=mlp.experts, top=mlp.top, activation="silu", weight_on_input=False,
                      renormalize=True, renorm_eps=1e-20, score="sigmoid", correction_name="correction",
                      groups=(mlp.groups, mlp.keep_groups), shared=None, shared_gate=False)


def build_senavik(cfg: SenavikConfig) -> CausalLM:
    W = cfg.hidden_size
    embedding = build_part("embedding", "token_embedding", vocab_size=cfg.vocab_size, hidden_size=W,
                           weight_name="embed", float32_stream=True, norm=_norm(cfg))
    blocks = []
    for layer in cfg.layers:
        ffn = _feed_forward(cfg, layer.mlp)
        # one float32 stream with a plain residual sum: the hyper-connection block without coefficients
        blocks.append(build_part("block", "hyper_connections", hidden_size=W, streams=1, mixer=_mixer(cfg, layer),
                                 mixer_norm=_norm(cfg), feed_forward=ffn,
                                 ffn_norm=_norm(cfg) if ffn is not None else None, learned=False))
    cache_layers = [b.cache_spec() for b in blocks]
    schedule = [LayerCall(i, i, True) for i in range(len(blocks))]
    final_norm = _norm(cfg)
    head = build_part("head", "linear_head", vocab_size=cfg.vocab_size, hidden_size=W, weight_name="head")
    prefixes = [("", embedding)]
    for i, b in enumerate(blocks):
        for role, part in b.children().items():
            prefixes.append((f"l{i}.{SENAVIK_BLOCK_PREFIXES[role]}", part))
    prefixes += [("final.norm", final_norm), ("", head)]
    return CausalLM(cfg, embedding, blocks, final_norm, head, cache_layers, schedule, prefixes)


register_model("Senavik", SenavikConfig, build_senavik)
