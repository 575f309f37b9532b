"""``Matusun``: layers given as a list, each with one of two mixers (softmax attention inside a
sliding window with normed and rotated queries and keys; the selective scan of Mamba) and a routed
feed-forward or none, RMS norms in front of the sublayers, several residual streams mixed by
learned coefficients (hyper-connections), a range of layers that runs several times in a row with
the same weights and a cache or state of its own each time, and the embedding table as the head.
The model is a list of layer specs over the engine's parts; tensor names are the checkpoint's own
("l<i>.mix.q", "l<i>.mlp.e0.up", "l<i>.hc1.in", "l<i>.norm1", ...).
"""
from __future__ import annotations

from ..config.matusun_config import MatusunConfig
from ..config.registry import register_model
from ..parts.base import build_part
from .causal_lm import CausalLM, LayerCall

# role of a part inside a block -> what follows "l<i>." in its tensors' names
MATUSUN_BLOCK_PREFIXES = {"norm1": "norm1", "norm2": "norm2", "mixer": "mix.", "feed_forward": "mlp.",
                          "connections": ""}


def _norm(cfg: MatusunConfig, streams: int = 1):
    return build_part("norm", "rmsnorm", size=cfg.hidden_size, eps=cfg.norm_eps, weight_name="", streams=streams)


def _mixer(cfg: MatusunConfig, layer):
    W, m = cfg.hidden_size, layer.mixer
    if layer.kind == "attention":
        return build_part("mixer", "normed_attention", hidden_size=W, num_heads=m.heads, num_kv_heads=m.kv_heads,
                          dim=m.dim, vdim=m.vdim, scale=m.scale, eps=cfg.norm_eps, qk_norm="whole", maps=1,
                          bias=False, gated=False, rot_dims=m.rot_dims, rot_base=m.rot_base, window=m.window)
    return build_part("mixer", "selective_scan", hidden_size=W, inner=m.inner, state=m.state, dt_rank=m.dt_rank,
                      taps=m.conv)


def _feed_forward(cfg: MatusunConfig, mlp):
    if mlp is None:
        return None
    W = cfg.hidden_size
    shared = None
    if mlp.shared_ff:
        shared = build_part("feed_forward", "mlp", hidden_size=W, intermediate_size=mlp.shared_ff,
                            activation="relu2")
    return build_part("feed_forward", "routed_experts", hidden_size=W, intermediate_size=mlp.ff,
                      num_experts=mlp.experts, top=mlp.top, activation="relu2", weight_on_input=False,
                      renormalize=True, renorm_eps=1e-20, route_scale=mlp.scale, score="softmax",
                      correction_name="correction", identity=mlp.identity, shared=shared, shared_gate=False)


def build_matusun(cfg: MatusunConfig) -> CausalLM:
    W = cfg.hidden_size
    learned = cfg.streams is not None
    S = cfg.streams if learned else 1
    embedding = build_part("embedding", "token_embedding", vocab_size=cfg.vocab_size, hidden_size=W,
                           weight_name="embed", float32_stream=True, copies=S)
    blocks = []
    for layer in cfg.layers:
        ffn = _feed_forward(cfg, layer.mlp)
        blocks.append(build_part("block", "hyper_connections", hidden_size=W, streams=S, mixer=_mixer(cfg, layer),
                                 mixer_norm=_norm(cfg), feed_forward=ffn,
                                 ffn_norm=_norm(cfg) if ffn is not None else None, learned=learned))
    # every run of a layer keeps a cache layer of its own: a looped layer one a pass
    cache_layers, schedule = [], []
    for i, _ in cfg.run_order():
        spec = blocks[i].cache_spec()
        if spec is None:
            schedule.append(LayerCall(i, None, True))
            continue
        cache_layers.append(spec)
        schedule.append(LayerCall(i, len(cache_layers) - 1, True))
    final_norm = _norm(cfg, S)
    head = build_part("head", "linear_head", vocab_size=cfg.vocab_size, hidden_size=W, tied_to=embedding)
    prefixes = [("", embedding)]
    for i, b in enumerate(blocks):
        for role, part in b.children().items():
            prefixes.append((f"l{i}.{MATUSUN_BLOCK_PREFIXES[role]}", part))
    prefixes += [("final.norm", final_norm), ("", head)]
    return CausalLM(cfg, embedding, blocks, final_norm, head, cache_layers, schedule, prefixes)


register_model("Matusun", MatusunConfig, build_matusun)
