"""Typed configuration of the Senavik design: a list of pre-norm layers, each with one of two
mixers (grouped-query attention inside a sliding window that keeps a sequence's first tokens;
attention over a latent that all heads share, with queries through a latent of their own) and a
dense, routed or absent feed-forward; norms whose weights are stored around zero; a norm behind
the embedding; a learned term a head in every softmax denominator. Every size and every constant
that can differ between models of the design is read from config.json; nothing is defaulted from
a known model.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from .model_config import ConfigError
from .rubasun_config import _need
from .virusun_config import _positive


def _scaling(rot: Optional[Dict[str, Any]], keys: Tuple[str, ...], where: str) -> Optional[Dict[str, float]]:
    """The numbers of a frequency scaling, all of them or none."""
    s = None if rot is None else rot.get("scaling")
    if s is None:
        return None
    out = {k: float(_need(s, k, where + ".rot.scaling")) for k in keys}
    if out["factor"] <= 0 or out["original"] <= 0:
        raise ConfigError(f"{where}.rot.scaling: factor and original must be positive")
    return out


def _rotation(d, where: str, most: int, what: str):
    """(dims, base) of a mixer's ``rot`` entry; none: (0, 1.0)."""
    rot = d.get("rot")
    if rot is None:
        return 0, 1.0
    dims, base = int(_need(rot, "dims", where + ".rot")), float(_need(rot, "base", where + ".rot"))
    if dims < 0 or dims % 2 or dims > most:
        raise ConfigError(f"{where}.rot: dims {dims} must be even and at most {what} {most}")
    if dims and base <= 0:
        raise ConfigError(f"{where}.rot: base must be positive")
    return dims, base


@dataclass(frozen=True)
class KeptWindowAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: Optional[int]      # a query sees itself and the window - 1 tokens before it; None: all
    keep_first: int            # and the tokens at positions below this
    rot_dims: int              # entries of a head that turn (0: none)
    rot_base: float
    rot_scaling: Optional[Dict[str, float]]    # factor, low, high, original: by wavelength band

    @classmethod
    def from_dict(cls, d, where) -> "KeptWindowAttentionConfig":
        mask = d.get("mask")
        dim = int(_need(d, "dim", where))
        rot_dims, rot_base = _rotation(d, where, dim, "the head's")
        c = cls(heads=int(_need(d, "heads", where)), kv_heads=int(_need(d, "kv_heads", where)),
                dim=dim, vdim=int(_need(d, "vdim", where)), scale=float(_need(d, "scale", where)),
                window=None if mask is None else int(_need(mask, "size", where + ".mask")),
                keep_first=0 if mask is None else int(mask.get("keep_first") or 0),
                rot_dims=rot_dims, rot_base=rot_base,
                rot_scaling=_scaling(d.get("rot"), ("factor", "low", "high", "original"), where))
        _positive(where, heads=c.heads, kv_heads=c.kv_heads, dim=c.dim, vdim=c.vdim)
        if c.heads % c.kv_heads:
            raise ConfigError(f"{where}: {c.heads} heads are not a multiple of {c.kv_heads} kv_heads")
        if c.window is not None and c.window <= 0:
            raise ConfigError(f"{where}.mask: size must be positive")
        if c.keep_first < 0:
            raise ConfigError(f"{where}.mask: keep_first must not be negative")
        return c


@dataclass(frozen=True)
class QueryLatentAttentionConfig:
    heads: int
    dim: int                   # unrotated query/key entries a head
    rot_dim: int               # rotated entries a head (and of the shared key part)
    vdim: int
    kv_rank: int
    q_rank: int
    scale: float
    rot_dims: int
    rot_base: float
    rot_scaling: Optional[Dict[str, float]]    # factor, original, fast, slow: a ramp

    @classmethod
    def from_dict(cls, d, where) -> "QueryLatentAttentionConfig":
        rot_dim = int(_need(d, "rot_dim", where))
        rot_dims, rot_base = _rotation(d, where, rot_dim, "rot_dim")
        c = cls(heads=int(_need(d, "heads", where)), dim=int(_need(d, "dim", where)), rot_dim=rot_dim,
                vdim=int(_need(d, "vdim", where)), kv_rank=int(_need(d, "kv_rank", where)),
                q_rank=int(_need(d, "q_rank", where)), scale=float(_need(d, "scale", where)),
                rot_dims=rot_dims, rot_base=rot_base,
                rot_scaling=_scaling(d.get("rot"), ("factor", "original", "fast", "slow"), where))
        _positive(where, heads=c.heads, vdim=c.vdim, kv_rank=c.kv_rank, q_rank=c.q_rank)
        if c.dim < 0 or c.rot_dim < 0 or c.rot_dim % 2 or c.dim + c.rot_dim <= 0:
            raise ConfigError(f"{where}: dim and rot_dim must not be negative (one of them positive), rot_dim even")
        if c.kv_rank + c.rot_dim > 640:
            raise ConfigError(f"{where}: kv_rank + rot_dim = {c.kv_rank + c.rot_dim}; the attention kernels take "
                              "up to 640")
        if c.rot_scaling is not None and (c.rot_scaling["fast"] <= 0 or c.rot_scaling["slow"] <= 0):
            raise ConfigError(f"{where}.rot.scaling: fast and slow must be positive")
        return c


@dataclass(frozen=True)
class SenavikMLPConfig:
    kind: str                  # "dense" | "moe"
    ff: int                    # hidden size of the dense layer, or of an expert
    experts: int = 0
    top: int = 0
    groups: int = 1            # equal groups of neighbouring experts
    keep_groups: int = 1       # groups a token may choose from

    @classmethod
    def from_dict(cls, d, where) -> "SenavikMLPConfig":
        kind = _need(d, "kind", where)
        if kind == "dense":
            c = cls("dense", int(_need(d, "ff", where)))
            _positive(where, ff=c.ff)
            return c
        if kind != "moe":
            raise ConfigError(f"{where}: unknown feed-forward kind {kind!r} (known: 'dense', 'moe')")
        r = _need(d, "router", where)
        g = r.get("groups")
        c = cls("moe", int(_need(_need(d, "expert", where), "ff", where + ".expert")),
                experts=int(_need(r, "experts", where + ".router")), top=int(_need(r, "top", where + ".router")),
                groups=1 if g is None else int(_need(g, "count", where + ".router.groups")),
                keep_groups=1 if g is None else int(_need(g, "keep", where + ".router.groups")))
        _positive(where, ff=c.ff, experts=c.experts, top=c.top, groups=c.groups, keep=c.keep_groups)
        if c.top > c.experts:
            raise ConfigError(f"{where}: top {c.top} of {c.experts} experts")
        if c.experts % c.groups or c.keep_groups > c.groups or c.keep_groups * (c.experts // c.groups) < c.top:
            raise ConfigError(f"{where}.router.groups: {c.groups} groups of which {c.keep_groups} are kept do not "
                              f"fit {c.experts} experts with {c.top} chosen")
        return c


MIXER_CONFIGS = {"attention": KeptWindowAttentionConfig, "latent_attention": QueryLatentAttentionConfig}


@dataclass(frozen=True)
class SenavikLayerConfig:
    kind: str                  # "attention" | "latent_attention"
    mixer: Any
    mlp: Optional[SenavikMLPConfig]


@dataclass(frozen=True)
class SenavikConfig:
    vocab_size: int
    hidden_size: int
    norm_eps: float
    layers: Tuple[SenavikLayerConfig, ...]
    eos_token_id: Any = None
    initializer_range: float = 0.05
    architectures: Tuple[str, ...] = ("Senavik",)
    raw: Any = None

    @property
    def eos_token_ids(self) -> Tuple[int, ...]:
        e = self.eos_token_id
        if e is None:
            return ()
        return tuple(int(x) for x in e) if isinstance(e, (list, tuple)) else (int(e),)

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "SenavikConfig":
        layers = []
        for i, e in enumerate(_need(d, "layers", "the model")):
            where = f"layers[{i}]"
            kind = _need(e, "type", where)
            if kind not in MIXER_CONFIGS:
                raise ConfigError(f"{where}: unknown layer type {kind!r} (known: {sorted(MIXER_CONFIGS)})")
            m = MIXER_CONFIGS[kind].from_dict(_need(e, "mixer", where), where + ".mixer")
            mlp = None if e.get("mlp") is None else SenavikMLPConfig.from_dict(e["mlp"], where + ".mlp")
            layers.append(SenavikLayerConfig(kind, m, mlp))
        if not layers:
            raise ConfigError("config.json: 'layers' is empty")
        cfg = cls(vocab_size=int(_need(d, "vocab", "the model")), hidden_size=int(_need(d, "width", "the model")),
                  norm_eps=float(_need(_need(d, "norm", "the model"), "eps", "norm")), layers=tuple(layers),
                  eos_token_id=d.get("eos_token_id"),
                  initializer_range=float(d.get("initializer_range", 0.05)), raw=dict(d))
        if cfg.vocab_size <= 0 or cfg.hidden_size <= 0 or cfg.norm_eps < 0:
            raise ConfigError("vocab and width must be positive, norm.eps not negative")
        return cfg

    def to_dict(self) -> Dict[str, Any]:
        return dict(self.raw)
