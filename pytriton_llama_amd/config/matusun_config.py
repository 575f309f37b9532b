"""Typed configuration of the Matusun design: a list of layers, each with one of two mixers
(softmax attention inside a sliding window; the selective scan of Mamba) and a routed
feed-forward or none, RMS norms in front of the sublayers, several residual streams that learned
coefficients mix (hyper-connections), and a range of layers that runs several times in a row.
Every size and every constant that can differ between models of the design is read from
config.json; nothing is defaulted from a known model.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from .model_config import ConfigError
from .rubasun_config import _need
from .virusun_config import _positive


@dataclass(frozen=True)
class WindowAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: Optional[int]      # a query sees itself and the window - 1 tokens before it; None: all
    rot_dims: int              # entries of a head that turn (0: none)
    rot_base: float

    @classmethod
    def from_dict(cls, d, where) -> "WindowAttentionConfig":
        mask, rot = d.get("mask"), d.get("rot")
        c = cls(heads=int(_need(d, "heads", where)), kv_heads=int(_need(d, "kv_heads", where)),
                dim=int(_need(d, "dim", where)), vdim=int(_need(d, "vdim", where)),
                scale=float(_need(d, "scale", where)),
                window=None if mask is None else int(_need(mask, "size", where + ".mask")),
                rot_dims=0 if rot is None else int(_need(rot, "dims", where + ".rot")),
                rot_base=1.0 if rot is None else float(_need(rot, "base", where + ".rot")))
        _positive(where, heads=c.heads, kv_heads=c.kv_heads, dim=c.dim, vdim=c.vdim)
        if c.heads % c.kv_heads:
            raise ConfigError(f"{where}: {c.heads} heads are not a multiple of {c.kv_heads} kv_heads")
        if c.window is not None and c.window <= 0:
            raise ConfigError(f"{where}.mask: size must be positive")
        if c.rot_dims < 0 or c.rot_dims % 2 or c.rot_dims > c.dim:
            raise ConfigError(f"{where}.rot: dims {c.rot_dims} must be even and at most the head's {c.dim}")
        if c.rot_dims and c.rot_base <= 0:
            raise ConfigError(f"{where}.rot: base must be positive")
        return c


@dataclass(frozen=True)
class SelectiveScanConfig:
    inner: int                 # channels
    state: int                 # state entries a channel
    dt_rank: int
    conv: int                  # taps of the causal convolution

    @classmethod
    def from_dict(cls, d, where) -> "SelectiveScanConfig":
        c = cls(inner=int(_need(d, "inner", where)), state=int(_need(d, "state", where)),
                dt_rank=int(_need(d, "dt_rank", where)), conv=int(_need(d, "conv", where)))
        _positive(where, inner=c.inner, state=c.state, dt_rank=c.dt_rank, conv=c.conv)
        return c


@dataclass(frozen=True)
class RoutedMLPConfig:
    ff: int                    # hidden size of an expert
    experts: int               # experts with tensors of their own
    identity: int              # router outputs behind them whose expert returns its input
    top: int
    scale: float
    shared_ff: int             # 0: no shared expert

    @classmethod
    def from_dict(cls, d, where) -> "RoutedMLPConfig":
        if _need(d, "kind", where) != "moe":
            raise ConfigError(f"{where}: unknown feed-forward kind {d['kind']!r} (known: 'moe')")
        r = _need(d, "router", where)
        shared = d.get("shared")
        c = cls(ff=int(_need(_need(d, "expert", where), "ff", where + ".expert")),
                experts=int(_need(r, "experts", where + ".router")), identity=int(r.get("identity") or 0),
                top=int(_need(r, "top", where + ".router")), scale=float(_need(r, "scale", where + ".router")),
                shared_ff=0 if shared is None else int(_need(shared, "ff", where + ".shared")))
        _positive(where, ff=c.ff, experts=c.experts, top=c.top)
        if c.identity < 0 or c.shared_ff < 0:
            raise ConfigError(f"{where}: router.identity and shared.ff must not be negative")
        if c.top > c.experts + c.identity:
            raise ConfigError(f"{where}: top {c.top} of {c.experts} + {c.identity} router outputs")
        return c


MIXER_CONFIGS = {"attention": WindowAttentionConfig, "mamba1": SelectiveScanConfig}


@dataclass(frozen=True)
class MatusunLayerConfig:
    kind: str                  # "attention" | "mamba1"
    mixer: Any
    mlp: Optional[RoutedMLPConfig]


@dataclass(frozen=True)
class LoopConfig:
    start: int
    stop: int
    times: int


@dataclass(frozen=True)
class MatusunConfig:
    vocab_size: int
    hidden_size: int
    norm_eps: float
    layers: Tuple[MatusunLayerConfig, ...]
    streams: Optional[int]     # None: one residual stream and a plain residual sum
    loop: Optional[LoopConfig]
    eos_token_id: Any = None
    initializer_range: float = 0.05
    architectures: Tuple[str, ...] = ("Matusun",)
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

    def run_order(self) -> Tuple[Tuple[int, int], ...]:
        """(layer, pass) of every layer run, in order: the looped range ``times`` times in a row."""
        n = len(self.layers)
        if self.loop is None:
            return tuple((i, 0) for i in range(n))
        a, b, times = self.loop.start, self.loop.stop, self.loop.times
        out = [(i, 0) for i in range(a)]
        for p in range(times):
            out += [(i, p) for i in range(a, b)]
        return tuple(out + [(i, 0) for i in range(b, n)])

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "MatusunConfig":
        layers = []
        for i, e in enumerate(_need(d, "layers", "the model")):
            where = f"layers[{i}]"
            kind = _need(e, "type", where)
            if kind not in MIXER_CONFIGS:
                raise ConfigError(f"{where}: unknown layer type {kind!r} (known: {sorted(MIXER_CONFIGS)})")
            m = MIXER_CONFIGS[kind].from_dict(_need(e, "mixer", where), where + ".mixer")
            mlp = None if e.get("mlp") is None else RoutedMLPConfig.from_dict(e["mlp"], where + ".mlp")
            layers.append(MatusunLayerConfig(kind, m, mlp))
        if not layers:
            raise ConfigError("config.json: 'layers' is empty")
        loop = None
        if d.get("loop") is not None:
            l = d["loop"]
            loop = LoopConfig(int(_need(l, "start", "loop")), int(_need(l, "stop", "loop")),
                              int(_need(l, "times", "loop")))
            if not 0 <= loop.start <= loop.stop <= len(layers) or loop.times < 1:
                raise ConfigError(f"loop: layers {loop.start}..{loop.stop - 1} {loop.times} times does not fit "
                                  f"{len(layers)} layers")
        streams = None if d.get("streams") is None else int(d["streams"])
        if streams is not None and not 1 <= streams <= 16:
            raise ConfigError(f"streams must be 1 to 16, got {streams}")
        cfg = cls(vocab_size=int(_need(d, "vocab", "the model")), hidden_size=int(_need(d, "width", "the model")),
                  norm_eps=float(_need(_need(d, "norm", "the model"), "eps", "norm")), layers=tuple(layers),
                  streams=streams, loop=loop, eos_token_id=d.get("eos_token_id"),
                  initializer_range=float(d.get("initializer_range", 0.05)), raw=dict(d))
        if cfg.vocab_size <= 0 or cfg.hidden_size <= 0 or cfg.norm_eps < 0:
            raise ConfigError("vocab and width must be positive, norm.eps not negative")
        return cfg

    def to_dict(self) -> Dict[str, Any]:
        return dict(self.raw)
