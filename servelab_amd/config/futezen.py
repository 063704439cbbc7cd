"""Configuration of the Futezen design: a decoder whose config.json lists its layers, each with
one of three mixers and a dense or routed feed-forward, and that may run a stretch of its layers
several times.

    {"architecture": "Futezen", "width", "vocab", "norm": {"eps"},
     "layers": [{"type", "mixer": {...}, "mlp": {...} | null}],
     "loop": {"start", "stop", "times"} | absent}

Mixers: ``attention`` (grouped heads: heads, kv_heads, dim, vdim, scale, rot {base, dims}: the
leading ``dims`` channels of a head turn in halves), ``latent_attention`` (queries through a
normed latent of ``q_rank`` channels, keys and values from a cached latent of ``kv_rank``, one
rotated key part of ``rot_dim`` channels shared by the heads, turning in neighbouring pairs) and
``mamba2`` (a state-space mixer: heads, vdim, state, groups, conv taps, norm_groups).
Feed-forward: ``{"kind": "dense", "ff"}`` or ``{"kind": "moe", "router": {"experts", "top"},
"expert": {"ff"}, "shared": {"ff"} | absent}``.  ``loop``: layers start .. stop - 1 run ``times``
times in a row with the same tensors and a cache of their own each time.
Nothing here is a default for a size or a constant of the model.
"""
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from .layered import _section
from .model import ConfigError, read_key


@dataclass(frozen=True)
class RotatedAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_base: float
    rot_dims: int                # 0: no rotation


@dataclass(frozen=True)
class QueryLatentAttentionConfig:
    heads: int
    dim: int                     # channels of a head that are not rotated
    rot_dim: int                 # rotated channels of a head, and of the shared key part
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    rot_base: float
    rot_dims: int


@dataclass(frozen=True)
class StateSpaceConfig:
    heads: int
    vdim: int                    # channels of a head
    state: int                   # rows of a head's state matrix
    groups: int                  # heads share the B and C of their group
    conv: int                    # taps of the short convolution
    norm_groups: int             # equal parts of the read-out that are normed one by one


@dataclass(frozen=True)
class DenseFfConfig:
    ff: int


@dataclass(frozen=True)
class ExpertsFfConfig:
    experts: int
    top: int
    ff: int
    shared_ff: int               # 0: no shared expert


@dataclass(frozen=True)
class FutezenLayer:
    kind: str                    # "attention" | "latent_attention" | "mamba2"
    mixer: Any
    mlp: Any                     # DenseFfConfig | ExpertsFfConfig | None


@dataclass(frozen=True)
class LoopConfig:
    start: int
    stop: int
    times: int


def _rotation(m, where):
    rot = _section(m, "rot", where, required=False)
    if rot is None:
        return 0.0, 0
    base, dims = read_key(rot, "base", kind=float), read_key(rot, "dims", kind=int)
    if dims < 0 or dims % 2 or (dims and not base > 0):
        raise ConfigError(f"config.json: {where}: rot.dims must be even and rot.base positive")
    return base, dims


def _read_mixer(kind: str, m: Dict[str, Any], where: str):
    if kind == "attention":
        base, dims = _rotation(m, where)
        c = RotatedAttentionConfig(
            heads=read_key(m, "heads", kind=int), kv_heads=read_key(m, "kv_heads", kind=int),
            dim=read_key(m, "dim", kind=int), vdim=read_key(m, "vdim", kind=int),
            scale=read_key(m, "scale", kind=float), rot_base=base, rot_dims=dims)
        if min(c.heads, c.kv_heads, c.dim, c.vdim) < 1 or c.heads % c.kv_heads or c.rot_dims > c.dim:
            raise ConfigError(f"config.json: {where}: heads must be a positive multiple of kv_heads, dim and "
                              "vdim positive, rot.dims within dim")
        return c
    if kind == "latent_attention":
        base, dims = _rotation(m, where)
        c = QueryLatentAttentionConfig(
            heads=read_key(m, "heads", kind=int), dim=read_key(m, "dim", kind=int),
            rot_dim=read_key(m, "rot_dim", kind=int), vdim=read_key(m, "vdim", kind=int),
            q_rank=read_key(m, "q_rank", kind=int), kv_rank=read_key(m, "kv_rank", kind=int),
            scale=read_key(m, "scale", kind=float), rot_base=base, rot_dims=dims)
        if min(c.heads, c.dim, c.rot_dim, c.vdim, c.q_rank, c.kv_rank) < 1 or c.rot_dims > c.rot_dim:
            raise ConfigError(f"config.json: {where}: heads, dim, rot_dim, vdim, q_rank and kv_rank must be "
                              "positive, rot.dims within rot_dim")
        return c
    if kind == "mamba2":
        c = StateSpaceConfig(
            heads=read_key(m, "heads", kind=int), vdim=read_key(m, "vdim", kind=int),
            state=read_key(m, "state", kind=int), groups=read_key(m, "groups", kind=int),
            conv=read_key(m, "conv", kind=int), norm_groups=read_key(m, "norm_groups", kind=int))
        if min(c.heads, c.vdim, c.state, c.groups, c.conv, c.norm_groups) < 1 or c.heads % c.groups \
                or (c.heads * c.vdim) % c.norm_groups:
            raise ConfigError(f"config.json: {where}: sizes must be positive, heads a multiple of groups, "
                              "heads * vdim a multiple of norm_groups")
        return c
    raise ConfigError(f"config.json: {where}: type {kind!r} is not one of attention, latent_attention, mamba2")


def _read_mlp(raw: Optional[Dict[str, Any]], where: str):
    if raw is None:
        return None
    kind = read_key(raw, "kind", kind=str)
    if kind == "dense":
        c = DenseFfConfig(read_key(raw, "ff", kind=int))
        if c.ff < 1:
            raise ConfigError(f"config.json: {where}: mlp.ff must be positive")
        return c
    if kind == "moe":
        router, expert = _section(raw, "router", where), _section(raw, "expert", where)
        shared = _section(raw, "shared", where, required=False)
        c = ExpertsFfConfig(experts=read_key(router, "experts", kind=int), top=read_key(router, "top", kind=int),
                            ff=read_key(expert, "ff", kind=int),
                            shared_ff=read_key(shared, "ff", kind=int) if shared else 0)
        if c.ff < 1 or c.shared_ff < 0 or not 1 <= c.top <= c.experts:
            raise ConfigError(f"config.json: {where}: mlp needs 1 <= router.top <= router.experts and positive widths")
        return c
    raise ConfigError(f"config.json: {where}: mlp.kind {kind!r} is not one of dense, moe")


def _read_layer(i: int, entry: Dict[str, Any]) -> FutezenLayer:
    where = f"layers[{i}]"
    if not isinstance(entry, dict):
        raise ConfigError(f"config.json: {where} must be an object")
    kind = read_key(entry, "type", kind=str)
    mixer = _read_mixer(kind, _section(entry, "mixer", where), where)
    return FutezenLayer(kind, mixer, _read_mlp(_section(entry, "mlp", where, required=False), where))


@dataclass
class FutezenConfig:
    width: int
    vocab: int
    norm_eps: float
    layers: List[FutezenLayer]
    loop: Optional[LoopConfig] = None
    architecture: str = "Futezen"
    dtype: str = "bfloat16"
    path: str = ""
    raw: Dict[str, Any] = field(default_factory=dict, repr=False, compare=False)

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def hidden_size(self) -> int:
        return self.width

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    def order(self) -> List[int]:
        """The layers in the order they run."""
        n = len(self.layers)
        if self.loop is None:
            return list(range(n))
        a, b, times = self.loop.start, self.loop.stop, self.loop.times
        return list(range(a)) + list(range(a, b)) * times + list(range(b, n))

    @classmethod
    def from_hf(cls, cfg: Dict[str, Any], path: str = "") -> "FutezenConfig":
        norm = _section(cfg, "norm", "model")
        layers = cfg.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        raw_loop = _section(cfg, "loop", "model", required=False)
        loop = None
        if raw_loop is not None:
            loop = LoopConfig(read_key(raw_loop, "start", kind=int), read_key(raw_loop, "stop", kind=int),
                              read_key(raw_loop, "times", kind=int))
        out = cls(width=read_key(cfg, "width", kind=int), vocab=read_key(cfg, "vocab", kind=int),
                  norm_eps=read_key(norm, "eps", kind=float),
                  layers=[_read_layer(i, e) for i, e in enumerate(layers)], loop=loop,
                  architecture=str(cfg.get("architecture") or "Futezen"),
                  dtype=str(cfg.get("torch_dtype") or "bfloat16"), path=path, raw=dict(cfg))
        out.validate()
        return out

    def validate(self) -> None:
        if self.width < 1 or self.vocab < 1 or not self.norm_eps > 0:
            raise ConfigError("config.json: width and vocab must be positive, norm.eps > 0")
        if self.loop is not None:
            l = self.loop
            if not 0 <= l.start <= l.stop <= len(self.layers) or l.times < 1:
                raise ConfigError("config.json: loop needs 0 <= start <= stop <= number of layers and times >= 1")

    def to_hf(self) -> Dict[str, Any]:
        layers = []
        for l in self.layers:
            m = l.mixer
            if l.kind == "attention":
                mixer = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale,
                         "rot": {"base": m.rot_base, "dims": m.rot_dims} if m.rot_dims else None}
            elif l.kind == "latent_attention":
                mixer = {"heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "vdim": m.vdim, "q_rank": m.q_rank,
                         "kv_rank": m.kv_rank, "scale": m.scale,
                         "rot": {"base": m.rot_base, "dims": m.rot_dims} if m.rot_dims else None}
            else:
                mixer = {"heads": m.heads, "vdim": m.vdim, "state": m.state, "groups": m.groups, "conv": m.conv,
                         "norm_groups": m.norm_groups}
            if l.mlp is None:
                mlp = None
            elif isinstance(l.mlp, DenseFfConfig):
                mlp = {"kind": "dense", "ff": l.mlp.ff}
            else:
                mlp = {"kind": "moe", "router": {"experts": l.mlp.experts, "top": l.mlp.top},
                       "expert": {"ff": l.mlp.ff}}
                if l.mlp.shared_ff:
                    mlp["shared"] = {"ff": l.mlp.shared_ff}
            layers.append({"type": l.kind, "mixer": mixer, "mlp": mlp})
        out = {"architecture": self.architecture, "width": self.width, "vocab": self.vocab,
               "norm": {"eps": self.norm_eps}, "layers": layers, "torch_dtype": self.dtype}
        if self.loop is not None:
            out["loop"] = {"start": self.loop.start, "stop": self.loop.stop, "times": self.loop.times}
        return out
