"""Configuration of the Vunadra design: a pre-norm decoder whose config.json lists its layers,
each with one of three attention mixers and a dense or routed feed-forward, and that may walk a
stretch of its layers several times, each pass entered through a product of the stream and the
embedding output.

    {"architecture": "Vunadra", "width", "vocab", "norm": {"eps"}, "embedding": {"scale"},
     "logit_scale", "layers": [{"type", "mixer": {...}, "mlp": {...} | null}],
     "loop": {"start", "stop", "times"} | absent}

Mixers (``rot`` = {base, dims[, scaling]}: the leading ``dims`` channels of a head turn in
neighbouring pairs; ``mask`` = {size}: a window, absent: every earlier key):
  ``attention``         heads, kv_heads, dim, vdim, scale, conv (taps of a short convolution on q, k
                        and v; absent or 0: none), rot, mask, softcap
  ``attention_2``       heads, kv_heads, dim (= vdim: the values are the keys as projected), scale,
                        softcap, rot, mask; biases and a norm over the whole projection
  ``latent_attention``  heads, dim, rot_dim, vdim, kv_rank, scale, rot, mask
``rot.scaling``: {factor, original, fast, slow} blends every frequency f between f and f / factor by
how often its pair turns within ``original`` positions and enlarges cos and sin by 0.1 ln(factor)
+ 1; {factor, original, low, high} stretches frequencies by wavelength.
Feed-forward: ``{"kind": "dense", "ff"}`` (biases, the tanh form of gelu as gate) or ``{"kind":
"moe", "router": {"experts", "top", "identity", "scale"}, "expert": {"ff", "limit"}}``.
Nothing here is a default for a size or a constant of the model.
"""
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from .layered import _section
from .model import ConfigError, read_key


@dataclass(frozen=True)
class RotationConfig:
    """dims 0: no rotation.  scaling: None, ("blended", factor, original, fast, slow) or
    ("wavelength", factor, original, low, high)."""
    base: float = 0.0
    dims: int = 0
    scaling: Optional[tuple] = None

    def to_hf(self):
        if not self.dims:
            return None
        out = {"base": self.base, "dims": self.dims}
        if self.scaling is not None:
            kind, factor, original, a, b = self.scaling
            names = ("fast", "slow") if kind == "blended" else ("low", "high")
            out["scaling"] = {"factor": factor, "original": original, names[0]: a, names[1]: b}
        return out


@dataclass(frozen=True)
class GroupedAttentionConfig:
    """``attention`` (values projected, an optional short convolution) and ``attention_2``
    (``values_are_keys``: biases, a norm over the projection, no value projection)."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: RotationConfig
    window: int = 0              # 0: every earlier key
    softcap: float = 0.0         # 0: scores are not capped
    conv: int = 0                # taps; 0: no convolution
    values_are_keys: bool = False


@dataclass(frozen=True)
class WindowLatentConfig:
    heads: int
    dim: int                     # channels of a head that are not rotated
    rot_dim: int                 # rotated channels of a head, and of the shared key part
    vdim: int
    kv_rank: int
    scale: float
    rot: RotationConfig
    window: int = 0


@dataclass(frozen=True)
class BiasedDenseConfig:
    ff: int


@dataclass(frozen=True)
class SharesExpertsConfig:
    experts: int                 # experts with matrices
    identity: int                # router outputs behind them whose expert hands its input through
    top: int
    scale: float
    ff: int
    limit: float


@dataclass(frozen=True)
class VunadraLayer:
    kind: str                    # "attention" | "attention_2" | "latent_attention"
    mixer: Any
    mlp: Any                     # BiasedDenseConfig | SharesExpertsConfig | None


@dataclass(frozen=True)
class PassesConfig:
    start: int
    stop: int
    times: int


def _rotation(m, where) -> RotationConfig:
    rot = _section(m, "rot", where, required=False)
    if rot is None or not rot.get("dims"):
        return RotationConfig()
    base, dims = read_key(rot, "base", kind=float), read_key(rot, "dims", kind=int)
    if dims < 0 or dims % 2 or not base > 1:
        raise ConfigError(f"config.json: {where}: rot.dims must be even and rot.base above 1")
    sc = _section(rot, "scaling", where, required=False)
    scaling = None
    if sc is not None:
        factor, original = read_key(sc, "factor", kind=float), read_key(sc, "original", kind=float)
        if "fast" in sc or "slow" in sc:
            scaling = ("blended", factor, original, read_key(sc, "fast", kind=float), read_key(sc, "slow", kind=float))
        else:
            scaling = ("wavelength", factor, original, read_key(sc, "low", kind=float), read_key(sc, "high", kind=float))
            if scaling[3] == scaling[4]:
                raise ConfigError(f"config.json: {where}: rot.scaling.low and .high must differ")
        if not factor > 0 or not original > 0 or not scaling[3] > 0 or not scaling[4] > 0:
            raise ConfigError(f"config.json: {where}: rot.scaling needs positive numbers")
    return RotationConfig(base, dims, scaling)


def _window(m, where) -> int:
    mask = _section(m, "mask", where, required=False)
    if mask is None:
        return 0
    size = read_key(mask, "size", 0, kind=int)
    if size < 0:
        raise ConfigError(f"config.json: {where}: mask.size must not be negative")
    return size


def _read_mixer(kind: str, m: Dict[str, Any], where: str):
    if kind in ("attention", "attention_2"):
        keys = kind == "attention_2"
        dim = read_key(m, "dim", kind=int)
        c = GroupedAttentionConfig(
            heads=read_key(m, "heads", kind=int), kv_heads=read_key(m, "kv_heads", kind=int), dim=dim,
            vdim=read_key(m, "vdim", dim, kind=int) if keys else read_key(m, "vdim", kind=int),
            scale=read_key(m, "scale", kind=float), rot=_rotation(m, where), window=_window(m, where),
            softcap=read_key(m, "softcap", 0.0, kind=float), conv=read_key(m, "conv", 0, kind=int),
            values_are_keys=keys)
        if min(c.heads, c.kv_heads, c.dim, c.vdim) < 1 or c.heads % c.kv_heads or c.rot.dims > c.dim \
                or c.conv < 0 or c.softcap < 0 or (keys and c.vdim != c.dim):
            raise ConfigError(f"config.json: {where}: heads must be a positive multiple of kv_heads, dim and vdim "
                              "positive (equal where the values are the keys), rot.dims within dim, conv and "
                              "softcap not negative")
        return c
    if kind == "latent_attention":
        c = WindowLatentConfig(
            heads=read_key(m, "heads", kind=int), dim=read_key(m, "dim", kind=int),
            rot_dim=read_key(m, "rot_dim", kind=int), vdim=read_key(m, "vdim", kind=int),
            kv_rank=read_key(m, "kv_rank", kind=int), scale=read_key(m, "scale", kind=float),
            rot=_rotation(m, where), window=_window(m, where))
        if min(c.heads, c.dim, c.rot_dim, c.vdim, c.kv_rank) < 1 or c.rot.dims > c.rot_dim:
            raise ConfigError(f"config.json: {where}: heads, dim, rot_dim, vdim and kv_rank must be positive, "
                              "rot.dims within rot_dim")
        return c
    raise ConfigError(f"config.json: {where}: type {kind!r} is not one of attention, attention_2, latent_attention")


def _read_mlp(raw: Optional[Dict[str, Any]], where: str):
    if raw is None:
        return None
    kind = read_key(raw, "kind", kind=str)
    if kind == "dense":
        c = BiasedDenseConfig(read_key(raw, "ff", kind=int))
        if c.ff < 1:
            raise ConfigError(f"config.json: {where}: mlp.ff must be positive")
        return c
    if kind == "moe":
        router, expert = _section(raw, "router", where), _section(raw, "expert", where)
        c = SharesExpertsConfig(experts=read_key(router, "experts", kind=int),
                                identity=read_key(router, "identity", 0, kind=int),
                                top=read_key(router, "top", kind=int), scale=read_key(router, "scale", kind=float),
                                ff=read_key(expert, "ff", kind=int), limit=read_key(expert, "limit", kind=float))
        if c.ff < 1 or c.experts < 1 or c.identity < 0 or not 1 <= c.top <= c.experts + c.identity or not c.limit > 0:
            raise ConfigError(f"config.json: {where}: mlp needs 1 <= router.top <= router.experts + "
                              "router.identity, a positive width and a positive limit")
        return c
    raise ConfigError(f"config.json: {where}: mlp.kind {kind!r} is not one of dense, moe")


def _read_layer(i: int, entry: Dict[str, Any]) -> VunadraLayer:
    where = f"layers[{i}]"
    if not isinstance(entry, dict):
        raise ConfigError(f"config.json: {where} must be an object")
    kind = read_key(entry, "type", kind=str)
    mixer = _read_mixer(kind, _section(entry, "mixer", where), where)
    return VunadraLayer(kind, mixer, _read_mlp(_section(entry, "mlp", where, required=False), where))


@dataclass
class VunadraConfig:
    width: int
    vocab: int
    norm_eps: float
    embedding_scale: float
    logit_scale: float
    layers: List[VunadraLayer]
    loop: Optional[PassesConfig] = None
    architecture: str = "Vunadra"
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

    def stretches(self):
        """(layers before the repeated stretch, the stretch, its passes, layers behind it)."""
        n = len(self.layers)
        if self.loop is None:
            return list(range(n)), [], 0, []
        a, b = self.loop.start, self.loop.stop
        return list(range(a)), list(range(a, b)), self.loop.times, list(range(b, n))

    @classmethod
    def from_hf(cls, cfg: Dict[str, Any], path: str = "") -> "VunadraConfig":
        norm = _section(cfg, "norm", "model")
        embedding = _section(cfg, "embedding", "model")
        layers = cfg.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        raw_loop = _section(cfg, "loop", "model", required=False)
        loop = None
        if raw_loop is not None:
            loop = PassesConfig(read_key(raw_loop, "start", kind=int), read_key(raw_loop, "stop", kind=int),
                                read_key(raw_loop, "times", kind=int))
        out = cls(width=read_key(cfg, "width", kind=int), vocab=read_key(cfg, "vocab", kind=int),
                  norm_eps=read_key(norm, "eps", kind=float),
                  embedding_scale=read_key(embedding, "scale", kind=float),
                  logit_scale=read_key(cfg, "logit_scale", kind=float),
                  layers=[_read_layer(i, e) for i, e in enumerate(layers)], loop=loop,
                  architecture=str(cfg.get("architecture") or "Vunadra"),
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
            if l.kind == "latent_attention":
                mixer = {"heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "vdim": m.vdim,
                         "kv_rank": m.kv_rank, "scale": m.scale}
            else:
                mixer = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale}
                if m.conv:
                    mixer["conv"] = m.conv
                if m.softcap:
                    mixer["softcap"] = m.softcap
            if m.rot.dims:
                mixer["rot"] = m.rot.to_hf()
            if m.window:
                mixer["mask"] = {"size": m.window}
            if l.mlp is None:
                mlp = None
            elif isinstance(l.mlp, BiasedDenseConfig):
                mlp = {"kind": "dense", "ff": l.mlp.ff}
            else:
                mlp = {"kind": "moe", "router": {"experts": l.mlp.experts, "identity": l.mlp.identity,
                                                 "top": l.mlp.top, "scale": l.mlp.scale},
                       "expert": {"ff": l.mlp.ff, "limit": l.mlp.limit}}
            layers.append({"type": l.kind, "mixer": mixer, "mlp": mlp})
        out = {"architecture": self.architecture, "width": self.width, "vocab": self.vocab,
               "norm": {"eps": self.norm_eps}, "embedding": {"scale": self.embedding_scale},
               "logit_scale": self.logit_scale, "layers": layers, "torch_dtype": self.dtype}
        if self.loop is not None:
            out["loop"] = {"start": self.loop.start, "stop": self.loop.stop, "times": self.loop.times}
        return out
