"""Configuration of decoders that list their layers one by one.

config.json of such a model gives ``width``, ``vocab``, ``norm.eps`` and a list
``layers``; every entry names the kind of its mixer (``type``), the mixer's
sizes and constants (``mixer``) and its feed-forward (``mlp``, or null).  The
Topelorn design is read this way: two kinds of mixer, ``attention`` (grouped
heads with a distance bias, a window that keeps the first tokens, a sink in the
softmax, values mixed with those of an earlier layer, an output gate) and
``latent_attention`` (keys and values made from a cached low-rank latent, a
rotated key part shared by the heads).  Nothing here is a default for a size
or a constant of the model: a key that the kind of layer needs and config.json
lacks is an error that names it.
"""
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from .model import ConfigError, read_key


def _section(cfg: Dict[str, Any], key: str, where: str, required=True) -> Optional[Dict[str, Any]]:
    value = cfg.get(key)
    if value is None:
        if required:
            raise ConfigError(f"config.json: {where}: required key '{key}' is missing")
        return None
    if not isinstance(value, dict):
        raise ConfigError(f"config.json: {where}: '{key}' must be an object, is {value!r}")
    return value


@dataclass(frozen=True)
class WindowConfig:
    """Query i sees key j <= i when i - j < size or j < keep_first; size 0: every j <= i."""
    size: int
    keep_first: int = 0


@dataclass(frozen=True)
class BiasedAttentionConfig:
    heads: int
    kv_heads: int
    dim: int                     # query/key channels of a head
    vdim: int                    # value channels of a head
    scale: float
    window: WindowConfig
    v_mix: bool = False


@dataclass(frozen=True)
class LatentAttentionConfig:
    heads: int
    dim: int                     # channels of a head that are not rotated
    rot_dim: int                 # rotated channels of a head (and of the shared key part)
    vdim: int
    kv_rank: int
    scale: float
    rot_base: float
    rot_dims: int
    window: WindowConfig


@dataclass(frozen=True)
class DenseMlpConfig:
    ff: int


@dataclass(frozen=True)
class LayerConfig:
    kind: str                    # "attention" | "latent_attention"
    mixer: Any
    mlp: Optional[DenseMlpConfig]


def _window(mixer: Dict[str, Any], where: str, keeps: bool) -> WindowConfig:
    mask = _section(mixer, "mask", where, required=False)
    if mask is None:
        return WindowConfig(0, 0)                   # no mask: every earlier key
    size = read_key(mask, "size", kind=int)
    keep = read_key(mask, "keep_first", 0, kind=int) if keeps else 0
    if size < 1 or keep < 0:
        raise ConfigError(f"config.json: {where}: mask.size must be >= 1 and mask.keep_first >= 0")
    return WindowConfig(size, keep)


def _read_layer(i: int, entry: Dict[str, Any]) -> LayerConfig:
    where = f"layers[{i}]"
    if not isinstance(entry, dict):
        raise ConfigError(f"config.json: {where} must be an object")
    kind = read_key(entry, "type", kind=str)
    m = _section(entry, "mixer", where)
    if kind == "attention":
        mixer = BiasedAttentionConfig(
            heads=read_key(m, "heads", kind=int), kv_heads=read_key(m, "kv_heads", kind=int),
            dim=read_key(m, "dim", kind=int), vdim=read_key(m, "vdim", kind=int),
            scale=read_key(m, "scale", kind=float), window=_window(m, where, True),
            v_mix=bool(read_key(m, "v_mix", False)))
        if min(mixer.heads, mixer.kv_heads, mixer.dim, mixer.vdim) < 1 or mixer.heads % mixer.kv_heads:
            raise ConfigError(f"config.json: {where}: heads must be a positive multiple of kv_heads, "
                              "dim and vdim positive")
    elif kind == "latent_attention":
        rot = _section(m, "rot", where)
        mixer = LatentAttentionConfig(
            heads=read_key(m, "heads", kind=int), dim=read_key(m, "dim", kind=int),
            rot_dim=read_key(m, "rot_dim", kind=int), vdim=read_key(m, "vdim", kind=int),
            kv_rank=read_key(m, "kv_rank", kind=int), scale=read_key(m, "scale", kind=float),
            rot_base=read_key(rot, "base", kind=float), rot_dims=read_key(rot, "dims", kind=int),
            window=_window(m, where, False))
        if min(mixer.heads, mixer.dim, mixer.rot_dim, mixer.vdim, mixer.kv_rank) < 1:
            raise ConfigError(f"config.json: {where}: heads, dim, rot_dim, vdim and kv_rank must be positive")
        if mixer.rot_dims % 2 or not 0 < mixer.rot_dims <= mixer.rot_dim or not mixer.rot_base > 0:
            raise ConfigError(f"config.json: {where}: rot.dims must be even and within rot_dim, rot.base positive")
    else:
        raise ConfigError(f"config.json: {where}: type {kind!r} is not one of attention, latent_attention")
    mlp = None
    if entry.get("mlp") is not None:
        raw = _section(entry, "mlp", where)
        mlp_kind = read_key(raw, "kind", kind=str)
        if mlp_kind != "dense":
            raise ConfigError(f"config.json: {where}: mlp.kind {mlp_kind!r} is not supported (dense)")
        mlp = DenseMlpConfig(read_key(raw, "ff", kind=int))
        if mlp.ff < 1:
            raise ConfigError(f"config.json: {where}: mlp.ff must be positive")
    return LayerConfig(kind, mixer, mlp)


@dataclass
class TopelornConfig:
    width: int
    vocab: int
    norm_eps: float
    layers: List[LayerConfig]
    architecture: str = "Topelorn"
    dtype: str = "bfloat16"
    path: str = ""
    raw: Dict[str, Any] = field(default_factory=dict, repr=False, compare=False)

    # the names the rest of the engine reads a model's sizes by
    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def hidden_size(self) -> int:
        return self.width

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_hf(cls, cfg: Dict[str, Any], path: str = "") -> "TopelornConfig":
        norm = _section(cfg, "norm", "model")
        layers = cfg.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        out = cls(width=read_key(cfg, "width", kind=int), vocab=read_key(cfg, "vocab", kind=int),
                  norm_eps=read_key(norm, "eps", kind=float),
                  layers=[_read_layer(i, e) for i, e in enumerate(layers)],
                  architecture=str(cfg.get("architecture") or "Topelorn"),
                  dtype=str(cfg.get("torch_dtype") or "bfloat16"), path=path, raw=dict(cfg))
        out.validate()
        return out

    def validate(self) -> None:
        if self.width < 1 or self.vocab < 1 or not self.norm_eps > 0:
            raise ConfigError("config.json: width and vocab must be positive, norm.eps > 0")
        mixing = [l.mixer for l in self.layers if l.kind == "attention" and l.mixer.v_mix]
        if any(m.kv_heads * m.vdim != mixing[0].kv_heads * mixing[0].vdim for m in mixing):
            raise ConfigError("config.json: layers that mix values (v_mix) must have values of one width "
                              "(kv_heads * vdim)")

    def to_hf(self) -> Dict[str, Any]:
        def mask(w, keeps):
            if not w.size:
                return None
            return {"size": w.size, "keep_first": w.keep_first} if keeps else {"size": w.size}
        layers = []
        for l in self.layers:
            m = l.mixer
            if l.kind == "attention":
                mixer = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim,
                         "scale": m.scale, "mask": mask(m.window, True), "v_mix": m.v_mix}
            else:
                mixer = {"heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "vdim": m.vdim,
                         "kv_rank": m.kv_rank, "scale": m.scale, "mask": mask(m.window, False),
                         "rot": {"base": m.rot_base, "dims": m.rot_dims}}
            layers.append({"type": l.kind, "mixer": mixer,
                           "mlp": {"kind": "dense", "ff": l.mlp.ff} if l.mlp else None})
        return {"architecture": self.architecture, "width": self.width, "vocab": self.vocab,
                "norm": {"eps": self.norm_eps}, "layers": layers, "torch_dtype": self.dtype}
