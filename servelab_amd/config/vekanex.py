"""Configuration of the Vekanex design: a decoder whose config.json lists its layers, each with
one of three mixers and a routed feed-forward.

    {"architecture": "Vekanex", "width", "vocab", "norm": {"eps"}, "residual_mult",
     "logit_softcap", "layers": [{"type", "mixer": {...}, "mlp": {...} | null, "weights_of"?}]}

Mixers: ``mlstm`` (matrix memory with exponential gates: heads, dim, vdim, gate_cap), ``gla``
(gated linear attention with a decay per key channel: heads, dim, vdim, tau) and ``parallel``
(a softmax attention ``left`` beside a gated delta rule ``right``, added with ``left_scale`` and
``right_scale``).  Feed-forward: ``{"kind": "moe", "router": {"experts", "top"}, "expert":
{"ff"}, "shared": {"ff"} | absent}``.  A layer with ``weights_of: j`` runs layer j's tensors
against a cache of its own.

The widths of the low-rank projections (the decay's and the output gate's) are no config.json
keys: they are the shapes of the checkpoint's tensors and are read from there; a configuration
made without a checkpoint (random weights) names them as ``decay_rank`` / ``gate_rank``.
Nothing here is a default for a size or a constant of the model.
"""
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from .layered import _section
from .model import ConfigError, read_key


@dataclass(frozen=True)
class MatrixLSTMConfig:
    heads: int
    dim: int
    vdim: int
    gate_cap: float


@dataclass(frozen=True)
class GatedLinearConfig:
    heads: int
    dim: int
    vdim: int
    tau: float
    decay_rank: int


@dataclass(frozen=True)
class SoftmaxSideConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_base: float
    rot_dims: int


@dataclass(frozen=True)
class DeltaSideConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    decay_rank: int
    gate_rank: int


@dataclass(frozen=True)
class SideBySideConfig:
    left: SoftmaxSideConfig
    right: DeltaSideConfig
    left_scale: float
    right_scale: float


@dataclass(frozen=True)
class RoutedMlpConfig:
    experts: int
    top: int
    ff: int
    shared_ff: int               # 0: no shared expert


@dataclass(frozen=True)
class VekanexLayer:
    kind: str                    # "mlstm" | "gla" | "parallel"
    mixer: Any
    mlp: Optional[RoutedMlpConfig]
    weights_of: Optional[int] = None


def _positive(where, **values):
    bad = [k for k, v in values.items() if v < 1]
    if bad:
        raise ConfigError(f"config.json: {where}: {', '.join(bad)} must be positive")


def _rank(m: Dict[str, Any], key: str, tensor: str, shapes, where: str) -> int:
    """A low-rank projection's inner width: config.json's own key if it has one, else the first
    axis of the checkpoint's tensor."""
    if m.get(key) is not None:
        return read_key(m, key, kind=int)
    if shapes is None or tensor not in shapes:
        raise ConfigError(f"config.json: {where}: '{key}' is not given and the checkpoint has no "
                          f"tensor '{tensor}' to take it from")
    return int(shapes[tensor][0])


def _read_mixer(kind: str, m: Dict[str, Any], prefix: str, shapes, where: str):
    if kind == "mlstm":
        out = MatrixLSTMConfig(read_key(m, "heads", kind=int), read_key(m, "dim", kind=int),
                               read_key(m, "vdim", kind=int), read_key(m, "gate_cap", kind=float))
        _positive(where, heads=out.heads, dim=out.dim, vdim=out.vdim)
        if not out.gate_cap > 0:
            raise ConfigError(f"config.json: {where}: gate_cap must be positive")
        return out
    if kind == "gla":
        out = GatedLinearConfig(read_key(m, "heads", kind=int), read_key(m, "dim", kind=int),
                                read_key(m, "vdim", kind=int), read_key(m, "tau", kind=float),
                                _rank(m, "decay_rank", prefix + "a1", shapes, where))
        _positive(where, heads=out.heads, dim=out.dim, vdim=out.vdim, decay_rank=out.decay_rank)
        if not out.tau > 0:
            raise ConfigError(f"config.json: {where}: tau must be positive")
        return out
    if kind == "parallel":
        l, r = _section(m, "left", where), _section(m, "right", where)
        rot = _section(l, "rot", where + ".left")
        left = SoftmaxSideConfig(
            read_key(l, "heads", kind=int), read_key(l, "kv_heads", kind=int),
            read_key(l, "dim", kind=int), read_key(l, "vdim", kind=int),
            read_key(l, "scale", kind=float), read_key(rot, "base", kind=float),
            read_key(rot, "dims", kind=int))
        _positive(where + ".left", heads=left.heads, kv_heads=left.kv_heads, dim=left.dim, vdim=left.vdim)
        if left.heads % left.kv_heads:
            raise ConfigError(f"config.json: {where}.left: heads must be a multiple of kv_heads")
        if left.rot_dims % 2 or not 0 <= left.rot_dims <= left.dim or not left.rot_base > 0:
            raise ConfigError(f"config.json: {where}.left: rot.dims must be even and within dim, "
                              "rot.base positive")
        right = DeltaSideConfig(
            read_key(r, "heads", kind=int), read_key(r, "kv_heads", kind=int),
            read_key(r, "dim", kind=int), read_key(r, "vdim", kind=int),
            read_key(r, "conv", kind=int),
            _rank(r, "decay_rank", prefix + "right.a1", shapes, where + ".right"),
            _rank(r, "gate_rank", prefix + "right.g1", shapes, where + ".right"))
        _positive(where + ".right", heads=right.heads, kv_heads=right.kv_heads, dim=right.dim,
                  vdim=right.vdim, conv=right.conv, decay_rank=right.decay_rank,
                  gate_rank=right.gate_rank)
        if right.heads % right.kv_heads:
            raise ConfigError(f"config.json: {where}.right: heads must be a multiple of kv_heads")
        return SideBySideConfig(left, right, read_key(m, "left_scale", kind=float),
                                read_key(m, "right_scale", kind=float))
    raise ConfigError(f"config.json: {where}: type {kind!r} is not one of mlstm, gla, parallel")


def _read_mlp(raw, where: str) -> Optional[RoutedMlpConfig]:
    if raw is None:
        return None
    if not isinstance(raw, dict):
        raise ConfigError(f"config.json: {where}: 'mlp' must be an object or null")
    kind = read_key(raw, "kind", kind=str)
    if kind != "moe":
        raise ConfigError(f"config.json: {where}: mlp.kind {kind!r} is not supported (moe)")
    router, expert = _section(raw, "router", where), _section(raw, "expert", where)
    shared = _section(raw, "shared", where, required=False)
    out = RoutedMlpConfig(read_key(router, "experts", kind=int), read_key(router, "top", kind=int),
                          read_key(expert, "ff", kind=int),
                          read_key(shared, "ff", kind=int) if shared is not None else 0)
    _positive(where, experts=out.experts, top=out.top, ff=out.ff)
    if out.top > out.experts or out.shared_ff < 0:
        raise ConfigError(f"config.json: {where}: router.top must not exceed router.experts")
    return out


@dataclass
class VekanexConfig:
    width: int
    vocab: int
    norm_eps: float
    residual_mult: float
    logit_softcap: float
    layers: List[VekanexLayer]
    architecture: str = "Vekanex"
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

    @classmethod
    def from_hf(cls, cfg: Dict[str, Any], path: str = "") -> "VekanexConfig":
        norm = _section(cfg, "norm", "model")
        entries = cfg.get("layers")
        if not isinstance(entries, list) or not entries:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        shapes = None
        if path:
            try:
                from ..weights.loader import Checkpoint
                shapes = Checkpoint(path).shapes()
            except Exception:
                shapes = None                     # a folder without weights: the ranks must be keys
        layers = []
        for i, entry in enumerate(entries):
            where = f"layers[{i}]"
            if not isinstance(entry, dict):
                raise ConfigError(f"config.json: {where} must be an object")
            owner = entry.get("weights_of")
            if owner is not None:
                # the layer whose tensors these are, through any layers that borrow them in turn
                owner, seen = read_key(entry, "weights_of", kind=int), {i}
                while True:
                    if not 0 <= owner < len(entries) or owner in seen or not isinstance(entries[owner], dict):
                        raise ConfigError(f"config.json: {where}: weights_of must lead to another layer "
                                          "that has tensors of its own")
                    if entries[owner].get("weights_of") is None:
                        break
                    seen.add(owner)
                    owner = read_key(entries[owner], "weights_of", kind=int)
                # what the entry leaves out it takes from the owner's
                entry = dict(entries[owner], **{k: v for k, v in entry.items() if k != "weights_of"})
            kind = read_key(entry, "type", kind=str)
            prefix = f"l{i if owner is None else owner}.mix."
            mixer = _read_mixer(kind, _section(entry, "mixer", where), prefix, shapes, where)
            layers.append(VekanexLayer(kind, mixer, _read_mlp(entry.get("mlp"), where), owner))
        out = cls(width=read_key(cfg, "width", kind=int), vocab=read_key(cfg, "vocab", kind=int),
                  norm_eps=read_key(norm, "eps", kind=float),
                  residual_mult=read_key(cfg, "residual_mult", 1.0, kind=float),
                  logit_softcap=read_key(cfg, "logit_softcap", 0.0, kind=float), layers=layers,
                  architecture=str(cfg.get("architecture") or "Vekanex"),
                  dtype=str(cfg.get("torch_dtype") or "bfloat16"), path=path, raw=dict(cfg))
        out.validate()
        return out

    def validate(self) -> None:
        if self.width < 1 or self.vocab < 1 or not self.norm_eps > 0:
            raise ConfigError("config.json: width and vocab must be positive, norm.eps > 0")
        if self.logit_softcap < 0:                # 0 (or no key): the logits stay as they are
            raise ConfigError("config.json: logit_softcap must not be negative")
        for i, l in enumerate(self.layers):
            if l.weights_of is not None:
                o = self.layers[l.weights_of]
                if (o.kind, o.mixer, o.mlp) != (l.kind, l.mixer, l.mlp):
                    raise ConfigError(f"config.json: layers[{i}] uses the tensors of layer "
                                      f"{l.weights_of} but describes another layer")

    def to_hf(self) -> Dict[str, Any]:
        def mixer(l):
            m = l.mixer
            if l.kind == "mlstm":
                return {"heads": m.heads, "dim": m.dim, "vdim": m.vdim, "gate_cap": m.gate_cap}
            if l.kind == "gla":
                return {"heads": m.heads, "dim": m.dim, "vdim": m.vdim, "tau": m.tau,
                        "decay_rank": m.decay_rank}
            a, b = m.left, m.right
            return {"left": {"heads": a.heads, "kv_heads": a.kv_heads, "dim": a.dim, "vdim": a.vdim,
                             "scale": a.scale, "rot": {"base": a.rot_base, "dims": a.rot_dims}},
                    "right": {"heads": b.heads, "kv_heads": b.kv_heads, "dim": b.dim, "vdim": b.vdim,
                              "conv": b.conv, "decay_rank": b.decay_rank, "gate_rank": b.gate_rank},
                    "left_scale": m.left_scale, "right_scale": m.right_scale}

        def mlp(c):
            if c is None:
                return None
            out = {"kind": "moe", "router": {"experts": c.experts, "top": c.top}, "expert": {"ff": c.ff}}
            if c.shared_ff:
                out["shared"] = {"ff": c.shared_ff}
            return out
        layers = []
        for l in self.layers:
            entry = {"type": l.kind, "mixer": mixer(l), "mlp": mlp(l.mlp)}
            if l.weights_of is not None:
                entry["weights_of"] = l.weights_of
            layers.append(entry)
        return {"architecture": self.architecture, "width": self.width, "vocab": self.vocab,
                "norm": {"eps": self.norm_eps}, "residual_mult": self.residual_mult,
                "logit_softcap": self.logit_softcap, "layers": layers, "torch_dtype": self.dtype}
