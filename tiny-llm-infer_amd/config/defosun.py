"""Typed configuration of the Defosun decoder, read from its config.json.

Keys: ``architecture`` ("Defosun"), ``vocab``, ``width``, ``norm.eps``, ``streams`` (optional: the
number of copies of the residual that hyper-connections keep; without it one plain residual),
``loop`` (optional: ``start``, ``stop``, ``times``: layers start .. stop - 1 run ``times`` times in a
row with the same tensors, every pass with a cache or state of its own), ``max_positions``
(optional: the design itself sets no limit) and ``layers``: a list with one entry a layer,
``{"type": "attention" | "latent_attention" | "lightning", "mixer": {...}, "mlp": {...} or null}``.

An attention mixer gives ``heads``, ``kv_heads``, ``dim`` (of a query/key head, and of a value
head: the values are the keys), ``scale``, ``rot.dims`` and ``rot.base``.  A latent mixer gives
``heads``, ``dim`` and ``rot_dim`` (the parts of a query/key head that are not and that are
turned), ``vdim``, ``kv_rank`` (of the latent vector a position), ``scale`` and ``rot.base``.  A
lightning mixer gives ``heads``, ``dim``, ``vdim`` and ``decay`` (one number a head).  A
feed-forward gives ``kind``: "dense" with ``ff``, or "moe" with ``expert.ff``, ``expert.limit``,
``router.experts``, ``router.top`` and optionally ``shared.ff`` with ``shared.limit``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple, Union

from .base import ConfigError, JsonReader

ARCHITECTURE = "Defosun"
NO_POSITION_LIMIT = 1 << 20          # what a config.json without ``max_positions`` is taken to allow


@dataclass(frozen=True)
class DefosunAttention:
    heads: int
    kv_heads: int
    dim: int
    scale: float
    rot_dims: int
    rot_base: float

    def to_dict(self) -> Dict[str, Any]:
        return {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.dim, "scale": self.scale,
                "rot": {"dims": self.rot_dims, "base": self.rot_base}}


@dataclass(frozen=True)
class DefosunLatent:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    scale: float
    rot_base: float

    def to_dict(self) -> Dict[str, Any]:
        return {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim, "kv_rank": self.kv_rank,
                "scale": self.scale, "rot": {"dims": self.rot_dim, "base": self.rot_base}}


@dataclass(frozen=True)
class DefosunLightning:
    heads: int
    dim: int
    vdim: int
    decay: Tuple[float, ...]

    def to_dict(self) -> Dict[str, Any]:
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "decay": list(self.decay)}


@dataclass(frozen=True)
class DefosunDense:
    ff: int

    def to_dict(self) -> Dict[str, Any]:
        return {"kind": "dense", "ff": self.ff}


@dataclass(frozen=True)
class DefosunExperts:
    experts: int
    top: int
    ff: int
    limit: float
    shared_ff: Optional[int]          # None: no shared expert
    shared_limit: float

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"kind": "moe", "expert": {"ff": self.ff, "limit": self.limit},
                               "router": {"experts": self.experts, "top": self.top}}
        if self.shared_ff is not None:
            out["shared"] = {"ff": self.shared_ff, "limit": self.shared_limit}
        return out


@dataclass(frozen=True)
class DefosunLayer:
    kind: str                                         # "attention", "latent_attention" or "lightning"
    mixer: Union[DefosunAttention, DefosunLatent, DefosunLightning]
    mlp: Union[None, DefosunDense, DefosunExperts]

    def to_dict(self) -> Dict[str, Any]:
        return {"type": self.kind, "mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict()}


def _rotation(m: JsonReader, where: str, default_dims: int, most: int) -> Tuple[int, float]:
    rot = JsonReader(m.raw("rot") or {}, where + ".rot")
    dims = rot.integer("dims", default_dims, minimum=2)
    if dims % 2 or dims > most:
        raise ConfigError(f"{where}: rot.dims {dims} must be even and at most {most}")
    base = rot.number("base")
    if base <= 0.0:
        raise ConfigError(f"{where}: rot.base must be positive")
    return dims, base


def _attention(m: JsonReader, where: str) -> DefosunAttention:
    heads = m.integer("heads", minimum=1)
    kv_heads = m.integer("kv_heads", heads, minimum=1)
    dim = m.integer("dim", minimum=2)
    vdim = m.integer("vdim", dim, minimum=1)
    if heads % kv_heads:
        raise ConfigError(f"{where}: heads {heads} must be a multiple of kv_heads {kv_heads}")
    if vdim != dim:
        raise ConfigError(f"{where}: the values of this attention are its keys, so vdim {vdim} must equal dim {dim}")
    dims, base = _rotation(m, where, dim, dim)
    return DefosunAttention(heads, kv_heads, dim, m.number("scale"), dims, base)


def _latent(m: JsonReader, where: str) -> DefosunLatent:
    heads = m.integer("heads", minimum=1)
    dim = m.integer("dim", minimum=1)
    rot_dim = m.integer("rot_dim", minimum=2)
    dims, base = _rotation(m, where, rot_dim, rot_dim)
    if dims != rot_dim:
        raise ConfigError(f"{where}: the whole turned part is turned: rot.dims {dims} must equal rot_dim {rot_dim}")
    return DefosunLatent(heads, dim, rot_dim, m.integer("vdim", dim, minimum=1), m.integer("kv_rank", minimum=1),
                         m.number("scale"), base)


def _lightning(m: JsonReader, where: str) -> DefosunLightning:
    heads = m.integer("heads", minimum=1)
    dim = m.integer("dim", minimum=1)
    decay = m.raw("decay")
    if isinstance(decay, (int, float)) and not isinstance(decay, bool):
        decay = [decay] * heads
    if (not isinstance(decay, (list, tuple)) or len(decay) != heads
            or any(isinstance(x, bool) or not isinstance(x, (int, float)) for x in decay)):
        raise ConfigError(f"{where}: 'decay' must be a list of {heads} numbers, one a head")
    return DefosunLightning(heads, dim, m.integer("vdim", dim, minimum=1), tuple(float(x) for x in decay))


def _limit(r: JsonReader, where: str) -> float:
    limit = r.number("limit")
    if limit <= 0.0:
        raise ConfigError(f"{where}: limit must be positive")
    return limit


def _mlp(f: JsonReader, where: str) -> Union[DefosunDense, DefosunExperts]:
    kind = f.string("kind")
    if kind == "dense":
        return DefosunDense(f.integer("ff", minimum=1))
    if kind != "moe":
        raise ConfigError(f"{where}: feed-forward kind '{kind}' is not known; known: dense, moe")
    r = JsonReader(f.raw("router") or {}, where + ".router")
    experts = r.integer("experts", minimum=1)
    top = r.integer("top", minimum=1)
    if top > experts:
        raise ConfigError(f"{where}: {experts} experts cannot give {top}")
    e = JsonReader(f.raw("expert") or {}, where + ".expert")
    ff, limit = e.integer("ff", minimum=1), _limit(e, where + ".expert")
    shared_ff, shared_limit = None, limit
    if f.raw("shared") is not None:
        s = JsonReader(f.raw("shared"), where + ".shared")
        shared_ff, shared_limit = s.integer("ff", minimum=1), _limit(s, where + ".shared")
    return DefosunExperts(experts, top, ff, limit, shared_ff, shared_limit)


_MIXERS = {"attention": _attention, "latent_attention": _latent, "lightning": _lightning}


@dataclass(frozen=True)
class DefosunConfig:
    vocab: int
    width: int
    norm_eps: float
    layers: Tuple[DefosunLayer, ...]
    streams: Optional[int] = None                     # None: one plain residual
    loop: Optional[Tuple[int, int, int]] = None       # (start, stop, times)
    max_positions: Optional[int] = None
    eos_token_ids: Tuple[int, ...] = ()

    def run_order(self) -> Tuple[int, ...]:
        """The layers in the order they run, a looped layer once a pass."""
        n = len(self.layers)
        if self.loop is None:
            return tuple(range(n))
        start, stop, times = self.loop
        return tuple(range(start)) + tuple(range(start, stop)) * times + tuple(range(stop, n))

    @staticmethod
    def from_dict(data: Dict[str, Any], origin: str = "config.json") -> "DefosunConfig":
        r = JsonReader(data, origin)
        name = r.string("architecture")
        if name != ARCHITECTURE:
            raise ConfigError(f"{origin}: architecture '{name}' is not '{ARCHITECTURE}'")
        vocab = r.integer("vocab", minimum=1)
        width = r.integer("width", minimum=1)
        eps = JsonReader(r.raw("norm") or {}, origin + ": norm").number("eps")
        if eps <= 0.0:
            raise ConfigError(f"{origin}: norm.eps must be positive")
        raw_layers = r.raw("layers")
        if not isinstance(raw_layers, list) or not raw_layers:
            raise ConfigError(f"{origin}: 'layers' must be a non-empty list")
        layers = []
        for i, entry in enumerate(raw_layers):
            where = f"{origin}: layers[{i}]"
            lr = JsonReader(entry, where)
            kind = lr.string("type")
            if kind not in _MIXERS:
                raise ConfigError(f"{where}: layer type '{kind}' is not known; known: {', '.join(sorted(_MIXERS))}")
            mixer = _MIXERS[kind](JsonReader(lr.raw("mixer") or {}, where + ".mixer"), where + ".mixer")
            mlp = lr.raw("mlp")
            layers.append(DefosunLayer(kind, mixer, None if mlp is None else _mlp(JsonReader(mlp, where + ".mlp"), where + ".mlp")))
        loop = None
        if r.raw("loop") is not None:
            lp = JsonReader(r.raw("loop"), origin + ": loop")
            start, stop, times = lp.integer("start", minimum=0), lp.integer("stop", minimum=0), lp.integer("times", 1, minimum=1)
            if not start <= stop <= len(layers):
                raise ConfigError(f"{origin}: loop {start}..{stop} does not lie within the {len(layers)} layers")
            if stop > start and times > 1:
                loop = (start, stop, times)
        return DefosunConfig(vocab=vocab, width=width, norm_eps=eps, layers=tuple(layers),
                             streams=r.integer("streams", None, minimum=1), loop=loop,
                             max_positions=r.integer("max_positions", None, minimum=1),
                             eos_token_ids=tuple(r.int_list("eos_token_id", [])))

    def to_dict(self) -> Dict[str, Any]:
        """The config.json this configuration is read back from."""
        out: Dict[str, Any] = {
            "architecture": ARCHITECTURE, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
            "layers": [layer.to_dict() for layer in self.layers],
        }
        if self.streams is not None:
            out["streams"] = self.streams
        if self.loop is not None:
            out["loop"] = {"start": self.loop[0], "stop": self.loop[1], "times": self.loop[2]}
        if self.max_positions is not None:
            out["max_positions"] = self.max_positions
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids)
        return out
