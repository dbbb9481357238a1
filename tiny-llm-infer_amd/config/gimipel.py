"""Typed configuration of the Gimipel decoder, read from its config.json.

Keys: ``architecture`` ("Gimipel"), ``vocab``, ``width``, ``embedding.scale``, ``norm.eps``,
``max_positions`` (optional: the design itself sets no limit) and ``layers``: a list with one entry
a layer, ``{"type": "attention" | "latent_attention", "mixer": {...}, "mlp": {...} or null}``, and
optionally ``"weights_of": j``: the layer has no tensors of its own and runs with those of layer j
(of equal sizes), keeping a cache of its own.

An attention mixer (two softmax maps a head) gives ``heads``, ``kv_heads``, ``dim`` (of a query and
a key head of one map), ``vdim`` (of a value head), ``scale`` (of the scores), ``diff`` (the constant
in the weight of the second map) and optionally ``mask.size`` with ``mask.keep_first`` (a row sees
itself, the size - 1 before it and the first keep_first positions of its sequence).  A latent mixer
gives ``heads``, ``dim`` and ``rot_dim`` (the parts of a query/key head that are not and that are
turned), ``vdim``, ``kv_rank`` (of the latent vector a position), ``scale``, ``rot.dims`` and
``rot.base``.  A feed-forward gives ``kind`` ("moe"), ``expert.ff``, ``router.experts|top|identity``,
``router.groups.count|keep`` and optionally ``shared.ff``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple, Union

from .base import ConfigError, JsonReader

ARCHITECTURE = "Gimipel"
NO_POSITION_LIMIT = 1 << 20          # what a config.json without ``max_positions`` is taken to allow


@dataclass(frozen=True)
class GimipelAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    diff: float
    window: Optional[int]             # None: every earlier position is seen
    keep_first: int

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim,
                               "scale": self.scale, "diff": self.diff}
        if self.window is not None:
            out["mask"] = {"size": self.window, "keep_first": self.keep_first}
        return out


@dataclass(frozen=True)
class GimipelLatent:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    scale: float
    rot_dims: int
    rot_base: float

    def to_dict(self) -> Dict[str, Any]:
        return {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim, "kv_rank": self.kv_rank,
                "scale": self.scale, "rot": {"dims": self.rot_dims, "base": self.rot_base}}


@dataclass(frozen=True)
class GimipelExperts:
    experts: int                      # experts with matrices
    identity: int                     # further router outputs whose expert hands its input on
    top: int
    groups: int
    keep: int
    ff: int
    shared_ff: Optional[int]          # None: no shared expert

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"kind": "moe", "expert": {"ff": self.ff},
                               "router": {"experts": self.experts, "top": self.top, "identity": self.identity,
                                          "groups": {"count": self.groups, "keep": self.keep}}}
        if self.shared_ff is not None:
            out["shared"] = {"ff": self.shared_ff}
        return out


@dataclass(frozen=True)
class GimipelLayer:
    kind: str                                         # "attention" or "latent_attention"
    mixer: Union[GimipelAttention, GimipelLatent]
    mlp: Optional[GimipelExperts]
    weights_of: Optional[int] = None

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"type": self.kind, "mixer": self.mixer.to_dict(),
                               "mlp": None if self.mlp is None else self.mlp.to_dict()}
        if self.weights_of is not None:
            out["weights_of"] = self.weights_of
        return out


def _attention(m: JsonReader, where: str) -> GimipelAttention:
    heads = m.integer("heads", minimum=1)
    kv_heads = m.integer("kv_heads", heads, minimum=1)
    dim = m.integer("dim", minimum=1)
    vdim = m.integer("vdim", dim, minimum=1)
    if heads % kv_heads:
        raise ConfigError(f"{where}: heads {heads} must be a multiple of kv_heads {kv_heads}")
    window, keep_first = None, 0
    raw_mask = m.raw("mask")
    if raw_mask is not None:
        mask = JsonReader(raw_mask, where + ".mask")
        window = mask.integer("size", None, minimum=1)
        keep_first = mask.integer("keep_first", 0, minimum=0)
        if window is None:
            keep_first = 0
    return GimipelAttention(heads, kv_heads, dim, vdim, m.number("scale"), m.number("diff"), window, keep_first)


def _latent(m: JsonReader, where: str) -> GimipelLatent:
    heads = m.integer("heads", minimum=1)
    dim = m.integer("dim", minimum=1)
    rot_dim = m.integer("rot_dim", minimum=2)
    rot = JsonReader(m.raw("rot") or {}, where + ".rot")
    dims = rot.integer("dims", rot_dim, minimum=2)
    if dims % 2 or dims > rot_dim:
        raise ConfigError(f"{where}: rot.dims {dims} must be even and at most rot_dim {rot_dim}")
    return GimipelLatent(heads, dim, rot_dim, m.integer("vdim", dim, minimum=1), m.integer("kv_rank", minimum=1),
                         m.number("scale"), dims, rot.number("base"))


def _experts(f: JsonReader, where: str) -> GimipelExperts:
    kind = f.string("kind")
    if kind != "moe":
        raise ConfigError(f"{where}: feed-forward kind '{kind}' is not known; known: moe")
    r = JsonReader(f.raw("router") or {}, where + ".router")
    g = JsonReader(r.raw("groups") or {}, where + ".router.groups")
    experts = r.integer("experts", minimum=0)
    identity = r.integer("identity", 0, minimum=0)
    top = r.integer("top", minimum=1)
    groups = g.integer("count", 1, minimum=1)
    keep = g.integer("keep", groups, minimum=1)
    outputs = experts + identity
    if outputs < 1 or outputs % groups:
        raise ConfigError(f"{where}: {outputs} router outputs do not form {groups} equal groups")
    if keep > groups or keep * (outputs // groups) < top:
        raise ConfigError(f"{where}: {keep} of {groups} groups of {outputs // groups} cannot give {top} experts")
    ff = JsonReader(f.raw("expert") or {}, where + ".expert").integer("ff", minimum=1)
    shared = f.raw("shared")
    shared_ff = None if shared is None else JsonReader(shared, where + ".shared").integer("ff", minimum=1)
    return GimipelExperts(experts, identity, top, groups, keep, ff, shared_ff)


@dataclass(frozen=True)
class GimipelConfig:
    vocab: int
    width: int
    embedding_scale: float
    norm_eps: float
    layers: Tuple[GimipelLayer, ...]
    max_positions: Optional[int] = None
    eos_token_ids: Tuple[int, ...] = ()

    @staticmethod
    def from_dict(data: Dict[str, Any], origin: str = "config.json") -> "GimipelConfig":
        r = JsonReader(data, origin)
        name = r.string("architecture")
        if name != ARCHITECTURE:
            raise ConfigError(f"{origin}: architecture '{name}' is not '{ARCHITECTURE}'")
        vocab = r.integer("vocab", minimum=1)
        width = r.integer("width", minimum=1)
        scale = JsonReader(r.raw("embedding") or {}, origin + ": embedding").number("scale", 1.0)
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
            m = JsonReader(lr.raw("mixer") or {}, where + ".mixer")
            if kind == "attention":
                mixer = _attention(m, where + ".mixer")
            elif kind == "latent_attention":
                mixer = _latent(m, where + ".mixer")
            else:
                raise ConfigError(f"{where}: layer type '{kind}' is not known; known: attention, latent_attention")
            mlp = lr.raw("mlp")
            mlp = None if mlp is None else _experts(JsonReader(mlp, where + ".mlp"), where + ".mlp")
            layers.append(GimipelLayer(kind, mixer, mlp, lr.integer("weights_of", None)))
        for i, layer in enumerate(layers):
            of, hops = layer.weights_of, 0
            while of is not None:                       # (a layer may name one that itself names another)
                if not 0 <= of < len(layers) or of == i or hops > len(layers):
                    raise ConfigError(f"{origin}: layers[{i}]: weights_of must name another layer with tensors of its own")
                owner = layers[of]
                if owner.weights_of is None:
                    break
                of, hops = owner.weights_of, hops + 1
            if of is not None:
                if (owner.kind, owner.mixer, owner.mlp) != (layer.kind, layer.mixer, layer.mlp):
                    raise ConfigError(f"{origin}: layers[{i}] runs with the weights of layer {of} but has other sizes")
                layers[i] = GimipelLayer(layer.kind, layer.mixer, layer.mlp, of)
        return GimipelConfig(vocab=vocab, width=width, embedding_scale=scale, norm_eps=eps, layers=tuple(layers),
                             max_positions=r.integer("max_positions", None, minimum=1),
                             eos_token_ids=tuple(r.int_list("eos_token_id", [])))

    def to_dict(self) -> Dict[str, Any]:
        """The config.json this configuration is read back from."""
        out: Dict[str, Any] = {
            "architecture": ARCHITECTURE, "vocab": self.vocab, "width": self.width,
            "embedding": {"scale": self.embedding_scale}, "norm": {"eps": self.norm_eps},
            "layers": [layer.to_dict() for layer in self.layers],
        }
        if self.max_positions is not None:
            out["max_positions"] = self.max_positions
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids)
        return out
