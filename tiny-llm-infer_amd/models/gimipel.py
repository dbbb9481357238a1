"""Gimipel: from its typed configuration to a ``ModelSpec``.

A decoder whose blocks norm what a sublayer gives, not what it reads:  x <- x + n1(mixer(x)),
x <- x + n2(ff(x))  with n1, n2 RMS norms (a weight each).  Embedding: scale * E[token].  A layer's
mixer is either attention with two softmax maps a head over a sliding window that also keeps the
first positions of a sequence (no rotation; q and k of every head and map normed with one weight
vector; the heads' outputs gated), or attention whose keys and values are made from one normed
latent vector a position beside a turned key part that all heads share (only those two are kept in
the cache).  Its feed-forward, if it has one, is a set of routed experts (softmax scores, a
correction added for the choice only, the best groups of neighbouring router outputs first, the
last outputs standing for experts that hand their input on) beside a shared expert.  A layer may run
with another layer's weights and keeps a cache of its own all the same.  After the blocks: RMS norm
and the head (a matrix of its own).

Tensor names: ``embed``, ``final.norm``, ``head``, and for layer i ``l<i>.norm1|norm2``; an attention
mixer ``l<i>.mix.q|k|v|g|o``, ``.q.norm``, ``.k.norm``, ``.lq1|lk1|lq2|lk2``; a latent mixer
``l<i>.mix.q|dkv|uk|uv|o``, ``.dkv.norm``; ``l<i>.mlp.router``, ``l<i>.mlp.correction``,
``l<i>.mlp.e<j>.gate|up|down``, ``l<i>.mlp.shared.gate|up|down``.
"""
from __future__ import annotations

from ..config.base import BlockSpec, LayerCall, ModelSpec, PartSpec
from ..config.gimipel import ARCHITECTURE, NO_POSITION_LIMIT, GimipelConfig
from ..registry import register_architecture


def gimipel_spec(cfg: GimipelConfig) -> ModelSpec:
    limit = cfg.max_positions or NO_POSITION_LIMIT

    def rms(name: str, size: int) -> PartSpec:
        return PartSpec("rmsnorm", {"size": size, "eps": cfg.norm_eps}, {"weight": name})

    blocks, block_of = [], {}
    for i, layer in enumerate(cfg.layers):
        if layer.weights_of is not None:
            continue
        p = f"l{i}."
        m = layer.mixer
        if layer.kind == "attention":
            mixer = PartSpec(
                "differential_attention",
                {"hidden_size": cfg.width, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "head_dim": m.dim,
                 "value_dim": m.vdim, "scale": m.scale, "diff": m.diff, "window": m.window, "keep_first": m.keep_first,
                 "norm_eps": cfg.norm_eps},
                {"q": p + "mix.q", "k": p + "mix.k", "v": p + "mix.v", "gate": p + "mix.g", "o": p + "mix.o",
                 "lq1": p + "mix.lq1", "lk1": p + "mix.lk1", "lq2": p + "mix.lq2", "lk2": p + "mix.lk2"},
                {"q_norm": rms(p + "mix.q.norm", m.dim), "k_norm": rms(p + "mix.k.norm", m.dim)})
        else:
            mixer = PartSpec(
                "latent_attention",
                {"hidden_size": cfg.width, "num_heads": m.heads, "head_dim": m.dim, "rotary_dim": m.rot_dim,
                 "value_dim": m.vdim, "kv_rank": m.kv_rank, "scale": m.scale},
                {"q": p + "mix.q", "down": p + "mix.dkv", "up_k": p + "mix.uk", "up_v": p + "mix.uv", "o": p + "mix.o"},
                {"position": PartSpec("rope_neox", {"head_dim": m.rot_dim, "rotary_dim": m.rot_dims,
                                                    "theta": m.rot_base, "max_positions": limit}),
                 "latent_norm": rms(p + "mix.dkv.norm", m.kv_rank)})
        ffn, norms = None, {"mixer": rms(p + "norm1", cfg.width)}
        if layer.mlp is not None:
            f = layer.mlp
            names = {"router": p + "mlp.router", "correction": p + "mlp.correction", "experts": p + "mlp.e{}."}
            if f.shared_ff is not None:
                names.update({"shared_gate": p + "mlp.shared.gate", "shared_up": p + "mlp.shared.up",
                              "shared_down": p + "mlp.shared.down"})
            ffn = PartSpec("routed_experts",
                           {"hidden_size": cfg.width, "experts": f.experts, "identity": f.identity, "top": f.top,
                            "groups": f.groups, "keep": f.keep, "intermediate_size": f.ff,
                            "shared_intermediate_size": f.shared_ff, "score": "softmax", "group_score": "max",
                            "normalize": False}, names)
            norms["ffn"] = rms(p + "norm2", cfg.width)
        block_of[i] = len(blocks)
        blocks.append(BlockSpec("sublayer_postnorm", mixer, ffn, norms))
    schedule = []
    for i, layer in enumerate(cfg.layers):
        owner = i if layer.weights_of is None else layer.weights_of
        schedule.append(LayerCall(block=block_of[owner], cache=i))
    return ModelSpec(
        architecture=ARCHITECTURE,
        hidden_size=cfg.width,
        vocab_size=cfg.vocab,
        max_positions=limit,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab, "hidden_size": cfg.width,
                                               "scale": cfg.embedding_scale}, {"weight": "embed"}),
        blocks=tuple(blocks),
        schedule=tuple(schedule),
        final_norm=rms("final.norm", cfg.width),
        head=PartSpec("linear_head", {"vocab_size": cfg.vocab, "hidden_size": cfg.width, "tied": False},
                      {"weight": "head"}),
        eos_token_ids=cfg.eos_token_ids)


register_architecture(ARCHITECTURE, GimipelConfig.from_dict, gimipel_spec)
