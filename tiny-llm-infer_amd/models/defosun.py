"""Defosun: from its typed configuration to a ``ModelSpec``.

A pre-norm decoder, x <- x + mixer(n1(x)), x <- x + ff(n2(x)), whose RMS norms store their weight
around zero (the multiplier is 1 + w), optionally over several copies of the residual
(hyper-connections: a sublayer reads a weighted sum of the streams and is written back into all of
them).  A layer's mixer is one of: attention with grouped heads whose values are its keys before
they are turned, with biases, a partial rotation of the pairs (i, i + dims/2) and a sink in the
softmax's denominator; attention whose keys and values are made from one normed latent vector a
position beside a key part, turned in pairs of neighbours, that all heads share, with a sink;
lightning attention, a matrix of state a head that decays by a constant a token.  Its
feed-forward, if it has one, is the gated dense one or routed experts (softmax scores, the largest
chosen and weighing as they are, a limited gated activation) beside a shared expert with a gate of
its own.  A run of layers may be passed several times with the same tensors; every pass keeps a
cache or state of its own.  After the blocks: the norm and the head (a matrix of its own).

Tensor names: ``embed``, ``final.norm``, ``head``, and for layer i ``l<i>.norm1|norm2``,
``l<i>.hc1|hc2.in|out|mix`` (with streams); an attention mixer ``l<i>.mix.q|k|o``, ``.q.b``,
``.k.b``, ``.o.b``, ``.sink``; a latent mixer ``l<i>.mix.q|dkv|uk|uv|o``, ``.dkv.norm``, ``.sink``;
a lightning mixer ``l<i>.mix.q|k|v|g|o``, ``.norm``; a dense feed-forward ``l<i>.mlp.gate|up|down``;
routed experts ``l<i>.mlp.router``, ``l<i>.mlp.e<j>.gate|up|down``, ``l<i>.mlp.shared.gate|up|down|sg``.
"""
from __future__ import annotations

from ..config.base import BlockSpec, LayerCall, ModelSpec, PartSpec
from ..config.defosun import ARCHITECTURE, NO_POSITION_LIMIT, DefosunConfig, DefosunDense
from ..registry import register_architecture

GATE_SLOPE = 1.702       # of the experts' activation g * sigmoid(slope * g) * (u + 1)


def defosun_spec(cfg: DefosunConfig) -> ModelSpec:
    limit = cfg.max_positions or NO_POSITION_LIMIT

    def norm(name: str) -> PartSpec:          # the model's norm: the weight is stored around zero
        return PartSpec("rmsnorm", {"size": cfg.width, "eps": cfg.norm_eps, "weight_offset": 1.0}, {"weight": name})

    def plain_norm(name: str, size: int) -> PartSpec:
        return PartSpec("rmsnorm", {"size": size, "eps": cfg.norm_eps}, {"weight": name})

    blocks = []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        m = layer.mixer
        if layer.kind == "attention":
            mixer = PartSpec(
                "sink_attention",
                {"hidden_size": cfg.width, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "head_dim": m.dim,
                 "scale": m.scale, "values": "keys"},
                {"q": p + "mix.q", "k": p + "mix.k", "o": p + "mix.o", "q_bias": p + "mix.q.b", "k_bias": p + "mix.k.b",
                 "o_bias": p + "mix.o.b", "sink": p + "mix.sink"},
                {"position": PartSpec("rope_neox", {"head_dim": m.dim, "rotary_dim": m.rot_dims, "theta": m.rot_base,
                                                    "max_positions": limit})})
        elif layer.kind == "latent_attention":
            mixer = PartSpec(
                "latent_attention",
                {"hidden_size": cfg.width, "num_heads": m.heads, "head_dim": m.dim, "rotary_dim": m.rot_dim,
                 "value_dim": m.vdim, "kv_rank": m.kv_rank, "scale": m.scale},
                {"q": p + "mix.q", "down": p + "mix.dkv", "up_k": p + "mix.uk", "up_v": p + "mix.uv", "o": p + "mix.o",
                 "sink": p + "mix.sink"},
                {"position": PartSpec("rope_interleaved", {"head_dim": m.rot_dim, "rotary_dim": m.rot_dim,
                                                           "theta": m.rot_base, "max_positions": limit}),
                 "latent_norm": plain_norm(p + "mix.dkv.norm", m.kv_rank)})
        else:
            mixer = PartSpec(
                "lightning_attention",
                {"hidden_size": cfg.width, "num_heads": m.heads, "key_dim": m.dim, "value_dim": m.vdim,
                 "decay": list(m.decay), "norm_eps": cfg.norm_eps},
                {"q": p + "mix.q", "k": p + "mix.k", "v": p + "mix.v", "gate": p + "mix.g", "o": p + "mix.o",
                 "norm": p + "mix.norm"})
        ffn, norms = None, {"mixer": norm(p + "norm1")}
        f = layer.mlp
        if isinstance(f, DefosunDense):
            ffn = PartSpec("swiglu", {"hidden_size": cfg.width, "intermediate_size": f.ff},
                           {"gate": p + "mlp.gate", "up": p + "mlp.up", "down": p + "mlp.down"})
        elif f is not None:
            names = {"router": p + "mlp.router", "experts": p + "mlp.e{}."}
            if f.shared_ff is not None:
                names.update({"shared_gate": p + "mlp.shared.gate", "shared_up": p + "mlp.shared.up",
                              "shared_down": p + "mlp.shared.down", "shared_scale": p + "mlp.shared.sg"})
            ffn = PartSpec("routed_experts",
                           {"hidden_size": cfg.width, "experts": f.experts, "top": f.top, "intermediate_size": f.ff,
                            "shared_intermediate_size": f.shared_ff, "score": "softmax", "group_score": "max",
                            "normalize": False, "activation": "limited", "limit": f.limit, "shared_limit": f.shared_limit,
                            "gate_slope": GATE_SLOPE}, names)
        if ffn is not None:
            norms["ffn"] = norm(p + "norm2")
        if cfg.streams is None:
            blocks.append(BlockSpec("prenorm", mixer, ffn, norms))
        else:
            own = {"in1": p + "hc1.in", "out1": p + "hc1.out", "mix1": p + "hc1.mix"}
            if ffn is not None:
                own.update({"in2": p + "hc2.in", "out2": p + "hc2.out", "mix2": p + "hc2.mix"})
            blocks.append(BlockSpec("hyper_prenorm", mixer, ffn, norms, {"streams": cfg.streams, "width": cfg.width}, own))
    # a layer that is passed several times keeps a cache layer (or, by its place in the run order, state) a pass
    schedule, cache_layers = [], 0
    for i in cfg.run_order():
        if cfg.layers[i].kind == "lightning":
            schedule.append(LayerCall(block=i))
        else:
            schedule.append(LayerCall(block=i, cache=cache_layers))
            cache_layers += 1
    return ModelSpec(
        architecture=ARCHITECTURE,
        hidden_size=cfg.width,
        vocab_size=cfg.vocab,
        max_positions=limit,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab, "hidden_size": cfg.width}, {"weight": "embed"}),
        blocks=tuple(blocks),
        schedule=tuple(schedule),
        final_norm=norm("final.norm"),
        head=PartSpec("linear_head", {"vocab_size": cfg.vocab, "hidden_size": cfg.width, "tied": False},
                      {"weight": "head"}),
        eos_token_ids=cfg.eos_token_ids)


register_architecture(ARCHITECTURE, DefosunConfig.from_dict, defosun_spec)
