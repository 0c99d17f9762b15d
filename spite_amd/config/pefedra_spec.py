"""A Pefedra model as a list of parts.

Every layer is a ``parallel`` block: mixer and feed-forward read the same stream through a norm
each and join it together, and the mixer's input passes a ``token_shift`` first.  Both kinds of
mixer are ``wide_attention`` with biases and a sliding window: ``attention`` with two score maps a
head and linearly scaled rotation frequencies where the configuration says so, ``attention_2`` with
the norm over the whole q and k projections, values that turn with the rotation's base (unscaled)
and a gate per head.  The feed-forward is ``dense_mlp`` with the erf form of gelu.  The embedding's
rows are multiplied by ``embedding.scale``.  Tensor names: ``l<i>.norm1``, ``.norm2``, ``.shift``,
``.mix.q|k|v`` with ``.b`` for the biases, ``.mix.o``, ``.mix.q.norm|k.norm|g`` or
``.mix.lq1|lk1|lq2|lk2``, ``.mlp.up|down``; ``embed``, ``final.norm``, ``head``.
"""
from __future__ import annotations

from .pefedra import PefedraConfig
from .registry import register_architecture
from ..parts.base import PartSpec, BlockSpec, LayerCall, ModelSpec


def build_spec(cfg: PefedraConfig) -> ModelSpec:
    d, eps = cfg.width, cfg.norm_eps
    blocks, order = [], []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        mx = layer.mixer
        norm = lambda name: PartSpec("rms", {"width": d, "eps": eps}, {"weight": p + name})
        position = None
        if mx.rot_base is not None and mx.rot_dims > 0:
            scaling = None if mx.rot_factor == 1.0 else {"rope_type": "linear", "factor": mx.rot_factor}
            position = PartSpec("rotary", {"head_dim": mx.dim, "theta": mx.rot_base, "rotary_dim": mx.rot_dims,
                                           "scaling": scaling})
        names = {"q_proj": p + "mix.q", "k_proj": p + "mix.k", "v_proj": p + "mix.v", "o_proj": p + "mix.o",
                 "q_bias": p + "mix.q.b", "k_bias": p + "mix.k.b", "v_bias": p + "mix.v.b"}
        args = dict(hidden_size=d, n_heads=mx.heads, n_kv_heads=mx.kv_heads, key_dim=mx.dim, value_dim=mx.vdim,
                    scale=mx.scale, position=position, visibility="full" if mx.window is None else "window",
                    span=mx.window or 0, bias=True, norm_eps=eps)
        if layer.type == "attention":
            args.update(maps=2, diff=mx.diff)
            names.update({f"lambda_{k}": f"{p}mix.l{k}" for k in ("q1", "k1", "q2", "k2")})
        else:
            args.update(projection_norm=True, head_gate=True,
                        value_position=PartSpec("rotary", {"head_dim": mx.vdim, "theta": mx.rot_base}))
            names.update({"q_norm": p + "mix.q.norm", "k_norm": p + "mix.k.norm", "gate_proj": p + "mix.g"})
        mixer = PartSpec("wide_attention", args, names)
        norm2 = ffn = None
        if layer.mlp is not None:
            norm2 = norm("norm2")
            ffn = PartSpec("dense_mlp", dict(hidden_size=d, intermediate_size=layer.mlp.ff, activation="gelu"),
                           {"up_proj": p + "mlp.up", "down_proj": p + "mlp.down"})
        shift = PartSpec("token_shift", {"width": d}, {"weight": p + "shift"})
        blocks.append(BlockSpec("parallel", norm("norm1"), mixer, norm2, ffn, {"shift": shift}))
        order.append(LayerCall(block=i, cache={"mixer": 2 * i, "shift": 2 * i + 1}))
    return ModelSpec(
        architecture=cfg.architecture, vocab_size=cfg.vocab, hidden_size=d, blocks=blocks, order=order,
        final_norm=PartSpec("rms", {"width": d, "eps": eps}, {"weight": "final.norm"}),
        embedding=PartSpec("token_table", {"vocab_size": cfg.vocab, "width": d, "scale": cfg.embed_scale}, {"weight": "embed"}),
        head_name="head", eos_token_ids=cfg.eos_token_ids, max_position=cfg.max_position, strip_prefixes=())


register_architecture("Pefedra", PefedraConfig.from_dict, build_spec)
