"""A Ravenex model as a list of parts.

Every layer is a ``sandwich`` block (a norm before and after each sublayer, the normed result
times ``residual_mult`` into the stream) around a ``latent_attention`` mixer, a dense gated
feed-forward (tanh-form gelu), a top-k sigmoid mixture of experts (silu) or none, and the
per-layer token input (``gated_token_table``) when the model has one.  A layer with ``kv_from``
reads the cache of the layer it names; that layer's cache keeps what the widest of its readers
needs.  Tensor names: ``l<i>.norm1``, ``.norm1b``, ``.norm2``, ``.norm2b``, ``.mix.*``, ``.mlp.*``,
``.side.*``; ``embed``, ``side.embed``, ``final.norm``, ``head``.
"""
from __future__ import annotations

from .ravenex import RavenexConfig
from .registry import register_architecture
from ..parts.base import PartSpec, BlockSpec, LayerCall, ModelSpec


def build_spec(cfg: RavenexConfig) -> ModelSpec:
    d, eps, m = cfg.width, cfg.norm_eps, cfg.residual_mult
    n_layers = len(cfg.layers)
    # what every cache has to keep: the widest reach of the layers that read it
    reach = {}
    for i, layer in enumerate(cfg.layers):
        owner = i if layer.mixer.kv_from is None else layer.mixer.kv_from
        w = layer.mixer.window
        if owner not in reach:
            reach[owner] = w
        elif reach[owner] is not None:
            reach[owner] = None if w is None else max(reach[owner], w)
    blocks, order = [], []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        mx = layer.mixer
        owner = i if mx.kv_from is None else mx.kv_from
        norm = lambda name: PartSpec("rms", {"width": d, "eps": eps}, {"weight": p + name})
        position = PartSpec("rotary", {"head_dim": mx.rot_dims, "theta": mx.rot_base, "pairing": "adjacent",
                                       "rotary_dim": mx.rot_dims})
        names = {k: f"{p}mix.{k}" for k in ("q", "uk", "uv", "o")}
        if mx.kv_from is None:
            names.update({"dkv": p + "mix.dkv", "dkv.norm": p + "mix.dkv.norm"})
        keep = reach[owner]
        mixer = PartSpec("latent_attention", dict(
            hidden_size=d, n_heads=mx.heads, dim=mx.dim, rot_dim=mx.rot_dim, v_dim=mx.vdim, kv_rank=mx.kv_rank,
            scale=mx.scale, position=position, norm_eps=eps,
            visibility="full" if mx.window is None else "window", span=mx.window or 0, own_kv=mx.kv_from is None,
            cache_visibility="full" if keep is None else "window", cache_span=keep or 0), names)
        ffn = norm2 = None
        extra = {"norm1b": norm("norm1b"), "residual_mult": m}
        if layer.mlp is not None:
            f = p + "mlp."
            norm2, extra["norm2b"] = norm("norm2"), norm("norm2b")
            if layer.mlp.kind == "dense":
                ffn = PartSpec("dense_glu", dict(hidden_size=d, intermediate_size=layer.mlp.ff, activation="gelu_tanh"),
                               {"gate_proj": f + "gate", "up_proj": f + "up", "down_proj": f + "down"})
            else:
                ml = layer.mlp
                fn = {"router": f + "router", "correction": f + "correction"}
                for e in range(ml.experts):
                    fn.update({f"e{e}.{k}": f"{f}e{e}.{k}" for k in ("gate", "up", "down")})
                if ml.shared_ff is not None:
                    fn.update({f"shared.{k}": f"{f}shared.{k}" for k in ("gate", "up", "down")})
                ffn = PartSpec("moe_topk_sigmoid", dict(
                    hidden_size=d, intermediate_size=ml.expert_ff, n_experts=ml.experts, top_k=ml.top,
                    shared_intermediate_size=ml.shared_ff, score_bias=True, renormalize=False, activation="silu"), fn)
        if cfg.side_dim is not None:
            extra["side"] = PartSpec("gated_token_table", dict(
                vocab_size=cfg.vocab, width=d, dim=cfg.side_dim, n_layers=n_layers, layer=i, eps=eps, mult=m),
                {"embed": "side.embed", "gate": p + "side.gate", "proj": p + "side.proj", "norm": p + "side.norm"})
        blocks.append(BlockSpec("sandwich", norm("norm1"), mixer, norm2, ffn, extra))
        order.append(LayerCall(block=i, cache=owner, write=owner == i))
    return ModelSpec(
        architecture=cfg.architecture, vocab_size=cfg.vocab, hidden_size=d, blocks=blocks, order=order,
        final_norm=PartSpec("rms", {"width": d, "eps": eps}, {"weight": "final.norm"}),
        embed_name="embed", head_name="head", eos_token_ids=cfg.eos_token_ids, max_position=cfg.max_position,
        strip_prefixes=())


register_architecture("Ravenex", RavenexConfig.from_dict, build_spec)
