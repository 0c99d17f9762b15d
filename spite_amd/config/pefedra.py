"""Typed configuration of the Pefedra design, read from the keys of its ``config.json``.

``architecture`` names the design; ``vocab``, ``width``, ``norm.eps`` and ``embedding.scale`` are
the model's own; ``layers`` lists the layers in order, each with its ``type`` (the kind of mixer:
``attention``, with two score maps a head, or ``attention_2``, with a norm over the whole q and k
projections, turned values and a gate per head), the mixer's sizes and constants under ``mixer``
and its feed-forward under ``mlp`` (``null``: none).  Every size and constant is read here; every
problem found is reported in one ``ConfigError``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Optional, Tuple

from .llama4 import ConfigError

MIXER_TYPES = ("attention", "attention_2")
MLP_KINDS = ("dense",)


@dataclass(frozen=True)
class PefedraMixer:
    heads: int
    kv_heads: int
    dim: int                      # query/key size of a head (of each of its maps)
    vdim: int                     # value size of a head
    scale: float
    window: Optional[int]         # mask.size; None: every earlier key
    rot_base: Optional[float]     # None: no rotation of q and k
    rot_dims: int                 # how many leading elements of a head turn
    rot_factor: float             # rot.scaling.factor: every frequency divided by it (1: none)
    diff: float = 0.0             # ``attention`` only


@dataclass(frozen=True)
class PefedraMlp:
    kind: str
    ff: int


@dataclass(frozen=True)
class PefedraLayer:
    type: str
    mixer: PefedraMixer
    mlp: Optional[PefedraMlp]


@dataclass(frozen=True)
class PefedraConfig:
    architecture: str
    vocab: int
    width: int
    norm_eps: float
    embed_scale: float
    layers: Tuple[PefedraLayer, ...]
    torch_dtype: str = "bfloat16"
    eos_token_ids: Tuple[int, ...] = ()
    max_position: int = 1 << 20

    @staticmethod
    def from_dict(raw: Mapping[str, Any]) -> "PefedraConfig":
        problems = []

        def need(d, key, kind, where, positive=True):
            if not isinstance(d, Mapping) or key not in d or d[key] is None:
                problems.append(f"{where}{key} is missing")
                return kind(1)
            try:
                v = kind(d[key])
            except (TypeError, ValueError):
                problems.append(f"{where}{key} = {d[key]!r} is no {kind.__name__}")
                return kind(1)
            if positive and not v > 0:
                problems.append(f"{where}{key} = {v} must be positive")
            return v

        layers = []
        raw_layers = raw.get("layers")
        if not isinstance(raw_layers, (list, tuple)) or not raw_layers:
            problems.append("layers is missing or empty")
            raw_layers = []
        for i, L in enumerate(raw_layers):
            w = f"layers[{i}]."
            kind = L.get("type") if isinstance(L, Mapping) else None
            if kind not in MIXER_TYPES:
                problems.append(f"{w}type = {kind!r} (known: {', '.join(MIXER_TYPES)})")
                continue
            mx = L.get("mixer") or {}
            wm = w + "mixer."
            mask, rot = mx.get("mask"), mx.get("rot")
            window = None if mask is None else need(mask, "size", int, wm + "mask.")
            rot_base, rot_dims, rot_factor = None, 0, 1.0
            if rot is not None:
                rot_base, rot_dims = need(rot, "base", float, wm + "rot."), need(rot, "dims", int, wm + "rot.")
                if rot.get("scaling") is not None:
                    rot_factor = need(rot["scaling"], "factor", float, wm + "rot.scaling.")
            mixer = PefedraMixer(
                heads=need(mx, "heads", int, wm), kv_heads=need(mx, "kv_heads", int, wm), dim=need(mx, "dim", int, wm),
                vdim=need(mx, "vdim", int, wm), scale=need(mx, "scale", float, wm), window=window,
                rot_base=rot_base, rot_dims=rot_dims, rot_factor=rot_factor,
                diff=need(mx, "diff", float, wm, positive=False) if kind == "attention" else 0.0)
            if mixer.heads % mixer.kv_heads:
                problems.append(f"{wm}heads = {mixer.heads} is no multiple of kv_heads = {mixer.kv_heads}")
            if mixer.rot_dims % 2 or mixer.rot_dims > mixer.dim:
                problems.append(f"{wm}rot.dims = {mixer.rot_dims} must be even and at most dim = {mixer.dim}")
            if kind == "attention_2":
                if rot is None:
                    problems.append(f"{wm}rot is missing (the values turn with its base)")
                if mixer.vdim % 2:
                    problems.append(f"{wm}vdim = {mixer.vdim} must be even (the values turn in pairs)")
            mlp = None
            rm = L.get("mlp")
            if rm is not None:
                k = rm.get("kind") if isinstance(rm, Mapping) else None
                if k == "dense":
                    mlp = PefedraMlp("dense", ff=need(rm, "ff", int, w + "mlp."))
                else:
                    problems.append(f"{w}mlp.kind = {k!r} (known: {', '.join(MLP_KINDS)})")
            layers.append(PefedraLayer(kind, mixer, mlp))
        emb = raw.get("embedding")
        cfg = PefedraConfig(
            architecture=str(raw.get("architecture", "Pefedra")),
            vocab=need(raw, "vocab", int, ""), width=need(raw, "width", int, ""),
            norm_eps=need(raw.get("norm") or {}, "eps", float, "norm."),
            embed_scale=1.0 if emb is None else need(emb, "scale", float, "embedding.", positive=False),
            layers=tuple(layers), torch_dtype=str(raw.get("torch_dtype", "bfloat16")),
            eos_token_ids=tuple(int(t) for t in raw.get("eos_token_ids", ()) or ()),
            max_position=int(raw.get("max_position", 1 << 20)))
        if problems:
            raise ConfigError("config.json does not describe a Pefedra model: " + "; ".join(problems))
        return cfg
