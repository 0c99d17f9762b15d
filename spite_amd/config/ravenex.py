"""Typed configuration of the Ravenex design, read from the keys of its ``config.json``.

``architecture`` names the design; ``vocab``, ``width``, ``residual_mult``, ``norm.eps`` and
``token_side.dim`` are the model's own; ``layers`` lists the layers in order, each with its
``type`` (the kind of mixer), the mixer's sizes and constants under ``mixer`` and its
feed-forward under ``mlp`` (``null``: none).  Every size and constant is read here; every
problem found is reported in one ``ConfigError``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Optional, Tuple

from .llama4 import ConfigError

MIXER_TYPES = ("latent_attention",)
MLP_KINDS = ("dense", "moe")


@dataclass(frozen=True)
class LatentAttentionConfig:
    heads: int
    dim: int                      # unrotated query/key size of a head
    rot_dim: int                  # rotated query/key size of a head (the key's part is shared by the heads)
    vdim: int                     # value size of a head
    kv_rank: int                  # size of the latent
    scale: float
    rot_base: float
    rot_dims: int                 # how many leading elements of the rotated part turn
    window: Optional[int]         # mask.size; None: every earlier key
    kv_from: Optional[int]        # the layer whose latent and rotated key part this one reads


@dataclass(frozen=True)
class MlpConfig:
    kind: str                     # "dense" | "moe"
    ff: int = 0                   # dense: inner width
    experts: int = 0
    top: int = 0
    expert_ff: int = 0
    shared_ff: Optional[int] = None


@dataclass(frozen=True)
class LayerConfig:
    type: str
    mixer: LatentAttentionConfig
    mlp: Optional[MlpConfig]


@dataclass(frozen=True)
class RavenexConfig:
    architecture: str
    vocab: int
    width: int
    residual_mult: float
    norm_eps: float
    side_dim: Optional[int]       # token_side.dim; None: no per-layer token input
    layers: Tuple[LayerConfig, ...]
    torch_dtype: str = "bfloat16"
    eos_token_ids: Tuple[int, ...] = ()
    max_position: int = 1 << 20

    @staticmethod
    def from_dict(raw: Mapping[str, Any]) -> "RavenexConfig":
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
            rot = mx.get("rot") or {}
            mask = mx.get("mask")
            window = None
            if mask is not None:
                window = need(mask, "size", int, wm + "mask.")
            kv_from = mx.get("kv_from")
            mixer = LatentAttentionConfig(
                heads=need(mx, "heads", int, wm), dim=need(mx, "dim", int, wm), rot_dim=need(mx, "rot_dim", int, wm),
                vdim=need(mx, "vdim", int, wm), kv_rank=need(mx, "kv_rank", int, wm), scale=need(mx, "scale", float, wm),
                rot_base=need(rot, "base", float, wm + "rot."), rot_dims=need(rot, "dims", int, wm + "rot."),
                window=window, kv_from=None if kv_from is None else int(kv_from))
            if mixer.rot_dims % 2 or mixer.rot_dims > mixer.rot_dim:
                problems.append(f"{wm}rot.dims = {mixer.rot_dims} must be even and at most rot_dim = {mixer.rot_dim}")
            mlp = None
            rm = L.get("mlp")
            if rm is not None:
                wl = w + "mlp."
                k = rm.get("kind")
                if k == "dense":
                    mlp = MlpConfig("dense", ff=need(rm, "ff", int, wl))
                elif k == "moe":
                    router, shared = rm.get("router") or {}, rm.get("shared")
                    mlp = MlpConfig("moe", experts=need(router, "experts", int, wl + "router."),
                                    top=need(router, "top", int, wl + "router."),
                                    expert_ff=need(rm.get("expert") or {}, "ff", int, wl + "expert."),
                                    shared_ff=None if shared is None else need(shared, "ff", int, wl + "shared."))
                    if mlp.top > mlp.experts:
                        problems.append(f"{wl}router.top = {mlp.top} of {mlp.experts} experts")
                else:
                    problems.append(f"{wl}kind = {k!r} (known: {', '.join(MLP_KINDS)})")
            layers.append(LayerConfig(kind, mixer, mlp))
        for i, L in enumerate(layers):
            j = L.mixer.kv_from
            if j is None:
                continue
            if not 0 <= j < i or layers[j].mixer.kv_from is not None:
                problems.append(f"layers[{i}].mixer.kv_from = {j} must name an earlier layer with a latent of its own")
                continue
            a, b = L.mixer, layers[j].mixer
            if (a.kv_rank, a.rot_dim, a.rot_base, a.rot_dims) != (b.kv_rank, b.rot_dim, b.rot_base, b.rot_dims):
                problems.append(f"layers[{i}] reads the latent of layers[{j}] but differs in kv_rank, rot_dim or rot")
        side = raw.get("token_side")
        cfg = RavenexConfig(
            architecture=str(raw.get("architecture", "Ravenex")),
            vocab=need(raw, "vocab", int, ""), width=need(raw, "width", int, ""),
            residual_mult=need(raw, "residual_mult", float, "", positive=False),
            norm_eps=need(raw.get("norm") or {}, "eps", float, "norm.", positive=False),
            side_dim=None if side is None else need(side, "dim", int, "token_side."),
            layers=tuple(layers), torch_dtype=str(raw.get("torch_dtype", "bfloat16")),
            eos_token_ids=tuple(int(t) for t in raw.get("eos_token_ids", ()) or ()),
            max_position=int(raw.get("max_position", 1 << 20)))
        if problems:
            raise ConfigError("config.json does not describe a Ravenex model: " + "; ".join(problems))
        return cfg
