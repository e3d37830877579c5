"""Typed configuration of the Rovidra decoder, read from ``config.json``.

The file lists the model's layers one by one: ``{"architecture": "Rovidra", "vocab": V, "width": D,
"embedding": {"scale": s}, "norm": {"eps": e}, "layers": [{"type": ..., "mixer": {...}, "mlp": {...} | null},
...]}``.  A layer's ``type`` names its mixer; ``mixer`` holds the mixer's sizes and constants; ``mlp`` its
feed-forward (``null``: the layer has none).  Nothing is implied: every size and constant that can differ
between two models of the design is a key of the file, and a key this reader does not know is an error.

Mixer ``latent_attention``: ``heads``, ``dim`` (unrotated query/key elements per head), ``rot_dim`` (rotated
ones), ``vdim`` (value elements per head), ``kv_rank`` (the latent's width), ``scale`` (of the scores),
``rot = {"base", "dims"}`` (the rotation's base and how many leading elements of the rotated part turn),
``mask = {"size": W}`` (a query sees itself and the ``W - 1`` tokens before it; absent: every earlier token)
and optionally ``kv_from = j``: the layer projects no latent of its own and reads what layer ``j`` cached.
Feed-forward ``dense``: ``ff`` (its width).
"""
from __future__ import annotations

import dataclasses
from typing import Any, Mapping, Optional

from .llama4 import ConfigError
from .specs import LayerSpec, ModelPlan, OrderEntry, part


def _need(d: Mapping[str, Any], key: str, where: str):
    if not isinstance(d, Mapping) or d.get(key) is None:
        raise ConfigError(f"config.json: {where} lacks the key {key!r}")
    return d[key]


def _only(d: Mapping[str, Any], known: tuple, where: str) -> None:
    extra = sorted(set(d) - set(known))
    if extra:
        raise ConfigError(f"config.json: {where} has unknown key(s) {', '.join(extra)}")


@dataclasses.dataclass(frozen=True)
class LatentAttentionConfig:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    scale: float
    rot_base: float
    rot_dims: int
    window: Optional[int]  # None: every earlier token
    kv_from: Optional[int]  # None: the layer has a latent of its own

    @classmethod
    def from_dict(cls, m: Mapping[str, Any], where: str) -> "LatentAttentionConfig":
        _only(m, ("heads", "dim", "rot_dim", "vdim", "kv_rank", "scale", "rot", "mask", "kv_from"), where)
        rot = _need(m, "rot", where)
        _only(rot, ("base", "dims"), where + ".rot")
        mask = m.get("mask")
        if mask is not None:
            _only(mask, ("size",), where + ".mask")
        c = cls(heads=int(_need(m, "heads", where)), dim=int(_need(m, "dim", where)),
                rot_dim=int(_need(m, "rot_dim", where)), vdim=int(_need(m, "vdim", where)),
                kv_rank=int(_need(m, "kv_rank", where)), scale=float(_need(m, "scale", where)),
                rot_base=float(_need(rot, "base", where + ".rot")), rot_dims=int(_need(rot, "dims", where + ".rot")),
                window=None if mask is None else int(_need(mask, "size", where + ".mask")),
                kv_from=None if m.get("kv_from") is None else int(m["kv_from"]))
        if min(c.heads, c.dim, c.rot_dim, c.vdim, c.kv_rank) < 1:
            raise ConfigError(f"config.json: {where}: sizes must be positive")
        if c.rot_dims % 2 or not 0 < c.rot_dims <= c.rot_dim:
            raise ConfigError(f"config.json: {where}.rot.dims must be even and at most rot_dim, got {c.rot_dims}")
        if c.window is not None and c.window < 1:
            raise ConfigError(f"config.json: {where}.mask.size must be positive")
        return c

    def to_dict(self) -> dict:
        d = {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim,
             "kv_rank": self.kv_rank, "scale": self.scale, "rot": {"base": self.rot_base, "dims": self.rot_dims}}
        if self.window is not None:
            d["mask"] = {"size": self.window}
        if self.kv_from is not None:
            d["kv_from"] = self.kv_from
        return d


@dataclasses.dataclass(frozen=True)
class DenseFeedForwardConfig:
    ff: int

    @classmethod
    def from_dict(cls, m: Mapping[str, Any], where: str) -> "DenseFeedForwardConfig":
        _only(m, ("kind", "ff"), where)
        if _need(m, "kind", where) != "dense":
            raise ConfigError(f"config.json: {where}.kind {m['kind']!r} is not known (dense)")
        return cls(ff=int(_need(m, "ff", where)))

    def to_dict(self) -> dict:
        return {"kind": "dense", "ff": self.ff}


@dataclasses.dataclass(frozen=True)
class RovidraLayerConfig:
    type: str
    mixer: LatentAttentionConfig
    mlp: Optional[DenseFeedForwardConfig]


_MIXERS = {"latent_attention": LatentAttentionConfig}


@dataclasses.dataclass(frozen=True)
class RovidraConfig:
    vocab: int
    width: int
    embedding_scale: float
    norm_eps: float
    layers: tuple

    @classmethod
    def from_dict(cls, top: Mapping[str, Any]) -> "RovidraConfig":
        _only(top, ("architecture", "architectures", "model_type", "vocab", "width", "embedding", "norm", "layers"),
              "the top level")
        layers = []
        raw = _need(top, "layers", "the top level")
        for i, entry in enumerate(raw):
            where = f"layers[{i}]"
            _only(entry, ("type", "mixer", "mlp"), where)
            kind = _need(entry, "type", where)
            if kind not in _MIXERS:
                raise ConfigError(f"config.json: {where}.type {kind!r} is not known ({', '.join(sorted(_MIXERS))})")
            mixer = _MIXERS[kind].from_dict(_need(entry, "mixer", where), where + ".mixer")
            mlp = entry.get("mlp")
            layers.append(RovidraLayerConfig(kind, mixer, None if mlp is None else
                                             DenseFeedForwardConfig.from_dict(mlp, where + ".mlp")))
        for i, lc in enumerate(layers):
            j = lc.mixer.kv_from
            if j is None:
                continue
            if not 0 <= j < i or layers[j].mixer.kv_from is not None:
                raise ConfigError(f"config.json: layers[{i}].mixer.kv_from = {j} must name an earlier layer that "
                                  "has a latent of its own")
            a, b = lc.mixer, layers[j].mixer
            if (a.kv_rank, a.rot_dim, a.rot_base, a.rot_dims) != (b.kv_rank, b.rot_dim, b.rot_base, b.rot_dims):
                raise ConfigError(f"config.json: layers[{i}] reads the latent of layers[{j}], whose kv_rank, "
                                  "rot_dim or rotation differ from its own")
        if not layers:
            raise ConfigError("config.json: no layers")
        return cls(vocab=int(_need(top, "vocab", "the top level")), width=int(_need(top, "width", "the top level")),
                   embedding_scale=float(_need(_need(top, "embedding", "the top level"), "scale", "embedding")),
                   norm_eps=float(_need(_need(top, "norm", "the top level"), "eps", "norm")), layers=tuple(layers))

    def to_dict(self, architecture: str = "Rovidra") -> dict:
        return {"architecture": architecture, "vocab": self.vocab, "width": self.width,
                "embedding": {"scale": self.embedding_scale}, "norm": {"eps": self.norm_eps},
                "layers": [{"type": lc.type, "mixer": lc.mixer.to_dict(),
                            "mlp": None if lc.mlp is None else lc.mlp.to_dict()} for lc in self.layers]}

    # ------------------------------------------------------------------ plan
    def cache_of(self, i: int) -> int:
        j = self.layers[i].mixer.kv_from
        return i if j is None else j

    def kept_window(self, cache: int) -> Optional[int]:
        """How far back the readers of a cache look at most: what its pages have to keep (``None``: everything)."""
        sizes = [lc.mixer.window for i, lc in enumerate(self.layers) if self.cache_of(i) == cache]
        return None if any(s is None for s in sizes) else max(sizes)

    def plan(self) -> ModelPlan:
        D, eps = self.width, self.norm_eps
        norm = part("rmsnorm", eps=eps, size=D)
        layers, order = [], []
        for i, lc in enumerate(self.layers):
            m = lc.mixer
            kept = self.kept_window(self.cache_of(i))
            mixer = part(
                "latent_attention", hidden_size=D, num_heads=m.heads, nope_dim=m.dim, rope_dim=m.rot_dim,
                value_dim=m.vdim, kv_rank=m.kv_rank, softmax_scale=m.scale, window=m.window,
                retention=("all",) if kept is None else ("window", kept), own_latent=m.kv_from is None,
                latent_norm_eps=eps,
                position=part("rope_half", theta=m.rot_base, rotary_dim=m.rot_dims))
            ff = None if lc.mlp is None else part("dense_polynorm", hidden_size=D, intermediate_size=lc.mlp.ff, eps=eps)
            layers.append(LayerSpec(mixer=mixer, feed_forward=ff, mixer_norm=norm, feed_forward_norm=norm,
                                    arrangement="sandwich_gated",
                                    options={"hidden_size": D, "post_norm": norm, "token_shift": True}))
            order.append(OrderEntry(layer=i, cache=self.cache_of(i), writes_cache=m.kv_from is None))
        return ModelPlan(vocab_size=self.vocab, hidden_size=D, layers=tuple(layers), order=tuple(order),
                         final_norm=norm, tie_word_embeddings=False,
                         embedding=part("token_embedding", vocab_size=self.vocab, hidden_size=D,
                                        multiplier=self.embedding_scale),
                         head=part("linear_head", vocab_size=self.vocab, hidden_size=D))
