"""Typed configuration of the Tiradra decoder, read from ``config.json``.

The file lists the model's layers one by one: ``{"architecture": "Tiradra", "vocab": V, "width": D, "norm": {"eps": e},
"embedding": {"bigram": {"buckets", "mul_prev", "mul_cur"}}, "loop": {"start", "stop", "times"}, "logit_softcap": c,
"layers": [{"type": ..., "mixer": {...}, "mlp": {...} | null}, ...]}``.  A layer's ``type`` names its mixer.  Every
size and constant that can differ between two models of the design is a key of the file; ``embedding.bigram``,
``loop``, ``logit_softcap``, a mixer's ``conv`` and a rotation's ``scaling`` may be absent (the model then has no
such thing), and a key this reader does not know is an error.

Mixer ``attention``: ``heads``, ``kv_heads``, ``dim`` (query/key elements per head), ``vdim`` (value elements per
head), ``scale`` (of the scores), ``conv`` (taps of the causal convolution over q, k and v), ``rot``.
Mixer ``latent_attention``: ``heads``, ``dim`` (unrotated query/key elements per head), ``rot_dim`` (rotated ones),
``vdim``, ``kv_rank`` (the latent's width), ``scale``, ``rot``.
``rot = {"base", "dims", "scaling": {"factor", "original", "fast", "slow"}}``: adjacent element pairs of the
leading ``dims`` elements turn; ``scaling`` stretches the slow pairs (see ``parts/position.py``: ``rope_yarn``).
Feed-forward ``dense``: ``ff`` (its width).
"""
from __future__ import annotations

import dataclasses
from typing import Any, Mapping, Optional

from .llama4 import ConfigError
from .rovidra import DenseFeedForwardConfig, _need, _only
from .specs import LayerSpec, ModelPlan, OrderEntry, part


@dataclasses.dataclass(frozen=True)
class RotationConfig:
    base: float
    dims: int
    scaling: Optional[tuple]  # (factor, original, fast, slow) or None

    @classmethod
    def from_dict(cls, m: Mapping[str, Any], where: str, limit: int) -> "RotationConfig":
        _only(m, ("base", "dims", "scaling"), where)
        sc = m.get("scaling")
        if sc is not None:
            _only(sc, ("factor", "original", "fast", "slow"), where + ".scaling")
            sc = tuple(float(_need(sc, k, where + ".scaling")) for k in ("factor", "original", "fast", "slow"))
            if sc[0] <= 0 or sc[1] <= 0 or sc[2] <= 0 or sc[3] <= 0:
                raise ConfigError(f"config.json: {where}.scaling: every number must be positive")
        c = cls(base=float(_need(m, "base", where)), dims=int(_need(m, "dims", where)), scaling=sc)
        if c.dims % 2 or not 0 < c.dims <= limit:
            raise ConfigError(f"config.json: {where}.dims must be even and at most {limit}, got {c.dims}")
        if c.base <= 1.0:
            raise ConfigError(f"config.json: {where}.base must be larger than 1")
        return c

    def to_dict(self) -> dict:
        d = {"base": self.base, "dims": self.dims}
        if self.scaling is not None:
            d["scaling"] = dict(zip(("factor", "original", "fast", "slow"), self.scaling))
        return d

    def spec(self):
        return part("rope_yarn", theta=self.base, rotary_dim=self.dims, scaling=self.scaling)


@dataclasses.dataclass(frozen=True)
class ConvAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    conv: int  # taps; 0: no convolution
    rot: RotationConfig

    @classmethod
    def from_dict(cls, m: Mapping[str, Any], where: str) -> "ConvAttentionConfig":
        _only(m, ("heads", "kv_heads", "dim", "vdim", "scale", "conv", "rot"), where)
        heads, dim = int(_need(m, "heads", where)), int(_need(m, "dim", where))
        c = cls(heads=heads, kv_heads=int(m["kv_heads"]) if m.get("kv_heads") is not None else heads, dim=dim,
                vdim=int(m["vdim"]) if m.get("vdim") is not None else dim, scale=float(_need(m, "scale", where)),
                conv=int(m.get("conv") or 0), rot=RotationConfig.from_dict(_need(m, "rot", where), where + ".rot", dim))
        if min(c.heads, c.kv_heads, c.dim, c.vdim) < 1 or c.conv < 0:
            raise ConfigError(f"config.json: {where}: sizes must be positive")
        if c.heads % c.kv_heads:
            raise ConfigError(f"config.json: {where}: {c.heads} heads are no multiple of {c.kv_heads} kv_heads")
        return c

    def to_dict(self) -> dict:
        d = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale,
             "rot": self.rot.to_dict()}
        if self.conv:
            d["conv"] = self.conv
        return d


@dataclasses.dataclass(frozen=True)
class SinkLatentAttentionConfig:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    scale: float
    rot: RotationConfig

    @classmethod
    def from_dict(cls, m: Mapping[str, Any], where: str) -> "SinkLatentAttentionConfig":
        _only(m, ("heads", "dim", "rot_dim", "vdim", "kv_rank", "scale", "rot"), where)
        rot_dim = int(_need(m, "rot_dim", where))
        c = cls(heads=int(_need(m, "heads", where)), dim=int(_need(m, "dim", where)), rot_dim=rot_dim,
                vdim=int(_need(m, "vdim", where)), kv_rank=int(_need(m, "kv_rank", where)),
                scale=float(_need(m, "scale", where)),
                rot=RotationConfig.from_dict(_need(m, "rot", where), where + ".rot", rot_dim))
        if min(c.heads, c.dim, c.rot_dim, c.vdim, c.kv_rank) < 1:
            raise ConfigError(f"config.json: {where}: sizes must be positive")
        return c

    def to_dict(self) -> dict:
        return {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim,
                "kv_rank": self.kv_rank, "scale": self.scale, "rot": self.rot.to_dict()}


@dataclasses.dataclass(frozen=True)
class TiradraLayerConfig:
    type: str
    mixer: Any
    mlp: Optional[DenseFeedForwardConfig]


@dataclasses.dataclass(frozen=True)
class BigramConfig:
    buckets: int
    mul_prev: int
    mul_cur: int


@dataclasses.dataclass(frozen=True)
class LoopConfig:
    start: int
    stop: int
    times: int


_MIXERS = {"attention": ConvAttentionConfig, "latent_attention": SinkLatentAttentionConfig}


@dataclasses.dataclass(frozen=True)
class TiradraConfig:
    vocab: int
    width: int
    norm_eps: float
    bigram: Optional[BigramConfig]
    loop: Optional[LoopConfig]
    logit_softcap: Optional[float]
    layers: tuple

    @classmethod
    def from_dict(cls, top: Mapping[str, Any]) -> "TiradraConfig":
        _only(top, ("architecture", "architectures", "model_type", "vocab", "width", "embedding", "norm", "layers",
                    "loop", "logit_softcap"), "the top level")
        layers = []
        for i, entry in enumerate(_need(top, "layers", "the top level")):
            where = f"layers[{i}]"
            _only(entry, ("type", "mixer", "mlp"), where)
            kind = _need(entry, "type", where)
            if kind not in _MIXERS:
                raise ConfigError(f"config.json: {where}.type {kind!r} is not known ({', '.join(sorted(_MIXERS))})")
            mixer = _MIXERS[kind].from_dict(_need(entry, "mixer", where), where + ".mixer")
            mlp = entry.get("mlp")
            layers.append(TiradraLayerConfig(kind, mixer, None if mlp is None else
                                             DenseFeedForwardConfig.from_dict(mlp, where + ".mlp")))
        if not layers:
            raise ConfigError("config.json: no layers")
        bigram = None
        emb = top.get("embedding")
        if emb is not None:
            _only(emb, ("bigram",), "embedding")
            b = emb.get("bigram")
            if b is not None:
                _only(b, ("buckets", "mul_prev", "mul_cur"), "embedding.bigram")
                bigram = BigramConfig(*(int(_need(b, k, "embedding.bigram")) for k in ("buckets", "mul_prev", "mul_cur")))
                if bigram.buckets < 1 or bigram.mul_prev < 0 or bigram.mul_cur < 0:
                    raise ConfigError("config.json: embedding.bigram: buckets must be positive, the multipliers not negative")
        loop = None
        lp = top.get("loop")
        if lp is not None:
            _only(lp, ("start", "stop", "times"), "loop")
            loop = LoopConfig(*(int(_need(lp, k, "loop")) for k in ("start", "stop", "times")))
            if not 0 <= loop.start <= loop.stop <= len(layers) or loop.times < 1:
                raise ConfigError(f"config.json: loop {lp} does not fit {len(layers)} layers")
        cap = top.get("logit_softcap")
        if cap is not None and float(cap) <= 0:
            raise ConfigError("config.json: logit_softcap must be positive")
        return cls(vocab=int(_need(top, "vocab", "the top level")), width=int(_need(top, "width", "the top level")),
                   norm_eps=float(_need(_need(top, "norm", "the top level"), "eps", "norm")), bigram=bigram, loop=loop,
                   logit_softcap=None if cap is None else float(cap), layers=tuple(layers))

    def to_dict(self, architecture: str = "Tiradra") -> dict:
        d = {"architecture": architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
             "layers": [{"type": lc.type, "mixer": lc.mixer.to_dict(),
                         "mlp": None if lc.mlp is None else lc.mlp.to_dict()} for lc in self.layers]}
        if self.bigram is not None:
            d["embedding"] = {"bigram": dataclasses.asdict(self.bigram)}
        if self.loop is not None:
            d["loop"] = dataclasses.asdict(self.loop)
        if self.logit_softcap is not None:
            d["logit_softcap"] = self.logit_softcap
        return d

    # ------------------------------------------------------------------ plan
    def run_order(self) -> list:
        """``(layer, number of the pass this run starts or None)`` in the order the layers run: the looped stretch
        ``times`` times in a row."""
        n = len(self.layers)
        if self.loop is None:
            return [(i, None) for i in range(n)]
        lo, hi, times = self.loop.start, self.loop.stop, self.loop.times
        order = [(i, None) for i in range(lo)]
        for t in range(times):
            order += [(i, t if i == lo else None) for i in range(lo, hi)]
        return order + [(i, None) for i in range(hi, n)]

    def plan(self) -> ModelPlan:
        D, eps = self.width, self.norm_eps
        norm = part("rmsnorm", eps=eps, size=D, unit_offset=True)
        layers = []
        for lc in self.layers:
            m = lc.mixer
            if lc.type == "attention":
                mixer = part("attention", hidden_size=D, num_heads=m.heads, num_kv_heads=m.kv_heads, head_dim=m.dim,
                             value_dim=m.vdim, softmax_scale=m.scale, retention=("all",), bias=True, conv_taps=m.conv,
                             qk_norm=part("rmsnorm", eps=eps, weighted=False), position=m.rot.spec())
            else:
                mixer = part("latent_attention", hidden_size=D, num_heads=m.heads, nope_dim=m.dim, rope_dim=m.rot_dim,
                             value_dim=m.vdim, kv_rank=m.kv_rank, softmax_scale=m.scale, window=None,
                             retention=("all",), own_latent=True, latent_norm_eps=eps, sink=True, output_gate=True,
                             position=m.rot.spec())
            ff = None if lc.mlp is None else part("dense_swiglu", hidden_size=D, intermediate_size=lc.mlp.ff,
                                                  activation="gelu_tanh")
            layers.append(LayerSpec(mixer=mixer, feed_forward=ff, mixer_norm=norm, feed_forward_norm=norm,
                                    arrangement="parallel"))
        # every run of a layer has a cache (and state) of its own
        order = tuple(OrderEntry(layer=i, cache=k, enters_pass=t) for k, (i, t) in enumerate(self.run_order()))
        loop = None if self.loop is None else part("pass_entry", hidden_size=D, times=self.loop.times)
        if self.bigram is None:
            embedding = part("token_embedding", vocab_size=self.vocab, hidden_size=D)
        else:
            embedding = part("token_pair_embedding", vocab_size=self.vocab, hidden_size=D, buckets=self.bigram.buckets,
                             mul_prev=self.bigram.mul_prev, mul_cur=self.bigram.mul_cur)
        return ModelPlan(vocab_size=self.vocab, hidden_size=D, layers=tuple(layers), order=order, final_norm=norm,
                         tie_word_embeddings=False, embedding=embedding, loop=loop,
                         head=part("linear_head", vocab_size=self.vocab, hidden_size=D, softcap=self.logit_softcap))
