"""The Tiradra decoder as an architecture: its configuration, its plan and the names of its checkpoint tensors.

The model's ends: ``embed``, ``bigram`` (the token-pair table, its last row for a sequence's first token),
``loop.step`` (one vector per pass of the looped layers), ``final.norm``, ``head``.  A layer ``i`` stores, under
``l<i>.``: its two norms (``norm1`` for the mixer, ``norm2`` for the feed-forward; weights around zero), the mixer's
tensors under ``mix.`` and the feed-forward's under ``mlp.`` (``gate``, ``up``, ``down``).  Mixer ``attention``:
``q``, ``k``, ``v`` with biases (``.b``) and convolution taps (``.conv``, ``[channels, taps]``), ``o``.  Mixer
``latent_attention``: ``q``, ``dkv`` with the latent's norm ``dkv.norm``, ``uk``, ``uv``, ``sink`` (one number a
head), ``g`` (the output gate), ``o``.  Linear weights are ``[out, in]``.
"""
from __future__ import annotations

import math
from typing import Any, Mapping

from ..config.registry import register_architecture
from ..config.specs import ModelPlan
from ..config.tiradra import TiradraConfig
from ..weights.bindings import TensorBinding


class TiradraArchitecture:
    names = ("Tiradra", "tiradra")
    # what of csrc/ a model of this design calls (a first run on a machine without a built library compiles these)
    kernel_sources = ("elementwise.hip", "parallel.hip", "attention_conv.hip", "attention_prep.hip", "attention_latent.hip",
                      "attention_mfma.hip", "attention_generic.hip", "attention_f32.hip", "gemm_skinny.hip",
                      "gemm_stream.hip", "gemm_grouped.hip", "gemm_generic.hip", "sampling.hip")

    def parse_config(self, top: Mapping[str, Any]) -> TiradraConfig:
        return TiradraConfig.from_dict(top)

    def plan(self, cfg: TiradraConfig) -> ModelPlan:
        return cfg.plan()

    def config_to_dict(self, cfg: TiradraConfig, architecture: str | None = None) -> dict:
        return cfg.to_dict(architecture or "Tiradra")

    def unused_prefixes(self, cfg: TiradraConfig) -> tuple:
        """Tensors that a checkpoint may hold and this model does not read: the feed-forward's norm of a layer that
        has no feed-forward."""
        return tuple(f"l{i}.norm2" for i, lc in enumerate(cfg.layers) if lc.mlp is None)

    def bindings(self, cfg: TiradraConfig, plan: ModelPlan) -> list[TensorBinding]:
        D, V = cfg.width, cfg.vocab
        mat = lambda fan_in: ("normal", 1.0 / math.sqrt(fan_in))
        norm = ("normal", 0.1)  # (stored as the distance from one)
        out = [TensorBinding("embed", (V, D), "embed.weight", init=("normal", 1.0))]
        if cfg.bigram is not None:
            out.append(TensorBinding("bigram", (cfg.bigram.buckets + 1, D), "embed.pair", init=("normal", 0.5)))
        if cfg.loop is not None:
            out.append(TensorBinding("loop.step", (cfg.loop.times, D), "loop.step", init=("normal", 0.3)))
        for i, lc in enumerate(cfg.layers):
            p, t = f"l{i}.", f"layers.{i}."
            m = lc.mixer
            out.append(TensorBinding(p + "norm1", (D,), t + "mixer_norm.weight", init=norm))
            if lc.type == "attention":
                nq, nk, nv = m.heads * m.dim, m.kv_heads * m.dim, m.kv_heads * m.vdim
                o = 0
                for name, rows in (("q", nq), ("k", nk), ("v", nv)):
                    out += [TensorBinding(p + f"mix.{name}", (rows, D), t + "mixer.wqkv", rows=(o, o + rows), init=mat(D)),
                            TensorBinding(p + f"mix.{name}.b", (rows,), t + "mixer.bqkv", rows=(o, o + rows),
                                          init=("normal", 0.3))]
                    if m.conv:
                        out.append(TensorBinding(p + f"mix.{name}.conv", (rows, m.conv), t + "mixer.conv",
                                                 rows=(o, o + rows), init=("normal", 0.6)))
                    o += rows
                out.append(TensorBinding(p + "mix.o", (D, m.heads * m.vdim), t + "mixer.wo", init=mat(m.heads * m.vdim)))
            else:
                hq, hv = m.heads * (m.dim + m.rot_dim), m.heads * m.vdim
                kv = m.kv_rank + m.rot_dim
                out += [
                    TensorBinding(p + "mix.q", (hq, D), t + "mixer.w_in", rows=(0, hq), init=mat(D)),
                    TensorBinding(p + "mix.dkv", (kv, D), t + "mixer.w_in", rows=(hq, hq + kv), init=mat(D)),
                    TensorBinding(p + "mix.g", (hv, D), t + "mixer.w_in", rows=(hq + kv, hq + kv + hv), init=mat(D)),
                    TensorBinding(p + "mix.dkv.norm", (m.kv_rank,), t + "mixer.latent_norm", init=("uniform", 0.5, 1.5)),
                    TensorBinding(p + "mix.uk", (m.heads * m.dim, m.kv_rank), t + "mixer.w_uk", init=mat(m.kv_rank)),
                    TensorBinding(p + "mix.uv", (hv, m.kv_rank), t + "mixer.w_uv", init=mat(m.kv_rank)),
                    TensorBinding(p + "mix.sink", (m.heads,), t + "mixer.sink", init=("normal", 1.0)),
                    TensorBinding(p + "mix.o", (D, hv), t + "mixer.wo", init=mat(hv)),
                ]
            if lc.mlp is not None:
                F = lc.mlp.ff
                out += [
                    TensorBinding(p + "norm2", (D,), t + "feed_forward_norm.weight", init=norm),
                    TensorBinding(p + "mlp.gate", (F, D), t + "feed_forward.w_gate_up", rows=(0, F), init=mat(D)),
                    TensorBinding(p + "mlp.up", (F, D), t + "feed_forward.w_gate_up", rows=(F, 2 * F), init=mat(D)),
                    TensorBinding(p + "mlp.down", (D, F), t + "feed_forward.w_down", init=mat(F)),
                ]
        out += [
            TensorBinding("final.norm", (D,), "final_norm.weight", init=norm),
            TensorBinding("head", (V, D), "lm_head.weight", init=mat(D)),
        ]
        return out


TIRADRA = register_architecture(TiradraArchitecture())
