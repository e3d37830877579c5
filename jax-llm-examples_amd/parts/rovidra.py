"""The Rovidra decoder as an architecture: its configuration, its plan and the names of its checkpoint tensors.

A layer ``i`` stores, under ``l<i>.``: the four norms of its sandwich arrangement (``norm1`` / ``norm1b`` before
and behind the mixer, ``norm2`` / ``norm2b`` round the feed-forward), the two residual gates (``rg1``, ``rg2``
with biases ``.b``), the token shift's weights (``shift``), the mixer's matrices under ``mix.`` (``q``, ``dkv``
with the latent's norm ``dkv.norm``, ``uk``, ``uv``, ``o``; a layer that reads another layer's latent has no
``dkv``) and the feed-forward's under ``mlp.`` (``up``, ``down`` with biases, the activation's four numbers
``act``).  Linear weights are ``[out, in]``.  The model's ends: ``embed``, ``final.norm``, ``head``.
"""
from __future__ import annotations

import math
from typing import Any, Mapping

from ..config.registry import register_architecture
from ..config.rovidra import RovidraConfig
from ..config.specs import ModelPlan
from ..weights.bindings import TensorBinding


class RovidraArchitecture:
    names = ("Rovidra", "rovidra")
    # what of csrc/ a model of this design calls (a first run on a machine without a built library compiles these)
    kernel_sources = ("elementwise.hip", "sandwich.hip", "attention_latent.hip", "gemm_skinny.hip", "gemm_stream.hip",
                      "gemm_grouped.hip", "gemm_generic.hip", "sampling.hip")

    def parse_config(self, top: Mapping[str, Any]) -> RovidraConfig:
        return RovidraConfig.from_dict(top)

    def plan(self, cfg: RovidraConfig) -> ModelPlan:
        return cfg.plan()

    def config_to_dict(self, cfg: RovidraConfig, architecture: str | None = None) -> dict:
        return cfg.to_dict(architecture or "Rovidra")

    def bindings(self, cfg: RovidraConfig, plan: ModelPlan) -> list[TensorBinding]:
        D, V = cfg.width, cfg.vocab
        mat = lambda fan_in: ("normal", 1.0 / math.sqrt(fan_in))
        norm = ("uniform", 0.5, 1.5)
        out = [TensorBinding("embed", (V, D), "embed.weight", init=("normal", 1.0 / math.sqrt(D)))]
        for i, lc in enumerate(cfg.layers):
            p, t = f"l{i}.", f"layers.{i}."
            m = lc.mixer
            hq = m.heads * (m.dim + m.rot_dim)
            out += [
                TensorBinding(p + "norm1", (D,), t + "mixer_norm.weight", init=norm),
                TensorBinding(p + "norm1b", (D,), t + "mixer_post_norm.weight", init=norm),
                TensorBinding(p + "rg1", (D, D), t + "mixer_gate.weight", init=mat(D)),
                TensorBinding(p + "rg1.b", (D,), t + "mixer_gate.bias", init=("normal", 1.0)),
                TensorBinding(p + "shift", (D,), t + "token_shift.weight", init=("uniform", 0.0, 1.0)),
                TensorBinding(p + "mix.q", (hq, D), t + "mixer.w_in", rows=(0, hq), init=mat(D)),
                TensorBinding(p + "mix.uk", (m.heads * m.dim, m.kv_rank), t + "mixer.w_uk", init=mat(m.kv_rank)),
                TensorBinding(p + "mix.uv", (m.heads * m.vdim, m.kv_rank), t + "mixer.w_uv", init=mat(m.kv_rank)),
                TensorBinding(p + "mix.o", (D, m.heads * m.vdim), t + "mixer.wo", init=mat(m.heads * m.vdim)),
            ]
            if m.kv_from is None:
                out += [
                    TensorBinding(p + "mix.dkv", (m.kv_rank + m.rot_dim, D), t + "mixer.w_in",
                                  rows=(hq, hq + m.kv_rank + m.rot_dim), init=mat(D)),
                    TensorBinding(p + "mix.dkv.norm", (m.kv_rank,), t + "mixer.latent_norm", init=norm),
                ]
            if lc.mlp is not None:
                F = lc.mlp.ff
                out += [
                    TensorBinding(p + "norm2", (D,), t + "feed_forward_norm.weight", init=norm),
                    TensorBinding(p + "norm2b", (D,), t + "feed_forward_post_norm.weight", init=norm),
                    TensorBinding(p + "rg2", (D, D), t + "feed_forward_gate.weight", init=mat(D)),
                    TensorBinding(p + "rg2.b", (D,), t + "feed_forward_gate.bias", init=("normal", 1.0)),
                    TensorBinding(p + "mlp.up", (F, D), t + "feed_forward.w_up", init=mat(D)),
                    TensorBinding(p + "mlp.up.b", (F,), t + "feed_forward.b_up", init=("normal", 0.1)),
                    TensorBinding(p + "mlp.down", (D, F), t + "feed_forward.w_down", init=mat(F)),
                    TensorBinding(p + "mlp.down.b", (D,), t + "feed_forward.b_down", init=("normal", 0.1)),
                    TensorBinding(p + "mlp.act", (4,), t + "feed_forward.coef", init=("uniform", -1.0, 1.0)),
                ]
        out += [
            TensorBinding("final.norm", (D,), "final_norm.weight", init=norm),
            TensorBinding("head", (V, D), "lm_head.weight", init=mat(D)),
        ]
        return out


ROVIDRA = register_architecture(RovidraArchitecture())
