"""Attention over a cached low-rank latent.

A token leaves two things in the cache: a latent ``c`` (``kv_rank`` numbers, RMS-normed with a weight) and one
rotated key part ``k_r`` (``rope_dim`` numbers) that all heads share.  A head's key is ``[W_uk c, k_r]``, its
value ``W_uv c``; its query ``[q_n, q_r]`` (``nope_dim`` unrotated and ``rope_dim`` rotated numbers), and

    score = (q_n . W_uk c + q_r . k_r) * softmax_scale.

Neither keys nor values are ever formed.  ``q_n . W_uk c = (W_uk^T q_n) . c``, so the query is taken into the
latent's space (one batched product per step), the attention kernel runs over the cached ``[c, k_r]`` rows
with all heads sharing them and sums the latents with the softmax weights, and ``W_uv`` is applied to that sum
(a second batched product).  Prefill and decode are the same computation, so a token's result does not depend
on how its request was cut into steps.

Options as data: ``window`` (a query sees itself and the ``window - 1`` tokens before it; ``None``: all),
``retention`` (what the cache keeps: at least the window of every run that reads it), ``own_latent`` (False: the
run projects no latent and reads a cache that another run writes), ``position`` (a rotary kind for ``q_r`` and
``k_r``), ``latent_norm_eps``, ``sink`` (a learned number per head whose exponential is one more term of the
softmax's denominator: it has no key and no value, is not scaled, and counts once) and ``output_gate`` (the heads'
outputs are multiplied element by element with ``sigmoid(W_g h)`` before ``W_o``; ``W_g``'s rows ride behind the
other projections' in ``w_in``).
"""
from __future__ import annotations

import torch

from .base import CacheNeed, Mixer, ParamSpec, build_position, register_mixer


@register_mixer("latent_attention")
class LatentAttention(Mixer):
    def __init__(self, spec) -> None:
        super().__init__()
        self.hidden = int(spec.hidden_size)
        self.num_heads = int(spec.num_heads)
        self.nope_dim, self.rope_dim = int(spec.nope_dim), int(spec.rope_dim)
        self.value_dim, self.kv_rank = int(spec.value_dim), int(spec.kv_rank)
        self.softmax_scale = float(spec.softmax_scale)
        w = spec.get("window")
        self.window = None if w is None else int(w)
        self.retention = tuple(spec.get("retention") or (("all",) if self.window is None else ("window", self.window)))
        if self.retention[0] == "window" and (self.window is None or self.window > int(self.retention[1])):
            raise ValueError(f"the cache keeps {self.retention}, less than the window {self.window} of a run that reads it")
        if self.retention[0] not in ("all", "window"):
            raise ValueError(f"the latent attention reads its cache under 'all' or 'window', not {self.retention!r}")
        self.own_latent = bool(spec.get("own_latent", True))
        self.latent_norm_eps = float(spec.latent_norm_eps)
        self.position = build_position(spec.position, self.rope_dim)
        self.rotation = None
        self.has_sink = bool(spec.get("sink", False))
        self.output_gate = bool(spec.get("output_gate", False))

    @property
    def q_rows(self) -> int:
        return self.num_heads * (self.nope_dim + self.rope_dim)

    def param_specs(self):
        h, d = self.num_heads, self.hidden
        kv = self.kv_rank + self.rope_dim if self.own_latent else 0
        gate = h * self.value_dim if self.output_gate else 0
        specs = {
            # rows: the heads' queries ([unrotated, rotated] per head), then the latent, then the shared rotated key,
            # then the output gate's
            "w_in": ParamSpec((self.q_rows + kv + gate, d), init=("normal", d ** -0.5)),
            "w_uk": ParamSpec((h * self.nope_dim, self.kv_rank), init=("normal", self.kv_rank ** -0.5)),
            "w_uv": ParamSpec((h * self.value_dim, self.kv_rank), init=("normal", self.kv_rank ** -0.5)),
            "wo": ParamSpec((d, h * self.value_dim), init=("normal", (h * self.value_dim) ** -0.5)),
        }
        if self.own_latent:
            specs["latent_norm"] = ParamSpec((self.kv_rank,), policy="float32", init=("uniform", 0.5, 1.5))
        if self.has_sink:
            specs["sink"] = ParamSpec((h,), policy="float32", init=("normal", 1.0))
        return specs

    def allocate(self, dtype, device) -> None:
        super().allocate(dtype, device)
        # In bfloat16, at sizes the matrix-core attention kernel takes, the cache holds the latent twice: token by
        # token for the scores, and per page with the page's tokens side by side for the weighted sum.
        self.transposed_copy = (dtype == torch.bfloat16 and self.kv_rank % 32 == 0 and self.kv_rank <= 512
                                and self.rope_dim % 8 == 0 and self.rope_dim <= 64)  # (of the cache's sizes alone:
        # every run that shares the cache must say the same)

    transposed_copy = False

    def cache_need(self) -> CacheNeed:
        paged = (("latent", (self.kv_rank,)), ("rope_key", (self.rope_dim,)))
        if self.transposed_copy:
            paged += (("latent_t", (self.kv_rank,)),)
        return CacheNeed(paged=paged, retention=self.retention)

    graph_safe = True

    def finalize(self) -> None:
        rot = self.position.rotation()
        if rot is not None:
            rot.inv_freq = rot.inv_freq.to(self.params["w_in"].device)
        self.rotation = rot

    def mixing_flops(self, start: int, count: int) -> float:
        """Scores and sums over the visible latents, and the two batched products that take queries into the
        latent's space and the sums out of it."""
        w = self.window
        keys = sum(min(p + 1, w) if w is not None else p + 1 for p in range(start, start + count))
        h, r = self.num_heads, self.kv_rank
        return (2.0 * h * (2 * r + self.rope_dim) * keys + 2.0 * count * h * r * (self.nope_dim + self.value_dim))

    def flops_per_token(self) -> float:
        return 2.0 * (self.params["w_in"].numel() + self.params["wo"].numel())

    @property
    def gate_offset(self) -> int:
        return self.q_rows + (self.kv_rank + self.rope_dim if self.own_latent else 0)

    def forward(self, h: torch.Tensor, ctx, cache) -> torch.Tensor:
        ops = ctx.ops
        H, dn, dr, dv, r = self.num_heads, self.nope_dim, self.rope_dim, self.value_dim, self.kv_rank
        n = h.shape[0]
        rows = ops.linear(h, self.params["w_in"])  # [N, H * (dn + dr) (+ r + dr)]
        if self.own_latent != bool(cache.writes):
            raise ValueError("a run with a latent of its own writes its cache, one without reads another's")
        # rotates q_r in place, norms the latent, rotates the shared key part and writes both into their pages
        ops.latent_prepare(rows, H, dn, dr, r, ctx.positions, self.rotation,
                           self.params.get("latent_norm"), self.latent_norm_eps,
                           cache.pages["latent"], cache.pages["rope_key"], cache.slot_mapping, cache.writes,
                           latent_t_pages=cache.pages.get("latent_t"))
        q = rows[:, : self.q_rows].view(n, H, dn + dr)
        # queries into the latent's space: [H, N, dn] x [H, dn, r]
        q_lat = ops.batched_linear(q[:, :, :dn].transpose(0, 1), self.params["w_uk"].view(H, dn, r))
        o_lat = ops.latent_attention(q_lat, q, dn, cache.pages["latent"], cache.pages["rope_key"], cache.block_table,
                                     ctx.positions, ctx.token_segment, self.window, self.softmax_scale,
                                     cache.attn_meta, latent_t_pages=cache.pages.get("latent_t"),
                                     sink=self.params.get("sink"))  # [N, H, r]
        # the sums out of it: [H, N, r] x [H, r, dv], laid out [N, H * dv]
        o = ops.batched_linear(o_lat.transpose(0, 1), self.params["w_uv"].view(H, dv, r).transpose(1, 2), tokens_first=True)
        o = o.view(n, H * dv)
        if self.output_gate:
            o = ops.sigmoid_mul(o, rows[:, self.gate_offset: self.gate_offset + H * dv])
        return ops.linear(o, self.params["wo"])
