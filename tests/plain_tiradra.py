"""A plain, slow implementation of the Tiradra decoder, written from its equations: one function per mechanism,
whole sequences at a time, float64 unless told otherwise.  It shares no code with the engine: it reads
config.json and model.safetensors itself (with the safetensors package), forms every head's keys and values
(from the latent too, as the definition says) and masks a full score matrix.

    x_0 = E[tok_t] + B[(tok_{t-1} * a + tok_t * b) mod n]            (row n of B for the first token)
    layers lo..hi-1 run T times with the same weights; before pass t:  x += x_0 (t > 0);  x += S[t]
    per layer:  x = x + mixer(N(x; w1)) + ff(N(x; w2))               N(v; w) = v / sqrt(mean(v^2) + eps) * (1 + w)
    logits = cap * tanh(head N(x; w_final) / cap)
"""
import json
import math
import os

import torch
from safetensors import safe_open


# --------------------------------------------------------------------------------------------------- small pieces
def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def centred_norm(x, weight, eps):
    """The weight is stored as its distance from one."""
    return unit_rms(x, eps) * (1.0 + weight)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def soft_cap(z, cap):
    return cap * torch.tanh(z / cap)


def bigram_rows(tokens, buckets, mul_prev, mul_cur):
    """Which row of the pair table each token adds: a hash of (token before, token); the extra last row for the
    first token of a sequence."""
    rows = [buckets]
    for before, tok in zip(tokens[:-1], tokens[1:]):
        rows.append((before * mul_prev + tok * mul_cur) % buckets)
    return rows


def causal_conv(u, taps_w):
    """u [T, C], taps_w [C, K]: y[t] = sum_j taps_w[:, j] * u[t - K + 1 + j], nothing before the start."""
    n, k = u.shape[0], taps_w.shape[1]
    y = torch.zeros_like(u)
    for j in range(k):
        back = k - 1 - j  # tap j reads the row this many steps earlier
        if back < n:
            y[back:] += taps_w[:, j] * u[: n - back]
    return y


def rotary_frequencies(base, dims, scaling=None):
    """f_i = base^(-2i/dims), i < dims/2, and the factor on sines and cosines.  With ``scaling`` (factor, original,
    fast, slow): slow-turning pairs are slowed by ``factor``, fast ones kept, a linear ramp between, and the
    sines and cosines grow by 0.1 ln(factor) + 1."""
    half = dims // 2
    f = [float(base) ** (-2.0 * i / dims) for i in range(half)]
    if not scaling:
        return f, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])
    where = lambda turns: dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(where(float(scaling["fast"]))), 0)
    hi = min(math.ceil(where(float(scaling["slow"]))), dims - 1)
    out = []
    for i in range(half):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f[i] / factor * ramp + f[i] * (1.0 - ramp))
    return out, 0.1 * math.log(factor) + 1.0


def rotate_adjacent(x, positions, freqs, grow):
    """x [T, ..., D]: elements (2i, 2i+1), i < len(freqs), turn by positions[t] * freqs[i]; the rest stay."""
    out = x.clone()
    pos = torch.tensor(positions, dtype=x.dtype).reshape(-1, *([1] * (x.dim() - 2)))
    for i, f in enumerate(freqs):
        a = pos * f
        c, s = torch.cos(a) * grow, torch.sin(a) * grow
        u, v = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = u * c - v * s
        out[..., 2 * i + 1] = v * c + u * s
    return out


def causal_softmax(scores, sink=None):
    """scores [T, T]; row i sees columns j <= i.  ``sink``: one more term exp(sink) in every row's denominator,
    with no column of its own."""
    n = scores.shape[0]
    seen = torch.tril(torch.ones(n, n, dtype=torch.bool))
    s = torch.where(seen, scores, torch.full_like(scores, -math.inf))
    if sink is None:
        return torch.softmax(s, dim=-1)
    top = torch.maximum(s.max(dim=-1, keepdim=True).values, sink.reshape(1, 1))
    e = torch.exp(s - top)
    return e / (e.sum(dim=-1, keepdim=True) + torch.exp(sink - top))


# --------------------------------------------------------------------------------------------------- the two mixers
def conv_attention(h, m, w, p, positions, eps):
    """Grouped-query attention whose q, k, v pass a short causal convolution, then rotation and a weightless
    norm of q and k per head."""
    n = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = h @ w[p + "q"].T + w[p + "q.b"]
    k = h @ w[p + "k"].T + w[p + "k.b"]
    v = h @ w[p + "v"].T + w[p + "v.b"]
    if m.get("conv"):
        q, k, v = causal_conv(q, w[p + "q.conv"]), causal_conv(k, w[p + "k.conv"]), causal_conv(v, w[p + "v.conv"])
    q, k, v = q.view(n, H, d), k.view(n, G, d), v.view(n, G, dv)
    freqs, grow = rotary_frequencies(m["rot"]["base"], m["rot"]["dims"], m["rot"].get("scaling"))
    q = unit_rms(rotate_adjacent(q, positions, freqs, grow), eps)
    k = unit_rms(rotate_adjacent(k, positions, freqs, grow), eps)
    out = torch.zeros(n, H, dv, dtype=h.dtype)
    for head in range(H):
        g = head // (H // G)
        out[:, head] = causal_softmax((q[:, head] @ k[:, g].T) * m["scale"]) @ v[:, g]
    return out.reshape(n, H * dv) @ w[p + "o"].T


def latent_sink_attention(h, m, w, p, positions, eps):
    """Keys and values of every head from one normed latent per token plus one rotated key part shared by the
    heads; a sink in the softmax; a sigmoid gate on the heads' outputs."""
    n = h.shape[0]
    H, dn, dr, dv, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    q = (h @ w[p + "q"].T).view(n, H, dn + dr)
    down = h @ w[p + "dkv"].T
    latent = unit_rms(down[:, :r], eps) * w[p + "dkv.norm"]
    freqs, grow = rotary_frequencies(m["rot"]["base"], m["rot"]["dims"], m["rot"].get("scaling"))
    key_r = rotate_adjacent(down[:, r:], positions, freqs, grow)
    q_r = rotate_adjacent(q[:, :, dn:], positions, freqs, grow)
    k_n = (latent @ w[p + "uk"].T).view(n, H, dn)
    v = (latent @ w[p + "uv"].T).view(n, H, dv)
    out = torch.zeros(n, H, dv, dtype=h.dtype)
    for head in range(H):
        s = (q[:, head, :dn] @ k_n[:, head].T + q_r[:, head] @ key_r.T) * m["scale"]
        out[:, head] = causal_softmax(s, w[p + "sink"][head]) @ v[:, head]
    out = out.reshape(n, H * dv) * torch.sigmoid(h @ w[p + "g"].T)
    return out @ w[p + "o"].T


def gated_feed_forward(h, w, p):
    return (gelu_tanh(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


MIXERS = {"attention": conv_attention, "latent_attention": latent_sink_attention}


def run_order(num_layers, loop):
    """[(layer, pass number or None if the run starts no pass)] in the order the layers run."""
    if not loop:
        return [(i, None) for i in range(num_layers)]
    lo, hi, times = loop["start"], loop["stop"], loop["times"]
    order = [(i, None) for i in range(lo)]
    for t in range(times):
        order += [(i, t if i == lo else None) for i in range(lo, hi)]
    return order + [(i, None) for i in range(hi, num_layers)]


class PlainTiradra:
    def __init__(self, folder, dtype=torch.float64):
        with open(os.path.join(folder, "config.json")) as f:
            self.cfg = json.load(f)
        self.w = {}
        with safe_open(os.path.join(folder, "model.safetensors"), "pt") as f:
            for k in f.keys():
                t = f.get_tensor(k)
                self.w[k] = t.to(dtype) if t.is_floating_point() else t
        self.dtype = dtype

    def embedding(self, tokens):
        cfg, w = self.cfg, self.w
        x = w["embed"][torch.tensor(tokens)]
        pair = (cfg.get("embedding") or {}).get("bigram")
        if pair:
            x = x + w["bigram"][torch.tensor(bigram_rows(tokens, pair["buckets"], pair["mul_prev"], pair["mul_cur"]))]
        return x

    def logits(self, tokens, residuals=None):
        """Logits ``[T, vocab]`` of a whole sequence; ``residuals``: a list that gets the stream behind every run
        of a layer."""
        cfg, w = self.cfg, self.w
        eps = cfg["norm"]["eps"]
        positions = list(range(len(tokens)))
        x0 = self.embedding(tokens)
        x = x0.clone()
        for i, enters in run_order(len(cfg["layers"]), cfg.get("loop")):
            layer, p = cfg["layers"][i], f"l{i}."
            if enters is not None:
                if enters > 0:
                    x = x + x0
                x = x + w["loop.step"][enters]
            y = MIXERS[layer["type"]](centred_norm(x, w[p + "norm1"], eps), layer["mixer"], w, p + "mix.", positions, eps)
            if layer.get("mlp") is not None:
                y = y + gated_feed_forward(centred_norm(x, w[p + "norm2"], eps), w, p + "mlp.")
            x = x + y
            if residuals is not None:
                residuals.append(x.clone())
        z = centred_norm(x, w["final.norm"], eps) @ w["head"].T
        cap = cfg.get("logit_softcap")
        return z if cap is None else soft_cap(z, cap)
