"""A plain, slow implementation of the Rovidra decoder, written from its equations: one function per mechanism,
whole sequences at a time, float64 unless told otherwise.  It shares no code with the engine: it reads
config.json and model.safetensors itself (with the safetensors package), forms every head's keys and values
from the latent as the definition says, and masks a full score matrix.

    x_0 = embed[token] * s
    per layer:  h = N(x; w1);  h' = h + (h_prev - h) * shift          (h_prev: h of the token before, 0 at the start)
                x = x + N(mixer(h') * sigmoid(G1 h + b1); w1b)
                h = N(x; w2);   x = x + N(ff(h) * sigmoid(G2 h + b2); w2b)        (if the layer has a feed-forward)
    logits = head N(x; w_final)
    N(v; w) = v / sqrt(mean(v^2) + eps) * w
"""
import json
import math
import os

import torch
from safetensors import safe_open


def rms_norm(x, weight, eps):
    y = x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)
    return y if weight is None else y * weight


def token_shift(h, shift):
    """Row t becomes h[t] + (h[t - 1] - h[t]) * shift; row 0 mixes with zeros."""
    before = torch.zeros_like(h)
    before[1:] = h[:-1]
    return h + (before - h) * shift


def gate(y, h, w, b):
    return y * torch.sigmoid(h @ w.T + b)


def rotate_half(x, positions, base, dims):
    """x: [tokens, ..., D]; the first ``dims`` elements turn, element j with element j + dims/2."""
    half = dims // 2
    out = x.clone()
    for t, p in enumerate(positions):
        for j in range(half):
            a = float(p) * float(base) ** (-2.0 * j / dims)
            u, v = x[t, ..., j], x[t, ..., j + half]
            out[t, ..., j] = u * math.cos(a) - v * math.sin(a)
            out[t, ..., j + half] = v * math.cos(a) + u * math.sin(a)
    return out


def visible(i, j, window):
    return 0 <= i - j and (window is None or i - j < window)


def latent_of(hs, w_dkv, norm_w, eps, kv_rank, positions, base, dims):
    """What a token leaves for others to read: the normed latent and the rotated shared key part."""
    dkv = hs @ w_dkv.T
    return rms_norm(dkv[:, :kv_rank], norm_w, eps), rotate_half(dkv[:, kv_rank:], positions, base, dims)


def latent_attention(hs, latent, rope_key, m, w_q, w_uk, w_uv, w_o, positions):
    """Keys and values of every head formed from the latent; full scores, masked; softmax; W_o."""
    n = hs.shape[0]
    H, dn, dr, dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    window = m["mask"]["size"] if m.get("mask") else None
    q = (hs @ w_q.T).view(n, H, dn + dr)
    q_r = rotate_half(q[:, :, dn:], positions, m["rot"]["base"], m["rot"]["dims"])
    k_n = (latent @ w_uk.T).view(n, H, dn)
    v = (latent @ w_uv.T).view(n, H, dv)
    out = torch.zeros(n, H, dv, dtype=hs.dtype)
    seen = torch.tensor([[visible(positions[i], positions[j], window) for j in range(n)] for i in range(n)])
    for h in range(H):
        s = (q[:, h, :dn] @ k_n[:, h].T + q_r[:, h] @ rope_key.T) * m["scale"]
        s = torch.where(seen, s, torch.full_like(s, -math.inf))
        out[:, h] = torch.softmax(s, dim=-1) @ v[:, h]
    return out.reshape(n, H * dv) @ w_o.T


def poly_norm(z, coef, eps):
    n = lambda v: v / torch.sqrt((v * v).mean(dim=-1, keepdim=True) + eps)
    return coef[0] * n(z) + coef[1] * n(z ** 2) + coef[2] * n(z ** 3) + coef[3]


def dense_feed_forward(h, w_up, b_up, w_down, b_down, coef, eps):
    return poly_norm(h @ w_up.T + b_up, coef, eps) @ w_down.T + b_down


class PlainRovidra:
    def __init__(self, folder, dtype=torch.float64):
        with open(os.path.join(folder, "config.json")) as f:
            self.cfg = json.load(f)
        self.w = {}
        with safe_open(os.path.join(folder, "model.safetensors"), "pt") as f:
            for k in f.keys():
                self.w[k] = f.get_tensor(k).to(dtype)
        self.dtype = dtype

    def logits(self, tokens, residuals=None):
        """Logits ``[T, vocab]`` of a whole sequence; ``residuals``: a list that gets the stream behind every layer."""
        cfg, w = self.cfg, self.w
        eps = cfg["norm"]["eps"]
        n = len(tokens)
        positions = list(range(n))
        x = w["embed"][torch.tensor(tokens)] * cfg["embedding"]["scale"]
        kept = {}
        for i, layer in enumerate(cfg["layers"]):
            p, m = f"l{i}.", layer["mixer"]
            h = rms_norm(x, w[p + "norm1"], eps)
            hs = token_shift(h, w[p + "shift"])
            if m.get("kv_from") is None:
                kept[i] = latent_of(hs, w[p + "mix.dkv"], w[p + "mix.dkv.norm"], eps, m["kv_rank"], positions,
                                    m["rot"]["base"], m["rot"]["dims"])
            latent, rope_key = kept[i if m.get("kv_from") is None else m["kv_from"]]
            y = latent_attention(hs, latent, rope_key, m, w[p + "mix.q"], w[p + "mix.uk"], w[p + "mix.uv"],
                                 w[p + "mix.o"], positions)
            x = x + rms_norm(gate(y, h, w[p + "rg1"], w[p + "rg1.b"]), w[p + "norm1b"], eps)
            if layer.get("mlp") is not None:
                h = rms_norm(x, w[p + "norm2"], eps)
                y = dense_feed_forward(h, w[p + "mlp.up"], w[p + "mlp.up.b"], w[p + "mlp.down"], w[p + "mlp.down.b"],
                                       w[p + "mlp.act"], eps)
                x = x + rms_norm(gate(y, h, w[p + "rg2"], w[p + "rg2.b"]), w[p + "norm2b"], eps)
            if residuals is not None:
                residuals.append(x.clone())
        return rms_norm(x, w["final.norm"], eps) @ w["head"].T
