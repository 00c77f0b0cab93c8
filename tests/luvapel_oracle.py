"""A plain, slow restatement of the Luvapel design for the tests: torch on the CPU in one float type (float64 by
default), token-by-token loops for everything that carries state, one function per mechanism, no code shared with the
package.  Notation: x [T, W] is the stream of one sequence from its first token; weights are a dict of tensors under the
checkpoint's names ([out, in] matrices applied as x @ M^T)."""
from __future__ import annotations

import math

import torch


def rms(x, eps):
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def unit(x):
    return x / torch.sqrt(x.pow(2).sum(-1, keepdim=True) + 1e-6)


def relu2_ff(h, up, down):
    return torch.relu(h @ up.T).pow(2) @ down.T


def residual_step(x, y, gate_w, gate_b, norm_w, eps):
    """the sublayer's result y, gated by what the sublayer read (x), normed, added"""
    return x + rms(y * torch.sigmoid(x @ gate_w.T + gate_b), eps) * norm_w


def rotate_pairs(v, pos, dims, base):
    """v [T, heads, D]; the pair (2i, 2i + 1), i < dims / 2, turns by pos * base^(-2i / dims)"""
    if dims == 0:
        return v
    i = torch.arange(dims // 2, dtype=v.dtype)
    ang = pos.to(v.dtype)[:, None] * torch.pow(torch.tensor(float(base), dtype=v.dtype), -2 * i / dims)[None]
    c, s = torch.cos(ang)[:, None], torch.sin(ang)[:, None]
    out = v.clone()
    a, b = v[..., 0:dims:2], v[..., 1:dims:2]
    out[..., 0:dims:2] = a * c - b * s
    out[..., 1:dims:2] = b * c + a * s
    return out


def window_attention(h, W, p, m, eps):
    """softmax attention whose values are the projected keys; query i sees keys j with 0 <= i - j < mask.size"""
    T = h.shape[0]
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    q, k = (h @ W[p + "q"].T).view(T, H, D), (h @ W[p + "k"].T).view(T, G, D)
    v = k
    pos = torch.arange(T)
    rot, size = m.get("rot") or {"dims": 0, "base": 1.0}, (m.get("mask") or {}).get("size")      # absent: no rotation, no window
    qn = rotate_pairs(rms(q, eps) * W[p + "q.norm"], pos, rot["dims"], rot["base"])
    kn = rotate_pairs(rms(k, eps) * W[p + "k.norm"], pos, rot["dims"], rot["base"])
    out = torch.zeros(T, H, D, dtype=h.dtype)
    for i in range(T):
        lo = max(0, i - size + 1) if size else 0
        for hh in range(H):
            g = hh // (H // G)
            s = (kn[lo:i + 1, g] @ qn[i, hh]) * m["scale"] * W[p + "temp"][hh]
            out[i, hh] = torch.softmax(s, 0) @ v[lo:i + 1, g]
    return (out.reshape(T, H * D) * torch.sigmoid(h @ W[p + "g"].T)) @ W[p + "o"].T


def short_conv_silu(x, w):
    """x [T, C], w [C, taps] with the current token's tap last, zeros before the first token"""
    T, taps = x.shape[0], w.shape[1]
    y = torch.zeros_like(x)
    for t in range(T):
        for j in range(taps):
            s = t - (taps - 1) + j
            if s >= 0:
                y[t] += w[:, j] * x[s]
    return torch.nn.functional.silu(y)


def gated_delta(h, W, p, m, eps):
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = unit(short_conv_silu(h @ W[p + "q"].T, W[p + "q.conv"]).view(T, G, D)) * D ** -0.5
    k = unit(short_conv_silu(h @ W[p + "k"].T, W[p + "k.conv"]).view(T, G, D))
    v = short_conv_silu(h @ W[p + "v"].T, W[p + "v.conv"]).view(T, H, Dv)
    beta = torch.sigmoid(h @ W[p + "b"].T)
    decay = torch.exp(-torch.exp(W[p + "A_log"]) * torch.nn.functional.softplus(h @ W[p + "a"].T + W[p + "dt_bias"]))
    out = torch.zeros(T, H, Dv, dtype=h.dtype)
    for hh in range(H):
        g = hh // (H // G)
        S = torch.zeros(D, Dv, dtype=h.dtype)
        for t in range(T):
            S = decay[t, hh] * S
            u = beta[t, hh] * (v[t, hh] - S.T @ k[t, g])
            S = S + torch.outer(k[t, g], u)
            out[t, hh] = S.T @ q[t, g]
    out = rms(out, eps) * W[p + "norm"]
    return (out.reshape(T, H * Dv) * torch.nn.functional.silu(h @ W[p + "g"].T)) @ W[p + "o"].T


def general_delta(h, W, p, m, eps):
    T = h.shape[0]
    H, D = m["heads"], m["dim"]
    r, k, v = ((h @ W[p + n].T).view(T, H, D) for n in ("r", "k", "v"))
    w = torch.exp(-math.exp(-0.5) * torch.sigmoid(torch.tanh(h @ W[p + "w1"].T) @ W[p + "w2"].T + W[p + "w0"])).view(T, H, D)
    a = torch.sigmoid(h @ W[p + "a"].T + W[p + "a.b"]).view(T, H, D)
    u = unit(k)
    out = torch.zeros(T, H, D, dtype=h.dtype)
    for hh in range(H):
        S = torch.zeros(D, D, dtype=h.dtype)
        for t in range(T):
            S = w[t, hh][:, None] * S - torch.outer(a[t, hh] * u[t, hh], S.T @ u[t, hh]) + torch.outer(k[t, hh], v[t, hh])
            out[t, hh] = S.T @ r[t, hh]
    out = rms(out, eps).reshape(T, H * D) * W[p + "norm"]
    return (out * torch.sigmoid(h @ W[p + "g"].T)) @ W[p + "o"].T


def parallel_mixer(h, W, p, m, eps):
    a = window_attention(h, W, p + "left.", m["left"], eps)
    b = gated_delta(h, W, p + "right.", m["right"], eps)
    return 0.5 * (rms(a, eps) * W[p + "left.out"] + rms(b, eps) * W[p + "right.out"])


class Oracle:
    def __init__(self, cfg, W, dtype=torch.float64):
        self.cfg, self.dtype = cfg, dtype
        self.W = {k: v.to(dtype) for k, v in W.items()}

    def forward(self, ids, layers_out=None):
        """ids: one whole sequence from its first token -> logits [T, vocab]"""
        cfg, W, eps = self.cfg, self.W, self.cfg["norm"]["eps"]
        x = W["embed"][torch.as_tensor(ids).long()] * cfg["embedding"]["scale"]
        for i, L in enumerate(cfg["layers"]):
            src = L.get("weights_of")
            p = f"l{i if src is None else src}."
            y = general_delta(x, W, p + "mix.", L["mixer"], eps) if L["type"] == "general_delta" else parallel_mixer(x, W, p + "mix.", L["mixer"], eps)
            x = residual_step(x, y, W[p + "rg1"], W[p + "rg1.b"], W[p + "norm1"], eps)
            if L.get("mlp"):
                x = residual_step(x, relu2_ff(x, W[p + "mlp.up"], W[p + "mlp.down"]), W[p + "rg2"], W[p + "rg2.b"], W[p + "norm2"], eps)
            if layers_out is not None:
                layers_out.append(x.clone())
        return (rms(x, eps) * W["final.norm"]) @ W["head"].T
