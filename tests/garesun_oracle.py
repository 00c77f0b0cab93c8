"""Plain, slow restatement of the Garesun decoder for the tests: one function per mechanism, torch on the CPU,
token-by-token recurrences, dense attention, every expert evaluated by a Python loop.  It shares no code with the
product path (`mlx-vlm_amd/models/garesun`, `csrc/*.hip`) and is written for clarity, not speed.

Notation: x [T, W] is the residual stream of ONE sequence, h its normed copy; weights are [out, in] and applied as
`h @ w.T`; `W` is the dict of tensors of a checkpoint (names `l<i>.mix.q`, `l<i>.mlp.e<j>.up`, ...); `cfg` is the parsed
config.json.  `dt` is the working dtype (float64 for a sharp comparison)."""
from __future__ import annotations

import math

import torch


def layer_norm_nobias(x, w, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rope_angles(pos, dims, base, dt):
    i = torch.arange(dims // 2, dtype=dt)
    f = torch.as_tensor(base, dtype=dt) ** (-2.0 * i / dims)
    return pos.to(dt)[:, None] * f[None]                     # [T, dims / 2]


def rope_half(x, pos, dims, base):
    """x [T, H, D]: dimension i pairs with i + dims / 2 inside the first `dims` dimensions"""
    a = rope_angles(pos, dims, base, x.dtype)
    c, s = a.cos()[:, None], a.sin()[:, None]
    u, v = x[..., : dims // 2], x[..., dims // 2: dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


def rope_interleaved(x, pos, dims, base):
    """x [T, H, D]: dimension 2 i pairs with 2 i + 1 inside the first `dims` dimensions"""
    a = rope_angles(pos, dims, base, x.dtype)
    c, s = a.cos()[:, None], a.sin()[:, None]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    rot = torch.stack([u * c - v * s, v * c + u * s], dim=-1).flatten(-2)
    return torch.cat([rot, x[..., dims:]], dim=-1)


# ------------------------------------------------------------------------------------------------ mixers
def retention(h, pos, W, p, m, eps, state=None):
    """fixed per-head decay, no softmax, no denominator.  state: S [H, D, Dv] or None -> (out [T, W], S)"""
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = (h @ W[p + "q"].T).view(T, H, D)
    k = (h @ W[p + "k"].T).view(T, H, D)
    v = (h @ W[p + "v"].T).view(T, H, Dv)
    q = rope_half(q, pos, m["rot"]["dims"], m["rot"]["base"])
    k = rope_half(k, pos, m["rot"]["dims"], m["rot"]["base"]) * D ** -0.5
    decay = torch.tensor(m["decay"], dtype=h.dtype)
    S = torch.zeros(H, D, Dv, dtype=h.dtype) if state is None else state.clone()
    o = torch.zeros(T, H, Dv, dtype=h.dtype)
    for t in range(T):
        S = decay[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hdv,hd->hv", S, q[t])
    o = unit_rms(o, eps).reshape(T, H * Dv)
    g = h @ W[p + "g"].T
    return (o * torch.nn.functional.silu(g)) @ W[p + "o"].T, S


def mlstm(h, pos, W, p, m, eps, state=None):
    """matrix memory with exponential input gate, stabilised by a running maximum that starts at 0.
    state: (S [H, D, Dv], n [H, D], mx [H]) or None"""
    H, D, Dv, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    T = h.shape[0]
    q = (h @ W[p + "q"].T).view(T, H, D) * D ** -0.5
    k = (h @ W[p + "k"].T).view(T, H, D)
    v = (h @ W[p + "v"].T).view(T, H, Dv)
    ig = cap * torch.tanh((h @ W[p + "i"].T + W[p + "i.b"]) / cap)
    fg = torch.nn.functional.logsigmoid(cap * torch.tanh((h @ W[p + "f"].T + W[p + "f.b"]) / cap))
    if state is None:
        S, n, mx = torch.zeros(H, D, Dv, dtype=h.dtype), torch.zeros(H, D, dtype=h.dtype), torch.zeros(H, dtype=h.dtype)
    else:
        S, n, mx = (s.clone() for s in state)
    o = torch.zeros(T, H, Dv, dtype=h.dtype)
    for t in range(T):
        m_new = torch.maximum(fg[t] + mx, ig[t])
        a, b = torch.exp(fg[t] + mx - m_new), torch.exp(ig[t] - m_new)
        S = a[:, None, None] * S + b[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        n = a[:, None] * n + b[:, None] * k[t]
        mx = m_new
        num = torch.einsum("hdv,hd->hv", S, q[t])
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-mx)) + 1e-6
        o[t] = num / den[:, None]
    o = unit_rms(o, eps).reshape(T, H * Dv) * W[p + "norm"]
    g = h @ W[p + "g"].T
    return (o * torch.sigmoid(g)) @ W[p + "o"].T, (S, n, mx)


def latent_kv(h, pos, W, p, m, eps):
    """what a latent-attention layer caches: (c [T, R] normed latent, kr [T, Dr] rotated shared key part)"""
    R, Dr = m["kv_rank"], m["rot_dim"]
    d = h @ W[p + "dkv"].T
    c = unit_rms(d[:, :R], eps) * W[p + "dkv.norm"]
    kr = rope_interleaved(d[:, None, R:], pos, m["rot"]["dims"], m["rot"]["base"])[:, 0]
    return c, kr


def latent_attention(h, pos, W, p, m, eps, c, kr, kpos):
    """c / kr / kpos: the latents, rotated key parts and positions of EVERY key of the sequence so far (this call's own
    tokens included, possibly another layer's); causal softmax attention with a per-head sigmoid output gate"""
    H, D, Dr, Dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    T = h.shape[0]
    q = (h @ W[p + "q"].T).view(T, H, D + Dr)
    qn, qr = q[..., :D], rope_interleaved(q[..., D:], pos, m["rot"]["dims"], m["rot"]["base"])
    kn = (c @ W[p + "uk"].T).view(-1, H, D)
    v = (c @ W[p + "uv"].T).view(-1, H, Dv)
    s = (torch.einsum("thd,jhd->htj", qn, kn) + torch.einsum("thd,jd->htj", qr, kr)) * m["scale"]
    s = s.masked_fill(kpos[None, None, :] > pos[None, :, None], float("-inf"))
    o = torch.einsum("htj,jhv->thv", torch.softmax(s, dim=-1), v)
    gate = torch.sigmoid(h @ W[p + "g"].T)                   # [T, H]
    return (o * gate[:, :, None]).reshape(T, H * Dv) @ W[p + "o"].T


# ------------------------------------------------------------------------------------------------ feed-forward
def relu2_expert(h, up, down):
    return torch.relu(h @ up.T) ** 2 @ down.T


def moe(h, W, p, mlp):
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    z = h.float() @ W[p + "router"].float().T if h.dtype != torch.float64 else h @ W[p + "router"].T
    val, idx = torch.topk(z, top, dim=-1)
    wgt = torch.softmax(val, dim=-1).to(h.dtype)
    out = torch.zeros(h.shape[0], W[p + "e0.down"].shape[0], dtype=h.dtype)
    for t in range(h.shape[0]):
        for j in range(top):
            e = int(idx[t, j])
            out[t] += wgt[t, j] * relu2_expert(h[t], W[p + f"e{e}.up"], W[p + f"e{e}.down"])
    if mlp.get("shared"):
        out = out + relu2_expert(h, W[p + "shared.up"], W[p + "shared.down"])
    return out


def token_side(x, tokens, W, i, dim, eps):
    """per-layer token input: a gated slice of a second embedding table, unit-RMS normed with a weight, added to x"""
    e = W["side.embed"][tokens][:, i * dim:(i + 1) * dim]
    g = gelu_tanh(x @ W[f"l{i}.side.gate"].T) * e
    y = g @ W[f"l{i}.side.proj"].T
    return x + unit_rms(y, eps) * W[f"l{i}.side.norm"]


# ------------------------------------------------------------------------------------------------ the model
class Oracle:
    """Holds one sequence's state, so that a prompt can be fed in pieces: `forward(tokens)` continues where the last
    call stopped.  -> logits [T, V]; `self.trace` = the residual stream after every layer of the last call."""

    def __init__(self, cfg, W, dt=torch.float64):
        self.cfg, self.dt = cfg, dt
        self.W = {k: (v.to(dt) if v.is_floating_point() else v) for k, v in W.items()}
        self.reset()

    def reset(self):
        self.n = 0
        self.state = {}

    def forward(self, tokens):
        cfg, W, dt = self.cfg, self.W, self.dt
        eps = cfg["norm"]["eps"]
        tokens = torch.as_tensor(tokens, dtype=torch.long)
        T = tokens.numel()
        pos = torch.arange(self.n, self.n + T)
        x = W["embed"][tokens] * cfg["embedding"]["scale"]
        side = (cfg.get("token_side") or {}).get("dim")
        self.trace = []
        for i, L in enumerate(cfg["layers"]):
            p, m = f"l{i}.mix.", L["mixer"]
            h = layer_norm_nobias(x, W[f"l{i}.norm1"], eps)
            if L["type"] == "retention":
                y, self.state[i] = retention(h, pos, W, p, m, eps, self.state.get(i))
            elif L["type"] == "mlstm":
                y, self.state[i] = mlstm(h, pos, W, p, m, eps, self.state.get(i))
            elif L["type"] == "latent_attention":
                src = m.get("kv_from")
                if src is None:
                    c, kr = latent_kv(h, pos, W, p, m, eps)
                    if i in self.state:
                        c, kr = torch.cat([self.state[i][0], c]), torch.cat([self.state[i][1], kr])
                    self.state[i] = (c, kr)
                    src = i
                c, kr = self.state[src]
                y = latent_attention(h, pos, W, p, m, eps, c, kr, torch.arange(c.shape[0]))
            else:
                raise ValueError(L["type"])
            if L.get("mlp"):
                y = y + moe(h, W, f"l{i}.mlp.", L["mlp"])
            x = x + y
            if side:
                x = token_side(x, tokens, W, i, side, eps)
            self.trace.append(x)
        self.n += T
        return layer_norm_nobias(x, W["final.norm"], eps) @ W["head"].T
