"""Small random Luvapel checkpoints for the tests: config dicts, bf16 weights with the checkpoint's tensor names, a folder
on disk for the loader.  Sizes are deliberately unequal (heads != kv_heads, dim differs between the two sides, partial
rotation, short windows, different tap counts) so that a swapped size shows."""
from __future__ import annotations

import json
import os

import torch

from tests.garesun_helpers import rel_rms, write_checkpoint  # noqa: F401


def general(heads=3, dim=24, ff=40):
    return dict(type="general_delta", mixer=dict(heads=heads, dim=dim), mlp=(dict(kind="dense", ff=ff) if ff else None))


def parallel(heads=4, kv_heads=2, dim=24, window=9, rot_dims=16, base=10000.0, scale=None, rheads=6, rkv=3, rdim=16, rvdim=24, conv=4,
             ff=40):
    left = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, scale=(dim ** -0.5 if scale is None else scale),
                rot=dict(base=base, dims=rot_dims), mask=dict(size=window))
    right = dict(heads=rheads, kv_heads=rkv, dim=rdim, vdim=rvdim, conv=conv)
    return dict(type="parallel", mixer=dict(left=left, right=right), mlp=(dict(kind="dense", ff=ff) if ff else None))


def shared(layers, j):
    """a further layer that uses layer j's tensors"""
    L = json.loads(json.dumps(layers[j]))
    L["weights_of"] = j
    return L


def config(layers, vocab=101, width=56, scale=3.0, eps=1e-5):
    return dict(architecture="Luvapel", vocab=vocab, width=width, layers=layers, norm=dict(eps=eps), embedding=dict(scale=scale))


def weights(cfg, seed=0, gain=1.0):
    g = torch.Generator().manual_seed(seed)
    W, width = {}, cfg["width"]

    def lin(name, out, inn, s=1.0):
        W[name] = (torch.randn(out, inn, generator=g) * (s * gain / inn ** 0.5)).to(torch.bfloat16)

    def vec(name, n, center=1.0, s=0.1):
        W[name] = (center + s * torch.randn(n, generator=g)).to(torch.bfloat16)

    W["embed"] = (torch.randn(cfg["vocab"], width, generator=g) * 0.5).to(torch.bfloat16)
    for i, L in enumerate(cfg["layers"]):
        if L.get("weights_of") is not None:
            continue
        p, m = f"l{i}.", L["mixer"]
        vec(p + "norm1", width, 0.5)
        lin(p + "rg1", width, width, 2.0)
        vec(p + "rg1.b", width, 0.0, 0.5)
        if L["type"] == "general_delta":
            HD = m["heads"] * m["dim"]
            for n in ("r", "k", "v", "g", "a"):
                lin(p + "mix." + n, HD, width, 2.0)
            lin(p + "mix.w1", 8, width, 2.0)
            lin(p + "mix.w2", HD, 8, 2.0)
            vec(p + "mix.w0", HD, -1.0, 1.0)
            vec(p + "mix.a.b", HD, 0.0, 1.0)
            vec(p + "mix.norm", HD)
            lin(p + "mix.o", width, HD)
        else:
            a, r = m["left"], m["right"]
            pl, pr = p + "mix.left.", p + "mix.right."
            lin(pl + "q", a["heads"] * a["dim"], width, 2.0)
            lin(pl + "k", a["kv_heads"] * a["dim"], width, 2.0)
            lin(pl + "g", a["heads"] * a["dim"], width, 2.0)
            lin(pl + "o", width, a["heads"] * a["dim"])
            vec(pl + "q.norm", a["dim"])
            vec(pl + "k.norm", a["dim"])
            vec(pl + "temp", a["heads"], 1.5, 0.4)
            vec(pl + "out", width)
            lin(pr + "q", r["kv_heads"] * r["dim"], width, 2.0)
            lin(pr + "k", r["kv_heads"] * r["dim"], width, 2.0)
            lin(pr + "v", r["heads"] * r["vdim"], width, 2.0)
            lin(pr + "g", r["heads"] * r["vdim"], width, 2.0)
            lin(pr + "b", r["heads"], width, 3.0)
            lin(pr + "a", r["heads"], width, 3.0)
            lin(pr + "o", width, r["heads"] * r["vdim"])
            for n, c in (("q", r["kv_heads"] * r["dim"]), ("k", r["kv_heads"] * r["dim"]), ("v", r["heads"] * r["vdim"])):
                W[pr + n + ".conv"] = (torch.randn(c, r["conv"], generator=g) * 0.6).to(torch.bfloat16)
            vec(pr + "A_log", r["heads"], -1.0, 1.0)
            vec(pr + "dt_bias", r["heads"], 0.0, 1.0)
            vec(pr + "norm", r["vdim"])
            vec(pr + "out", width)
        if L.get("mlp"):
            lin(p + "mlp.up", L["mlp"]["ff"], width, 1.5)
            lin(p + "mlp.down", width, L["mlp"]["ff"])
            vec(p + "norm2", width, 0.5)
            lin(p + "rg2", width, width, 2.0)
            vec(p + "rg2.b", width, 0.0, 0.5)
    vec("final.norm", width)
    lin("head", cfg["vocab"], width)
    return W


def mixed_layers():
    L = [general(), parallel(), general(heads=2, dim=40, ff=0), parallel(heads=3, kv_heads=3, dim=20, window=70, rot_dims=20, rheads=2,
                                                                          rkv=2, rdim=72, rvdim=8, conv=2, ff=24)]
    return L + [shared(L, 1), general(heads=5, dim=8)]
