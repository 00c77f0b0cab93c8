"""Small random Garesun checkpoints for the tests: config dicts, bf16 weights with the checkpoint's tensor names, a
folder on disk for the loader.  Sizes are deliberately unequal (dim != vdim, heads differ between layers, rot.dims <
dim, kv_rank not a multiple of 64) so that a swapped size shows."""
from __future__ import annotations

import json
import os

import torch


def layer(kind, **kw):
    if kind == "retention":
        H = kw.get("heads", 3)
        m = dict(heads=H, dim=kw.get("dim", 16), vdim=kw.get("vdim", 24), decay=kw.get("decay", [1 - 2.0 ** -(4 + h) for h in range(H)]),
                 rot=dict(base=kw.get("base", 10000.0), dims=kw.get("rot_dims", 8)))
    elif kind == "mlstm":
        m = dict(heads=kw.get("heads", 2), dim=kw.get("dim", 24), vdim=kw.get("vdim", 40), gate_cap=kw.get("gate_cap", 12.0))
    else:
        D, Dr = kw.get("dim", 24), kw.get("rot_dim", 8)
        m = dict(heads=kw.get("heads", 5), dim=D, rot_dim=Dr, vdim=kw.get("vdim", 16), kv_rank=kw.get("kv_rank", 40),
                 scale=kw.get("scale", (D + Dr) ** -0.5), rot=dict(base=kw.get("base", 50000.0), dims=Dr))
        if "kv_from" in kw:
            m["kv_from"] = kw["kv_from"]
    mlp = kw.get("mlp", "moe")
    if mlp == "moe":
        mlp = dict(kind="moe", router=dict(experts=kw.get("experts", 5), top=kw.get("top", 2)), expert=dict(ff=kw.get("ff", 24)))
        if kw.get("shared_ff", 16):
            mlp["shared"] = dict(ff=kw.get("shared_ff", 16))
    return dict(type=kind, mixer=m, mlp=mlp)


def config(layers, vocab=97, width=72, side=8, scale=2.0, eps=1e-5):
    cfg = dict(architecture="Garesun", vocab=vocab, width=width, layers=layers, norm=dict(eps=eps), embedding=dict(scale=scale))
    if side:
        cfg["token_side"] = dict(dim=side)
    return cfg


def weights(cfg, seed=0, gain=1.0):
    g = torch.Generator().manual_seed(seed)
    W, width = {}, cfg["width"]

    def lin(name, out, inn, s=1.0):
        W[name] = (torch.randn(out, inn, generator=g) * (s * gain / inn ** 0.5)).to(torch.bfloat16)

    def vec(name, n, center=1.0, s=0.1):
        W[name] = (center + s * torch.randn(n, generator=g)).to(torch.bfloat16)

    W["embed"] = (torch.randn(cfg["vocab"], width, generator=g) * 0.5).to(torch.bfloat16)
    side = (cfg.get("token_side") or {}).get("dim", 0)
    if side:
        W["side.embed"] = torch.randn(cfg["vocab"], side * len(cfg["layers"]), generator=g).to(torch.bfloat16)
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        vec(p + "norm1", width)
        H = m["heads"]
        if L["type"] in ("retention", "mlstm"):
            for n, rows in (("q", H * m["dim"]), ("k", H * m["dim"]), ("v", H * m["vdim"]), ("g", H * m["vdim"])):
                lin(p + "mix." + n, rows, width, 2.0)
            lin(p + "mix.o", width, H * m["vdim"])
            if L["type"] == "mlstm":
                lin(p + "mix.i", H, width, 3.0)
                lin(p + "mix.f", H, width, 3.0)
                vec(p + "mix.i.b", H, 0.0, 1.0)
                vec(p + "mix.f.b", H, 2.0, 1.0)
                vec(p + "mix.norm", H * m["vdim"])
        else:
            lin(p + "mix.q", H * (m["dim"] + m["rot_dim"]), width, 2.0)
            lin(p + "mix.g", H, width, 2.0)
            lin(p + "mix.uk", H * m["dim"], m["kv_rank"], 2.0)
            lin(p + "mix.uv", H * m["vdim"], m["kv_rank"])
            lin(p + "mix.o", width, H * m["vdim"])
            if m.get("kv_from") is None:
                lin(p + "mix.dkv", m["kv_rank"] + m["rot_dim"], width, 2.0)
                vec(p + "mix.dkv.norm", m["kv_rank"])
        if L["mlp"]:
            E, ff = L["mlp"]["router"]["experts"], L["mlp"]["expert"]["ff"]
            for e in range(E):
                lin(p + f"mlp.e{e}.up", ff, width, 1.5)
                lin(p + f"mlp.e{e}.down", width, ff)
            lin(p + "mlp.router", E, width, 4.0)
            if L["mlp"].get("shared"):
                lin(p + "mlp.shared.up", L["mlp"]["shared"]["ff"], width, 1.5)
                lin(p + "mlp.shared.down", width, L["mlp"]["shared"]["ff"])
        if side:
            lin(p + "side.gate", side, width)
            lin(p + "side.proj", width, side)
            vec(p + "side.norm", width, 0.3, 0.05)
    vec("final.norm", width)
    lin("head", cfg["vocab"], width)
    return W


def write_checkpoint(folder, cfg, W):
    from safetensors.torch import save_file

    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in W.items()}, os.path.join(folder, "model.safetensors"))
    return folder


MIXED = [layer("mlstm"), layer("latent_attention"), layer("retention"), layer("latent_attention", kv_from=1, heads=3),
         layer("retention", heads=2, dim=40, vdim=8, rot_dims=40, mlp=None), layer("mlstm", heads=3, dim=8, vdim=72, top=1, shared_ff=0)]


def rel_rms(got, want, q=1.0):
    """row-wise rms of the mean-free difference over the rms of the mean-free reference; the worst row, or the q-quantile of
    the rows.  bf16 runs are judged at q < 1: a router logit pair closer than the rounding of a 16-bit activation picks another
    expert for that token, which is a property of the random test weights, not an error."""
    d = got.double() - want.double()
    d = d - d.mean(-1, keepdim=True)
    w = want.double() - want.double().mean(-1, keepdim=True)
    e = (d.pow(2).mean(-1).sqrt() / w.pow(2).mean(-1).sqrt().clamp_min(1e-30)).reshape(-1)
    return e.max().item() if q >= 1.0 else torch.quantile(e, q).item()
