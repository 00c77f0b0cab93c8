"""`bench.py --workload luvapel-compare`: prefill and decode throughput of the Luvapel design (generalized and gated delta
rules, sliding-window attention, dense relu^2 feed-forwards, fp32 residual stream, un-normed readers) next to the framework's
closest model, Garesun (the other hybrid of recurrences and attention on the same ragged step), at the same width, depth,
head count and head size - random weights, synthetic token ids, bf16.  Not the headline metric: one JSON line of its own."""
from __future__ import annotations

import torch

from benchlib.garesun import SIZES, _measure, garesun_cfg, garesun_weights


def luvapel_cfg(s, window=1024):
    H, hd, W = s["heads"], s["hd"], s["width"]
    ff = s["inter"] * 3 // 4 // 8 * 8           # the comparison model runs 2 of 8 experts + a shared one of inter / 4 each
    mlp = dict(kind="dense", ff=ff)
    general = dict(type="general_delta", mixer=dict(heads=H, dim=hd), mlp=mlp)
    par = dict(type="parallel", mlp=mlp,
               mixer=dict(left=dict(heads=H, kv_heads=s["kv_heads"], dim=hd, vdim=hd, scale=hd ** -0.5, rot=dict(base=500000.0, dims=hd // 2),
                                    mask=dict(size=window)),
                          right=dict(heads=H, kv_heads=H // 2, dim=hd, vdim=hd, conv=4)))
    layers = [dict(par if i % 3 == 1 else general) for i in range(s["layers"])]
    return dict(architecture="Luvapel", vocab=s["vocab"], width=W, layers=layers, norm=dict(eps=1e-6), embedding=dict(scale=W ** 0.5))


def luvapel_weights(cfg, dev, seed=0, rank=64):
    g = torch.Generator(device=dev).manual_seed(seed)
    W, width = {}, cfg["width"]

    def lin(name, o, i, s=1.0):
        W[name] = (torch.randn(o, i, generator=g, device=dev, dtype=torch.float32) * (s * i ** -0.5)).to(torch.bfloat16)

    def const(name, n, v=1.0):
        W[name] = torch.full((n,), v, dtype=torch.bfloat16, device=dev)

    lin("embed", cfg["vocab"], width)
    lin("head", cfg["vocab"], width)
    const("final.norm", width)
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        const(p + "norm1", width)
        const(p + "norm2", width)
        for r in ("rg1", "rg2"):
            lin(p + r, width, width, 1.0 / width ** 0.5)
            const(p + r + ".b", width, 0.0)
        if L["type"] == "general_delta":
            HD = m["heads"] * m["dim"]
            for n in ("r", "k", "v", "g", "a"):
                lin(p + "mix." + n, HD, width, 1.0 / width ** 0.5)
            lin(p + "mix.w1", rank, width, 1.0 / width ** 0.5)
            lin(p + "mix.w2", HD, rank)
            const(p + "mix.w0", HD, -2.0)
            const(p + "mix.a.b", HD, 0.0)
            const(p + "mix.norm", HD)
            lin(p + "mix.o", width, HD)
        else:
            a, r = m["left"], m["right"]
            pl, pr = p + "mix.left.", p + "mix.right."
            for n, rows in (("q", a["heads"] * a["dim"]), ("k", a["kv_heads"] * a["dim"]), ("g", a["heads"] * a["dim"])):
                lin(pl + n, rows, width, 1.0 / width ** 0.5)
            lin(pl + "o", width, a["heads"] * a["dim"])
            const(pl + "q.norm", a["dim"])
            const(pl + "k.norm", a["dim"])
            const(pl + "temp", a["heads"])
            const(pl + "out", width)
            for n, rows in (("q", r["kv_heads"] * r["dim"]), ("k", r["kv_heads"] * r["dim"]), ("v", r["heads"] * r["vdim"]),
                            ("g", r["heads"] * r["vdim"]), ("b", r["heads"]), ("a", r["heads"])):
                lin(pr + n, rows, width, 1.0 / width ** 0.5)
            for n, c in (("q", r["kv_heads"] * r["dim"]), ("k", r["kv_heads"] * r["dim"]), ("v", r["heads"] * r["vdim"])):
                lin(pr + n + ".conv", c, r["conv"])
            const(pr + "A_log", r["heads"], -2.0)
            const(pr + "dt_bias", r["heads"], 0.0)
            const(pr + "norm", r["vdim"])
            const(pr + "out", width)
            lin(pr + "o", width, r["heads"] * r["vdim"])
        lin(p + "mlp.up", L["mlp"]["ff"], width, 1.0 / width ** 0.5)
        lin(p + "mlp.down", width, L["mlp"]["ff"])
    return W


def workload_luvapel_compare(args):
    from mlx_vlm_amd.models import garesun, luvapel

    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    prompt_lens, rows, ctx, steps = (512, 2048), (1, 8), 512, max(8, int(args.steps) * 8)
    ids_in = lambda ids: (torch.as_tensor(ids, dtype=torch.int32, device=dev).reshape(-1, 1), None)      # noqa: E731
    res = {}
    for name, s in SIZES.items():
        cfg = luvapel_cfg(s)
        lm_ = luvapel.Model(luvapel.ModelConfig.from_dict(cfg), device=dev, dtype="bfloat16", kv_pool_tokens=16384, max_seqs=12)
        lm_.load_weights(luvapel_weights(cfg, dev))
        r = {"luvapel": _measure(lm_.language_model, ids_in, s["vocab"], prompt_lens, rows, ctx, steps)}
        del lm_
        torch.cuda.empty_cache()
        cfg = garesun_cfg(s)
        gm = garesun.Model(garesun.ModelConfig.from_dict(cfg), device=dev, dtype="bfloat16", kv_pool_tokens=16384, max_seqs=12)
        gm.load_weights(garesun_weights(cfg, dev))
        r["garesun"] = _measure(gm.language_model, ids_in, s["vocab"], prompt_lens, rows, ctx, steps)
        del gm
        torch.cuda.empty_cache()
        r["ratio_luvapel_over_garesun"] = {
            "prefill_" + k: round(r["luvapel"]["prefill"][k]["tokens_per_s"] / r["garesun"]["prefill"][k]["tokens_per_s"], 3) for k in r["garesun"]["prefill"]}
        r["ratio_luvapel_over_garesun"].update({
            "decode_" + k: round(r["luvapel"]["decode"][k]["tokens_per_s"] / r["garesun"]["decode"][k]["tokens_per_s"], 3) for k in r["garesun"]["decode"]})
        res[name] = dict(sizes=s, **r)
    return {"metric": "luvapel_vs_garesun", "unit": "tokens/s", "dtype": "bf16", "data": "synthetic", "n_gpus": 1,
            "config": {"layers": "6 per model: (general_delta, parallel[window attention | gated delta], general_delta) x 2, dense relu^2 "
                                 "feed-forward of 3/4 of the dense intermediate | (mlstm, latent_attention, retention) x 2 with 8-expert "
                                 "top-2 MoE + shared expert", "window": 1024, "prompt_lens": list(prompt_lens), "decode_rows": list(rows),
                       "decode_context": ctx},
            "results": res}
