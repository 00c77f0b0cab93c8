"""`bench.py --workload garesun-compare`: prefill and decode throughput of the Garesun design (matrix-state recurrences +
latent attention + mixture of experts, fp32 residual stream) next to the Qwen2 text decoder of the same width, depth and
head size on the native engine - random weights, synthetic token ids, bf16.  Not the headline metric: one JSON line of
its own."""
from __future__ import annotations

import time

import numpy as np
import torch

SIZES = {
    # name: width, heads, head dim, dense intermediate of the comparison decoder, layers (both models), vocab
    "2b-dims": dict(width=1536, heads=12, hd=128, inter=8960, kv_heads=2, layers=6, vocab=32768),
    "7b-dims": dict(width=3584, heads=28, hd=128, inter=18944, kv_heads=4, layers=6, vocab=32768),
}


def garesun_cfg(s):
    H, hd, W = s["heads"], s["hd"], s["width"]
    ff = s["inter"] // 4 // 8 * 8
    mlp = dict(kind="moe", router=dict(experts=8, top=2), expert=dict(ff=ff), shared=dict(ff=ff))
    kinds = [dict(type="mlstm", mixer=dict(heads=H, dim=hd, vdim=hd, gate_cap=12.0)),
             dict(type="latent_attention", mixer=dict(heads=H, dim=hd, rot_dim=64, vdim=hd, kv_rank=512, scale=(hd + 64) ** -0.5,
                                                      rot=dict(base=100000.0, dims=64))),
             dict(type="retention", mixer=dict(heads=H, dim=hd, vdim=hd, decay=[1 - 2.0 ** -(5 + h % 4) for h in range(H)],
                                               rot=dict(base=10000.0, dims=hd)))]
    layers = [dict(kinds[i % 3], mlp=mlp) for i in range(s["layers"])]
    return dict(architecture="Garesun", vocab=s["vocab"], width=W, layers=layers, norm=dict(eps=1e-5), embedding=dict(scale=1.0),
                token_side=dict(dim=64))


def garesun_weights(cfg, dev, seed=0):
    g = torch.Generator(device=dev).manual_seed(seed)
    W, width = {}, cfg["width"]

    def lin(name, o, i):
        W[name] = (torch.randn(o, i, generator=g, device=dev, dtype=torch.float32) * i ** -0.5).to(torch.bfloat16)

    def ones(name, n):
        W[name] = torch.ones(n, dtype=torch.bfloat16, device=dev)

    lin("embed", cfg["vocab"], width)
    lin("head", cfg["vocab"], width)
    ones("final.norm", width)
    sd = cfg["token_side"]["dim"]
    lin("side.embed", cfg["vocab"], sd * len(cfg["layers"]))
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        ones(p + "norm1", width)
        H = m["heads"]
        if L["type"] == "latent_attention":
            lin(p + "mix.q", H * (m["dim"] + m["rot_dim"]), width)
            lin(p + "mix.g", H, width)
            lin(p + "mix.dkv", m["kv_rank"] + m["rot_dim"], width)
            ones(p + "mix.dkv.norm", m["kv_rank"])
            lin(p + "mix.uk", H * m["dim"], m["kv_rank"])
            lin(p + "mix.uv", H * m["vdim"], m["kv_rank"])
        else:
            for n, r in (("q", H * m["dim"]), ("k", H * m["dim"]), ("v", H * m["vdim"]), ("g", H * m["vdim"])):
                lin(p + "mix." + n, r, width)
            if L["type"] == "mlstm":
                lin(p + "mix.i", H, width)
                lin(p + "mix.f", H, width)
                W[p + "mix.i.b"] = torch.zeros(H, dtype=torch.bfloat16, device=dev)
                W[p + "mix.f.b"] = torch.full((H,), 3.0, dtype=torch.bfloat16, device=dev)
                ones(p + "mix.norm", H * m["vdim"])
        lin(p + "mix.o", width, H * m["vdim"])
        E, ff = L["mlp"]["router"]["experts"], L["mlp"]["expert"]["ff"]
        for e in range(E):
            lin(p + f"mlp.e{e}.up", ff, width)
            lin(p + f"mlp.e{e}.down", width, ff)
        lin(p + "mlp.router", E, width)
        lin(p + "mlp.shared.up", L["mlp"]["shared"]["ff"], width)
        lin(p + "mlp.shared.down", width, L["mlp"]["shared"]["ff"])
        lin(p + "side.gate", sd, width)
        lin(p + "side.proj", width, sd)
        ones(p + "side.norm", width)
    return W


def _median_ms(fn, reps=3):
    ts = []
    for _ in range(reps):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        fn()
        torch.cuda.synchronize()
        ts.append((time.perf_counter() - t0) * 1e3)
    return sorted(ts)[len(ts) // 2]


def _measure(lm, embed_ids, vocab, prompt_lens, decode_rows, ctx, steps):
    """prefill ms per prompt length (one sequence), decode ms per step for B rows at context ctx.  `embed_ids(ids [T]) ->
    (inputs, position_ids)` hides what the language model's prefill takes (embeddings or ids)."""
    from mlx_vlm_amd.sample_utils import make_sampler

    out = {"prefill": {}, "decode": {}}
    rng = np.random.default_rng(0)
    for T in prompt_lens:
        ids = rng.integers(0, vocab, T)
        inp, pos = embed_ids(ids)

        def run():
            c = lm.make_cache()
            lm.prefill(inp, pos, [c], [T], "last")
            torch.cuda.synchronize()
            c[0]._seq.release()
        run()
        ms = _median_ms(run)
        out["prefill"][str(T)] = {"ms": round(ms, 3), "tokens_per_s": round(T / ms * 1e3, 1)}
    sargs = make_sampler().engine_args()
    for B in decode_rows:
        caches = lm.make_cache_batch(B)
        ids = rng.integers(0, vocab, B * ctx)
        inp, pos = embed_ids(ids)
        if pos is not None:
            pos = np.concatenate([pos[:, :ctx]] * B, axis=1)
        lm.prefill(inp, pos, caches, [ctx] * B, "last", reserve_extra=3 * steps + 8)
        st = lm.decode_begin(caches, rng.integers(0, vocab, B), np.zeros((B, 1), np.int64), max_new_tokens=3 * steps + 8)
        lm.decode_run(st, 4, sargs)
        ms = _median_ms(lambda: lm.decode_run(st, steps, sargs), reps=2) / steps
        out["decode"][str(B)] = {"ms_per_step": round(ms, 4), "tokens_per_s": round(B / ms * 1e3, 1), "context": ctx}
        for c in caches:
            c[0]._seq.release()
    return out


def workload_garesun_compare(args):
    from mlx_vlm_amd import synthetic
    from mlx_vlm_amd.models import garesun, qwen2_vl

    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    prompt_lens, rows, ctx, steps = (512, 2048), (1, 8), 512, max(8, int(args.steps) * 8)
    res = {}
    for name, s in SIZES.items():
        cfg = garesun_cfg(s)
        gm = garesun.Model(garesun.ModelConfig.from_dict(cfg), device=dev, dtype="bfloat16", kv_pool_tokens=16384, max_seqs=12)
        gm.load_weights(garesun_weights(cfg, dev))
        glm = gm.language_model
        r = {"garesun": _measure(glm, lambda ids: (torch.as_tensor(ids, dtype=torch.int32, device=dev).reshape(-1, 1), None),
                                 s["vocab"], prompt_lens, rows, ctx, steps)}
        r["garesun"]["params_per_layer_M"] = round(sum(v.numel() for k, v in glm._L[0].__dict__.items() if isinstance(v, torch.Tensor)) / 1e6, 1)
        del gm, glm
        torch.cuda.empty_cache()
        qd = dict(synthetic.QWEN2_VL_2B, hidden_size=s["width"], num_hidden_layers=s["layers"], intermediate_size=s["inter"],
                  num_attention_heads=s["heads"], num_key_value_heads=s["kv_heads"], vocab_size=s["vocab"], tie_word_embeddings=False,
                  image_token_id=s["vocab"] - 3, video_token_id=s["vocab"] - 2, vision_start_token_id=s["vocab"] - 4,
                  vision_config=dict(synthetic.QWEN2_VL_2B["vision_config"], depth=1, hidden_size=s["width"]))
        qc = qwen2_vl.ModelConfig.from_dict(qd)
        qm = qwen2_vl.Model(qc, device=dev, kv_pool_tokens=16384, max_seqs=24)
        qm.load_weights(synthetic.random_weights(qc, seed=0, device=dev))
        qlm = qm.language_model

        def q_embed(ids):
            e = qlm.embed_tokens(np.asarray(ids).reshape(1, -1))[0]
            p = np.broadcast_to(np.arange(len(ids))[None], (3, len(ids))).copy()
            return e, p
        r["qwen2"] = _measure(qlm, q_embed, s["vocab"], prompt_lens, rows, ctx, steps)
        del qm, qlm
        torch.cuda.empty_cache()
        r["ratio_garesun_over_qwen2"] = {
            "prefill_" + k: round(r["garesun"]["prefill"][k]["tokens_per_s"] / r["qwen2"]["prefill"][k]["tokens_per_s"], 3) for k in r["qwen2"]["prefill"]}
        r["ratio_garesun_over_qwen2"].update({
            "decode_" + k: round(r["garesun"]["decode"][k]["tokens_per_s"] / r["qwen2"]["decode"][k]["tokens_per_s"], 3) for k in r["qwen2"]["decode"]})
        res[name] = dict(sizes=s, **r)
    return {"metric": "garesun_vs_qwen2_text_decoder", "unit": "tokens/s", "dtype": "bf16", "data": "synthetic", "n_gpus": 1,
            "config": {"layers": "6 per model: (mlstm, latent_attention, retention) x 2 with 8-expert top-2 MoE + shared expert | "
                                 "6 Qwen2 decoder layers", "prompt_lens": list(prompt_lens), "decode_rows": list(rows), "decode_context": ctx},
            "results": res}
