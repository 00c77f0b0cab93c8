"""Luvapel language model on the HIP operator library (the ragged step of models/ragged.py).

The sublayers read the fp32 stream x itself (rounded once to the serving dtype, `h`); what is normed is their RESULT:
    x <- x + rms(mixer(x) * sigmoid(W_rg1 x + b_rg1)) * w_norm1          x <- x + rms(ff(x) * sigmoid(W_rg2 x + b_rg2)) * w_norm2
Per layer:
    proj = h @ [mixer projections | W_rg1]^T                              one GEMM (rows packed at load)
    general_delta : prepare (unit key, decay through the low-rank map, removal rate) -> delta-rule scan -> head norm, gate
    parallel      : left  = head-normed, rotated q / k, sliding-window softmax attention over the paged k cache whose values
                            are the keys as projected, sigmoid output gate
                    right = short convolutions + silu, unit q / k, gated delta-rule scan, head norm, silu gate
                    result = (rms(left W_o) w_left + rms(right W_o) w_right) / 2
    residual step : gate, RMS norm, add - one kernel, which also rounds the new stream for the next reader
    ff            : h @ [W_up | W_rg2]^T, relu^2, W_down, residual step
A layer with `weights_of` shares another layer's tensors and has a cache / state of its own.
"""
from __future__ import annotations

from types import SimpleNamespace
from typing import Dict

import torch

from ... import _lib, ops
from ..cache import HybridPool, PagedSequence, RecurrentCache
from ..ragged import RaggedLanguageModel, _al8, inv_freq, pack_rows
from .config import ModelConfig


class LanguageModel(RaggedLanguageModel):
    NAME = "Luvapel"

    def __init__(self, config: ModelConfig, **kwargs):
        super().__init__(config, **kwargs)

    # ------------------------------------------------------------------ weights
    def load_weights(self, W: Dict[str, torch.Tensor]):
        cfg, dev, T = self.config, self.device, self.dtype

        def g(name):
            if name not in W:
                raise KeyError(f"Luvapel checkpoint: tensor {name!r} missing")
            return W[name].to(device=dev, dtype=T).contiguous()

        def shaped(t, shape, name):
            if tuple(t.shape) != tuple(shape):
                raise ValueError(f"Luvapel checkpoint: {name} is {tuple(t.shape)}, the config says {tuple(shape)}")
            return t

        Wd = cfg.width
        self._w = dict(embed=shaped(g("embed"), (cfg.vocab, Wd), "embed"), final_norm=shaped(g("final.norm"), (Wd,), "final.norm"),
                       head=shaped(g("head"), (cfg.vocab, Wd), "head"))
        rows, states, aux = {}, {}, {}
        self._L = [None] * len(cfg.layers)
        # layers with tensors of their own first: a borrowing layer may stand before its source
        for i, L in sorted(enumerate(cfg.layers), key=lambda e: (e[1].weights_of is not None, e[0])):
            if L.weights_of is not None:
                ns = SimpleNamespace(**vars(self._L[L.weights_of]))
                if L.type == "parallel":                 # what is no tensor comes from the layer's own entry
                    self._left_constants(ns, L.mixer["left"])
            else:
                p, m = f"l{i}.", L.mixer
                ns = SimpleNamespace(type=L.type, norm1=shaped(g(p + "norm1"), (Wd,), p + "norm1"), rg1b=g(p + "rg1.b"))
                if L.type == "general_delta":
                    H, D = int(m["heads"]), int(m["dim"])
                    ns.H, ns.D = H, D
                    parts = [(n, shaped(g(p + "mix." + n), (H * D, Wd), p + "mix." + n)) for n in ("r", "k", "v", "g", "a")]
                    w1 = g(p + "mix.w1")
                    ns.R = w1.shape[0]
                    parts.append(("w1", w1))
                    ns.w2, ns.w0 = shaped(g(p + "mix.w2"), (H * D, ns.R), p + "mix.w2"), shaped(g(p + "mix.w0"), (H * D,), p + "mix.w0")
                    ns.ab, ns.normw = shaped(g(p + "mix.a.b"), (H * D,), p + "mix.a.b"), shaped(g(p + "mix.norm"), (H * D,), p + "mix.norm")
                    ns.wo = shaped(g(p + "mix.o"), (Wd, H * D), p + "mix.o")
                else:
                    a, r = m["left"], m["right"]
                    ns.aH, ns.aG, ns.aD = int(a["heads"]), int(a["kv_heads"]), int(a["dim"])
                    self._left_constants(ns, a)
                    ns.H, ns.G, ns.D, ns.Dv, ns.taps = int(r["heads"]), int(r["kv_heads"]), int(r["dim"]), int(r["vdim"]), int(r["conv"])
                    pl, pr = p + "mix.left.", p + "mix.right."
                    parts = [("lq", shaped(g(pl + "q"), (ns.aH * ns.aD, Wd), pl + "q")), ("lk", shaped(g(pl + "k"), (ns.aG * ns.aD, Wd), pl + "k")),
                             ("lg", shaped(g(pl + "g"), (ns.aH * ns.aD, Wd), pl + "g")),
                             ("rq", shaped(g(pr + "q"), (ns.G * ns.D, Wd), pr + "q")), ("rk", shaped(g(pr + "k"), (ns.G * ns.D, Wd), pr + "k")),
                             ("rv", shaped(g(pr + "v"), (ns.H * ns.Dv, Wd), pr + "v")), ("rb", shaped(g(pr + "b"), (ns.H, Wd), pr + "b")),
                             ("ra", shaped(g(pr + "a"), (ns.H, Wd), pr + "a")), ("rg", shaped(g(pr + "g"), (ns.H * ns.Dv, Wd), pr + "g"))]
                    ns.qnorm, ns.knorm = shaped(g(pl + "q.norm"), (ns.aD,), pl + "q.norm"), shaped(g(pl + "k.norm"), (ns.aD,), pl + "k.norm")
                    ns.temp = shaped(g(pl + "temp"), (ns.aH,), pl + "temp")
                    ns.left_o, ns.right_o = shaped(g(pl + "o"), (Wd, ns.aH * ns.aD), pl + "o"), shaped(g(pr + "o"), (Wd, ns.H * ns.Dv), pr + "o")
                    ns.left_out, ns.right_out = shaped(g(pl + "out"), (Wd,), pl + "out"), shaped(g(pr + "out"), (Wd,), pr + "out")
                    ns.qconv = shaped(g(pr + "q.conv"), (ns.G * ns.D, ns.taps), pr + "q.conv")
                    ns.kconv = shaped(g(pr + "k.conv"), (ns.G * ns.D, ns.taps), pr + "k.conv")
                    ns.vconv = shaped(g(pr + "v.conv"), (ns.H * ns.Dv, ns.taps), pr + "v.conv")
                    ns.A_log, ns.dt_bias = shaped(g(pr + "A_log"), (ns.H,), pr + "A_log"), shaped(g(pr + "dt_bias"), (ns.H,), pr + "dt_bias")
                    # (one weight of vdim for every head: laid out per head for the finish pass)
                    ns.normw = shaped(g(pr + "norm"), (ns.Dv,), pr + "norm").repeat(ns.H).contiguous()
                parts.append(("rg1", shaped(g(p + "rg1"), (Wd, Wd), p + "rg1")))
                ns.wproj, ns.off = pack_rows(parts, T, dev)
                ns.ff = int(L.mlp["ff"]) if L.mlp is not None else 0
                if ns.ff:
                    ns.wff, ns.foff = pack_rows([("up", shaped(g(p + "mlp.up"), (ns.ff, Wd), p + "mlp.up")),
                                                 ("rg2", shaped(g(p + "rg2"), (Wd, Wd), p + "rg2"))], T, dev)
                    ns.down, ns.rg2b = shaped(g(p + "mlp.down"), (Wd, ns.ff), p + "mlp.down"), g(p + "rg2.b")
                    ns.norm2 = shaped(g(p + "norm2"), (Wd,), p + "norm2")
            if L.type == "general_delta":
                states[i] = (ns.H, ns.D, ns.D, False)
            else:
                states[i] = (ns.H, ns.D, ns.Dv, False)
                rows[(i, "k")] = (ns.aG * ns.aD, torch.float32)           # normed and rotated, never rounded
                rows[(i, "v")] = (ns.aG * ns.aD, T)                       # the keys as projected
                if ns.taps > 1:
                    aux[i] = (ns.taps - 1, 2 * ns.G * ns.D + ns.H * ns.Dv)
            self._L[i] = ns
        self.pool = HybridPool(len(cfg.layers), rows, states, self._kv_pool_tokens, self._max_seqs, device=dev, dtype=T, aux_layers=aux)
        return self

    def _left_constants(self, ns, a):
        ns.scale, ns.rot_dims = float(a["scale"]), int(a["rot"]["dims"])
        ns.window = int(a["mask"]["size"]) if a["mask"]["size"] is not None else 0        # 0: every earlier key is seen
        ns.inv_freq = inv_freq(ns.rot_dims, a["rot"]["base"], self.device) if ns.rot_dims else None

    # ------------------------------------------------------------------ cache
    def make_cache(self):
        seq = PagedSequence(self.pool)
        return [RecurrentCache(seq, i) for i in range(len(self.config.layers))]

    def make_cache_batch(self, n: int):
        return [self.make_cache() for _ in range(n)]

    # ------------------------------------------------------------------ mixers
    def _finish_args(self, a, ns, pl, i, raw, gate, out, H, KH, D, Dv, gate_act):
        a.seg_start, a.seg_slot, a.seg_pos0 = pl.cu.data_ptr(), pl.slot.data_ptr(), pl.pos0.data_ptr()
        a.state, a.raw = self.pool.state[i].data_ptr(), raw.data_ptr()
        a.gate, a.ldg, a.normw, a.gate_act, a.eps = gate.data_ptr(), gate.stride(0), ns.normw.data_ptr(), gate_act, self.config.norm_eps
        a.out, a.ldo = out.data_ptr(), out.stride(0)
        a.H, a.KH, a.D, a.Dv = H, KH, D, Dv

    def _general_delta(self, ns, proj, pl, i, keep):
        """-> [tokens, heads * dim] in the serving dtype: head-normed, weighted, gated read-outs"""
        Tn, H, D, dev = pl.Tn, ns.H, ns.D, self.device
        col = lambda name: proj[:, ns.off[name]:]          # noqa: E731
        f = torch.empty(6, Tn, H * D, dtype=torch.float32, device=dev)
        raw = torch.empty(Tn, H, D, dtype=torch.float32, device=dev)
        out = torch.empty(Tn, H * D, dtype=self.dtype, device=dev)
        a = _lib.DeltaPrepGeneralArgs()
        a.r, a.k, a.v_in, a.a = (col(n).data_ptr() for n in ("r", "k", "v", "a"))
        a.ld, a.a_bias, a.low, a.ld_low = proj.stride(0), ns.ab.data_ptr(), col("w1").data_ptr(), proj.stride(0)
        a.w2, a.w0 = ns.w2.data_ptr(), ns.w0.data_ptr()
        a.q, a.kw, a.kr, a.v, a.w, a.b = (f[j].data_ptr() for j in range(6))
        a.H, a.D, a.R = H, D, ns.R
        ops.delta_prep_general(a, Tn, self.dtype == torch.float32)
        s = _lib.DeltaRuleArgs()
        s.mode = 1
        s.q, s.kw, s.kr, s.v, s.w, s.b = (f[j].data_ptr() for j in range(6))
        s.ldk = s.ldv = H * D
        self._finish_args(s, ns, pl, i, raw, col("g"), out, H, H, D, D, 1)
        ops.delta_rule(s, pl.nseg, Tn, self.dtype == torch.float32)
        keep += [f, raw]
        return out

    def _gated_delta(self, ns, proj, pl, i, keep):
        """-> [tokens, heads * vdim] in the serving dtype"""
        Tn, H, G, D, Dv, dev = pl.Tn, ns.H, ns.G, ns.D, ns.Dv, self.device
        col = lambda name: proj[:, ns.off[name]:]          # noqa: E731
        f32 = torch.float32
        qk = torch.empty(2, Tn, G * D, dtype=f32, device=dev)
        v = torch.empty(Tn, H * Dv, dtype=f32, device=dev)
        bg = torch.empty(2, Tn, H, dtype=f32, device=dev)
        raw = torch.empty(Tn, H, Dv, dtype=f32, device=dev)
        out = torch.empty(Tn, H * Dv, dtype=self.dtype, device=dev)
        a = _lib.DeltaPrepGatedArgs()
        a.q_in, a.k_in, a.v_in, a.b_in, a.a_in = (col(n).data_ptr() for n in ("rq", "rk", "rv", "rb", "ra"))
        a.ld = proj.stride(0)
        a.q_conv, a.k_conv, a.v_conv = ns.qconv.data_ptr(), ns.kconv.data_ptr(), ns.vconv.data_ptr()
        a.A_log, a.dt_bias = ns.A_log.data_ptr(), ns.dt_bias.data_ptr()
        a.conv_state = self.pool.aux[i].data_ptr() if ns.taps > 1 else None
        a.seg_start, a.seg_slot, a.seg_pos0 = pl.cu.data_ptr(), pl.slot.data_ptr(), pl.pos0.data_ptr()
        a.q, a.k, a.v, a.beta, a.g = qk[0].data_ptr(), qk[1].data_ptr(), v.data_ptr(), bg[0].data_ptr(), bg[1].data_ptr()
        a.qscale = float(D) ** -0.5
        a.H, a.KH, a.D, a.Dv, a.taps = H, G, D, Dv, ns.taps
        ops.delta_prep_gated(a, pl.nseg, Tn, self.dtype == f32)
        s = _lib.DeltaRuleArgs()
        s.mode = 0
        s.q, s.kw, s.v, s.beta, s.g = qk[0].data_ptr(), qk[1].data_ptr(), v.data_ptr(), bg[0].data_ptr(), bg[1].data_ptr()
        s.ldk, s.ldv = G * D, H * Dv
        self._finish_args(s, ns, pl, i, raw, col("rg"), out, H, G, D, Dv, 0)
        ops.delta_rule(s, pl.nseg, Tn, self.dtype == f32)
        keep += [qk, v, bg, raw]
        return out

    def _window_attention(self, ns, proj, pl, i, keep):
        """-> [tokens, heads * dim] in the serving dtype: gated attention read-outs (the values are the projected keys)"""
        Tn, H, G, D, dev = pl.Tn, ns.aH, ns.aG, ns.aD, self.device
        col = lambda name: proj[:, ns.off[name]:]          # noqa: E731
        pool, eps = self.pool, self.config.norm_eps
        kpool, vpool = pool.rows[(i, "k")], pool.rows[(i, "v")]
        ops.headnorm_rope_rows(col("lk"), G, D, ns.knorm, eps, ns.rot_dims, ns.inv_freq, pl.tok_pos, kpool, tok_seq=pl.tok_seq,
                               block_table=pool.block_table, raw_pool=vpool)
        q = torch.empty(Tn, H * D, dtype=torch.float32, device=dev)
        ops.headnorm_rope_rows(col("lq"), H, D, ns.qnorm, eps, ns.rot_dims, ns.inv_freq, pl.tok_pos, q)
        out = torch.empty(Tn, H * D, dtype=self.dtype, device=dev)
        # prompt form wherever a step brings more than decode rows, and always in float32 serving - one kernel there, so that
        # a token's bits do not depend on the schedule
        if self.dtype == torch.float32 or Tn > 8:
            ops.window_attn_blocks(q, kpool, vpool, pl.qb_start, pl.qb_count, pl.tok_seq, pl.tok_pos, pool.block_table, H, G, D, D,
                                   ns.scale, out, temp=ns.temp, window=ns.window, gate=col("lg"))
        else:
            ops.window_attn_rows(q, kpool, vpool, pl.tok_seq, pl.tok_pos, pool.block_table, H, G, D, D, ns.scale, out, temp=ns.temp,
                                 window=ns.window, gate=col("lg"))
        keep.append(q)
        return out

    # ------------------------------------------------------------------ the device side of a step
    def _run(self, pl, logits_dtype=torch.float32):
        """Nothing here looks at host data that changes between two steps of the same shape, so a decode step can be
        captured once and replayed."""
        cfg, dev, T = self.config, self.device, self.dtype
        eps = cfg.norm_eps
        x = ops.embed_scale_f32(pl.ids, self._w["embed"], cfg.embedding_scale)
        h = ops.stream_cast(x, T)
        keep = [pl.md, pl.ids]
        for i, ns in enumerate(self._L):
            proj = self._linear(h, ns.wproj)
            rg1 = proj[:, ns.off["rg1"]:]
            if ns.type == "general_delta":
                o = self._general_delta(ns, proj, pl, i, keep)
                y = self._linear(o, ns.wo)
                ops.gated_rms_add_(x, y, ns.norm1, eps, gate=rg1, gate_bias=ns.rg1b, h=h)
                keep += [o, y]
            else:
                ol = self._window_attention(ns, proj, pl, i, keep)
                yl = self._linear(ol, ns.left_o)
                orr = self._gated_delta(ns, proj, pl, i, keep)
                yr = self._linear(orr, ns.right_o)
                ops.gated_rms_add_(x, yl, ns.norm1, eps, gate=rg1, gate_bias=ns.rg1b, b=yr, wa=ns.left_out, wb=ns.right_out, h=h)
                keep += [ol, yl, orr, yr]
            keep.append(proj)
            if ns.ff:
                up = self._linear(h, ns.wff)
                act = ops.relu2_rows(up[:, : ns.ff])
                y2 = self._linear(act, ns.down)
                ops.gated_rms_add_(x, y2, ns.norm2, eps, gate=up[:, ns.foff["rg2"]:], gate_bias=ns.rg2b, h=h)
                keep += [up, act, y2]
            if self._trace is not None:
                self._trace.append(x.clone())
        keep.append(h)
        self._keep = keep
        if pl.rows.size == 0:
            return None
        xl = x if pl.all_rows else x.index_select(0, pl.rows_d.long())
        hn = ops.rms_rows(xl, self._w["final_norm"], eps)
        # rows at a pitch of vocab rounded up to 8: 16-byte aligned bf16 rows for the samplers, whatever the vocabulary
        out = torch.empty(hn.shape[0], _al8(cfg.vocab), dtype=logits_dtype, device=dev)[:, : cfg.vocab]
        return self._linear(hn, self._w["head"], out=out)
